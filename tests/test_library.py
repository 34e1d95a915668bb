"""CPU-side checks of the C-ABI library and the host layer (no GPU, no compute calls)."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355_moe.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    from torchllmtuner_amd import _lib

    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 18
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} is declared in mi355_moe.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes prototype"
    assert set(_lib.SIGNATURES) == set(names)
    assert lib.mi355_moe_abi_version() == _lib.ABI_VERSION == 3
    assert lib.mi355_grouped_tile_m(1) == 256 and lib.mi355_grouped_tile_m(0) == 256


def test_argument_validation_reports_errors_without_a_gpu():
    from torchllmtuner_amd import _lib

    lib = _lib.load()
    # E = 0 is rejected before any launch
    rc = lib.mi355_router_select_fwd(None, None, None, None, None, None, 4, 0, 1, 0, 0, 1.0, 0, 0, 0, None)
    assert rc == -1
    assert b"E=0" in lib.mi355_moe_last_error()
    rc = lib.mi355_permute_plan(None, 4, 2, 8, 5, 3, 1, 128, None, None, None, None, None, None, 8, None,
                                None, None, 2, None, None)
    assert rc == -1 and b"local range" in lib.mi355_moe_last_error()
    with pytest.raises(ValueError, match="local range"):
        _lib.check(rc, "permute_plan")


def test_gather_entry_points_reject_unaddressable_token_matrices_without_launching():
    """The fused token gather addresses its source with 32-bit byte offsets and clamps the
    index to [0, num_tokens): a token matrix of 4 GiB or more, or an index with no rows to
    point at, is MI355_EINVAL from every entry point that takes token_of_row -- checked on
    the host, before anything is launched (this test runs without a GPU; the pointers are
    never dereferenced)."""
    from torchllmtuner_amd import _lib

    lib = _lib.load()
    p = 0x1000  # any non-null value
    El, D, F, R, tiles = 4, 2048, 768, 1024, 16
    too_many = (1 << 32) // (D * 2)  # T * D * 2 == 2^32 bytes
    for T, needle in ((too_many, b"exceeds the 4 GiB"), (0, b"num_tokens = 0")):
        rc = lib.mi355_grouped_swiglu_fwd(p, p, T, p, p, p, 1, p, p, p, p, p, tiles, p, p, p, p, El, D, F, R, None)
        assert rc == -1 and needle in lib.mi355_moe_last_error(), lib.mi355_moe_last_error()
        rc = lib.mi355_grouped_swiglu_bwd(p, p, p, T, p, p, p, p, p, p, 1, p, p, p, p, p, tiles, p, p, p, p, p, p,
                                          El, D, F, R, None)
        assert rc == -1 and needle in lib.mi355_moe_last_error()
        rc = lib.mi355_grouped_swiglu_stage(1, p, p, p, T, p, p, p, p, p, p, p, p, p, p, p, p, tiles, p, p, p, p, p,
                                            p, El, D, F, R, None)
        assert rc == -1 and needle in lib.mi355_moe_last_error()
        rc = lib.mi355_grouped_swiglu_combine_bwd(p, p, p, T, p, p, p, p, p, p, 1, p, p, p, p, p, tiles, p, p, p, p,
                                                  p, p, p, p, El, D, F, R, 0, None)
        assert rc == -1 and needle in lib.mi355_moe_last_error()
    # fp32 rows cannot be gathered at all
    rc = lib.mi355_grouped_swiglu_fwd(p, p, 8, p, p, p, 0, p, p, p, p, p, tiles, p, p, p, p, El, D, F, R, None)
    assert rc == -3 and b"bf16 only" in lib.mi355_moe_last_error()  # MI355_EUNSUP, as the header says
    # gate and up are omitted together or not at all, and only where the bf16 MFMA path runs
    rc = lib.mi355_grouped_swiglu_fwd(p, None, 8, p, p, p, 1, p, p, p, p, p, tiles, None, p, p, p, El, D, F, R, None)
    assert rc == -1 and b"together" in lib.mi355_moe_last_error()
    rc = lib.mi355_grouped_swiglu_fwd(p, None, 8, p, p, p, 0, p, p, p, p, p, tiles, None, None, p, p, El, D, F, R, None)
    assert rc == -1 and b"can only be omitted" in lib.mi355_moe_last_error()
    # the allocation-free plan refuses what its built-in scratch cannot hold
    assert lib.mi355_permute_plan_static_max_bytes() == 8 << 20
    rc = lib.mi355_permute_plan_static(p, 1 << 20, 8, 128, 0, 128, 1, 256, p, p, p, p, p, p, 1 << 23, p, p, p,
                                       1 << 16, None)
    assert rc == -1 and b"built-in array holds" in lib.mi355_moe_last_error()


def test_ops_refuse_cpu_tensors():
    from torchllmtuner_amd import ops

    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.router_gate_fwd(torch.zeros(2, 4), torch.zeros(3, 4))
    with pytest.raises(TypeError, match="float32 and bfloat16"):
        ops._dt(torch.zeros(1, dtype=torch.float16))
    assert ops._dt(torch.zeros(1, dtype=torch.float64)) == 2  # MI355_F64
    with pytest.raises(TypeError, match="float32 and bfloat16, got torch.float64"):
        ops._dt(torch.zeros(1, dtype=torch.float64), fp64=False)  # kernels without an fp64 form (rms_norm)


def test_module_surface_matches_the_reference_block():
    """Constructor validation, parameter names and buffers of the block
    (llmtuner/models/common/moe/layer.py:109-193, routing.py:64-144, experts.py:87-120)."""
    from torchllmtuner_amd import moe

    with pytest.raises(ValueError, match="num_limited_groups must be set"):
        moe.TokenChoiceTopKRouter(8, 16, 2, num_expert_groups=2)
    with pytest.raises(ValueError, match="must be divisible by num_expert_groups"):
        moe.TokenChoiceTopKRouter(8, 16, 2, num_expert_groups=3, num_limited_groups=1)
    with pytest.raises(ValueError, match="cannot exceed num_expert_groups"):
        moe.TokenChoiceTopKRouter(8, 16, 2, num_expert_groups=2, num_limited_groups=5)
    with pytest.raises(ValueError, match="must be >= 2"):
        moe.TokenChoiceTopKRouter(8, 16, 2, num_expert_groups=8, num_limited_groups=1)
    with pytest.raises(ValueError, match="top_k must be in"):
        moe.TokenChoiceTopKRouter(4, 16, 5)
    with pytest.raises(ValueError, match="Unknown score function"):
        moe.TokenChoiceTopKRouter(4, 16, 1, score_func="relu")
    for field in ("dim", "hidden_dim", "num_experts"):
        opts = {"dim": 4, "hidden_dim": 8, "num_experts": 2}
        opts[field] = True
        with pytest.raises(ValueError, match=field + " must be positive integer"):
            moe.GroupedExperts(**opts)
    with pytest.raises(TypeError, match="use_grouped_mm must be bool or None"):
        moe.GroupedExperts(4, 8, 2, use_grouped_mm=1)
    with pytest.raises(ValueError, match="pad_multiple"):
        moe.PaddedTokenDispatcher(4, 2, pad_multiple=0)

    router = moe.TokenChoiceTopKRouter(8, 16, 2, score_func="softmax", route_norm=True)
    experts = moe.RoutedExperts(moe.GroupedExperts(16, 32, 8), moe.LocalTokenDispatcher(8, 2))
    with pytest.raises(ValueError, match="must match router.num_experts"):
        moe.MoE(4, experts, router)
    with pytest.raises(ValueError, match="load_balance_coeff must be finite and positive"):
        moe.MoE(8, experts, router, load_balance_coeff=0.0)
    block = moe.MoE(8, experts, router, shared_experts=moe.DenseSwiGLU(16, 32))
    assert list(block.state_dict()) == [
        "expert_bias_E",
        "routed_experts.inner_experts.w1_EFD",
        "routed_experts.inner_experts.w3_EFD",
        "routed_experts.inner_experts.w2_EDF",
        "router.gate.weight",
        "shared_experts.gate_proj.weight",
        "shared_experts.up_proj.weight",
        "shared_experts.down_proj.weight",
    ]
    ie = block.routed_experts.inner_experts
    assert ie.w1_EFD.shape == (8, 32, 16) and ie.w3_EFD.shape == (8, 32, 16) and ie.w2_EDF.shape == (8, 16, 32)
    assert router.gate.bias is None and router.gate.weight.shape == (8, 16)
    # statistics buffers stay fp32 under a bf16 cast; the counter is not persistent
    block = block.to(torch.bfloat16)
    assert block.expert_bias_E.dtype == torch.float32 and block.tokens_per_expert_E.dtype == torch.float32
    assert "tokens_per_expert_E" not in block.state_dict()
    assert moe.MoE(8, experts, router, load_balance_coeff=None).expert_bias_E is None
    assert list(block.expert_parallel_parameters()) == list(ie.parameters())


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """A C99 translation unit that includes the header, takes the address of every declared
    entry point and links against the shared library: the boundary a cgo / JNI / ctypes binding
    sees has no C++ or torch types in it."""
    import shutil
    import subprocess

    from torchllmtuner_amd import _lib

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    _lib.load()
    names = _declared_functions()
    src = tmp_path / "abi.c"
    src.write_text(
        '#include "mi355_moe.h"\n#include <stdio.h>\nint main(void) {\n  const void* fns[] = {\n'
        + "".join(f"    (const void*)&{n},\n" for n in names)
        + '  };\n  printf("%d %d\\n", (int)(sizeof(fns) / sizeof(fns[0])), mi355_moe_abi_version());\n  return 0;\n}\n'
    )
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
         "-L", libdir, "-lmi355moe", f"-Wl,-rpath,{libdir}"],
        check=True, capture_output=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert out == [str(len(names)), str(_lib.ABI_VERSION)]


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: any other --gpus value exits with a message and no JSON line."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) and "{" not in r.stdout
