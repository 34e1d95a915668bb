#!/usr/bin/env python3
"""Benchmark: MoE layer forward+backward tokens/s at the Qwen3-30B-A3B shape.

One step = one forward + backward of the MoE block (router, permute, grouped
SwiGLU experts, combine and every gradient: dX, dW1/dW3/dW2, dW_router) over one
batch of T tokens that is already resident in HBM.  Prints one JSON line.

Besides the whole-step rate it reports, for the dominant kernel, the achieved
fraction of its roofline (timed alone with HIP events on the launch stream) and a
CPU baseline: the oracle restatement of the reference block timed on this
machine's host cores over a bounded token sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM bytes per launch at the default workload, measured with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (scaled by a 256 MiB copy: x2.0 and x1.0); the table these come from is
# profiles/moe_layer_qwen3_t8192_hbm_traffic.txt.  Only reported for the default workload.
MEASURED_HBM_BYTES = {
    "gate_up": 1511.8e6, "down": 844.8e6, "dh": 1255.4e6, "drows": 1434.6e6,
    "dw2": 828.0e6, "dw1": 895.9e6, "dw3": 895.9e6,
}

WORKLOADS = {
    # name: T, D, E, K, F
    "qwen3-30b-a3b-moe-layer fwd+bwd T=8192 bf16": dict(T=8192, D=2048, E=128, K=8, F=768),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=1024)
    ap.add_argument("--stage-iters", type=int, default=10)
    ap.add_argument("--no-probe", action="store_true",
                    help="skip the sustained-MFMA probe (about 0.8 s of matrix-core work)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (known traffic, for scaling rocprof FETCH_SIZE / WRITE_SIZE)")
    return ap.parse_args()


def time_events(fn, iters, warmup=2):
    """Average milliseconds of ``fn`` with HIP events on the current (launch) stream."""
    import torch

    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def sustained_mfma(dev):
    """What the matrix cores hold on v_mfma_f32_32x32x16_bf16 with register-resident
    operands of random bits (libmi355probe.so): rate and core clock, both under the
    card's own power management.  Returns None when the probe library is not built."""
    import ctypes

    import torch

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "torchllmtuner_amd", "libmi355probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.mi355_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_void_p]
    lib.mi355_probe_mfma.restype = ctypes.c_int
    blocks = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2 * blocks, dtype=torch.int64, device=dev)
    out = {}
    # 16x16x32 is the shape of the row-tiled grouped GEMMs, 32x32x16 that of the weight gradients
    for shape, name, iters in ((1, "16x16x32", 50000), (0, "32x32x16", 100000)):
        out[name] = {}
        for label, rnd in (("random_bits", 1), ("constant_bits", 0)):
            def launch():
                rc = lib.mi355_probe_mfma(sink.data_ptr(), clocks.data_ptr(), blocks, iters, rnd, shape,
                                          torch.cuda.current_stream().cuda_stream)
                assert rc == 0
            ms = time_events(launch, 2, warmup=1)
            flops = blocks * 8.0 * iters * 262144 * (shape + 1)
            c = clocks.view(blocks, 2).double()
            out[name][label] = {"TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1),
                                "core_clock_mhz": round(float((c[:, 0] / c[:, 1]).mean()) * 100.0, 0)}
    return out


def cpu_baseline(cfg, sample_tokens):
    """The oracle's forward+backward on host cores over ``sample_tokens`` tokens."""
    import torch

    from oracle import moe_ref as R
    from tests.helpers import make_params

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    D, E, K, F = cfg["D"], cfg["E"], cfg["K"], cfg["F"]
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=0)
    for name in ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF"):
        getattr(p, name).requires_grad_()

    def run(tokens):
        x = torch.randn(tokens, D, generator=torch.Generator().manual_seed(0)).bfloat16().requires_grad_()
        g = torch.randn(tokens, D, generator=torch.Generator().manual_seed(1)).bfloat16()
        t0 = time.perf_counter()
        out, _ = R.moe_forward(x, p, spec)
        out.backward(g)
        return time.perf_counter() - t0

    run(128)  # warm-up: thread pool, allocator
    dt = run(sample_tokens)
    return {
        "value": sample_tokens / dt,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"oracle fwd+bwd, {sample_tokens} tokens of the same layer (D={D},E={E},K={K},F={F}), "
                  f"bf16, 1 run after a 128-token warm-up, {dt:.2f} s",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    from oracle import moe_ref as R
    from tests.helpers import build_block, make_params
    from torchllmtuner_amd import ops

    name = next(iter(WORKLOADS))
    cfg = dict(WORKLOADS[name])
    cfg["T"] = args.tokens
    T, D, E, K, F = cfg["T"], cfg["D"], cfg["E"], cfg["K"], cfg["F"]
    dev = "cuda:0"
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=0)
    block = build_block(p, spec, D, F, torch.bfloat16, dev)
    block.train()
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0)).bfloat16().to(dev)
    gout = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).bfloat16().to(dev)

    def step():
        block.zero_grad(set_to_none=True)
        xin = x.detach().requires_grad_()
        out = block(xin)
        out.backward(gout)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = T * args.steps / dt

    # ---- per-kernel timing on the launch stream ---------------------------------
    with torch.no_grad():
        scores, ids = block.router.route(x)
        plan = block.routed_experts.token_dispatcher.plan(ids)
        rows = ops.permute_rows_fwd(x, plan)
        ie = block.routed_experts.inner_experts
        w1, w3, w2 = ie.w1_EFD.detach(), ie.w3_EFD.detach(), ie.w2_EDF.detach()
        y, gate, up, h = ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)
        dy, _ = ops.combine_bwd(gout, y, scores, plan)
        # as in the training step: the token matrix is read through the gather index
        # (gate/up A operand, dW1/dW3 B operand); no expert-major copy of the tokens
        buf = dict(rows=x, token_of_row=plan.token_of_row, w1=w1, w3=w3, w2=w2, gate=gate, up=up, h=h, y=y, dy=dy,
                   dgate=torch.empty_like(gate), dup=torch.empty_like(up), drows=torch.empty_like(rows),
                   dw1=torch.empty_like(w1), dw3=torch.empty_like(w3), dw2=torch.empty_like(w2))
        R_rows = int(plan.total_rows.item())
        it = args.stage_iters
        # The step's backward folds the combine into the expert kernels: dH reads the output
        # gradient through the token index and scales rows in its epilogue, dW2 contracts the
        # gathered rows with score * h.  Those two are timed in that form.
        folded = ops.combine_bwd_slots(x.dtype, D, F) > 0
        if folded:
            buf.update(dout=gout, row_scale=ops.combine_row_scale(scores, plan), hs=torch.empty_like(h),
                       dot_partial=torch.empty(rows.shape[0], ops.combine_bwd_slots(x.dtype, D, F),
                                               dtype=torch.float32, device=dev))

        def run_stage(s):
            if folded and s in ("dh", "dw2"):
                ops.grouped_swiglu_combine_stage(s, buf, plan)
            else:
                ops.grouped_swiglu_stage(s, buf, plan)

        stage_ms = {s: time_events(lambda s=s: run_stage(s), it) for s in ops.STAGES}
        logits = ops.router_gate_fwd(x, block.router.gate.weight)
        other_ms = {
            "router_gate_fwd": time_events(lambda: ops.router_gate_fwd(x, block.router.gate.weight), it),
            "router_select_fwd": time_events(lambda: ops.router_select_fwd(logits, None, K, "softmax", True, 1.0), it),
            "permute_plan": time_events(lambda: ops.permute_plan(ids, E), it),
            "permute_rows_fwd": time_events(lambda: ops.permute_rows_fwd(x, plan), it),
            "combine_fwd": time_events(lambda: ops.combine_fwd(y, scores, plan), it),
            "combine_bwd": time_events(lambda: ops.combine_bwd(gout, y, scores, plan), it),
            "permute_rows_bwd": time_events(lambda: ops.permute_rows_bwd(buf["drows"], plan), it),
            "router_gate_bwd": time_events(lambda: ops.router_gate_bwd(logits, x, block.router.gate.weight), it),
        }
        if folded:
            other_ms["combine_row_scale"] = time_events(lambda: ops.combine_row_scale(scores, plan), it)
            other_ms["combine_scores_bwd"] = time_events(lambda: ops.combine_scores_bwd(buf["dot_partial"], plan), it)
        # the callers' side of the path, outside the timed step: the decoder layer's norm in
        # front of the block and the statistics of a quantile-balanced router
        norm_w = torch.ones(D, dtype=torch.bfloat16, device=dev)
        normed, rstd = ops.rms_norm_fwd(x, norm_w, 1e-6)
        q_bias = torch.zeros(E, dtype=torch.float32, device=dev)
        _, _, q_scores, q_cut = ops.router_select_cutoff_fwd(logits, q_bias, K, "sigmoid", True, 1.0)
        q_hist = torch.zeros(E, 1000, dtype=torch.int64, device=dev)
        outside_ms = {
            "rms_norm_fwd": time_events(lambda: ops.rms_norm_fwd(x, norm_w, 1e-6), it),
            "rms_norm_bwd": time_events(lambda: ops.rms_norm_bwd(gout, x, norm_w, rstd), it),
            "router_select_cutoff_fwd": time_events(
                lambda: ops.router_select_cutoff_fwd(logits, q_bias, K, "sigmoid", True, 1.0), it),
            "quantile_observe": time_events(lambda: ops.quantile_observe(q_hist, q_scores, q_cut, q_bias), it),
        }
        other_ms.update(outside_ms)
    # algorithmic work per launch (padding excluded): 2*R*D*F per projection
    proj = 2.0 * R_rows * D * F
    stage_flops = {"gate_up": 2 * proj, "down": proj, "dh": proj, "drows": 2 * proj,
                   "dw2": proj, "dw1": proj, "dw3": proj}
    s_bytes = 2
    other_bytes = {
        "permute_rows_fwd": T * D * s_bytes + R_rows * D * s_bytes + 4 * R_rows,
        "combine_fwd": R_rows * D * s_bytes + 8 * T * K + T * D * s_bytes,
        "combine_bwd": T * D * s_bytes + 2 * R_rows * D * s_bytes + 4 * T * K,
        "permute_rows_bwd": R_rows * D * s_bytes + T * D * s_bytes,
        "rms_norm_fwd": 2 * T * D * s_bytes,
        "rms_norm_bwd": 3 * T * D * s_bytes,
    }
    kernels = {}
    for s, ms in stage_ms.items():
        tf = stage_flops[s] / (ms * 1e-3) / 1e12
        kernels[f"grouped_{s}"] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1), "frac_mfma": round(tf / PEAK_BF16_TFLOPS, 4)}
    for s, ms in other_ms.items():
        ent = {"ms": round(ms, 4)}
        if s == "permute_rows_fwd" or (s == "combine_bwd" and folded) or s in outside_ms:
            # permute_rows_fwd, combine_bwd: public dispatcher API only, the step gathers inside
            # the GEMMs and folds the combine's backward into them; the others belong to the
            # block's callers
            ent["in_step"] = False
        if s in other_bytes:
            gbs = other_bytes[s] / (ms * 1e-3) / 1e9
            ent.update({"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)})
        kernels[s] = ent
    dominant = max(stage_ms, key=stage_ms.get)
    ach = stage_flops[dominant] / (stage_ms[dominant] * 1e-3) / 1e12
    gemm_flops = sum(stage_flops.values())
    gemm_ms = sum(stage_ms.values())
    roofline = {
        "kernel": f"grouped_{dominant}",
        "bound": "mfma",
        "achieved": round(ach, 2),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(ach / PEAK_BF16_TFLOPS, 4),
        "traffic": MEASURED_HBM_BYTES.get(dominant) if T == 8192 else None,
        "avg_launch_ms": round(stage_ms[dominant], 4),
        "all_grouped_gemms": {"TFLOP/s": round(gemm_flops / (gemm_ms * 1e-3) / 1e12, 1),
                              "frac": round(gemm_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)},
    }

    probe = None if args.no_probe else sustained_mfma(dev)
    if probe is not None:
        # the same instruction with operands in registers: the rate the card holds under
        # its own power management, next to the data-sheet peak above
        roofline["sustained_mfma"] = probe
        shape = "32x32x16" if dominant.startswith("dw") else "16x16x32"
        roofline["frac_of_sustained"] = round(ach / probe[shape]["random_bits"]["TFLOP/s"], 4)

    if not args.no_probe:
        # The vendor library's dense GEMM with the dominant kernel's flops (all rows against
        # ONE expert's gate and up weights, random values, no SwiGLU, no routing): what a
        # tuned kernel holds on this card at this size, next to the data-sheet peak.
        a = torch.randn(R_rows, D, device=dev).bfloat16()
        b = torch.randn(2 * F, D, device=dev).bfloat16()
        ms = time_events(lambda: torch.mm(a, b.t()), 10, warmup=3)
        roofline["vendor_dense_gemm"] = {"shape_mnk": [R_rows, 2 * F, D], "ms": round(ms, 4),
                                         "TFLOP/s": round(2.0 * R_rows * 2 * F * D / (ms * 1e-3) / 1e12, 1)}
        del a, b

    result = {
        "metric": "MoE layer fwd+bwd tokens/s (Qwen3-30B-A3B shape, 1 GPU)",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": name if T == 8192 else f"{name} (tokens overridden to {T})",
                   "tokens": T, "hidden": D, "experts": E, "top_k": K, "moe_intermediate": F,
                   "router": "fp32 softmax top-k, norm_topk_prob", "routed_rows": R_rows},
        "roofline": roofline,
        "kernels": kernels,
    }
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
