"""The allocation-free plan entry point (mi355_permute_plan_static) against
mi355_permute_plan, through the C ABI: every output array bit for bit, on two calls in a row
that share the library's built-in scratch -- the second one smaller, so stale scratch from the
first call would show -- plus a padded one-rank-share layout, and the size limit."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _plan(lib, entry, ids, E, lo, hi, align, workspace):
    T, K = ids.shape
    N, El, tm = T * K, hi - lo, 256
    row_cap = N + (El * (align - 1) if align > 1 else 0)
    tile_cap = N // tm + El + 1
    i32 = dict(dtype=torch.int32, device=DEV)
    # filled with a sentinel so that "never written" cannot pass for "equal"
    out = {name: torch.full((n,), -7, **i32) for name, n in (
        ("counts_E", E), ("seg_offsets", El + 1), ("seg_counts", 2 * El), ("row_of_slot", N), ("slot_of_row", row_cap),
        ("token_of_row", row_cap), ("tile_expert", tile_cap), ("tile_row0", tile_cap), ("num_tiles", 1))}
    p = lambda k: out[k].data_ptr()
    args = [ids.data_ptr(), T, K, E, lo, hi, align, tm, p("counts_E"), p("seg_offsets"), p("seg_counts"),
            p("row_of_slot"), p("slot_of_row"), p("token_of_row"), row_cap, p("tile_expert"), p("tile_row0"),
            p("num_tiles"), tile_cap]
    if workspace is not None:
        args.append(workspace.data_ptr())
    stream = torch.cuda.current_stream().cuda_stream
    rc = getattr(lib, entry)(*args, stream)
    assert rc == 0, lib.mi355_moe_last_error()
    torch.cuda.synchronize()
    nt = int(out["num_tiles"])
    out["tile_expert"], out["tile_row0"] = out["tile_expert"][:nt], out["tile_row0"][:nt]
    return out


def test_static_plan_equals_the_workspace_plan_on_consecutive_calls():
    from torchllmtuner_amd import _lib

    lib = _lib.load()
    g = torch.Generator().manual_seed(21)
    cases = [  # (T, K, E, lo, hi, align): large first, then smaller ones over the same scratch
        (8192, 8, 128, 0, 128, 1),
        (700, 4, 16, 0, 16, 1),
        (1500, 6, 64, 8, 24, 16),
        (0, 2, 4, 0, 4, 1),
    ]
    for T, K, E, lo, hi, align in cases:
        print(f"static plan T={T} K={K} E={E} [{lo},{hi}) align={align}", flush=True)
        ids = torch.randint(0, E, (T, K), generator=g).to(DEV)
        nbytes = lib.mi355_permute_plan_workspace_bytes(T, K, E)
        assert nbytes <= lib.mi355_permute_plan_static_max_bytes()
        ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        want = _plan(lib, "mi355_permute_plan", ids, E, lo, hi, align, ws)
        got = _plan(lib, "mi355_permute_plan_static", ids, E, lo, hi, align, None)
        for name in want:
            assert torch.equal(got[name], want[name]), name
        # and it is the stable argsort (not merely equal to the other entry point)
        if align == 1 and (lo, hi) == (0, E):
            assert torch.equal(got["slot_of_row"].long().cpu(), torch.argsort(ids.reshape(-1).cpu(), stable=True))
    # beyond the built-in scratch: a clear refusal, nothing launched
    rc = lib.mi355_permute_plan_static(ids.data_ptr(), 1 << 20, 8, 128, 0, 128, 1, 256, *([ids.data_ptr()] * 6), 1 << 23,
                                       *([ids.data_ptr()] * 3), 1 << 16, None)
    assert rc == -1 and b"built-in array holds" in lib.mi355_moe_last_error()
