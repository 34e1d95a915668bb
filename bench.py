#!/usr/bin/env python3
"""Benchmark: MoE layer tokens/s on one MI355X, at each of the five workload shapes.

One step = one pass of the MoE block (router, permute, grouped SwiGLU experts, combine; with
the backward every gradient: dX, dW1/dW3/dW2, dW_router, shared-expert weights) over one batch
of tokens that is already resident in HBM.  Prints one JSON line.

``--workload c3`` (the default) is the headline: the Qwen3-30B-A3B-shaped layer, T=8192,
forward + backward in bf16.  c1 (tiny fp32), c2 (forward only), c4 (T=16384, skewed routing,
128-row padded segments) and c5 (DeepSeek-V3 shape, one rank's expert share, shared expert) are
the other configurations; all are built by ``torchllmtuner_amd.workloads`` from the product's
own modules.

Besides the whole-step rate the line carries per-kernel times (HIP events on the launch
stream), the roofline fraction of the kernel that takes the largest share of the step, and a
CPU baseline: the oracle restatement of the reference block timed on this machine's host cores
over a bounded token sample (warm-up, then the median of three runs).
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3   # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

PROFILE_TRAFFIC = {"c3": "moe_layer_qwen3_t8192_hbm_traffic.txt",
                   "c4": "moe_layer_qwen3_t16384_skewed_padded_hbm_traffic.txt",
                   "c5": "moe_layer_deepseek_v3_local_share_t4096_hbm_traffic.txt"}


def measured_traffic(workload):
    """HBM bytes per launch of the grouped stages as rocprofv3 counted them (FETCH_SIZE and
    WRITE_SIZE, scaled by a copy of known size), read from the summary under profiles/: its
    lines ``traffic <stage> <bytes>`` and ``measured at commit <sha>``.  Nothing is assumed when
    the file or a stage is missing: the figure belongs to the commit the file names, not to
    the run that prints it."""
    name = PROFILE_TRAFFIC.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return {}, None
    table, commit = {}, None
    for line in open(path):
        f = line.split()
        if len(f) == 3 and f[0] == "traffic":
            try:
                table[f[1]] = float(f[2])
            except ValueError:
                pass
        elif line.startswith("measured at commit") and len(f) >= 4:
            commit = f[3]
    return table, commit


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["c1", "c2", "c3", "c4", "c5"], default="c3")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=512)
    ap.add_argument("--stage-iters", type=int, default=10)
    ap.add_argument("--no-probe", action="store_true",
                    help="skip the sustained-MFMA probe (about 0.8 s of matrix-core work) and the vendor GEMM")
    ap.add_argument("--power", action="store_true",
                    help="also loop each grouped GEMM, the whole step, the vendor GEMM, the MFMA probe and a copy for "
                         "--power-seconds each while sampling the card's power sensor (hwmon); adds a \"power\" object")
    ap.add_argument("--power-seconds", type=float, default=2.5)
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the same step")
    ap.add_argument("--single-workload", dest="all_workloads", action="store_false",
                    help="measure --workload only (default: the other four configurations follow it, a short run "
                         "each, and are summarised under \"workloads\")")
    ap.add_argument("--settle-steps", type=int, default=30,
                    help="untimed steps before the warm-up that bring the card from its idle clocks to the ones it holds")
    ap.add_argument("--other-steps", type=int, default=20)
    ap.add_argument("--other-warmup", type=int, default=10)
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


def time_sequence(fns, iters, warmup=2):
    """Average milliseconds of each launch in ``fns`` (name -> callable), launched round after
    round in the given order -- the order of a training step -- with HIP events around every
    launch.  A kernel timed back to back with itself runs under a different power and cache
    state than in the step (the matrix-core kernels measure up to a fifth slower that way on
    this card); timed in sequence, the averages agree with a profiler's view of the step."""
    import torch

    for _ in range(warmup):
        for fn in fns.values():
            fn()
    events = {name: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                     for _ in range(iters)] for name in fns}
    torch.cuda.synchronize()
    for i in range(iters):
        for name, fn in fns.items():
            start, stop = events[name][i]
            start.record()
            fn()
            stop.record()
    torch.cuda.synchronize()
    return {name: sum(a.elapsed_time(b) for a, b in pairs) / iters for name, pairs in events.items()}


def mfma_probe(dev):
    """(launch(shape, random_bits, iters), blocks, clocks) over bench_probe/libmi355probe.so, or
    None when the probe is not built.  shape 1 = 16x16x32, 0 = 32x32x16."""
    import ctypes

    import torch

    path = os.path.join(ROOT, "bench_probe", "libmi355probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.mi355_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_void_p]
    lib.mi355_probe_mfma.restype = ctypes.c_int
    blocks = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2 * blocks, dtype=torch.int64, device=dev)

    def launch(shape, rnd, iters):
        rc = lib.mi355_probe_mfma(sink.data_ptr(), clocks.data_ptr(), blocks, iters, rnd, shape,
                                  torch.cuda.current_stream().cuda_stream)
        assert rc == 0

    return launch, blocks, clocks


def sustained_mfma(dev):
    """What the matrix cores hold on the two MFMA shapes the grouped GEMMs use, with
    register-resident operands of random bits (bench_probe/libmi355probe.so): rate and core
    clock, both under the card's own power management.  None when the probe is not built."""
    probe = mfma_probe(dev)
    if probe is None:
        return None
    run, blocks, clocks = probe
    out = {}
    # 16x16x32 is the shape of the row-tiled grouped GEMMs, 32x32x16 that of the weight gradients
    for shape, name, iters in ((1, "16x16x32", 50000), (0, "32x32x16", 100000)):
        out[name] = {}
        for label, rnd in (("random_bits", 1), ("constant_bits", 0)):
            ms = time_events(lambda: run(shape, rnd, iters), 2, warmup=1)
            flops = blocks * 8.0 * iters * 262144 * (shape + 1)
            c = clocks.view(blocks, 2).double()
            out[name][label] = {"TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1),
                                "core_clock_mhz": round(float((c[:, 0] / c[:, 1]).mean()) * 100.0, 0)}
    return out


def power_table(cases, seconds):
    """Average socket power (W) while each callable of ``cases`` runs in a loop for ``seconds``,
    read from the amdgpu hwmon sensor every 20 ms (the first 0.8 s of each loop are dropped: the
    sensor averages).  ``None`` in ``cases`` means idle.  Returns None when no sensor is readable."""
    import glob
    import threading

    import torch

    def read(path):
        try:
            return int(open(path).read().strip())
        except (OSError, ValueError):
            return None

    sensor = cap = None
    for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
        for name in ("power1_average", "power1_input"):
            if read(os.path.join(h, name)) is not None:
                sensor, cap = os.path.join(h, name), read(os.path.join(h, "power1_cap"))
                break
        if sensor:
            break
    if sensor is None:
        return None

    def sample(stop, out):
        while not stop.is_set():
            v = read(sensor)
            if v is not None:
                out.append((time.time(), v / 1e6))
            time.sleep(0.02)

    table = {}
    for name, fn in cases.items():
        out, stop = [], threading.Event()
        th = threading.Thread(target=sample, args=(stop, out))
        th.start()
        t0, n = time.time(), 0
        if fn is None:
            time.sleep(min(seconds, 1.5))
        else:
            while time.time() - t0 < seconds:
                for _ in range(20):
                    fn()
                torch.cuda.synchronize()
                n += 20
        dt = time.time() - t0
        stop.set()
        th.join()
        watts = [w for t, w in out if t - t0 > 0.8] or [w for _, w in out]
        table[name] = {"watts": round(sum(watts) / max(len(watts), 1), 1)}
        if n:
            table[name]["ms_per_call_looped"] = round(dt / n * 1e3, 4)
    return {"sensor": sensor, "cap_watts": None if cap is None else cap / 1e6, "cases": table}


def hip_graph_step(block, x, gout, wl, steps, warmup):
    """The same step captured once as a HIP graph and replayed ``steps`` times: what a caller
    gets who removes the host's per-kernel work (about thirty launches per step).  Every kernel
    of the block is asynchronous, allocates through PyTorch's allocator only and never reads a
    size back to the host, so the whole forward + backward captures as it is.  Returns
    ms per step, or a string saying why the capture failed."""
    import torch

    try:
        params = [p for p in block.parameters() if p.requires_grad]
        xin = x.detach().clone().requires_grad_(wl.backward)

        def step():
            if wl.backward:
                return torch.autograd.grad(block(xin), [xin] + params, gout)
            with torch.no_grad():
                return block(xin)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = step()  # noqa: F841  (the graph's output buffers stay alive with it)
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3
    except Exception as e:  # the eager figure stands on its own
        return f"{type(e).__name__}: {e}"


def cpu_baseline(wl, sample_tokens):
    """The oracle's pass (forward, + backward where the workload has one) on host cores at the
    workload's FULL token count: a short warm-up, then one timed run, reported as tokens/s.
    A second, small sample (``sample_tokens`` tokens) is timed beside it as ``fixed_cost_s``: the
    oracle's time hardly depends on the token count at the large shapes (its per-expert loop, like
    the reference's, indexes the stacked weights, so autograd materialises a full (E, F, D)
    gradient per expert and projection), which is why a rate taken over a sample would be an
    artefact of the sample's size."""
    import torch

    from oracle import moe_ref as R
    from torchllmtuner_amd import workloads as W

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)

    def runner(wl, dtype):
        w = W.make_weights(wl)
        cast = lambda t: t.to(dtype)
        p = R.MoEParams(router_w_ED=w["router"].clone(), w1_EFD=cast(w["w1"]), w3_EFD=cast(w["w3"]),
                        w2_EDF=cast(w["w2"]))
        if wl.shared_hidden_dim:
            p.shared_gate_FD, p.shared_up_FD, p.shared_down_DF = (cast(w[k]) for k in
                                                                  ("shared_gate", "shared_up", "shared_down"))
        if wl.expert_bias:
            p.expert_bias_E = w["expert_bias"]
        leaves = [getattr(p, n) for n in ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF", "shared_gate_FD", "shared_up_FD",
                                          "shared_down_DF") if getattr(p, n) is not None]
        for t in leaves:
            t.requires_grad_(wl.backward)
        spec = R.RouterSpec(wl.num_experts, wl.top_k, score_func=wl.score_func, route_norm=wl.route_norm,
                            route_scale=wl.route_scale, num_expert_groups=wl.num_expert_groups,
                            num_limited_groups=wl.num_limited_groups)
        kw = {}
        if wl.pad_multiple:
            kw["pad_multiple"] = wl.pad_multiple
        if wl.local_experts:
            kw["local_experts"] = wl.local_experts

        def run(n):
            x = torch.randn(n, wl.dim, generator=torch.Generator().manual_seed(0)).to(dtype).requires_grad_(wl.backward)
            g = torch.randn(n, wl.dim, generator=torch.Generator().manual_seed(1)).to(dtype)
            for t in leaves:
                t.grad = None
            t0 = time.perf_counter()
            with torch.set_grad_enabled(wl.backward):
                out, _ = R.moe_forward(x, p, spec, **kw)
                if wl.backward:
                    out.backward(g)
            return time.perf_counter() - t0

        return run

    name = {torch.float32: "fp32", torch.bfloat16: "bf16"}[wl.dtype]
    run = runner(wl, wl.dtype)
    small = min(sample_tokens, wl.tokens)
    run(min(128, wl.tokens))  # warm-up: thread pool, allocator
    if wl.tokens <= 1024:
        times = [run(wl.tokens) for _ in range(3)]
        full_s, how = statistics.median(times), f"median of 3 runs ({', '.join(f'{t:.3f}' for t in times)} s)"
    else:
        full_s = run(wl.tokens)
        how = f"one run ({full_s:.2f} s)"
    out = {
        "value": round(wl.tokens / full_s, 2),
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "seconds": round(full_s, 3),
        "sample": f"oracle {'fwd+bwd' if wl.backward else 'fwd'} of the whole {wl.key} layer at its full size, "
                  f"T={wl.tokens} (D={wl.dim},E={wl.num_experts},K={wl.top_k},F={wl.hidden_dim}), {name}, after a "
                  f"128-token warm-up: {how}",
    }
    if small < wl.tokens:
        fixed = run(small)
        out["fixed_cost_s"] = round(fixed, 3)
        out["fixed_cost_note"] = (f"the same pass over {small} tokens takes {fixed:.2f} s: most of the oracle's time "
                                  f"at this shape does not scale with the token count, so only the full-size run "
                                  f"above is a rate")
    if wl.key != "c1":
        c1 = W.WORKLOADS["c1"]
        run1 = runner(c1, c1.dtype)
        run1(c1.tokens)
        times1 = [run1(c1.tokens) for _ in range(3)]
        out["c1_full_size"] = {"value": round(c1.tokens / statistics.median(times1), 1), "unit": "tokens/s",
                               "sample": f"oracle fwd+bwd of the whole C1 block (T={c1.tokens}, fp32), median of 3"}
    return out


def swiglu_stage_bytes(rows, experts, D, F, s, saves_gate_up=True, dh_writes_scaled_h=True):
    """Algorithmic HBM bytes of each grouped SwiGLU stage: every operand and every result once
    (``rows`` routed rows or tokens, ``experts`` weight sets of (F, D), element size ``s``;
    ``dh_writes_scaled_h``: the combine's backward is folded into dH, which then also writes
    score * h for dW2)."""
    x, a, w = rows * D * s, rows * F * s, experts * D * F * s
    return {
        "gate_up": x + 2 * w + (3 if saves_gate_up else 1) * a,  # rows, w1, w3 -> (gate, up,) h
        "down": a + w + x,                                         # h, w2 -> y
        "dh": x + w + 2 * a + (3 if dh_writes_scaled_h else 2) * a,  # dy, w2, gate, up -> dgate, dup(, score * h)
        "drows": 2 * a + 2 * w + x,                                # dgate, dup, w1, w3 -> drows
        "dw2": x + a + w,                                          # dy, h -> dW2
        "dw1": x + a + w,                                          # rows, dgate -> dW1
        "dw3": x + a + w,                                          # rows, dup -> dW3
    }


def per_kernel_times(args, wl, block, x, gout, dev):
    """HIP-event averages of the kernels of one step, each launched alone on the buffers of a
    real step.  Returns (kernels, stage_ms, stage_flops, routed_rows)."""
    import torch

    from torchllmtuner_amd import ops

    it = args.stage_iters
    T, D, E, K, F = x.shape[0], wl.dim, wl.num_experts, wl.top_k, wl.hidden_dim
    s_bytes = x.element_size()
    peak = PEAK_BF16_TFLOPS if wl.dtype == torch.bfloat16 else PEAK_FP32_TFLOPS
    with torch.no_grad():
        scores, ids = block.router.route(x, block.expert_bias_E)
        plan = block.routed_experts.token_dispatcher.plan(ids)
        R_rows = int(plan.seg_counts.sum().item())       # real rows
        R_cover = int(plan.total_rows.item())            # rows in use, padding included
        ie = block.routed_experts.inner_experts
        w1, w3, w2 = ie.w1_EFD.detach(), ie.w3_EFD.detach(), ie.w2_EDF.detach()
        rows = ops.permute_rows_fwd(x, plan)
        y, gate, up, h = ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)
        dy, _ = ops.combine_bwd(gout, y, scores, plan)
        logits = ops.router_gate_fwd(x, block.router.gate.weight, block.router.gate.bias)
        proj = 2.0 * R_rows * D * F
        stage_flops = {"gate_up": 2 * proj, "down": proj, "dh": proj, "drows": 2 * proj,
                       "dw2": proj, "dw1": proj, "dw3": proj}
        if not wl.backward:
            stage_flops = {k: stage_flops[k] for k in ("gate_up", "down")}
        n_local = (wl.local_experts[1] - wl.local_experts[0]) if wl.local_experts else E
        stage_bytes = swiglu_stage_bytes(R_rows, n_local, D, F, s_bytes, saves_gate_up=wl.backward)
        stage_ms = {}
        folded = ops.gather_supported(x, F) and ops.combine_bwd_slots(x.dtype, D, F) > 0
        if folded:
            # as in the step: the token matrix is read through the gather index (gate/up A operand,
            # dW1/dW3 B operand), dH reads the output gradient through it and scales rows in its
            # epilogue, dW2 contracts the gathered rows with score * h
            buf = dict(rows=x, token_of_row=plan.token_of_row, w1=w1, w3=w3, w2=w2, gate=gate, up=up, h=h, y=y,
                       dy=dy, dgate=torch.empty_like(gate), dup=torch.empty_like(up), drows=torch.empty_like(rows),
                       dw1=torch.empty_like(w1), dw3=torch.empty_like(w3), dw2=torch.empty_like(w2),
                       dout=gout, row_scale=ops.combine_row_scale(scores, plan), hs=torch.empty_like(h),
                       dot_partial=torch.empty(rows.shape[0], ops.combine_bwd_slots(x.dtype, D, F),
                                               dtype=torch.float32, device=dev))

            if not wl.backward:
                # as in a step without gradients: gate and up are not written
                buf["gate"] = buf["up"] = None

            def run_stage(s):
                if s in ("dh", "dw2"):
                    ops.grouped_swiglu_combine_stage(s, buf, plan)
                else:
                    ops.grouped_swiglu_stage(s, buf, plan)

            stage_fns = {s: (lambda s=s: run_stage(s)) for s in stage_flops}
            drows = buf["drows"]
        else:
            # fp32 / odd shapes: the generic kernels, timed per call (forward: gate, up, SwiGLU, down;
            # backward: dh, SwiGLU', drows, three weight gradients)
            stage_flops = {"experts_fwd": 3 * proj}
            stage_fns = {"experts_fwd": lambda: ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)}
            if wl.backward:
                stage_flops["experts_bwd"] = 6 * proj
                stage_fns["experts_bwd"] = lambda: ops.grouped_swiglu_bwd(dy, rows, w1, w3, w2, gate, up, h, plan)
            drows = torch.empty_like(rows)
        gw, gb = block.router.gate.weight, block.router.gate.bias
        sel = lambda: ops.router_select_fwd(logits, block.expert_bias_E, K, wl.score_func, wl.route_norm,
                                            wl.route_scale, wl.num_expert_groups or 0, wl.num_limited_groups or 0,
                                            want_map=True)
        lo, hi = wl.local_experts or (0, E)
        shared_fns, shared_flops, shared_bytes = {}, {}, {}
        if wl.shared_hidden_dim and ops.gather_supported(x, wl.shared_hidden_dim):
            # the shared expert: a dense SwiGLU over all tokens on the same kernels (one segment)
            sh = block.shared_experts
            Fs = wl.shared_hidden_dim
            sp = ops.segments_from_counts(torch.full((1,), T, dtype=torch.int32, device=dev), T)
            s1, s3, s2 = (w.detach().unsqueeze(0) for w in (sh.gate_proj.weight, sh.up_proj.weight, sh.down_proj.weight))
            sy, sg, su, shh = ops.grouped_swiglu_fwd(x, s1, s3, s2, sp)
            sbuf = dict(rows=x, w1=s1, w3=s3, w2=s2, gate=sg, up=su, h=shh, y=sy, dy=gout,
                        dgate=torch.empty_like(sg), dup=torch.empty_like(su), drows=torch.empty_like(x),
                        dw1=torch.empty_like(s1), dw3=torch.empty_like(s3), dw2=torch.empty_like(s2))
            sproj = 2.0 * T * D * Fs
            shared_flops = {"gate_up": 2 * sproj, "down": sproj, "dh": sproj, "drows": 2 * sproj, "dw2": sproj,
                            "dw1": sproj, "dw3": sproj}
            shared_bytes = swiglu_stage_bytes(T, 1, D, Fs, s_bytes, dh_writes_scaled_h=False)
            if not wl.backward:
                shared_flops = {k: shared_flops[k] for k in ("gate_up", "down")}
            shared_fns = {s: (lambda s=s: ops.grouped_swiglu_stage(s, sbuf, sp)) for s in shared_flops}
        # ---- the launches of one step, in the step's order
        fwd_stages = [s for s in stage_fns if s in ("gate_up", "down", "experts_fwd")]
        bwd_stages = [s for s in stage_fns if s not in fwd_stages]
        seq = {"router_gate_fwd": lambda: ops.router_gate_fwd(x, gw, gb), "router_select_fwd": sel,
               "permute_plan": lambda: ops.permute_plan(ids, E, lo, hi, wl.pad_multiple or 1)}
        if not folded:
            seq["permute_rows_fwd"] = lambda: ops.permute_rows_fwd(x, plan)
        seq.update({f"grouped_{s}": stage_fns[s] for s in fwd_stages})
        seq["combine_fwd"] = lambda: ops.combine_fwd(y, scores, plan)
        seq.update({f"shared_{s}": shared_fns[s] for s in shared_fns if s in ("gate_up", "down")})
        if wl.backward:
            seq.update({f"shared_{s}": shared_fns[s] for s in shared_fns if s not in ("gate_up", "down")})
            if folded:
                seq["combine_row_scale"] = lambda: ops.combine_row_scale(scores, plan)
                order = [s for s in ("dh", "drows") if s in bwd_stages]
                seq.update({f"grouped_{s}": stage_fns[s] for s in order})
                seq["permute_rows_bwd"] = lambda: ops.permute_rows_bwd(drows, plan)
                seq["combine_scores_bwd"] = lambda: ops.combine_scores_bwd(buf["dot_partial"], plan)
                seq.update({f"grouped_{s}": stage_fns[s] for s in bwd_stages if s not in order})
            else:
                seq["combine_bwd"] = lambda: ops.combine_bwd(gout, y, scores, plan)
                seq.update({f"grouped_{s}": stage_fns[s] for s in bwd_stages})
                seq["permute_rows_bwd"] = lambda: ops.permute_rows_bwd(drows, plan)
            seq["router_select_bwd"] = lambda: ops.router_select_bwd(logits, ids, scores, None, wl.score_func,
                                                                     wl.route_norm, wl.route_scale)
            seq["router_gate_bwd"] = lambda: ops.router_gate_bwd(logits, x, gw)
        seq_ms = time_sequence(seq, it)
        stage_ms = {s: seq_ms[f"grouped_{s}"] for s in stage_fns}
        shared_ms = {s: seq_ms[f"shared_{s}"] for s in shared_fns}
        in_step = {k for k in seq if not k.startswith(("grouped_", "shared_"))}
        other_ms = {k: seq_ms[k] for k in in_step}
        # the public dispatcher API's movers, which the fused step does not launch
        if "permute_rows_fwd" not in other_ms:
            other_ms["permute_rows_fwd"] = time_events(lambda: ops.permute_rows_fwd(x, plan), it)
        if wl.backward and "combine_bwd" not in other_ms:
            other_ms["combine_bwd"] = time_events(lambda: ops.combine_bwd(gout, y, scores, plan), it)
        # the callers' side of the path, outside the timed step: the decoder layer's norm in
        # front of the block and the statistics of a quantile-balanced router
        outside_ms = {}
        if wl.key == "c3":
            norm_w = torch.ones(D, dtype=x.dtype, device=dev)
            _, rstd = ops.rms_norm_fwd(x, norm_w, 1e-6)
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
    other_bytes = {
        "permute_rows_fwd": T * D * s_bytes + R_cover * D * s_bytes + 4 * T * K,
        "combine_fwd": R_rows * D * s_bytes + 8 * T * K + T * D * s_bytes,
        "combine_bwd": T * D * s_bytes + 2 * R_rows * D * s_bytes + 4 * T * K,
        "permute_rows_bwd": R_rows * D * s_bytes + T * D * s_bytes,
        "rms_norm_fwd": 2 * T * D * s_bytes,
        "rms_norm_bwd": 3 * T * D * s_bytes,
    }
    kernels = {}

    def gemm_entry(ms, flops, nbytes):
        # both sides of the roofline: the product's flops against the MFMA peak and its algorithmic
        # bytes against the HBM peak; the one that bounds it is decided by flops per byte
        tf = flops / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
        ent = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1), "frac_mfma": round(tf / peak, 4)}
        if nbytes and ms > 0:
            gbs = nbytes / (ms * 1e-3) / 1e9
            ent.update({"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4),
                        "flop_per_byte": round(flops / nbytes, 1)})
        return ent

    for s, ms in stage_ms.items():
        kernels[f"grouped_{s}"] = gemm_entry(ms, stage_flops[s], stage_bytes.get(s) if folded else None)
    for s, ms in shared_ms.items():
        kernels[f"shared_{s}"] = gemm_entry(ms, shared_flops[s], shared_bytes.get(s))
    for s, ms in other_ms.items():
        ent = {"ms": round(ms, 4)}
        if s not in in_step:
            # public dispatcher API / the block's callers: not launched by the timed step
            ent["in_step"] = False
        if s in other_bytes:
            gbs = other_bytes[s] / (ms * 1e-3) / 1e9
            ent.update({"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)})
        kernels[s] = ent
    return (kernels, stage_ms, stage_flops, shared_ms, shared_flops, R_rows, folded, stage_fns,
            stage_bytes if folded else {}, shared_bytes)


def measure_workload(args, wl, steps, warmup, *, detail):
    """Build the block of ``wl``, time ``steps`` whole steps after ``warmup`` and each kernel of a
    step.  ``detail``: also the HIP-graph replay, the MFMA probe and the vendor GEMM (the
    headline workload); without it only what the summary of the other workloads needs."""
    import torch

    from torchllmtuner_amd import workloads as W

    dev = "cuda:0"
    x_cpu, gout_cpu = W.make_inputs(wl)
    block = W.build_block(wl, dev, x_for_skew=x_cpu)
    block.train(wl.backward)
    x, gout = x_cpu.to(dev), gout_cpu.to(dev)
    T = wl.tokens

    if wl.backward:
        # (gradients dropped through a list made once, as an optimizer's zero_grad does: walking the
        # module tree on every step costs 30 us of host time, a tenth of the smallest workload's step)
        params = list(block.parameters())

        def step():
            for p in params:
                p.grad = None
            xin = x.detach().requires_grad_()
            out = block(xin)
            out.backward(gout)
    else:
        def step():
            with torch.no_grad():
                block(x)

    # The card leaves its idle clocks over the first fifteen or so steps of a process (at C3:
    # 3.4, 3.1, 2.9, 2.75 ... ms, level from the fifteenth on), whatever the caller's warm-up
    # count: settle first, untimed, then do the W warm-up steps and time exactly K.
    for _ in range(args.settle_steps):
        step()
    torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / steps * 1e3
    tokens_per_s = T * steps / dt

    graph_ms = None if (args.no_graph or not detail) else hip_graph_step(block, x, gout, wl, steps, warmup)

    x2, g2 = x.reshape(-1, wl.dim), gout.reshape(-1, wl.dim)
    (kernels, stage_ms, stage_flops, shared_ms, shared_flops, R_rows, folded, stage_fns, stage_bytes,
     shared_bytes) = per_kernel_times(
        args, wl, block, x2, g2, dev)
    peak = PEAK_BF16_TFLOPS if wl.dtype == torch.bfloat16 else PEAK_FP32_TFLOPS

    # The kernel with the largest share of the step.  dW1 and dW3 are two launches of one kernel
    # (the gathered weight gradient), so they count together; the shared expert's stages are
    # launches of the same kernels over one dense segment and are listed under their own names.
    groups = {}
    for s in stage_ms:
        key = "dw1+dw3" if s in ("dw1", "dw3") else s
        g = groups.setdefault(f"grouped_{key}", {"ms": 0.0, "flops": 0.0, "launches": 0, "bytes": 0.0})
        g["ms"] += stage_ms[s]; g["flops"] += stage_flops[s]; g["launches"] += 1; g["bytes"] += stage_bytes.get(s, 0.0)
    for s in shared_ms:
        key = "dw1+dw3" if s in ("dw1", "dw3") else s
        g = groups.setdefault(f"shared_{key}", {"ms": 0.0, "flops": 0.0, "launches": 0, "bytes": 0.0})
        g["ms"] += shared_ms[s]; g["flops"] += shared_flops[s]; g["launches"] += 1; g["bytes"] += shared_bytes.get(s, 0.0)
    dominant = max(groups, key=lambda k: groups[k]["ms"])
    dg = groups[dominant]
    ach = dg["flops"] / (dg["ms"] * 1e-3) / 1e12
    gemm_flops = sum(stage_flops.values()) + sum(shared_flops.values())
    gemm_ms = sum(stage_ms.values()) + sum(shared_ms.values())
    traffic = traffic_commit = None
    tb, traffic_commit = measured_traffic(wl.key)
    if dominant.startswith("grouped_"):
        parts = dominant[len("grouped_"):].split("+")
        if parts and all(p in tb for p in parts):
            traffic = sum(tb[p] for p in parts) / len(parts)
    # The grouped and shared-expert products are matrix-core work: the fraction is their flops
    # (2*R*D*F per projection over real rows, padding excluded) per second against the dense
    # bf16 MFMA peak.  Their algorithmic bytes against the HBM peak, the flops per byte and the
    # ridge of the two published peaks (2500 TFLOP/s / 8 TB/s = 312 flop/B in bf16) are kept
    # beside it: at these shapes the products sit close to the ridge.
    ridge = peak * 1e12 / (PEAK_HBM_GBS * 1e9)
    intensity = dg["flops"] / dg["bytes"] if dg["bytes"] else None
    ach_gbs = dg["bytes"] / (dg["ms"] * 1e-3) / 1e9 if dg["bytes"] else None
    roofline = {
        "kernel": dominant,
        "launches_per_step": dg["launches"],
        "share_of_step": round(dg["ms"] / ms_per_step, 4),
        "bound": "mfma",
        "achieved": round(ach, 2),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(ach / peak, 4),
        "frac_mfma": round(ach / peak, 4),
        "frac_hbm": None if ach_gbs is None else round(ach_gbs / PEAK_HBM_GBS, 4),
        "flop_per_byte": None if intensity is None else round(intensity, 1),
        "ridge_flop_per_byte": round(ridge, 1),
        "algorithmic_bytes_per_launch": None if not dg["bytes"] else round(dg["bytes"] / dg["launches"]),
        "traffic": traffic,
        "traffic_measured_at_commit": traffic_commit if traffic is not None else None,
        "avg_launch_ms": round(dg["ms"] / dg["launches"], 4),
        "all_grouped_gemms": {"TFLOP/s": round(gemm_flops / (gemm_ms * 1e-3) / 1e12, 1),
                              "frac": round(gemm_flops / (gemm_ms * 1e-3) / 1e12 / peak, 4),
                              "ms": round(gemm_ms, 4)},
    }

    probe = None if (args.no_probe or not detail or wl.dtype != torch.bfloat16) else sustained_mfma(dev)
    if probe is not None:
        # the same instruction with operands in registers: the rate the card holds under
        # its own power management, next to the data-sheet peak above
        roofline["sustained_mfma"] = probe
        shape = "32x32x16" if "dw" in dominant else "16x16x32"
        roofline["frac_of_sustained"] = round(ach / probe[shape]["random_bits"]["TFLOP/s"], 4)
        # The vendor library's dense GEMM with the gate/up kernel's flops (all rows against ONE
        # expert's gate and up weights, random values, no SwiGLU, no routing): what a tuned
        # kernel holds on this card at this size, next to the data-sheet peak.
        a = torch.randn(max(R_rows, 1), wl.dim, device=dev).bfloat16()
        b = torch.randn(2 * wl.hidden_dim, wl.dim, device=dev).bfloat16()
        ms = time_events(lambda: torch.mm(a, b.t()), 10, warmup=3)
        roofline["vendor_dense_gemm"] = {"shape_mnk": [a.shape[0], 2 * wl.hidden_dim, wl.dim], "ms": round(ms, 4),
                                         "TFLOP/s": round(2.0 * a.shape[0] * 2 * wl.hidden_dim * wl.dim / (ms * 1e-3) / 1e12, 1)}
        del a, b

    config = W.describe(wl)
    config["routed_rows"] = R_rows
    if getattr(block, "skew_top20_share", None) is not None:
        config["skew_top20_share_solved"] = round(block.skew_top20_share, 4)
    if wl.zipf_top20_share:
        with torch.no_grad():
            _, ids = block.router.route(x2)
        load = torch.bincount(ids.reshape(-1), minlength=wl.num_experts).sort(descending=True).values
        config["load_histogram_sorted"] = {"max": int(load[0]), "median": int(load[wl.num_experts // 2]),
                                           "min": int(load[-1]),
                                           "top20_share": round(float(load[: wl.num_experts // 5].sum()) / ids.numel(), 4)}
    metric = ("MoE layer fwd+bwd tokens/s (Qwen3-30B-A3B shape, 1 GPU)" if wl.key == "c3"
              else f"MoE layer {'fwd+bwd' if wl.backward else 'fwd'} tokens/s ({wl.key}, 1 GPU)")
    result = {
        "metric": metric,
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if wl.dtype == torch.bfloat16 else "fp32",
        "data": "synthetic",
        "config": config,
        "roofline": roofline,
        "kernels": kernels,
    }
    if isinstance(graph_ms, float):
        # the same K steps replayed from one captured HIP graph (value / ms_per_step above are the eager calls)
        result["hip_graph"] = {"ms_per_step": round(graph_ms, 4), "tokens_per_s": round(T / (graph_ms * 1e-3), 1)}
    elif graph_ms is not None:
        result["hip_graph"] = {"error": graph_ms[:300]}
    if args.power and detail:
        cases = {"idle": None}
        cases.update({f"grouped_{s}": fn for s, fn in stage_fns.items()})
        cases["whole_step"] = step
        if wl.dtype == torch.bfloat16:
            a = torch.randn(max(R_rows, 1), wl.dim, device=dev).bfloat16()
            b = torch.randn(2 * wl.hidden_dim, wl.dim, device=dev).bfloat16()
            cases["vendor_dense_gemm"] = lambda: torch.mm(a, b.t())
            pl = mfma_probe(dev)
            if pl is not None:
                # operands in registers: matrix cores alone, with random and with constant operand bits
                cases["mfma_probe_16x16x32_random_bits"] = lambda: pl[0](1, 1, 2000)
                cases["mfma_probe_16x16x32_constant_bits"] = lambda: pl[0](1, 0, 2000)
        big = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        big2 = torch.empty_like(big)
        cases["copy_1GiB"] = lambda: big2.copy_(big)
        result["power"] = power_table(cases, args.power_seconds)
        if result["power"] is not None:
            for name, ent in result["power"]["cases"].items():
                key = name[len("grouped_"):]
                if key in stage_flops and "ms_per_call_looped" in ent:
                    ent["TFLOP/s_looped"] = round(stage_flops[key] / (ent["ms_per_call_looped"] * 1e-3) / 1e12, 1)
            if "vendor_dense_gemm" in result["power"]["cases"]:
                ent = result["power"]["cases"]["vendor_dense_gemm"]
                ent["TFLOP/s_looped"] = round(2.0 * a.shape[0] * b.shape[0] * wl.dim / (ent["ms_per_call_looped"] * 1e-3) / 1e12, 1)
            for name, ent in result["power"]["cases"].items():
                if name.startswith("mfma_probe"):
                    ent["TFLOP/s_looped"] = round(pl[1] * 8.0 * 2000 * 262144 * 2 / (ent["ms_per_call_looped"] * 1e-3) / 1e12, 1)
            ent = result["power"]["cases"]["copy_1GiB"]
            ent["GB/s_looped"] = round(2.0 * (1 << 30) / (ent["ms_per_call_looped"] * 1e-3) / 1e9, 1)
    return result


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    import gc

    import torch

    from torchllmtuner_amd import workloads as W

    wl = W.WORKLOADS[args.workload]
    result = measure_workload(args, wl, args.steps, args.warmup, detail=True)
    if args.all_workloads:
        # the other four configurations, a short run each (no CPU leg, no probe, no graph): whole-step
        # rate and the grouped products together against the MFMA peak; the top-level keys stay
        # those of the workload chosen above
        summary = {}
        for key in ("c1", "c2", "c3", "c4", "c5"):
            if key == wl.key:
                r = result
            else:
                gc.collect()
                torch.cuda.empty_cache()
                r = measure_workload(args, W.WORKLOADS[key], args.other_steps, args.other_warmup, detail=False)
            summary[key] = {"workload": r["config"]["workload"], "steps": r["steps"], "ms_per_step": r["ms_per_step"],
                            "tokens_per_s": r["value"],
                            "all_grouped_gemms_frac": r["roofline"]["all_grouped_gemms"]["frac"],
                            "all_grouped_gemms_TFLOP/s": r["roofline"]["all_grouped_gemms"]["TFLOP/s"],
                            "dtype": r["dtype"]}
        result["workloads"] = summary
        gc.collect()
        torch.cuda.empty_cache()
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(wl, args.cpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
