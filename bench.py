#!/usr/bin/env python3
"""Benchmark of the fused SAE decoder-loss path on one MI355X.

One "step" = forward + backward of the HierarchicalTopK loss through the public API
(``triton_hierarchical_sae_loss(...)``; ``loss.backward()``) on one batch of synthetic input that
is already resident in HBM.  Default workload: B=4096, F=65536, D=2304, K=128, bf16 tensors with
fp32 arithmetic, per-row unique uniform indices.  The TopK loss is timed on the same inputs for
the latency ratio, the two dominant kernels are timed alone with HIP events for the roofline
object, and a torch restatement of the reference's eager path is timed on the host cores on a
bounded row sample as the CPU baseline.

Prints ONE JSON line on stdout.  ``python bench.py`` = ``--gpus 1 --steps 100 --warmup 5``, the
protocol of the reference's timing script (5 warm-up + 100 timed iterations, events around
``loss = f(...); loss.backward()``, mean and standard deviation; reference example.py:30-36, 70-101).
"""
import argparse
import ctypes
import json
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
# what the "algorithmic_frac_of_peak" figures of whole steps and of the forward kernel are
ALGORITHMIC_NOTE = ("algorithmic bytes / time / 8 TB/s: every gathered row counted once per sweep whether HBM or a "
                    "cache served it, so this is not an HBM utilisation and exceeds 1 where hot rows come from the "
                    "L2 (skewed indices) or the weights fit the memory-side cache; roofline.traffic holds the "
                    "counter-measured bytes of the dominant kernel")

WORKLOADS = {
    # name: (B, K, F, D, dtype, index distribution, weight std)
    "c2_k128": (4096, 128, 65536, 2304, "bf16", "unique", 1.0),
    "c2_k64": (4096, 64, 65536, 2304, "bf16", "unique", 1.0),
    "c2_k32": (4096, 32, 65536, 2304, "bf16", "unique", 1.0),
    "c3": (2048, 256, 131072, 1024, "fp32", "randint", 1.0),
    "c4": (8192, 64, 262144, 4096, "bf16", "zipf", 0.02),
    "c5": (16384, 128, 524288, 8192, "bf16", "unique", 0.02),
    "c1": (64, 32, 4096, 256, "fp32", "randint", 1.0),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2_k128", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", default="", help="override B,K,F,D of the workload (tuning aid)")
    ap.add_argument("--dtype", default="", choices=["", "bf16", "fp16", "fp32"],
                    help="override the storage dtype of the workload (tuning aid)")
    ap.add_argument("--no-other-mode", action="store_true",
                    help="skip the extra timing of the hierarchical loss in its other memory mode (staged / flat)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows in the CPU-baseline sample (0 = auto)")
    return ap.parse_args()


def make_inputs(torch, B, K, F, D, dtype, dist, w_std, device):
    """Seeded synthetic inputs in the order indices, vals, weight, bias, target (seed 1234, the
    reference's test seed, reference tests/test_setup.py:3).  Workloads whose weight matrix has at
    most 2^28 elements are generated with the CPU generator and moved to the device, so the CPU
    baseline and the GPU see tensors anyone can regenerate; larger ones are generated on the device
    (the CPU legs still get the same tensors, copied back).  Returns (tensors, where)."""
    on_cpu = F * D <= (1 << 28)
    gdev = "cpu" if on_cpu else device
    g = torch.Generator(device=gdev).manual_seed(1234)
    if dist == "randint":
        idx = torch.randint(0, F, (B, K), generator=g, device=gdev, dtype=torch.long)
    else:
        idx = torch.empty(B, K, dtype=torch.long, device=gdev)
        step = max(1, ((1 << 24) if on_cpu else (1 << 26)) // F)
        if dist == "zipf":
            logp = -1.1 * torch.log(torch.arange(1, F + 1, dtype=torch.float32, device=gdev))
            perm = torch.randperm(F, generator=g, device=gdev)
        for b0 in range(0, B, step):
            n = min(step, B - b0)
            u = torch.rand(n, F, generator=g, device=gdev)
            if dist == "zipf":
                key = logp - torch.log(-torch.log(u.clamp_(1e-30, 1 - 1e-7)))
                idx[b0:b0 + n] = perm[key.topk(K, dim=1).indices]
            else:
                idx[b0:b0 + n] = u.topk(K, dim=1).indices
    vals = torch.randn(B, K, generator=g, device=gdev).abs()
    if dist == "zipf":
        vals = vals.sort(dim=1, descending=True).values
    weight = torch.empty(F, D, dtype=dtype, device=gdev)
    rows = max(1, (1 << 27) // D)
    for f0 in range(0, F, rows):
        n = min(rows, F - f0)
        weight[f0:f0 + n] = (torch.randn(n, D, generator=g, device=gdev) * w_std).to(dtype)
    bias = torch.randn(D, generator=g, device=gdev).to(dtype)
    target = torch.randn(B, D, generator=g, device=gdev).to(dtype)
    out = tuple(x.to(device) for x in (idx, weight, vals.to(dtype), bias, target))
    return out, ("cpu generator" if on_cpu else "device generator")


def algorithmic_bytes(B, K, F, D, sw, st, sv):
    """Conservative byte model: every gathered row once per sweep, every dense output once."""
    G = B * K * D * sw
    T = B * D * st
    I = B * K * (8 + sv)
    Wb = F * D * sw
    dv = B * K * 4
    R = B * D * 4  # the fp32 residual handed from forward to backward
    return {
        "hier_step": 2 * G + 2 * T + 2 * I + Wb + dv + 8 * D,
        "topk_step": (G + T + I) + (Wb + R + I + Wb + dv + 4 * D),
        "fwd_kernel": G + T + I + R + D * sw,
        "hier_bwd_kernel": G + R + I + Wb + dv + 4 * D,
        "topk_bwd_kernel": Wb + Wb + B * K * 4 + I + dv,
    }


def time_steps(torch, fn, steps, warmup):
    """W untimed steps, then exactly K steps between two synchronisations (wall clock); every timed
    step is also bracketed by a pair of events for the spread.  Returns (ms per step by the wall
    clock, mean of the per-step event times, their standard deviation)."""
    for _ in range(warmup):
        fn()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e0, e1 in events:
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps * 1e3
    per = [e0.elapsed_time(e1) for e0, e1 in events]
    mean = sum(per) / len(per)
    std = (sum((x - mean) ** 2 for x in per) / max(1, len(per) - 1)) ** 0.5
    return wall, mean, std


def time_kernel_events(torch, prepare, launch, steps, warmup):
    """Average duration (ms) of ``launch`` alone, HIP events on the launch stream."""
    for _ in range(max(1, warmup)):
        prepare()
        launch()
    torch.cuda.synchronize()
    total = 0.0
    for _ in range(steps):
        prepare()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        launch()
        e1.record()
        e1.synchronize()
        total += e0.elapsed_time(e1)
    return total / steps


def cpu_baseline(torch, mode_name, inputs, full_B, rows=0):
    """The reference's eager torch path (gather -> scale -> cumsum -> MSE -> autograd) restated in
    oracle.torch_loss, timed on the host cores on the first ``rows`` rows with the full weight
    matrix; the per-step figure is scaled to the full batch (the work is linear in B apart from
    the dense weight-gradient buffer, which the sample pays in full)."""
    import oracle

    # every host core the process may use: os.cpu_count(), unless the machine caps the thread pools
    # through OMP_NUM_THREADS (a one-GPU box of this pool exports 16, its share of the host)
    cap = os.environ.get("OMP_NUM_THREADS", "")
    threads = os.cpu_count() or 1
    threads_note = "os.cpu_count()"
    if cap.isdigit() and 0 < int(cap) < threads:
        threads, threads_note = int(cap), f"OMP_NUM_THREADS={cap} set by the machine (os.cpu_count() = {os.cpu_count()})"
    torch.set_num_threads(threads)
    mode = oracle.HIER if mode_name == "hier" else oracle.TOPK
    W, b = inputs[1].cpu(), inputs[3].cpu()
    K, D = inputs[0].shape[1], W.shape[1]
    chunk = max(1, (1 << 28) // (K * D * 4))  # keep [Bc,K,D] fp32 around 256 MiB

    def run(n):
        idx, v, t = inputs[0][:n].cpu(), inputs[2][:n].cpu(), inputs[4][:n].cpu()
        Wg, vg, bg = (x.detach().clone().requires_grad_() for x in (W, v, b))
        t0 = time.perf_counter()
        loss = oracle.torch_loss(mode, idx, Wg, vg, bg, t, chunk_rows=chunk)
        loss.backward()
        return time.perf_counter() - t0

    if not rows:
        probe_rows = min(full_B, 16)
        run(probe_rows)  # warm-up (allocator, thread pool)
        probe = run(probe_rows)
        rows = int(min(full_B, max(probe_rows, probe_rows * 4.0 / max(probe, 1e-3))))  # ~4 s per repetition
    else:
        run(min(rows, full_B))
    rows = min(rows, full_B)
    times = []
    t_all = time.perf_counter()
    while len(times) < 3 and (time.perf_counter() - t_all) < 20.0:
        times.append(run(rows))
    sec = sum(times) / len(times)
    std = (sum((x - sec) ** 2 for x in times) / max(1, len(times) - 1)) ** 0.5
    extrapolated = rows < full_B
    return {
        "value": round(sec * 1e3 * (full_B / rows), 1),
        "unit": "ms",
        "cores": threads,
        "cores_from": threads_note,
        "kind": "port",
        "extrapolated": extrapolated,
        "std_ms": round(std * 1e3 * (full_B / rows), 1),
        "sample": f"first {rows} of {full_B} rows with the full F x D weight, {len(times)} timed fwd+bwd "
                  f"repetitions after a warm-up, {sec * 1e3:.1f} ms each"
                  + (f"; value is EXTRAPOLATED to the full batch: that x {full_B}/{rows}" if extrapolated else ""),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build measures one GPU only (the path has no multi-GPU "
                         "code); run with --gpus 1\n")
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(3)
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import flexsae_amd as flex
    from flexsae_amd import _lib

    lib = _lib.load()  # fails loudly if the HIP library is not built
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    B, K, F, D, dt_name, dist, w_std = WORKLOADS[args.workload]
    if args.shape:
        B, K, F, D = (int(x) for x in args.shape.split(","))
    if args.dtype:
        dt_name = args.dtype
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dt_name]
    es = 4 if dtype == torch.float32 else 2
    inputs, generated_with = make_inputs(torch, B, K, F, D, dtype, dist, w_std, dev)
    idx, W, v, b, t = inputs
    torch.cuda.synchronize()
    abytes = algorithmic_bytes(B, K, F, D, es, es, es)

    Wp, vp, bp = (x.clone().requires_grad_() for x in (W, v, b))

    def step(fn):
        Wp.grad = vp.grad = bp.grad = None
        loss = fn(idx, Wp, vp, bp, t)
        loss.backward()
        return loss

    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    hier_ms, hier_ev_ms, hier_std = time_steps(torch, lambda: step(flex.triton_hierarchical_sae_loss), args.steps,
                                               args.warmup)
    hier_peak = torch.cuda.max_memory_allocated() - base_mem
    Wp.grad = vp.grad = bp.grad = None
    # the same step in the other memory mode of the API: with a stage budget that holds all per-pair
    # contributions between forward and backward (faster, memory grows with B*K*D) when the run
    # above kept memory flat (the default), and the other way round
    other_ms = other_peak = None
    main_staged = bool(flex.ops._stage_fits(idx, W)) and flex.ops._train_supported(W, K)
    if not args.no_other_mode and flex.ops._train_supported(W, K):
        stage_budget = flex.ops.hier_stage_bytes()
        flex.set_hier_stage_bytes(0 if main_staged else torch.cuda.get_device_properties(dev).total_memory // 8)
        if bool(flex.ops._stage_fits(idx, W)) != main_staged:
            torch.cuda.reset_peak_memory_stats()
            other_ms, _, _ = time_steps(torch, lambda: step(flex.triton_hierarchical_sae_loss), args.steps,
                                        args.warmup)
            other_peak = torch.cuda.max_memory_allocated() - base_mem
        flex.set_hier_stage_bytes(stage_budget)
    Wp.grad = vp.grad = bp.grad = None
    # the training step with the plain-SGD update of the decoder weight fused into the reduction
    # (no dense dW, untouched rows neither read nor written); a step size of zero keeps the weights
    # as they are while moving the same bytes
    sgd_ms = sgd_peak = None
    if not args.no_other_mode and flex.ops._train_supported(W, K) and D % (4 if dtype == torch.float32 else 8) == 0:
        zero_step = torch.zeros((), dtype=torch.float32, device=dev)
        torch.cuda.reset_peak_memory_stats()
        with torch.no_grad():
            sgd_ms, _, _ = time_steps(torch, lambda: flex.ops.hier_sgd_step(idx, W, v, b, t, zero_step),
                                      args.steps, args.warmup)
        sgd_peak = torch.cuda.max_memory_allocated() - base_mem
    torch.cuda.reset_peak_memory_stats()
    topk_ms, topk_ev_ms, topk_std = time_steps(torch, lambda: step(flex.triton_topk_sae_loss), args.steps, args.warmup)
    topk_peak = torch.cuda.max_memory_allocated() - base_mem
    Wp.grad = vp.grad = bp.grad = None

    # ---- kernels alone, HIP events on the launch stream -----------------------------------
    DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}
    sh = _lib.Shape(B, K, F, D, DT[dtype], DT[dtype], DT[dtype], DT[dtype])
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    st = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws_bytes = lib.flexsae_fwd_workspace_bytes(ctypes.byref(sh))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    loss = torch.empty(1, dtype=torch.float32, device=dev)
    resid = torch.empty(B, D, dtype=torch.float32, device=dev)
    g1 = torch.ones(1, dtype=torch.float32, device=dev)
    dvals = torch.empty(B, K, dtype=torch.float32, device=dev)
    dbias = torch.empty(D, dtype=torch.float32, device=dev)
    dW = torch.empty(F, D, dtype=dtype, device=dev)
    p_size = 2 if dtype == torch.bfloat16 else 4
    scratch = flex.ops._hier_scratch_budget(B, K, F, D, dtype)  # FLEXSAE_HIER_SCRATCH_MB, else the package's rule
    # same decision as the API: the fused training step runs when the stage budget holds every
    # per-pair contribution at once (one slice as wide as D); otherwise forward + sliced backward
    # (staged); failing that, the same kernel slice by slice with an immediate reduction (sliced);
    # shapes the training-step kernel does not cover run forward + sliced backward (unfused)
    fused = (os.environ.get("FLEXSAE_FUSED_TRAINING", "1") not in ("", "0") and scratch > 0
             and flex.ops._train_supported(W, K)
             and bool(lib.flexsae_hier_fwd_bwd_supported(ctypes.byref(sh))))
    staged = fused and flex.ops._stage_fits(idx, W)
    hier_mode = "staged" if staged else "sliced" if fused else "unfused"
    slice_cols = D if staged else flex.ops._hier_slice_cols(B, K, F, D, dtype)
    # hot-latent accumulators: the same decision as the API takes for a weight that needs its gradient
    hot = bool(fused and not staged and flex.ops._use_hot_latents(B, K, F, D, dtype, dev))
    # ... and whether shapes with few pairs per latent reduce without the row-count list
    dense = bool(fused and not staged and flex.ops._use_dense_latents(B, K, F, D, dtype, dev))
    HOTF = (_lib.BWD_HOT_LATENTS if hot else 0) | (_lib.BWD_DENSE_LATENTS if dense else 0)
    if hot:
        slice_cols = flex.ops._hot_slice_cols(B, slice_cols, dev)
    tile = 64 * (4 if D % 4 == 0 else 2 if D % 2 == 0 else 1)
    d_pad = -(-D // tile) * tile
    if fused:
        # slices are whole training tiles when the reduction can work on 256-byte pieces
        bws_bytes = lib.flexsae_hier_fwd_bwd_workspace_bytes_flags(ctypes.byref(sh), slice_cols,
                                                                   _lib.BWD_HOT_LATENTS if hot else 0)
        train_tile = 64 if (dtype == torch.float32 and K > 64) else 128
        granule = train_tile if D % (16 // p_size) == 0 else tile
    else:
        bws_bytes = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), slice_cols)
        granule = tile
    bws = torch.empty(bws_bytes, dtype=torch.uint8, device=dev)
    slice_w = min(d_pad, max(granule, -(-slice_cols // granule) * granule))
    n_slices = -(-D // slice_w)

    def fwd_launch():
        _lib.check(lib.flexsae_hier_fwd(ctypes.byref(sh), p(idx), p(W), p(v), p(b), p(t), p(loss), p(resid), p(ws),
                                        ws_bytes, None, st()), "flexsae_hier_fwd")

    def bwd_launch(flags=0, workspace=None):
        w = bws if workspace is None else workspace
        _lib.check(lib.flexsae_hier_bwd(ctypes.byref(sh), p(idx), p(W), p(v), p(resid), p(g1), p(dW), DT[dtype],
                                        p(dvals), p(dbias), p(w), w.numel(), flags, None, st()),
                   "flexsae_hier_bwd")

    PRE, REUSE, SWEEP, REDUCE, NO_DW, NO_EPILOGUE, REUSE_HOT = 1, 2, 4, 8, 32, 64, _lib.BWD_REUSE_HOT_TABLES
    fwd_k_ms = time_kernel_events(torch, lambda: None, fwd_launch, args.steps, args.warmup)
    step_entry_ms = None
    if fused:
        # the API step above went through the fused training-step entry point: time it and its phases
        def train_launch(flags=0):
            if flags & REUSE:
                flags |= REUSE_HOT
            _lib.check(lib.flexsae_hier_fwd_bwd(ctypes.byref(sh), p(idx), p(W), p(v), p(b), p(t), p(loss), p(dW),
                                                DT[dtype], p(dvals), p(dbias), p(bws), bws_bytes, flags | HOTF, None,
                                                st()), "flexsae_hier_fwd_bwd")

        step_entry_ms = time_kernel_events(torch, lambda: None, train_launch, args.steps, args.warmup)
        # the training-step kernel(s) alone: no pair list (kept), no reductions, no epilogue kernels
        sweep_ms = time_kernel_events(torch, lambda: None,
                                      lambda: train_launch(PRE | REUSE | NO_DW | NO_EPILOGUE), args.steps, 1)
        reduce_ms = time_kernel_events(torch, lambda: None, lambda: train_launch(PRE | REUSE | REDUCE | NO_EPILOGUE),
                                       args.steps, 1)
        # the separate backward entry point (whole 256-column tiles per slice) in a workspace of its own
        ubws = torch.empty(lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), slice_cols), dtype=torch.uint8,
                           device=dev)
        bwd_k_ms = time_kernel_events(torch, lambda: None, lambda: bwd_launch(0, ubws), args.steps, args.warmup)
        del ubws
        sweep_name = "hier_train_hot_kernel" if hot else "hier_train_kernel"
    elif scratch > 0:
        bwd_k_ms = time_kernel_events(torch, lambda: None, bwd_launch, args.steps, args.warmup)
        # the pair list is in the workspace now: time the two phases alone (n_slices launches each)
        sweep_ms = time_kernel_events(torch, lambda: None, lambda: bwd_launch(PRE | REUSE | SWEEP), args.steps, 1)
        reduce_ms = time_kernel_events(torch, lambda: None, lambda: bwd_launch(PRE | REUSE | REDUCE), args.steps, 1)
        sweep_name = "hier_sweep_kernel"
    else:
        # scratch budget 0 selects the single-pass atomic fallback (one launch, fp32 accumulator)
        dW_acc = torch.empty(F, D, dtype=torch.float32, device=dev)

        def atomic_launch():
            _lib.check(lib.flexsae_hier_bwd_atomic(ctypes.byref(sh), p(idx), p(W), p(v), p(resid), p(g1), p(dW_acc),
                                                   p(dvals), p(dbias), PRE, None, st()), "flexsae_hier_bwd_atomic")

        def atomic_prepare():
            dW_acc.zero_()
            dvals.zero_()
            dbias.zero_()

        bwd_k_ms = time_kernel_events(torch, atomic_prepare, atomic_launch, args.steps, args.warmup)
        sweep_ms, reduce_ms, n_slices, sweep_name = bwd_k_ms, 0.0, 1, "hier_bwd_kernel (atomic fallback)"
        del dW_acc
    del dW, bws

    def gbps(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9

    # algorithmic bytes of ONE sweep launch: its share of the gathered rows, indices/vals/slots,
    # and the residual slice (the staged contributions are traffic, not algorithmic bytes)
    # (the training-step kernel reads bias/target instead of the residual: same order of bytes)
    sweep_launch_bytes = (B * K * D * es + B * K * (8 + es + 4) * n_slices + B * D * 4) / n_slices
    sweep_launch_ms = sweep_ms / n_slices
    # HBM-side bytes per launch of the dominant kernel: a counter measurement (two rocprofv3 --pmc
    # runs of this script, FETCH_SIZE and WRITE_SIZE) kept in profiles/hbm_traffic.json under the
    # workload, the slice budget and the id of the build it was taken on.  A record of another build
    # is not reported as this build's traffic.
    traffic = None
    traffic_key = f"{args.workload}:{'fused' if staged else slice_w}"  # workload : columns per slice
    traffic_source = None
    traffic_file = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    build_id = _lib.build_id()
    if os.path.exists(traffic_file) and not args.shape:
        with open(traffic_file) as fh:
            rec = json.load(fh).get(traffic_key)
        if rec and rec.get("build_id") == build_id:
            traffic = rec.get(f"{sweep_name}_bytes_per_launch")
            traffic_source = f"profiles/hbm_traffic.json[{traffic_key}], build {build_id}"
        elif rec:
            traffic_source = (f"none: profiles/hbm_traffic.json[{traffic_key}] was measured on build "
                              f"{rec.get('build_id')}, this is build {build_id}")
    # What the memory system gives a plain kernel for the same number of bytes: the runtime's own
    # device-to-device copy of half the launch's traffic (read once, written once).
    moved = traffic if traffic else int(sweep_launch_bytes + B * K * slice_w * p_size)
    copy_src = torch.empty(moved // 2, dtype=torch.uint8, device=dev)
    copy_dst = torch.empty_like(copy_src)
    n_copies = max(1, n_slices)  # as many back-to-back launches per timed bracket as the kernel has

    def copy_launch():
        for _ in range(n_copies):
            copy_dst.copy_(copy_src)

    copy_ms = time_kernel_events(torch, lambda: None, copy_launch, max(10, args.steps // 2), 2) / n_copies
    del copy_src, copy_dst
    roofline = {
        "bound": "hbm",
        "kernel": sweep_name,
        "achieved": round(gbps(sweep_launch_bytes, sweep_launch_ms), 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(gbps(sweep_launch_bytes, sweep_launch_ms) / HBM_PEAK_GBPS, 4),
        "traffic": traffic,
        "traffic_source": traffic_source,
        "algorithmic_bytes_per_launch": int(sweep_launch_bytes),
        "avg_launch_ms": round(sweep_launch_ms, 4),
        "launches_per_step": n_slices,
        "traffic_GBps": round(gbps(traffic, sweep_launch_ms), 1) if traffic else None,
        "device_copy_same_bytes": {"bytes_moved": 2 * (moved // 2), "ms": round(copy_ms, 4),
                                   "GBps": round(gbps(2 * (moved // 2), copy_ms), 1),
                                   "what": "torch's device-to-device copy moving as many bytes as one launch of the "
                                           "kernel (half read, half written), timed the same way"},
    }

    out = {
        "metric": "fwd+bwd ms/step + HBM GB/s (% peak), HierTopK F=65536 D=2304 K=128",
        "value": round(hier_ms, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(hier_ms, 4),
        "ms_per_step_std": round(hier_std, 4),
        "ms_per_step_events": round(hier_ev_ms, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 arithmetic on %s storage" % dt_name,
        "data": "synthetic (seed 1234, %s)" % generated_with,
        "build_id": build_id,
        "config": {"workload": f"HierarchicalTopK fwd+bwd, {args.workload}: B={B} K={K} F={F} D={D} {dt_name}, "
                               f"indices {dist}", "B": B, "K": K, "F": F, "D": D,
                   "hier_scratch_mb": scratch >> 20, "hier_slice_cols": int(slice_w), "hot_latents": hot, "dense_latents": dense, "fused_training_step": bool(fused), "hier_mode": hier_mode,
                   "hier_stage_mb": flex.ops.hier_stage_bytes(dev) >> 20},
        "roofline": roofline,
        "step_hbm": {"algorithmic_bytes": abytes["hier_step"],
                     "achieved_GBps": round(gbps(abytes["hier_step"], hier_ms), 1),
                     "algorithmic_frac_of_peak": round(gbps(abytes["hier_step"], hier_ms) / HBM_PEAK_GBPS, 4),
                     "note": ALGORITHMIC_NOTE},
        "kernels": {
            "flexsae_hier_fwd (sae_fwd_kernel + loss_finalize)": {
                "ms": round(fwd_k_ms, 4), "algorithmic_bytes": abytes["fwd_kernel"],
                "GBps": round(gbps(abytes["fwd_kernel"], fwd_k_ms), 1),
                "algorithmic_frac_of_peak": round(gbps(abytes["fwd_kernel"], fwd_k_ms) / HBM_PEAK_GBPS, 4),
                "note": ALGORITHMIC_NOTE},
            "flexsae_hier_bwd (pair list + sweep + reduce)": {
                "ms": round(bwd_k_ms, 4), "algorithmic_bytes": abytes["hier_bwd_kernel"],
                "GBps": round(gbps(abytes["hier_bwd_kernel"], bwd_k_ms), 1)},
            "flexsae_hier_fwd_bwd (fused training step: pair list + train kernel + reduce)": (
                {"ms": round(step_entry_ms, 4)} if step_entry_ms is not None else None),
            "%s x%d" % (sweep_name, n_slices): {"ms": round(sweep_ms, 4)},
            "segment reduction x%d" % n_slices: {"ms": round(reduce_ms, 4)},
        },
        "topk": {"ms_per_step": round(topk_ms, 4), "ms_per_step_std": round(topk_std, 4),
                 "ms_per_step_events": round(topk_ev_ms, 4), "algorithmic_bytes": abytes["topk_step"],
                 "achieved_GBps": round(gbps(abytes["topk_step"], topk_ms), 1)},
        "hier_over_topk_latency": round(hier_ms / topk_ms, 3),
        ("hier_flat_memory_mode" if main_staged else "hier_staged_mode"): None if other_ms is None else {
            "ms_per_step": round(other_ms, 4), "over_topk_latency": round(other_ms / topk_ms, 3),
            "peak_mem_gib": round(other_peak / 2 ** 30, 3)},
        "hier_sgd_step": None if sgd_ms is None else {
            "ms_per_step": round(sgd_ms, 4), "over_topk_latency": round(sgd_ms / topk_ms, 3),
            "peak_mem_gib": round(sgd_peak / 2 ** 30, 3),
            "what": "flexsae_hier_sgd_step: loss, dvals, dbias and the in-place SGD update of W; no dense dW"},
        "peak_mem_gib": {"hier": round(hier_peak / 2 ** 30, 3), "topk": round(topk_peak / 2 ** 30, 3),
                         "inputs": round(base_mem / 2 ** 30, 3)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, "hier", inputs, B, rows=args.cpu_rows)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
