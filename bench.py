#!/usr/bin/env python3
"""Benchmark of the Gaussian-mixture evaluation path on one MI355X.

A step is one forward plus one backward (both gradients) of `evaluate_inversed` over one synthetic batch of the
named workload (default C4: 3-D, float32, B=32, L=64, M=512 Gaussians, N=8192 points per mixture, 8.59e9
Gaussian-point pairs).  Inputs are resident in HBM before the timed region.  Prints ONE JSON line:
  value            whole-step throughput, Gaussian-point pairs per second (forward + backward)
  fwd / fwd_bwd    pairs per second and fraction of the FP32 vector peak at the contract flop counts
                   (D=3: 20 flop per forward pair, 52 per backward pair; D=2: 12 / 30)
  roofline         dominant kernel (the backward pair kernel), HIP-event time on the launch stream
  cpu_baseline     the C/OpenMP restatement of the reference's CPU path on a bounded slice of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "gaussian-mixture-convolution-networks_amd"))

FLOP_FWD = {2: 12, 3: 20}
FLOP_BWD = {2: 30, 3: 52}
# forward flops per pair of the reference's literal arithmetic (determinant, square root and exp per pair,
# util/gaussian.h:82-95); reported for transparency only, never as the headline
FLOP_FWD_LITERAL = {2: 15, 3: 27}
PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}     # MI355X vector peaks
PEAK_CLOCK_MHZ = 2400.0                        # the engine clock those peaks are quoted at (256 CUs x 256 flop/cycle x 2.4 GHz)
# The dense kernels are bound by FP32 arithmetic.  MI355X's FP32 matrix rate equals its (packed) FP32 vector rate,
# 157.3 TFLOP/s, which is the peak the metric names.  `bound` says which unit issues the kernel's arithmetic: "valu"
# for the all-vector kernels, "mfma" for the forward kernel that takes the affine part from the matrix cores, "hbm"
# for the memory- and latency-bound paths.
VALU_NOTE = ("bound by vector-instruction issue against the FP32 peak of 157.3 TFLOP/s (MI355X's FP32 matrix rate equals "
             "its packed FP32 vector rate); the kernels issue unpacked FP32 vector instructions (measured: one wave64 FMA "
             "per 2.3 cycles and SIMD = 137 TFLOP/s)")
MFMA_NOTE = VALU_NOTE + "; this kernel takes y = u x - u b from the bf16 matrix cores and keeps |y|^2, exp2 and the sum on the vector ALU"
PROFILES = {"C4": "eval_dense_fwd_bwd_C4.md", "C5": "eval_bvh_build_fwd_bwd_C5.md", "C5dense": "eval_dense_fwd_bwd_C5_f64.md"}


def profile_traffic(workload: str, kernel_prefix: str):
    """HBM bytes per launch of the kernel whose name starts with `kernel_prefix`, read from the committed counter
    summary of this script under profiles/: FETCH_SIZE and WRITE_SIZE (KiB per dispatch), each scaled by what the
    same counter shows for the 1 GiB device copy in the same run.  None when the summary or the kernel is missing."""
    path = os.path.join(ROOT, "profiles", PROFILES.get(workload, ""))
    if not os.path.isfile(path):
        return None
    tables, header = {}, None
    for line in open(path):
        cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")] if line.startswith("|") else None
        if not cells:
            header = None
        elif cells[0] == "kernel":
            header = cells[1:]
        elif header and not set(cells[0]) <= set("-: "):
            for name, value in zip(header, cells[1:]):
                try:
                    tables.setdefault(name, {})[cells[0]] = float(value)
                except ValueError:
                    pass
    total = 0.0
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        rows = tables.get(counter, {})
        mine = [v for k, v in rows.items() if k.startswith(kernel_prefix)]
        copy = [v for k, v in rows.items() if k.startswith("__amd_rocclr_copyBuffer")]
        if not mine or not copy or copy[0] <= 0:
            return None
        total += mine[0] * 1024.0 * (1048576.0 / copy[0])            # the copy moves 1 GiB each way
    return total


def median(values):
    v = sorted(values)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


def cpu_baseline(name: str):
    """Times oracle/libcpu_ref.so (checker code, used here only as the reported CPU baseline)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import cpu_ref
    from gmc import synthetic
    base = synthetic.WORKLOADS[name]
    # bounded sample of the same distributions (about 10 s of CPU work at C4): four batch entries
    kw = dict(B=4) if name != "C5" else dict(N=2000)
    wl, mix, xes, gout = synthetic.make_workload(name, **kw)
    m, x, g = mix.numpy(), xes.numpy(), gout.numpy()
    threads = 128                                    # the reference's own choice (parallel_start.h:94-99)
    cores = len(os.sched_getaffinity(0))
    cpu_ref.forward(m[:, :1], x[:, :1], n_threads=threads)       # warm-up (thread pool, page faults)
    t0 = time.perf_counter()
    cpu_ref.forward(m, x, n_threads=threads)
    t_fwd = time.perf_counter() - t0
    t0 = time.perf_counter()
    cpu_ref.backward(g, m, x, n_threads=threads)
    t_bwd = time.perf_counter() - t0
    return {
        "value": wl.pairs / (t_fwd + t_bwd), "unit": "pairs/s (fwd+bwd)", "cores": cores, "threads": threads,
        "kind": "port", "fwd_pairs_per_s": wl.pairs / t_fwd, "bwd_pairs_per_s": wl.pairs / t_bwd,
        "sample": f"{name} slice B={wl.B} L={wl.L} M={wl.M} N={wl.N} ({wl.pairs:.3g} pairs), "
                  f"fwd {t_fwd:.2f} s + bwd {t_bwd:.2f} s, C/OpenMP restatement of the reference CPU path",
    }


def measure_bvh(aabb_mode: str, steps: int, warmup: int, copy_calibration: bool = False, name: str = "C5"):
    """LBVH-culled path on a workload (default C5: 3-D, float64, one mixture of 16384 Gaussians, 100000 points).  A step
    builds the trees (the mixtures change every training step), evaluates forward and backward.  Returns the step time
    (wall clock over all steps), the timings of its parts (HIP events on the launch stream, medians over a second run of
    the same steps) and the number of pairs actually evaluated."""
    import torch
    from gmc import _native, synthetic
    wl, mix, xes, gout = synthetic.make_workload(name)
    dev = torch.device("cuda:0")
    mix, xes, gout = mix.to(dev), xes.to(dev), gout.to(dev)
    torch.cuda.synchronize()

    def step(ev=None):
        if ev:
            ev[0].record()
        bvh = _native.Bvh(mix, xes, 0.001, aabb_mode)
        if ev:
            ev[1].record()
        out = _native.eval_bvh_fwd(mix, xes, bvh)
        if ev:
            ev[2].record()
        g = _native.eval_bvh_bwd(gout, mix, xes, bvh, True, True)
        if ev:
            ev[3].record()
        return out, g

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    if copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # the step time: wall clock over `steps` steps with nothing else in the stream (a step is 0.2 ms in 13 launches,
    # and four event records per step would add several microseconds of their own to it) ...
    t0 = time.perf_counter()
    for k in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # ... and its parts: the same steps again with HIP events between the calls
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for k in range(steps):
        step(events[k])
    torch.cuda.synchronize()
    build_ms, fwd_ms, bwd_ms = (median([e[i].elapsed_time(e[i + 1]) for e in events]) for i in range(3))
    # ... and without the host between the launches: ten builds, and ten whole steps, captured into HIP graphs and
    # replayed (the build of small trees is one launch of about 20 us, shorter than the host needs to enqueue it, so
    # the event pair above measures the host there)
    def in_graph(fn, repeats=10, replays=5):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = [fn() for _ in range(repeats)]
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        del keep
        return e0.elapsed_time(e1) / (repeats * replays)
    build_graph_ms = in_graph(lambda: _native.Bvh(mix, xes, 0.001, aabb_mode))
    step_graph_ms = in_graph(step)
    # pairs actually evaluated: points inside the cutoff box of a Gaussian (counted outside the timed region)
    bvh = _native.Bvh(mix, xes, 0.001, aabb_mode)
    lo, up = bvh.boxes()
    hits = 0
    for b in range(wl.B):
        for n0 in range(0, wl.N, 2048):
            x = xes[b, :, n0:n0 + 2048].unsqueeze(2)                   # [L, n, 1, D]
            hits += int(((x >= lo[b].unsqueeze(1)) & (x <= up[b].unsqueeze(1))).all(dim=-1).sum().item())
    return {"wl": wl, "ms_step": wall * 1e3 / steps, "build_ms": build_ms, "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "hits": hits,
            "build_graph_ms": build_graph_ms, "step_graph_ms": step_graph_ms}


def bvh_summary(r, aabb_mode):
    """the C5 numbers of one box rule as a compact object (entry of `other_workloads`)"""
    wl = r["wl"]
    return {"aabb_mode": aabb_mode, "ms_per_step": r["ms_step"], "build_ms": r["build_ms"], "fwd_ms": r["fwd_ms"],
            "bwd_ms": r["bwd_ms"], "build_ms_in_graph": r["build_graph_ms"], "ms_per_step_in_graph": r["step_graph_ms"],
            "dense_equivalent_pairs_per_s": wl.pairs / (r["ms_step"] * 1e-3),
            "evaluated_pairs": r["hits"], "evaluated_pairs_per_s": r["hits"] / (r["ms_step"] * 1e-3)}


def bench_bvh(args):
    """`--workload C5`: the LBVH-culled step (build + forward + backward).  Throughput is reported in dense-equivalent
    pairs (B L M N per step); the roofline entries are against HBM with the compulsory bytes of the pass (Gaussians,
    node boxes and links, points in, values and gradients out)."""
    r = measure_bvh(args.aabb_mode, args.steps, args.warmup, args.copy_calibration, name=args.workload)
    wl, ms_step, build_ms, fwd_ms, bwd_ms, hits = r["wl"], r["ms_step"], r["build_ms"], r["fwd_ms"], r["bwd_ms"], r["hits"]
    import torch
    s, M, N, D, BL = (8 if wl.dtype == torch.float64 else 4), wl.M, wl.N, wl.dims, wl.B * wl.L
    G = 1 + D + D * D
    bytes_fwd = BL * (M * G * s + (2 * M - 1) * (2 * D * s + 8) + N * (D + 1) * s)
    bytes_bwd = bytes_fwd + BL * (N * s + M * G * s + N * D * s)
    dt = "f64" if s == 8 else "f32"
    reference_rule = args.aabb_mode == "reference"
    line = {
        "metric": "Gaussian-point evals/sec fwd and fwd+bwd at 1 GPU; % of FP32 VALU peak",
        "value": wl.pairs / (ms_step * 1e-3), "unit": "dense-equivalent Gaussian-point pairs/s (LBVH build + forward + backward step)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{args.workload}: D={D} {dt} B={wl.B} L={wl.L} M={M} N={N}, LBVH-culled (aabb_mode={args.aabb_mode}, "
                               f"threshold 0.001), {wl.pairs:.4g} dense-equivalent pairs per step"},
        "build_ms": build_ms, "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "build_ms_in_graph": r["build_graph_ms"], "ms_per_step_in_graph": r["step_graph_ms"],
        "evaluated_pairs": hits, "evaluated_pairs_per_s": hits / (ms_step * 1e-3),
        "evaluated_fraction_of_dense": hits / wl.pairs,
        "roofline": {"kernel": "bvh_traverse_kernel (backward mode; event pair also holds its zero-fill and epilogue)",
                     "bound": "hbm", "achieved": bytes_bwd / (bwd_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": bytes_bwd / (bwd_ms * 1e-3) / 8e12,
                     "traffic": profile_traffic("C5", "bvh_traverse_kernel<double, 3, 1") if reference_rule and args.workload == "C5" else None,
                     "launch_ms": bwd_ms, "algorithmic_bytes": bytes_bwd,
                     "bound_detail": "latency-bound: dependent tree-node fetches and double-precision leaf "
                                     "evaluation; the tree (about 4 MB) is fetched once per XCD (8 L2 caches)"},
        "roofline_fwd": {"kernel": "bvh_traverse_kernel (forward mode)", "bound": "hbm",
                         "achieved": bytes_fwd / (fwd_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                         "frac": bytes_fwd / (fwd_ms * 1e-3) / 8e12,
                         "traffic": profile_traffic("C5", "bvh_traverse_kernel<double, 3, 0") if reference_rule and args.workload == "C5" else None,
                         "launch_ms": fwd_ms, "algorithmic_bytes": bytes_fwd},
    }
    if not args.no_cpu_baseline and args.workload == "C5":
        line["cpu_baseline"] = cpu_baseline_bvh(args.aabb_mode)
    print(json.dumps(line))


def cpu_baseline_bvh(mode: str):
    """CPU comparison for the culled path: the C restatement of the reference CPU loops with the per-pair box
    test in front of each evaluation (the reference has no CPU BVH evaluator to restate), on the whole C5
    workload with the boxes of the oracle's rule, five repetitions."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import cpu_ref
    import gm_oracle
    from gmc import synthetic
    wl, mix, xes, gout = synthetic.make_workload("C5")
    m, x, g = mix.numpy(), xes.numpy(), gout.numpy()
    lo, up = gm_oracle.gaussian_aabbs(m, mode=mode)
    threads, cores = 128, len(os.sched_getaffinity(0))
    reps = 5
    cpu_ref.forward(m, x[:, :, :2000], lo, up, n_threads=threads)        # warm-up (thread pool, page faults)
    t0 = time.perf_counter()
    for _ in range(reps):
        cpu_ref.forward(m, x, lo, up, n_threads=threads)
    t_fwd = (time.perf_counter() - t0) / reps
    t0 = time.perf_counter()
    for _ in range(reps):
        cpu_ref.backward(g, m, x, lo, up, n_threads=threads)
    t_bwd = (time.perf_counter() - t0) / reps
    return {"value": wl.pairs / (t_fwd + t_bwd), "unit": "dense-equivalent pairs/s (fwd+bwd)", "cores": cores,
            "threads": threads, "kind": "port",
            "sample": f"the whole C5 workload, {reps} repetitions (M=16384, N=100000: {wl.pairs:.3g} dense-equivalent pairs "
                      f"each), brute-force box test per pair, fwd {t_fwd:.2f} s + bwd {t_bwd:.2f} s per repetition"}


def bench_convolution(args):
    """Closed-form convolution on a layer-sized problem (2-D, float32, batch 100, 8 -> 16 channels, 128 data and 5
    kernel components per channel: 8.2e6 output Gaussians, 229 MB).  A step is forward plus backward (both
    gradients).  The path is streaming: the unit is output Gaussians per second and the roofline is HBM with the
    compulsory bytes (forward: operands in, result out; backward: grad_out once, operands in, gradients out)."""
    import torch
    from gmc import _native
    from gmc import mixture as gm
    B, Cin, Cout, Nd, Nk, D = 100, 8, 16, 128, 5, 2
    G = 1 + D + D * D
    gen = torch.Generator().manual_seed(20246)
    data = gm.generate_random_mixtures(B, Cin, Nd, n_dims=D, pos_radius=1, cov_radius=0.5)
    kernels = gm.generate_random_mixtures(Cout, Cin, Nk, n_dims=D, pos_radius=1, cov_radius=0.5)
    dev = torch.device("cuda:0")
    data, kernels = data.to(dev), kernels.to(dev)
    n_out = B * Cout * Nd * Cin * Nk
    gout = torch.randn((B, Cout, Nd * Cin * Nk, G), generator=gen).to(dev)
    torch.cuda.synchronize()

    def step(ev=None):
        if ev:
            ev[0].record()
        out = _native.convolution_fwd(data, kernels)
        if ev:
            ev[1].record()
        g = _native.convolution_bwd(gout, data, kernels, True, True)
        if ev:
            ev[2].record()
        return out, g

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(events[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_step = wall * 1e3 / args.steps
    fwd_ms, bwd_ms = (median([e[i].elapsed_time(e[i + 1]) for e in events]) for i in range(2))
    small = (data.numel() + kernels.numel()) * 4
    bytes_fwd = n_out * G * 4 + small
    bytes_bwd = n_out * G * 4 + 2 * small                    # grad_out once; operands in, gradients out
    line = {
        "metric": "closed-form mixture convolution, output Gaussians per second (forward + backward step)",
        "value": n_out / (ms_step * 1e-3), "unit": "output Gaussians/s (forward + backward step)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"conv: D={D} f32 data [{B},{Cin},{Nd}] * kernels [{Cout},{Cin},{Nk}] -> "
                               f"[{B},{Cout},{Nd * Cin * Nk}], {n_out:.4g} output Gaussians per step"},
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "roofline": {"kernel": "conv_bwd_fused_kernel (with the zero fill of grad_kernels in the event pair)", "bound": "hbm",
                     "achieved": bytes_bwd / (bwd_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": bytes_bwd / (bwd_ms * 1e-3) / 8e12, "traffic": None, "launch_ms": bwd_ms,
                     "algorithmic_bytes": bytes_bwd},
        "roofline_fwd": {"kernel": "conv_fwd_kernel", "bound": "hbm", "achieved": bytes_fwd / (fwd_ms * 1e-3) / 1e9,
                         "peak": 8000.0, "unit": "GB/s", "frac": bytes_fwd / (fwd_ms * 1e-3) / 8e12,
                         "launch_ms": fwd_ms, "algorithmic_bytes": bytes_fwd},
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import gm_oracle
        d, k, g = data.cpu().numpy(), kernels.cpu().numpy(), gout.cpu().numpy()
        t0 = time.perf_counter()
        gm_oracle.convolution_forward(d, k)
        t_fwd = time.perf_counter() - t0
        t0 = time.perf_counter()
        gm_oracle.convolution_backward(g, d, k)
        t_bwd = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": n_out / (t_fwd + t_bwd), "unit": "output Gaussians/s (fwd+bwd)", "cores": 1,
                                "kind": "port", "sample": f"the whole step once in numpy float32 (the oracle's "
                                f"restatement), fwd {t_fwd:.2f} s + bwd {t_bwd:.2f} s"}
    print(json.dumps(line))


def bench_componentwise(args):
    """Component-wise evaluation (values [B, L, N, M] without the sum over components) on the C2 shape: 2-D float32,
    B=100, L=8, M=128, N=784, 8.03e7 pairs.  A step is forward plus backward (both gradients).  One scalar per pair is
    written (forward) or read (backward), so the unit is pairs per second and the roofline is HBM with 4 bytes per
    pair plus the operands."""
    import torch
    from gmc import _native, synthetic
    wl, mix, xes, _ = synthetic.make_workload("C2")
    dev = torch.device("cuda:0")
    mix, xes = mix.to(dev), xes.to(dev)
    gen = torch.Generator().manual_seed(20247)
    gout = torch.randn((wl.B, wl.L, wl.N, wl.M), generator=gen).to(dev)
    torch.cuda.synchronize()

    def step(ev=None):
        if ev:
            ev[0].record()
        out = _native.eval_componentwise_fwd(mix, xes)
        if ev:
            ev[1].record()
        g = _native.eval_componentwise_bwd(gout, mix, xes, True, True)
        if ev:
            ev[2].record()
        return out, g

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(events[k])
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd_ms, bwd_ms = (median([e[i].elapsed_time(e[i + 1]) for e in events]) for i in range(2))
    small = (mix.numel() + xes.numel()) * 4
    bytes_fwd = wl.pairs * 4 + small
    bytes_bwd = wl.pairs * 4 + 2 * small
    line = {
        "metric": "component-wise Gaussian-point evaluations per second (forward + backward step)",
        "value": wl.pairs / (ms_step * 1e-3), "unit": "Gaussian-point pairs/s (forward + backward step)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"componentwise on C2: D=2 f32 B={wl.B} L={wl.L} M={wl.M} N={wl.N}, {wl.pairs:.3g} pairs "
                               f"per step, values [B,L,N,M] out, gradient of the same shape in"},
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "roofline": {"kernel": "componentwise_bwd_kernel (with its zero fill and epilogue in the event pair)", "bound": "hbm",
                     "achieved": bytes_bwd / (bwd_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": bytes_bwd / (bwd_ms * 1e-3) / 8e12, "traffic": None, "launch_ms": bwd_ms,
                     "algorithmic_bytes": bytes_bwd,
                     "bound_detail": "4 bytes per pair leave about 40 vector instructions per 64 pairs at the HBM "
                                     "rate; the pair math and the wavefront reductions of dL/dx take 38 (measured)"},
        "roofline_fwd": {"kernel": "componentwise_fwd_kernel", "bound": "hbm",
                         "achieved": bytes_fwd / (fwd_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                         "frac": bytes_fwd / (fwd_ms * 1e-3) / 8e12, "launch_ms": fwd_ms,
                         "algorithmic_bytes": bytes_fwd},
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import gm_oracle
        m, x = mix[:4].cpu().numpy().astype("float64"), xes[:4].cpu().numpy().astype("float64")
        t0 = time.perf_counter()
        gm_oracle.evaluate_inversed(m, x)
        t = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": 4 * wl.L * wl.M * wl.N / t, "unit": "pairs/s (forward only)", "cores": 1,
                                "kind": "port", "sample": f"the same pair values for four batch entries in numpy float64 "
                                f"(the oracle's evaluate_inversed, which forms every pair's value before it sums "
                                f"them), {t:.2f} s"}
    print(json.dumps(line))


def bench_layer(args):
    """The callers either side of the evaluation in a network layer, on the C2 shape (2-D float32, B=100, L=8, M=128):
    `gm.evaluate` on a mixture that holds covariances (the inverse is taken inside the kernels) forward + backward
    at the N=784 grid points, the ReLU fixed-point fitting (two evaluations at the mixture's own 128 centres plus
    the multiplicative update) and BatchNorm (one evaluation at 100 random samples per channel, moments, rescale).
    A step runs the three one after the other through the autograd-level API; the value counts the pairs of all
    evaluations in it."""
    import torch
    from gmc import fitting, mat_tools, modules, synthetic
    from gmc import mixture as gm
    wl, mix, xes, gout = synthetic.make_workload("C2")
    dev = torch.device("cuda:0")
    mix, xes, gout = mix.to(dev), xes.to(dev), gout.to(dev)
    mix_cov = gm.pack_mixture(gm.weights(mix), gm.positions(mix), mat_tools.inverse(gm.covariances(mix))).contiguous()
    constant = torch.randn((wl.B, wl.L), generator=torch.Generator().manual_seed(20248)).to(dev)
    norm = modules.BatchNorm(wl.L).to(dev)
    leaf = mix_cov.clone().requires_grad_(True)
    torch.cuda.synchronize()

    def step(ev=None):
        if ev:
            ev[0].record()
        leaf.grad = None
        gm.evaluate(leaf, xes).backward(gout)
        if ev:
            ev[1].record()
        with torch.no_grad():
            fitted, _ = fitting.fixed_point_iteration_to_relu(mix_cov, constant, mix_cov, n_iter=1)
        if ev:
            ev[2].record()
        with torch.no_grad():
            scaled, _ = norm((mix_cov, constant))
        if ev:
            ev[3].record()
        return fitted, scaled

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(events[k])
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    eval_ms, fit_ms, norm_ms = (median([e[i].elapsed_time(e[i + 1]) for e in events]) for i in range(3))
    mixtures = wl.B * wl.L
    pairs_eval = 2 * wl.pairs                                   # forward and backward
    pairs_fit = 2 * mixtures * wl.M * wl.M
    pairs_norm = mixtures * wl.M * (10000 // wl.B)
    pairs = pairs_eval + pairs_fit + pairs_norm
    line = {
        "metric": "Gaussian-point evaluations per second through gm.evaluate and its callers (autograd-level API)",
        "value": pairs / (ms_step * 1e-3), "unit": "Gaussian-point pairs/s (forward pairs + backward pairs)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"layer on C2: D=2 f32 B={wl.B} L={wl.L} M={wl.M}; evaluate(covariances) forward + "
                               f"backward at N={wl.N}, fixed_point_iteration_to_relu (n_iter=1), BatchNorm.forward"},
        "evaluate_fwd_bwd": {"ms": eval_ms, "pairs": pairs_eval},
        "fixed_point_iteration_to_relu": {"ms": fit_ms, "pairs": pairs_fit},
        "batch_norm_forward": {"ms": norm_ms, "pairs": pairs_norm},
        "roofline": {"kernel": "eval_bwd_rc_kernel (covariance form, inside evaluate_fwd_bwd)", "bound": "valu",
                     "bound_detail": "launch-bound at this size: the step is a chain of small launches and "
                                     "element-wise torch operations; the fraction is that of the whole evaluate "
                                     "forward + backward against the FP32 peak at 12 + 30 flop per pair",
                     "achieved": (FLOP_FWD[2] + FLOP_BWD[2]) * wl.pairs / (eval_ms * 1e-3) / 1e12,
                     "peak": PEAK_TFLOPS["f32"], "unit": "TFLOP/s",
                     "frac": (FLOP_FWD[2] + FLOP_BWD[2]) * wl.pairs / (eval_ms * 1e-3) / 1e12 / PEAK_TFLOPS["f32"],
                     "traffic": None, "launch_ms": eval_ms},
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import gm_oracle
        m = mix_cov[:2].cpu().numpy().astype("float64")
        c = constant[:2].cpu().numpy().astype("float64")
        t0 = time.perf_counter()
        gm_oracle.fixed_point_iteration_to_relu(m, c, m, 1)
        t = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": 2 * 2 * wl.L * wl.M * wl.M / t, "unit": "pairs/s (fixed-point fitting only)",
                                "cores": 1, "kind": "port",
                                "sample": f"the oracle's fixed_point_iteration_to_relu (numpy float64) on two batch "
                                          f"entries, {t:.2f} s"}
    print(json.dumps(line))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C4", choices=["C1", "C2", "C3", "C4", "C5", "C5dense", "conv", "cw", "layer"],
                    help="C1..C4: dense all-pairs path; C5: LBVH-culled path (build + forward + backward per step); C5dense: the C5 "
                         "inputs (float64, one mixture) through the dense path; "
                         "conv: closed-form convolution; cw: component-wise evaluation on the C2 shape (forward + "
                         "backward per step); layer: gm.evaluate on covariances forward + backward, the ReLU fixed-point "
                         "fitting and BatchNorm on the C2 shape")
    ap.add_argument("--aabb-mode", default="reference", choices=["reference", "tight"])
    ap.add_argument("--culled", action="store_true",
                    help="C2 or C3 through the LBVH-culled path (build + forward + backward per step), like C5")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="C4 only: leave out the `other_workloads` object (C1, C2, C3 and C5 measured after C4)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device-to-device copy (known HBM traffic) so that a counter run of "
                         "this command holds the calibration kernel next to the evaluation kernels")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU; --gpus N with N > 1 is not supported (nothing here uses a "
              "second GPU; mixtures would shard over batch x layers without communication)", file=sys.stderr)
        sys.exit(2)

    import torch
    from gmc import _native, synthetic

    if args.workload == "C5" or (args.culled and args.workload in ("C2", "C3")):
        return bench_bvh(args)
    if args.workload == "conv":
        return bench_convolution(args)
    if args.workload == "cw":
        return bench_componentwise(args)
    if args.workload == "layer":
        return bench_layer(args)
    dense_name = "C5" if args.workload == "C5dense" else args.workload
    r = measure_dense(dense_name, args.steps, args.warmup, args.copy_calibration)
    wl, ms_step, fwd_ms, bwd_ms = r["wl"], r["ms_step"], r["fwd_ms"], r["bwd_ms"]
    D = wl.dims
    dt = "f32" if wl.dtype == torch.float32 else "f64"
    peak = PEAK_TFLOPS[dt]
    fwd_tf = FLOP_FWD[D] * wl.pairs / (fwd_ms * 1e-3) / 1e12
    bwd_tf = FLOP_BWD[D] * wl.pairs / (bwd_ms * 1e-3) / 1e12
    step_tf = (FLOP_FWD[D] + FLOP_BWD[D]) * wl.pairs / (ms_step * 1e-3) / 1e12
    fwd_kernel = r["fwd_kernel"]
    fwd_mhz, bwd_mhz = r["clocks_mhz"]

    def at_measured_clock(frac, mhz):
        """what the fraction of the published peak (quoted at PEAK_CLOCK_MHZ) is against the clock the launch ran at"""
        return {"shader_clock_mhz": mhz, "frac_at_that_clock": frac * PEAK_CLOCK_MHZ / mhz} if mhz > 0 else {}

    line = {
        "metric": "Gaussian-point evals/sec fwd and fwd+bwd at 1 GPU; % of FP32 VALU peak",
        "value": wl.pairs / (ms_step * 1e-3), "unit": "Gaussian-point pairs/s (forward + backward step)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{args.workload}: D={D} {dt} B={wl.B} L={wl.L} M={wl.M} N={wl.N}, dense all-pairs, "
                               f"{wl.pairs:.4g} pairs per step, forward + backward (grad mixture and grad xes)"},
        "timing": "ms_per_step: wall clock over all steps / steps; fwd.ms, roofline launch_ms: medians of per-step HIP event pairs (launch_ms_mean: their means)",
        "fwd": {"ms": fwd_ms, "pairs_per_s": wl.pairs / (fwd_ms * 1e-3), "tflops": fwd_tf, "frac_of_peak": fwd_tf / peak,
                "tflops_by_reference_literal_count": FLOP_FWD_LITERAL[D] * wl.pairs / (fwd_ms * 1e-3) / 1e12},
        "fwd_bwd": {"ms": ms_step, "pairs_per_s": wl.pairs / (ms_step * 1e-3), "tflops": step_tf,
                    "frac_of_peak": step_tf / peak},
        "roofline": {"kernel": "eval_bwd_rc_kernel (backward pair kernel; its zero-fill and epilogue launches, <1% of "
                               "the time, are inside the event pair)",
                     "bound": "valu", "bound_detail": VALU_NOTE, "achieved": bwd_tf, "peak": peak, "unit": "TFLOP/s", "frac": bwd_tf / peak,
                     "traffic": profile_traffic(args.workload, "eval_bwd_rc_kernel"), "launch_ms": bwd_ms,
                     "launch_ms_mean": r["bwd_ms_mean"], "flop_per_pair": FLOP_BWD[D], **at_measured_clock(bwd_tf / peak, bwd_mhz)},
        "roofline_fwd": {"kernel": fwd_kernel, "bound": "mfma" if fwd_kernel == "eval_fwd_mfma_kernel" else "valu",
                         "bound_detail": MFMA_NOTE if fwd_kernel == "eval_fwd_mfma_kernel" else VALU_NOTE,
                         "achieved": fwd_tf, "peak": peak,
                         "unit": "TFLOP/s", "frac": fwd_tf / peak, "launch_ms": fwd_ms, "launch_ms_mean": r["fwd_ms_mean"],
                         "flop_per_pair": FLOP_FWD[D],
                         "traffic": profile_traffic(args.workload, fwd_kernel),
                         **(at_measured_clock(fwd_tf / peak, fwd_mhz) if fwd_kernel == "eval_fwd_mfma_kernel" else {})},
    }
    if args.workload == "C4" and not args.no_other_workloads:
        # every other configuration of the baseline, measured in the same process after the timed region of C4
        others = {}
        for name in ("C1", "C2", "C3"):
            o = measure_dense(name, 20, 3)
            w, d = o["wl"], o["wl"].dims
            others[name] = {
                "config": f"D={d} f32 B={w.B} L={w.L} M={w.M} N={w.N}, dense, {w.pairs:.4g} pairs",
                "fwd_ms": o["fwd_ms"], "bwd_ms": o["bwd_ms"], "ms_per_step": o["ms_step"],
                "fwd_pairs_per_s": w.pairs / (o["fwd_ms"] * 1e-3), "fwd_bwd_pairs_per_s": w.pairs / (o["ms_step"] * 1e-3),
                "fwd_frac_of_peak": FLOP_FWD[d] * w.pairs / (o["fwd_ms"] * 1e-3) / 1e12 / PEAK_TFLOPS["f32"],
                "fwd_bwd_frac_of_peak": (FLOP_FWD[d] + FLOP_BWD[d]) * w.pairs / (o["ms_step"] * 1e-3) / 1e12 / PEAK_TFLOPS["f32"],
                "fwd_kernel": o["fwd_kernel"],
                # short launches with gaps between them do not bring the clock up to what the long ones of C4 reach
                "bwd_shader_clock_mhz": o["clocks_mhz"][1]}
        o = measure_dense("C2", 20, 3, broadcast_xes=True)
        others["C2_broadcast_xes"] = {
            "config": "C2 with the points of the first mixture shared by all 800 ([1, 1, 784, 2]): grad_xes is summed over the mixtures",
            "fwd_ms": o["fwd_ms"], "bwd_ms": o["bwd_ms"], "ms_per_step": o["ms_step"]}
        o = measure_dense("C5", 10, 2)
        w = o["wl"]
        others["C5_dense_f64"] = {
            "config": f"the C5 inputs through the dense path: D=3 f64 B=1 L=1 M={w.M} N={w.N}, {w.pairs:.4g} pairs",
            "fwd_ms": o["fwd_ms"], "bwd_ms": o["bwd_ms"], "ms_per_step": o["ms_step"],
            "fwd_frac_of_f64_peak": FLOP_FWD[3] * w.pairs / (o["fwd_ms"] * 1e-3) / 1e12 / PEAK_TFLOPS["f64"],
            "bwd_frac_of_f64_peak": FLOP_BWD[3] * w.pairs / (o["bwd_ms"] * 1e-3) / 1e12 / PEAK_TFLOPS["f64"],
            "fwd_kernel": o["fwd_kernel"]}
        others["C5"] = {"config": "D=3 f64 B=1 L=1 M=16384 N=100000, LBVH-culled (threshold 0.001): build + forward + backward per step",
                        "by_aabb_mode": [bvh_summary(measure_bvh(mode, 20, 3), mode) for mode in ("reference", "tight")]}
        for name in ("C2", "C3"):
            r = measure_bvh("tight", 20, 3, name=name)
            w = r["wl"]
            others[name + "_culled"] = {
                "config": f"{name} through the LBVH-culled path (aabb_mode=tight, threshold 0.001): build + forward + backward per step",
                **bvh_summary(r, "tight"), "evaluated_fraction_of_dense": r["hits"] / w.pairs,
                "dense_ms_per_step": others[name]["ms_per_step"]}
        line["other_workloads"] = others
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(dense_name)
    print(json.dumps(line))


def measure_dense(name: str, steps: int, warmup: int, copy_calibration: bool = False, broadcast_xes: bool = False):
    """Forward + backward (both gradients) of the dense path on the named workload; timings from HIP events on the
    launch stream (medians over the steps), the step time from the wall clock over all steps.  broadcast_xes: all
    mixtures share the points of the first one ([1, 1, N, D]; grad_xes is then summed over the mixtures)."""
    import torch
    from gmc import _native, synthetic
    wl, mix, xes, gout = synthetic.make_workload(name)
    if broadcast_xes:
        xes = xes[:1, :1].contiguous()
    dev = torch.device("cuda:0")
    mix, xes, gout = mix.to(dev), xes.to(dev), gout.to(dev)
    torch.cuda.synchronize()

    def step(ev=None):
        if ev:
            ev[0].record()
        out = _native.eval_fwd(mix, xes)
        if ev:
            ev[1].record()
        gm_, gx_ = _native.eval_bwd(gout, mix, xes, True, True)
        if ev:
            ev[2].record()
        return out, gm_, gx_

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    if copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for k in range(steps):
        step(events[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    import ctypes
    shape = _native.check_input(mix, xes)
    # shader clock that one workgroup in the middle of the last forward (float32 matrix-core kernel) and backward
    # launch saw: under this load the clock settles below the 2400 MHz that the published peak assumes
    mhz = (ctypes.c_double * 2)()
    clocks = (mhz[0], mhz[1]) if _native.lib().gmc_export_launch_clocks(mhz) == 0 else (0.0, 0.0)
    return {"wl": wl, "ms_step": wall * 1e3 / steps, "clocks_mhz": clocks,
            "fwd_ms": median([e[0].elapsed_time(e[1]) for e in events]),
            "bwd_ms": median([e[1].elapsed_time(e[2]) for e in events]),
            "fwd_ms_mean": sum(e[0].elapsed_time(e[1]) for e in events) / steps,
            "bwd_ms_mean": sum(e[1].elapsed_time(e[2]) for e in events) / steps,
            "fwd_kernel": _native.lib().gmc_eval_fwd_kernel_name(ctypes.byref(shape)).decode()}


if __name__ == "__main__":
    main()
