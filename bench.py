#!/usr/bin/env python3
"""Benchmark of the point-cloud operator path on one MI355X.

Workload (config 2 of the baseline: "object-scale MCConv fwd+bwd"): 16 clouds x 4096 points sampled
on random primitives and scaled into the unit cube; radius 0.05; density by Gaussian KDE with bandwidth
0.2 * radius; MCConv with a 3 -> 16 hidden kernel, 64 -> 128 channels, fp32.  Inputs are synthetic
(seeded) and resident in HBM before anything is timed.

One step = one MCConv forward plus one backward over the batch through the autograd wrapper, producing every
gradient the reference's mc_conv_grads returns (weights, features, axis, bias, density, points, samples); the
neighborhood and the densities are built beforehand.  `value` = points / second = M / step time.  The time of
the same step restricted to the gradients config 2 names (features and weights) is reported as an extra key.
In the same run the neighbor pipeline (box, keys, radix sort, pillar table, count, scan, fill) and the
density pipeline are timed as well and reported as extra keys of the same JSON line, next to

  roofline      the dominant kernel of the step (the fp32 MFMA contraction): algorithmic flops per launch
                divided by its mean launch duration, taken live with HIP events on the launch stream;
  roofline_neighbors   the same for the neighbor fill kernel against HBM bandwidth, measured on the
                million-point room of config 4 (`scene` carries that leg's pairs / second);
  roofline_projection_forward / _backward   the two projection kernels of the step against HBM bandwidth;
  cpu_baseline  the same step on the host cores: the vectorised torch form of the oracle on all threads over the whole
                workload, and the scalar oracle (C + numpy, one thread) on two clouds beside it.

Exactly one JSON line goes to stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_FP32_PEAK_TFLOPS = 157.3     # MI355X dense fp32 matrix peak
MFMA_BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 matrix peak
HBM_PEAK_GBPS = 8000.0            # MI355X HBM3E peak



def traffic(workload, kernel):
    """Bytes per launch that a kernel moves past the L2 on one of the default workloads, from the table kept beside
    the rocprofv3 counter summaries (profiles/traffic_table.json: FETCH_SIZE / WRITE_SIZE runs of this command, scaled
    by the copy kernel of known size); None when the table has no entry (another size, a kernel not yet measured)."""
    global _TRAFFIC
    if _TRAFFIC is None:
        try:
            with open(os.path.join(ROOT, "profiles", "traffic_table.json")) as handle:
                _TRAFFIC = json.load(handle)
        except (OSError, ValueError):
            _TRAFFIC = {}
    entry = _TRAFFIC.get(workload, {}).get(kernel)
    return float(entry["bytes"]) if entry else None


_TRAFFIC = None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_workload(seed=2, batch=16, num_pts=4096, c_in=64, c_out=128, hidden=16):
    from pccnn_lib_amd import synthetic
    pts, ids = synthetic.primitives(seed, batch, num_pts)
    rng = np.random.default_rng(seed)
    n = pts.shape[0]
    return dict(
        pts=pts, ids=ids, batch=batch, num_pts=num_pts, radius=0.05, bandwidth=0.2 * 0.05,
        feats=rng.normal(size=(n, c_in)).astype(np.float32),
        axis=rng.normal(0, np.sqrt(1.0 / 3.0), (3, hidden)).astype(np.float32),
        bias=np.zeros((1, hidden), np.float32),
        weights=rng.normal(0, np.sqrt(1.0 / (hidden * c_in)), (1, hidden * c_in, c_out)).astype(np.float32),
        out_grads=rng.normal(size=(n, c_out)).astype(np.float32),
        c_in=c_in, c_out=c_out, hidden=hidden)


def cpu_baseline(wl, scalar_clouds=2):
    """The same MCConv forward + backward on the host cores: the vectorised torch form on all threads over the whole
    workload (the reported baseline), and the scalar oracle on one thread over the first clouds beside it."""
    import torch
    from oracle import oracle, torch_cpu
    try:
        from threadpoolctl import threadpool_limits
    except ImportError:                                           # pragma: no cover
        threadpool_limits = None
    n = wl["batch"] * wl["num_pts"]
    pts, ids, feats = wl["pts"], wl["ids"], wl["feats"]
    unnorm, _, _ = oracle.pointcloud_pdf(pts, ids, wl["bandwidth"])
    nb = oracle.neighborhood(pts, ids, pts, ids, wl["radius"])
    pdf = (unnorm * np.prod(nb["radii"])).astype(np.float32)

    def timed(run, budget_s, max_reps):
        run()                                                     # warm-up
        t0 = time.perf_counter()
        reps = 0
        while reps < max_reps and (reps == 0 or time.perf_counter() - t0 < budget_s):
            run()
            reps += 1
        return (time.perf_counter() - t0) / reps, reps

    threads = torch.get_num_threads()
    dt, reps = timed(lambda: torch_cpu.mcconv_step(pts, pdf, feats, nb["neighbors"], nb["ends"], nb["radii"], wl["axis"],
                                                   wl["bias"], wl["weights"], wl["out_grads"]), 15.0, 20)
    result = {"value": n / dt, "unit": "points/s", "cores": threads, "kind": "port",
              "sample": "vectorised torch-CPU MCConv forward + all gradients (oracle/torch_cpu.py) on all %d clouds "
                        "(%d points, %d pairs), %d repetition(s), neighbor search and density excluded like in `value`"
                        % (wl["batch"], n, nb["neighbors"].shape[0], reps)}

    ns = scalar_clouds * wl["num_pts"]
    pairs = int(nb["ends"][ns - 1])
    args = (pts[:ns], pdf[:ns], feats[:ns], pts[:ns], nb["neighbors"][:pairs], nb["ends"][:ns], nb["radii"], wl["axis"],
            wl["bias"], wl["weights"])

    def scalar():
        oracle.mcconv(*args)
        oracle.mcconv_grads(*args, wl["out_grads"][:ns])

    ctx = threadpool_limits(limits=1) if threadpool_limits else None
    try:
        dts, _ = timed(scalar, 8.0, 3)
    finally:
        if ctx is not None:
            ctx.unregister() if hasattr(ctx, "unregister") else ctx.restore_original_limits()
    result["scalar_oracle"] = {"value": ns / dts, "unit": "points/s", "cores": 1,
                               "sample": "oracle mcconv + mcconv_grads (scalar C + numpy) on %d of %d clouds"
                                         % (scalar_clouds, wl["batch"])}
    return result


def config3_leg(lib, dev, timed, steps, warmup, with_cpu):
    """Config 3: KPConv on 8 x 8192 surface points, radius 0.04, 15 kernel points, 128 -> 256 channels, fp32; forward
    plus the gradients w.r.t. features, weights and point positions through the autograd wrapper."""
    import torch
    from pccnn_lib_amd import synthetic
    from pccnn_lib_amd.op_wrappers import ComputeKPConv
    batch, num_pts, c_in, c_out, k, radius = 8, 8192, 128, 256, 15, 0.04
    pts, ids = synthetic.primitives(3, batch, num_pts)
    rng = np.random.default_rng(3)
    kp, sigma = synthetic.kernel_points_sphere(3, k)
    feats = rng.normal(size=(pts.shape[0], c_in)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / (k * c_in)), (k * c_in, c_out)).astype(np.float32)
    og = rng.normal(size=(pts.shape[0], c_out)).astype(np.float32)
    t = lambda a: torch.as_tensor(a, device=dev)
    pc = lib.pc.Pointcloud(t(pts), t(ids))
    radii = torch.full((3,), radius, dtype=torch.float32, device=dev)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    mirror = nbh.mirror()
    pairs = int(nbh.neighbors_.shape[0])
    leaves = [x.clone().requires_grad_(True) for x in (t(pts), t(feats), t(w))]
    tkp, tog = t(kp), t(og)

    def step():
        p, f, ww = leaves
        out = ComputeKPConv.apply(p, f, p, nbh.neighbors_, nbh.start_ids_, radii, tkp, float(sigma), ww, mirror)
        return torch.autograd.grad(out, leaves, tog)

    ms, kernels = timed(step, steps, warmup)
    m = pts.shape[0]
    flops = 2.0 * m * (k * c_in) * c_out
    g_n, g_ms = kernels.get("gemm", (0, 0.0))
    g_avg = g_ms / max(g_n, 1)
    tflops = flops / (g_avg * 1e-3) / 1e12 if g_n else 0.0
    leg = {"workload": "config 3: KPConv fwd + dFeat, dW, dPts, 8 x 8192 points on random primitives, radius 0.04, "
                       "15 kernel points, Cin 128 -> Cout 256, fp32",
           "points": m, "pairs": pairs, "ms_per_step": ms, "points_per_sec": m / (ms * 1e-3),
           "kernels_us": {kk: round(1e3 * v[1] / v[0], 2) for kk, v in kernels.items()},
           "roofline": {"kernel": "gemm_f32_full_tiles_kernel (all three products)", "bound": "mfma", "achieved": tflops,
                        "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_FP32_PEAK_TFLOPS,
                        "traffic": traffic("config3", "contraction_f32"), "flops_per_launch": flops,
                        "avg_launch_ms": g_avg, "launches": g_n,
                        "shapes": "P[65536,1920] W[1920,256]; P^T dOut; dOut W^T (mean of the three launches)"}}
    # the two projection kernels of this step against HBM (bytes as for config 2: pairs, offsets, coordinates and
    # features in, the projection out; backward: the projection gradient in, feature gradient, basis gradient and
    # per-pair point gradients out)
    geo = 8.0 * pairs + 4.0 * m + 12.0 * 2 * m + 4.0 * m * c_in
    proj = 4.0 * m * c_in * k
    for key, name, alg in (("proj_fwd", "conv_proj_fwd_kernel", geo + proj),
                           ("proj_bwd", "conv_proj_bwd_kernel", geo + proj + 4.0 * m * c_in + 4.0 * pairs * k + 16.0 * pairs)):
        k_n, k_ms = kernels.get(key, (0, 0.0))
        avg = k_ms / max(k_n, 1)
        gbps = alg / (avg * 1e-3) / 1e9 if k_n else 0.0
        leg["roofline_projection_" + ("forward" if key == "proj_fwd" else "backward")] = {
            "kernel": name, "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic("config3", name), "bytes_per_launch": alg,
            "avg_launch_ms": avg, "launches": k_n}
    log("config 3: %d pairs, step %.3f ms" % (pairs, ms),
        {kk: "%d x %.1f us" % (v[0], 1e3 * v[1] / v[0]) for kk, v in kernels.items()})
    if with_cpu:
        # the same step in torch on the host cores, on the first two of the eight clouds
        from oracle import oracle, torch_cpu
        ns = 2 * num_pts
        nb = oracle.neighborhood(pts[:ns], ids[:ns], pts[:ns], ids[:ns], radius)
        run = lambda: torch_cpu.kpconv_step(pts[:ns], feats[:ns], nb["neighbors"], nb["ends"], nb["radii"], kp, sigma, w,
                                            og[:ns])
        run()
        t0 = time.perf_counter()
        reps = 0
        while reps < 10 and (reps == 0 or time.perf_counter() - t0 < 8.0):
            run()
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        leg["cpu_baseline"] = {"value": ns / dt, "unit": "points/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "vectorised torch-CPU KPConv forward + weight, feature and position gradients "
                                         "(oracle/torch_cpu.py) on 2 of the 8 clouds (%d points, %d pairs), %d "
                                         "repetition(s)" % (ns, nb["neighbors"].shape[0], reps)}
        log("config 3 cpu baseline: %.0f points/s" % (ns / dt))
    return leg


def config5_leg(lib, dev, steps, warmup):
    """Config 5: 8 x 100 000 room points, four Poisson-disk levels (radii 0.025 / 0.05 / 0.1 / 0.2 of the room's
    longest side), each with neighbor search (2 x the pooling radius), density and an MCConv with division by the
    density, channels 8 -> 32 -> 64 -> 128 -> 256, bf16 contraction operands with fp32 accumulation; one forward pass
    through the four levels and one backward pass, host-synchronised only at the end.  As in a training step, the
    parameters' gradients are reset to none before the pass (what ``optimizer.zero_grad()`` does), and the backward
    pass starts from a gradient of ones on the last level's features (the gradient of their sum)."""
    import torch
    from pccnn_lib_amd import synthetic
    batch, num_pts = 8, 100000
    pts = np.concatenate([synthetic.room(70 + b, num_pts) / 10.0 for b in range(batch)]).astype(np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int32), num_pts)
    tp, ti = torch.as_tensor(pts, device=dev), torch.as_tensor(ids, device=dev)
    torch.manual_seed(5)
    layers, c_in = [], 8
    for c_out in (32, 64, 128, 256):
        layer = lib.pc.layers.MCConv(3, c_in, c_out, 8).to(dev)
        layer.contraction_ = "bf16"
        layers.append(layer)
        c_in = c_out
    feats0 = torch.randn(pts.shape[0], 8, device=dev)
    radii_levels = (0.025, 0.05, 0.1, 0.2)
    sizes, marks = [], []
    params = [p for layer in layers for p in layer.parameters()]
    ones = {}

    def drained():
        # the device has finished what was queued (a spin on an event query: torch.cuda.synchronize() returns some
        # tens of microseconds late, which would be charged to every level of the split run)
        mark = torch.cuda.Event()
        mark.record()
        while not mark.query():
            pass

    def whole(split=False, input_grad=True):
        for p in params:
            p.grad = None
        pc = lib.pc.Pointcloud(tp, ti)
        feats = feats0.clone().requires_grad_(input_grad)
        del sizes[:], marks[:]
        for level, radius in enumerate(radii_levels):
            if split:
                drained()
                marks.append(time.perf_counter())
            # (the density is queued between the pooling and the first use of its result: the device computes it
            # while the host waits for the size of the selection)
            pool = lib.pc.PointPooling(pc, radius)
            pc.compute_pdf(0.2 * radius)
            out_pc = lib.pc.Pointcloud(pool.pool_tensor(pc.pts_), pool.pool_tensor(pc.batch_ids_))
            feats, nbh = layers[level](pc, out_pc, feats, 2.0 * radius)
            feats = torch.nn.functional.leaky_relu(feats, 0.2)
            # (the pair count from the list the search kept: reading neighbors_ of a key-order list would make the
            # original-index copy just for its shape)
            kept = nbh.neighbors_original_ if nbh.neighbors_original_ is not None else nbh.neighbors_key_order_
            sizes.append((int(pc.pts_.shape[0]), int(out_pc.pts_.shape[0]), int(kept.shape[0])))
            pc = out_pc
        if split:
            drained()
            marks.append(time.perf_counter())
        shape = tuple(feats.shape)
        if shape not in ones:
            ones[shape] = torch.ones(shape, dtype=feats.dtype, device=dev)
        feats.backward(ones[shape])
        if split:
            drained()
            marks.append(time.perf_counter())
        return feats

    for _ in range(warmup):
        whole()
    stream = torch.cuda.current_stream()
    passes = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        passes[i].record(stream)
        whole()
    passes[steps].record(stream)
    torch.cuda.synchronize()
    mean_ms = (time.perf_counter() - t0) / steps * 1e3
    ms = float(np.median([passes[i].elapsed_time(passes[i + 1]) for i in range(steps)]))
    # the same pass with the input features as plain data (no gradient asked for them, as in a training step whose
    # first layer reads the raw point attributes): the first level's backward projection then has no feature rows to add
    data_passes = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    for i in range(steps):
        data_passes[i].record(stream)
        whole(input_grad=False)
    data_passes[steps].record(stream)
    torch.cuda.synchronize()
    data_ms = float(np.median([data_passes[i].elapsed_time(data_passes[i + 1]) for i in range(steps)]))
    split_ms = np.zeros(5)
    for _ in range(steps):
        whole(split=True)
        split_ms += np.diff(np.array(marks)) * 1e3
    split_ms /= steps
    levels = [{"level": i, "radius": radii_levels[i], "points_in": sizes[i][0], "points_out": sizes[i][1],
               "pairs": sizes[i][2], "forward_ms": float(split_ms[i])} for i in range(4)]
    leg = {"workload": "config 5: 8 x 100000 room points, four Poisson-disk levels (0.025/0.05/0.1/0.2), neighbor "
                       "search + density + MCConv 8->32->64->128->256 with bf16 contraction operands, forward + backward",
           "points": int(pts.shape[0]), "ms_per_pass": ms, "ms_per_pass_mean_wall": mean_ms,
           "ms_per_pass_input_features_without_gradient": data_ms, "points_per_sec": pts.shape[0] / (ms * 1e-3),
           "dtype": "bf16 operands, f32 accumulate", "levels": levels, "backward_ms": float(split_ms[4]),
           "note": "ms_per_pass is the median over the passes (HIP events around each), synchronised at the end only; the per-level times come from a second run with a "
                   "host synchronisation between the levels, so they add up to more"}
    log("config 5: pass %.3f ms (%.3f ms without a gradient for the input features)" % (ms, data_ms), [(l["points_in"], l["points_out"], l["pairs"], round(l["forward_ms"], 3))
                                        for l in levels], "backward %.3f ms" % split_ms[4])
    return leg


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: the first few milliseconds after an idle spell run at a lower shader clock and with the caching
    # allocator still growing (about 2 ms spread over the first steps), so the warm-up is 50 steps (40 ms) and the
    # timed region 100
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-scene", action="store_true", help="skip the million-point neighbor-search leg")
    ap.add_argument("--scene-points", type=int, default=1000000)
    ap.add_argument("--profile-leg", choices=["config3", "config5"], default=None,
                    help="run this leg only (for rocprofv3 runs of one leg)")
    ap.add_argument("--no-config3", action="store_true", help="skip the KPConv leg of config 3")
    ap.add_argument("--no-config5", action="store_true", help="skip the four-level bf16 encoder leg of config 5")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on one GPU only; --gpus %d is not supported "
            "(no collectives or sharding are part of it)" % args.gpus)
        return 2

    import torch
    from pccnn_lib_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        log("libpccnn_hip.so not found, building it")
        build.build(verbose=False)
    if not torch.cuda.is_available():
        log("bench.py needs a GPU (torch.cuda.is_available() is False)")
        return 3
    import pccnn_lib_amd as lib
    ops = lib.pccnn_lib_ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    def timed(fn, steps, warmup, stats=None):
        """(ms per step, per-kernel timings).  After the warm-up exactly `steps` steps run between two device
        synchronisations, each bracketed by HIP events on the launch stream; the step time reported is the MEDIAN of
        those per-step durations, and `stats` (a dict, optional) also receives the wall-clock mean over the same
        steps, the fastest and the slowest step.  That pass runs without the library's event hooks (they serialise
        the stream around every hooked launch); a second pass of the same steps with the hooks on gives the
        per-kernel durations."""
        for _ in range(warmup):
            fn()
        stream = torch.cuda.current_stream()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            marks[i].record(stream)
            fn()
        marks[steps].record(stream)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        per_step = np.array([marks[i].elapsed_time(marks[i + 1]) for i in range(steps)])
        if stats is not None:
            stats.update(median_ms=float(np.median(per_step)), mean_wall_ms=dt / steps * 1e3,
                         min_ms=float(per_step.min()), max_ms=float(per_step.max()), steps=steps)
        _lib.timing(enable=True, reset=True)
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        kernels = _lib.timing(enable=False)
        if stats is not None and stats.get("sustained"):
            # the same step once the device has been under this load for a while: after an idle spell the part's clock
            # management takes 30 - 40 ms of continuous work to settle (the first steps run up to 20 % slower), which
            # a short warm-up does not cover; 60 more untimed steps, then the median of 100
            for _ in range(60):
                fn()
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(101)]
            for i in range(100):
                marks[i].record(stream)
                fn()
            marks[100].record(stream)
            torch.cuda.synchronize()
            stats["sustained_ms"] = float(np.median([marks[i].elapsed_time(marks[i + 1]) for i in range(100)]))
        return float(np.median(per_step)), kernels

    # what a plain float4 copy reaches on this part, as the practical ceiling beside the published 8 TB/s: 1 GiB read
    # and 1 GiB written per launch (beyond every cache), timed with events on the launch stream.  The same launches
    # are the known-size yardstick that rocprofv3's traffic counters are scaled against.
    src = torch.ones(256 << 20, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    cs = torch.cuda.current_stream()
    copy_call = lambda: _lib.call("pccnn_calibration_copy", _lib.P(src.data_ptr()), _lib.P(dst.data_ptr()), src.numel(),
                                  _lib.P(cs.cuda_stream))
    for _ in range(2):
        copy_call()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(cs)
    for _ in range(5):
        copy_call()
    e1.record(cs)
    torch.cuda.synchronize()
    copy_gbps = 5 * 2.0 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    log("copy ceiling: %.0f GB/s" % copy_gbps)
    del src, dst

    if args.profile_leg:
        # one leg alone, for a profiler run of that leg (the JSON line then carries only that leg)
        leg = config3_leg(lib, dev, timed, args.steps, args.warmup, False) if args.profile_leg == "config3" \
            else config5_leg(lib, dev, args.steps, args.warmup)
        print(json.dumps({"leg": args.profile_leg, "result": leg}), flush=True)
        return 0

    wl = make_workload()
    t = lambda a: torch.as_tensor(a, device=dev)
    pts, ids, feats = t(wl["pts"]), t(wl["ids"]), t(wl["feats"])
    axis, bias, weights, out_grads = t(wl["axis"]), t(wl["bias"]), t(wl["weights"]), t(wl["out_grads"])
    radii = torch.full((3,), wl["radius"], dtype=torch.float32, device=dev)
    bw = torch.full((3,), wl["bandwidth"], dtype=torch.float32, device=dev)
    m = pts.shape[0]

    # ---- untimed set-up: density and neighborhood (they are inputs of the timed step)
    pc = lib.pc.Pointcloud(pts, ids)
    pc.compute_pdf(bw)
    nbh = lib.pc.layers.conv_base.build_neighborhood(pc, pc, radii, 0)
    neigh, ends = nbh.neighbors_, nbh.start_ids_
    pdf = (pc.pts_unnorm_pdf_ * torch.prod(radii)).contiguous()
    total_pairs = int(neigh.shape[0])
    torch.cuda.synchronize()
    log("workload: M=N=%d, T=%d pairs (%.1f per point)" % (m, total_pairs, total_pairs / m))

    # The step runs through the autograd wrapper, as a training loop would: forward, then backward for every
    # differentiable input (points - which are also the samples -, density, features, axis, bias, weights),
    # i.e. all the gradients the reference's mc_conv_grads returns.
    from pccnn_lib_amd.op_wrappers import ComputeMCConv
    leaves = [x.clone().requires_grad_(True) for x in (pts, pdf, feats, axis, bias, weights)]

    mirror = nbh.mirror()        # the samples are the points: symmetric pair list (built once per neighborhood)

    def mirror_step():
        return ops.mirror_pairs(neigh, ends)

    def conv_step():
        p, q, f, a, b, w = leaves
        out = ComputeMCConv.apply(p, q, f, p, neigh, ends, radii, a, b, w, mirror)
        return torch.autograd.grad(out, leaves, out_grads)

    def conv_step_fw_only():
        # gradients w.r.t. features and weights only (the gradient set config 2 names); with the neighborhood's
        # mirror index at hand the feature gradients go through per-pair rows and a gather instead of atomics
        f, w = leaves[2], leaves[5]
        out = ComputeMCConv.apply(pts, pdf, f, pts, neigh, ends, radii, axis, bias, w, mirror)
        return torch.autograd.grad(out, [f, w], out_grads)

    def conv_step_deterministic():
        # the headline step with the backward pass that uses no float atomics (bit-identical from run to run)
        before = ops.set_deterministic(True)
        try:
            return conv_step()
        finally:
            ops.set_deterministic(before)

    def forward_only():
        # inference: no projection is kept
        with torch.no_grad():
            return ComputeMCConv.apply(pts, pdf, feats, pts, neigh, ends, radii, axis, bias, weights)

    def forward_only_fused():
        before = ops.set_fused_forward(True)
        try:
            return forward_only()
        finally:
            ops.set_fused_forward(before)

    def conv_step_bf16():
        # the same step with the three contractions on the bf16 matrix pipe (bf16 operands, fp32 accumulation)
        p, q, f, a, b, w = leaves
        out = ComputeMCConv.apply(p, q, f, p, neigh, ends, radii, a, b, w, mirror, "bf16")
        return torch.autograd.grad(out, leaves, out_grads)

    def pc_fresh():
        p = lib.pc.Pointcloud.__new__(lib.pc.Pointcloud)         # same tensors, nothing cached: a cold build
        p.__dict__.update(pc.__dict__)
        p.__dict__.pop("aabb_cache_", None)
        return p

    def neighbor_step():
        p = pc_fresh()
        return lib.pc.layers.conv_base.build_neighborhood(p, p, radii, 0)

    def pdf_step():
        p = pc_fresh()
        p.compute_pdf(bw)
        return p

    # The headline step is timed twice with the same W warm-up and K timed steps: once as the first work the device
    # sees after the host-side set-up above (`ms_per_step_from_idle`: the part's clock management needs 30 - 40 ms of
    # continuous load to settle, so a short run from idle reads up to 10 % slow), and again behind the other
    # forward + backward legs of this workload, when the device has been under the same kind of load without a break
    # (`ms_per_step`, `value`): the state a training loop is in after its first few dozen steps.  (The forward-only
    # legs follow it: their kernels load the device less, and a measurement behind them reads 0.83 ms again.)
    idle_stats, conv_stats, fw_stats = {}, {"sustained": True}, {"sustained": True}
    idle_ms, _ = timed(conv_step, args.steps, args.warmup, idle_stats)
    fw_ms, _ = timed(conv_step_fw_only, args.steps, args.warmup, fw_stats)
    bf_ms, bf_kernels = timed(conv_step_bf16, args.steps, args.warmup)
    det_ms, _ = timed(conv_step_deterministic, args.steps, args.warmup)
    conv_ms, conv_kernels = timed(conv_step, args.steps, args.warmup, conv_stats)
    fwd_ms, _ = timed(forward_only, args.steps, args.warmup)
    fwd_fused_ms, _ = timed(forward_only_fused, args.steps, args.warmup)
    nb_ms, nb_kernels = timed(neighbor_step, args.steps, args.warmup)
    pdf_ms, pdf_kernels = timed(pdf_step, args.steps, args.warmup)
    mirror_ms, _ = timed(mirror_step, args.steps, args.warmup)
    log("conv fwd+bwd %.3f ms median, %.3f ms wall-clock mean (features+weights grads only: %.3f ms) | neighborhood "
        "%.3f ms | density %.3f ms | sustained %.3f / %.3f ms" % (conv_ms, conv_stats["mean_wall_ms"], fw_ms, nb_ms, pdf_ms,
                                                                  conv_stats["sustained_ms"], fw_stats["sustained_ms"]))
    log("conv fwd+bwd with bf16 contraction operands: %.3f ms | without atomics: %.3f ms | forward only %.3f ms "
        "(fused %.3f ms)" % (bf_ms, det_ms, fwd_ms, fwd_fused_ms))
    for name, ks in (("conv", conv_kernels), ("conv bf16", bf_kernels), ("neighbors", nb_kernels),
                     ("pdf", pdf_kernels)):
        log(name, {k: "%d x %.1f us" % (v[0], 1e3 * v[1] / v[0]) for k, v in ks.items()})

    # ---- roofline of the dominant kernel: the contraction (three launches per step, equal flops)
    kdim = wl["hidden"] * wl["c_in"]
    gemm_flops = 2.0 * m * kdim * wl["c_out"]
    gemm_n, gemm_total_ms = conv_kernels.get("gemm", (0, 0.0))
    gemm_avg_ms = gemm_total_ms / max(gemm_n, 1)
    gemm_tflops = gemm_flops / (gemm_avg_ms * 1e-3) / 1e12 if gemm_n else 0.0
    roofline = {"kernel": "gemm_f32_full_tiles_kernel (P W, Pt dOut), gemm_f32_mfma_kernel (dOut Wt)", "bound": "mfma", "achieved": gemm_tflops,
                "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": gemm_tflops / MFMA_FP32_PEAK_TFLOPS,
                "traffic": traffic("config2", "contraction_f32"), "flops_per_launch": gemm_flops, "avg_launch_ms": gemm_avg_ms,
                "launches": gemm_n}

    # ---- the two projection kernels against HBM bandwidth.  Algorithmic bytes, forward: pairs 8T + offsets 4M +
    # coordinates 12(N + M) + features 4 N Cin + density 4N in, projection 4 M Cin K out.  Backward: the projection
    # gradient 4 M Cin K, pairs, offsets, coordinates, features and density in; feature gradient 4 N Cin, basis
    # gradient 4 T K and the per-pair point gradients 16 T out.
    t_pairs = float(total_pairs)
    geo_bytes = 8.0 * t_pairs + 4.0 * m + 12.0 * 2 * m + 4.0 * m * wl["c_in"] + 4.0 * m
    proj_bytes = 4.0 * m * kdim
    rooflines_proj = {}
    for key, name, alg, moved in (
            ("proj_fwd", "conv_proj_fwd_kernel", geo_bytes + proj_bytes, traffic("config2", "conv_proj_fwd_kernel")),
            ("proj_bwd", "conv_proj_bwd_kernel", geo_bytes + proj_bytes + 4.0 * m * wl["c_in"] +
             4.0 * t_pairs * wl["hidden"] + 16.0 * t_pairs, traffic("config2", "conv_proj_bwd_kernel"))):
        k_n, k_ms = conv_kernels.get(key, (0, 0.0))
        avg = k_ms / max(k_n, 1)
        gbps = alg / (avg * 1e-3) / 1e9 if k_n else 0.0
        rooflines_proj[key] = {"kernel": name, "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                               "frac": gbps / HBM_PEAK_GBPS, "traffic": moved, "bytes_per_launch": alg,
                               "avg_launch_ms": avg, "launches": k_n}

    # the same three launches on the bf16 pipe (reported beside the fp32 figures; `value` is the fp32 step)
    bf_n, bf_total_ms = bf_kernels.get("gemm", (0, 0.0))
    bf_avg_ms = bf_total_ms / max(bf_n, 1)
    bf_tflops = gemm_flops / (bf_avg_ms * 1e-3) / 1e12 if bf_n else 0.0
    bf16_leg = {"ms_per_step": bf_ms, "points_per_sec": m / (bf_ms * 1e-3), "dtype": "bf16 operands, f32 accumulate",
                "kernels_us": {k: round(1e3 * v[1] / v[0], 2) for k, v in bf_kernels.items()},
                "roofline": {"kernel": "gemm_bf16_mfma_kernel", "bound": "mfma", "achieved": bf_tflops,
                             "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": bf_tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None,
                             "flops_per_launch": gemm_flops, "avg_launch_ms": bf_avg_ms, "launches": bf_n}}

    # ---- neighbor fill kernel against HBM: 8T out + 24M (sample xyz, key, order, offsets) + 20N (point xyz, key)
    grid_bytes = 8 * wl["batch"] * int(np.prod(nbh.grid_.num_cells_host()[0:2]))
    nb_bytes = 8.0 * total_pairs + 24.0 * m + 20.0 * m + grid_bytes
    fill_n, fill_total_ms = nb_kernels.get("nb_fill", (0, 0.0))
    fill_avg_ms = fill_total_ms / max(fill_n, 1)
    fill_gbps = nb_bytes / (fill_avg_ms * 1e-3) / 1e9 if fill_n else 0.0
    roofline_nb = {"kernel": "neighbors_group_kernel<fill, 8 lanes per sample>", "workload": "config 2", "bound": "hbm", "achieved": fill_gbps, "peak": HBM_PEAK_GBPS,
                   "unit": "GB/s", "frac": fill_gbps / HBM_PEAK_GBPS, "traffic": traffic("config2", "neighbors_fill"),
                   "bytes_per_launch": nb_bytes, "avg_launch_ms": fill_avg_ms, "launches": fill_n}

    # ---- scene-scale neighbor search (config 4: one room of 10^6 points, cell = radius = 0.05 m): the
    # neighbor kernels only show their throughput at this size, so their roofline entry is taken here
    scene = roofline_sort = roofline_pdf = roofline_pdf_grid = roofline_nb_count = roofline_nb_search = None
    if not args.no_scene:
        from pccnn_lib_amd import synthetic
        spts = t(synthetic.room(4, args.scene_points))
        sids = torch.zeros((spts.shape[0],), dtype=torch.int32, device=dev)
        sradii = torch.full((3,), 0.05, dtype=torch.float32, device=dev)
        spc = lib.pc.Pointcloud(spts, sids)

        def scene_step():
            p = lib.pc.Pointcloud.__new__(lib.pc.Pointcloud)
            p.__dict__.update(spc.__dict__)
            p.__dict__.pop("aabb_cache_", None)             # a cold build: the box is computed again
            return lib.pc.layers.conv_base.build_neighborhood(p, p, sradii, 0)

        snb = scene_step()
        s_pairs = int(snb.neighbors_.shape[0])
        s_ms, s_kernels = timed(scene_step, max(args.steps // 2, 3), 2)
        n_s = spts.shape[0]
        s_grid = 8 * int(np.prod(snb.grid_.num_cells_host()[0:2]))
        s_bytes = 8.0 * s_pairs + 24.0 * n_s + 20.0 * n_s + s_grid
        f_n, f_ms = s_kernels.get("nb_fill", (0, 0.0))
        f_avg = f_ms / max(f_n, 1)
        s_gbps = s_bytes / (f_avg * 1e-3) / 1e9 if f_n else 0.0
        roofline_nb = {"kernel": "neighbors_fill_masks_kernel", "workload": "config 4: %d room points, radius 0.05" % n_s,
                       "bound": "hbm", "achieved": s_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                       "frac": s_gbps / HBM_PEAK_GBPS,
                       "traffic": traffic("scene_%d" % n_s, "neighbors_fill"), "bytes_per_launch": s_bytes,
                       "avg_launch_ms": f_avg, "launches": f_n}
        # the count pass of the same search: the fill's inputs (24M + 20N + pillar table), per-sample counts 4M out
        c_n, c_ms = s_kernels.get("nb_count", (0, 0.0))
        c_avg = c_ms / max(c_n, 1)
        c_bytes = 24.0 * n_s + 20.0 * n_s + s_grid + 4.0 * n_s
        c_gbps = c_bytes / (c_avg * 1e-3) / 1e9 if c_n else 0.0
        roofline_nb_count = {"kernel": "neighbors_kernel<count>", "workload": roofline_nb["workload"], "bound": "hbm",
                             "achieved": c_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": c_gbps / HBM_PEAK_GBPS,
                             "traffic": traffic("scene_%d" % n_s, "neighbors_count"), "bytes_per_launch": c_bytes,
                             "avg_launch_ms": c_avg, "launches": c_n}
        # the whole search as a caller sees it (box, keys, sort, pillar table, count, scan, fill, the two read-backs
        # of sizes): the algorithmic bytes of its stages (keys 24N, sort 44N, table 8N + 8 B nc0 nc1, search
        # 8T + 24M + 20N + 8 B nc0 nc1) over the time of one neighborhood build
        e2e_bytes = 24.0 * n_s + 44.0 * n_s + 8.0 * n_s + s_grid + s_bytes
        e2e_gbps = e2e_bytes / (s_ms * 1e-3) / 1e9
        roofline_nb_search = {"kernel": "neighborhood build end to end (box, keys, sort, table, count, scan, fill)",
                              "workload": roofline_nb["workload"], "bound": "hbm", "achieved": e2e_gbps,
                              "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": e2e_gbps / HBM_PEAK_GBPS, "traffic": None,
                              "bytes_per_launch": e2e_bytes, "avg_launch_ms": s_ms, "launches": max(args.steps // 2, 3)}
        # the density of the same scene (Pointcloud.compute_pdf, bandwidth 0.2 x radius: its own grid of cell size
        # 4 x bandwidth, then the KDE walk on it)
        sbw = np.full(3, 0.2 * 0.05, np.float32)

        def scene_pdf_step():
            p = lib.pc.Pointcloud.__new__(lib.pc.Pointcloud)
            p.__dict__.update(spc.__dict__)
            p.__dict__.pop("aabb_cache_", None)             # a cold build: the box is computed again
            p.compute_pdf(sbw)
            return p

        scene_pdf_step()
        sp_ms, sp_kernels = timed(scene_pdf_step, max(args.steps // 2, 3), 2)
        # the key sort of the scene's grid: 44 N algorithmic bytes for one logical sort (keys 8N in, sorted keys 8N,
        # permutation 4N and gathered coordinates 12N + 12N out), however many digit passes it takes
        so_n, so_ms = s_kernels.get("sort", (0, 0.0))
        so_avg = so_ms / max(so_n, 1)
        so_gbps = 44.0 * n_s / (so_avg * 1e-3) / 1e9 if so_n else 0.0
        roofline_sort = {"kernel": "radix_hist / radix_scan / radix_scatter (all passes of one sort)",
                         "workload": "config 4: %d keys of %d significant bits" % (n_s, snb.grid_.key_bits()),
                         "bound": "hbm", "achieved": so_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": so_gbps / HBM_PEAK_GBPS, "traffic": None, "bytes_per_launch": 44.0 * n_s,
                         "avg_launch_ms": so_avg, "launches": so_n,
                         "traffic_last_pass": traffic("scene_%d" % n_s, "radix_scatter_kernel_last_pass")}
        # the density two ways: the walk on the grid that Pointcloud.compute_pdf runs (no pair list: sorted xyz 12N and
        # keys 8N in, estimate and normalised estimate 8N out), and the list form of the reference's op on the
        # radius-0.05 pair list (pairs 8T and xyz 12N in, offsets 4N in, estimate 4N out)
        pg_n, pg_ms = sp_kernels.get("pdf", (0, 0.0))
        pg_avg = pg_ms / max(pg_n, 1)
        pg_gbps = 28.0 * n_s / (pg_avg * 1e-3) / 1e9 if pg_n else 0.0
        roofline_pdf_grid = {"kernel": "pdf_grid_kernel", "workload": "config 4, bandwidth 0.01 (cell 0.04, cap 300)",
                             "bound": "hbm", "achieved": pg_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                             "frac": pg_gbps / HBM_PEAK_GBPS, "traffic": traffic("scene_%d" % n_s, "pdf_grid_kernel"),
                             "bytes_per_launch": 28.0 * n_s, "avg_launch_ms": pg_avg, "launches": pg_n}
        tbw = torch.as_tensor(sbw, device=dev)
        list_pdf_step = lambda: ops.compute_pdf(3, tbw, spts, snb.neighbors_, snb.start_ids_)
        list_pdf_step()
        _, pl_kernels = timed(list_pdf_step, max(args.steps // 2, 3), 2)
        pl_n, pl_ms = pl_kernels.get("pdf", (0, 0.0))
        pl_avg = pl_ms / max(pl_n, 1)
        pl_bytes = 8.0 * s_pairs + 20.0 * n_s
        pl_gbps = pl_bytes / (pl_avg * 1e-3) / 1e9 if pl_n else 0.0
        roofline_pdf = {"kernel": "pdf_kernel", "workload": "config 4: compute_pdf on the radius-0.05 pair list "
                                                            "(%d pairs), bandwidth 0.01" % s_pairs,
                        "bound": "hbm", "achieved": pl_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": pl_gbps / HBM_PEAK_GBPS, "traffic": traffic("scene_%d" % n_s, "pdf_kernel"),
                        "bytes_per_launch": pl_bytes,
                        "avg_launch_ms": pl_avg, "launches": pl_n}
        scene = {"points": n_s, "pairs": s_pairs, "neighborhood_ms": s_ms,
                 "neighbor_pairs_per_sec": s_pairs / (s_ms * 1e-3),
                 "kernels_us": {k: round(1e3 * v[1] / v[0], 2) for k, v in s_kernels.items()},
                 "density_ms": sp_ms, "density_bandwidth": 0.01,
                 # config 4 as the baseline words it: keys, grid, neighbors, then the density, per neighbor pair
                 "neighbor_pairs_per_sec_with_density": s_pairs / ((s_ms + sp_ms) * 1e-3),
                 "density_kernels_us": {k: round(1e3 * v[1] / v[0], 2) for k, v in sp_kernels.items()}}
        log("scene: %d points, %d pairs, neighborhood %.3f ms -> %.2f G pairs/s" % (n_s, s_pairs, s_ms,
                                                                                  s_pairs / s_ms / 1e6))
        log("scene", {k: "%d x %.1f us" % (v[0], 1e3 * v[1] / v[0]) for k, v in s_kernels.items()})
        log("scene density %.3f ms" % sp_ms, {k: "%d x %.1f us" % (v[0], 1e3 * v[1] / v[0]) for k, v in sp_kernels.items()})

    config3 = None if args.no_config3 else config3_leg(lib, dev, timed, args.steps, args.warmup,
                                                        not args.no_cpu_baseline)
    config5 = None if args.no_config5 else config5_leg(lib, dev, max(args.steps // 2, 3), 2)

    cpu = None
    if not args.no_cpu_baseline:
        log("timing the CPU oracle on a sample ...")
        cpu = cpu_baseline(wl)
        log("cpu baseline: %.0f points/s" % cpu["value"])

    result = {
        "metric": "mcconv_fwd_bwd_points_per_sec", "value": m / (conv_ms * 1e-3), "unit": "points/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": conv_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: MCConv fwd+bwd, 16 x 4096 points on random primitives, radius 0.05, "
                               "KDE bandwidth 0.01, hidden 16, Cin 64 -> Cout 128, fp32",
                   "points": m, "pairs": total_pairs, "seed": 2,
                   "gradients": "all inputs (features, weights, axis, bias, density, positions); the step with the "
                                "feature and weight gradients only is ms_per_step_feature_and_weight_grads_only"},
        "timing": "ms_per_step is the median of the per-step durations of the timed steps (HIP events on the launch "
                  "stream around every step); ms_per_step_mean_wall is the wall-clock mean over the same steps. The "
                  "step is timed twice with the same warm-up and step counts: as the first device work of the run "
                  "(ms_per_step_from_idle, clocks still ramping) and again behind the other forward + backward legs of this workload "
                  "(ms_per_step, value)",
        "ms_per_step_from_idle": idle_ms, "ms_per_step_from_idle_mean_wall": idle_stats["mean_wall_ms"],
        "ms_per_step_mean_wall": conv_stats["mean_wall_ms"], "ms_per_step_min": conv_stats["min_ms"],
        "ms_per_step_max": conv_stats["max_ms"],
        # (not `value`: the same step after 60 more untimed steps, median of 100 - what a training loop sees once the
        # part's clock management has settled under the load)
        "ms_per_step_sustained": conv_stats["sustained_ms"],
        "ms_per_step_feature_and_weight_grads_only": fw_ms,
        "ms_per_step_feature_and_weight_grads_only_mean_wall": fw_stats["mean_wall_ms"],
        "ms_per_step_feature_and_weight_grads_only_sustained": fw_stats["sustained_ms"],
        # the same step with the backward pass without float atomics (GRAD_DETERMINISTIC)
        "ms_per_step_deterministic": det_ms,
        # the forward pass alone under no_grad (no projection kept): the two-kernel path that is the default, and the
        # optional kernel that keeps the projection on chip
        "forward_only_ms": fwd_ms, "forward_only_fused_ms": fwd_fused_ms,
        # the symmetric-pair index that the step's point / density gradients use is built once per neighborhood
        # (outside ms_per_step); a step on a fresh neighborhood pays it once more
        "mirror_ms": mirror_ms, "ms_per_step_with_mirror": conv_ms + mirror_ms,
        "neighbor_pairs_per_sec": total_pairs / (nb_ms * 1e-3), "neighborhood_ms": nb_ms,
        "density_ms": pdf_ms,
        "kernels_us": {leg: {k: round(1e3 * v[1] / v[0], 2) for k, v in ks.items()}
                       for leg, ks in (("conv", conv_kernels), ("neighborhood", nb_kernels), ("density", pdf_kernels))},
        "bf16_contraction": bf16_leg, "scene": scene, "roofline": roofline, "roofline_neighbors": roofline_nb,
        "roofline_neighbors_count": roofline_nb_count, "roofline_neighbor_search": roofline_nb_search,
        "roofline_projection_forward": rooflines_proj["proj_fwd"],
        "roofline_projection_backward": rooflines_proj["proj_bwd"], "roofline_sort": roofline_sort,
        "roofline_pdf": roofline_pdf, "roofline_pdf_grid": roofline_pdf_grid, "config3": config3, "config5": config5,
        "hbm_copy_ceiling_gbps": copy_gbps,
        "cpu_baseline": cpu,
    }
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
