#!/usr/bin/env python3
"""Benchmark of the 3-D front end on one MI355X: voxelGenerator -> SpMiddleFHD conv stack -> sparse2Dense.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--points 20000] [--seed 0] [--dtype fp32|fp16]

A "step" is one frame: one pass of the whole path over one seeded synthetic LiDAR frame that is already
resident in device memory.  The timed region is exactly K pipeline enqueues bracketed by device
synchronisation.  One JSON line is printed with the frame time, the roofline position of the dominant
kernel (the 64->64 channel gather-GEMM, timed with HIP events on the pipeline's stream) and the CPU
baseline (the scalar oracle port, one core, same frame).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "se-ssd-ai-trt_amd"))

PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
PEAK_FP32_TFLOPS = 157.3    # MI355X dense FP32 (vector and matrix)
PEAK_FP16_TFLOPS = 2500.0   # MI355X dense FP16 MFMA


def layer_work(layer, n_in, n_out, pairs, esize):
    """Algorithmic work of one conv layer's gather-GEMM launch: flops = 2*P*Cin*Cout; bytes = gathered
    input rows + output rows written once + rulebook entries read + weights read once."""
    flops = 2.0 * pairs * layer.cin * layer.cout
    bytes_ = pairs * layer.cin * esize + n_out * layer.cout * esize + 8.0 * pairs + layer.kvol * layer.cin * layer.cout * esize
    return flops, bytes_


def profiled_traffic(kernel, dtype):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 summary (FETCH_SIZE and WRITE_SIZE
    runs, scaled by a copy kernel of known size), or None when no summary covers it."""
    path = os.path.join(ROOT, "profiles", "frame_pipeline_config3_%s.md" % dtype)
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.split("|")]
                if len(cells) >= 8 and cells[1] == kernel and cells[2].isdigit():
                    return float(round((float(cells[5]) + float(cells[6])) * 1e6))
    except (OSError, ValueError):
        pass
    return None


def cpu_model():
    """Model name of the host CPU as /proc/cpuinfo gives it."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def cpu_baseline(pts, layers, W, max_voxels, voxel_cap, budget_s=24.0):
    """The CPU port (the parity oracle) on the same frame, a bounded number of frames: once on one thread and
    once with the pairs of every kernel offset split over the host's cores (same bits either way)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    from sessd3d import backbone as B
    # (the oracle uses one capacity for every tensor; the voxelizer's cap equals it in the headline config)
    vg = B.voxelgen_desc(max_voxels=max_voxels if voxel_cap >= max_voxels else voxel_cap)
    dd = B.dense_desc(channel=layers[-1].cout)

    def median_ms(max_frames, budget):
        times, t_start = [], time.perf_counter()
        while len(times) < max_frames and (not times or (time.perf_counter() - t_start) < budget):
            t0 = time.perf_counter()
            O.frame(pts, vg, layers, W, dd)
            times.append((time.perf_counter() - t0) * 1e3)
        times.sort()
        return times[len(times) // 2], len(times)

    O.frame(pts, vg, layers, W, dd)          # warm-up (allocates the dense index grids)
    one, n_one = median_ms(3, budget_s / 2)
    # a one-GPU machine of this pool gives a job 16 cores, whatever os.cpu_count() reports
    threads = max(1, min(16, os.cpu_count() or 1))
    O.set_threads(threads)
    try:
        O.frame(pts, vg, layers, W, dd)
        many, n_many = median_ms(8, budget_s / 2)
    finally:
        O.set_threads(1)
    return {"value": round(many, 2), "unit": "ms/frame", "cores": threads, "kind": "port",
            "single_thread_ms": round(one, 2),
            "sample": "the same %d-point frame through oracle_frame (g++ -O2): median of %d frame(s) with the gather-GEMM's "
                      "pairs split over %d threads (value), median of %d frame(s) on one thread (single_thread_ms); "
                      "host reports %d logical CPUs (%s)" % (len(pts), n_many, threads, n_one, os.cpu_count() or 0,
                                                               cpu_model())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=[3, 4, 5],
                    help="benchmark configuration: 3 = 20k points FP32 (headline), 4 = 60k points, voxel cap 40k, FP16, "
                         "5 = 150k points over 360 degrees, voxel cap 60k, doubled channel widths, FP16")
    ap.add_argument("--points", type=int, default=None)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", default=None, choices=["fp32", "fp16"])
    ap.add_argument("--max-voxels", type=int, default=None, help="rows of the conv layers' tensors")
    ap.add_argument("--voxel-cap", type=int, default=None, help="the voxelizer's max_voxels")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels directly instead of replaying a hipGraph")
    ap.add_argument("--no-share", action="store_true", help="every SubM layer rebuilds its rulebook (as the reference does)")
    ap.add_argument("--pad-rows", action="store_true", help="write rows >= voxel_num of every tensor (reference behaviour)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="single stream: do not run the rulebook builds concurrently with the GEMMs of earlier layers")
    ap.add_argument("--no-two-in-flight", action="store_true",
                    help="skip the secondary throughput figure (two pipelines on two streams)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--profile-steps", type=int, default=50)
    ap.add_argument("--calibrate-mb", type=int, default=0,
                    help="after the timed region run a device-to-device copy of this many MiB three times: a kernel "
                         "of known traffic against which rocprofv3's FETCH_SIZE / WRITE_SIZE counters are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU (frames are independent; there is no multi-GPU mode); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from sessd3d import api, backbone as B, frames as F

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    preset = {3: dict(points=20000, dtype="fp32", max_voxels=60000, voxel_cap=60000, width=1, full=False),
              4: dict(points=60000, dtype="fp16", max_voxels=100000, voxel_cap=40000, width=1, full=False),
              5: dict(points=150000, dtype="fp16", max_voxels=200000, voxel_cap=60000, width=2, full=True)}[args.config]
    args.points = args.points or preset["points"]
    args.dtype = args.dtype or preset["dtype"]
    args.max_voxels = args.max_voxels or preset["max_voxels"]
    args.voxel_cap = args.voxel_cap or preset["voxel_cap"]
    layers = B.reference_layers(width_mult=preset["width"])
    W = B.random_weights(layers, seed=1, w_std=0.05 if args.dtype == "fp16" else 0.1)
    pts = F.lidar_frame(args.points, args.seed, full_circle=preset["full"])
    max_points = args.points
    pipe = api.Pipeline(layers, W, max_points, args.max_voxels, feature_dtype=args.dtype,
                        share_rulebooks=not args.no_share, skip_pad_rows=not args.pad_rows,
                        use_graph=not args.no_graph, overlap_streams=not args.no_overlap, voxel_cap=args.voxel_cap,
                        dense_size_xyz=B.DENSE_SIZE_XYZ)
    points = torch.as_tensor(pts).to(dev)
    size = torch.tensor([len(pts)], dtype=torch.int32, device=dev)
    dense = pipe.new_dense(dev)
    stream = torch.cuda.Stream()

    with torch.cuda.stream(stream):
        for _ in range(args.warmup):
            pipe.enqueue(points, size, dense, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        for _ in range(args.steps):
            pipe.enqueue(points, size, dense, stream)
    torch.cuda.synchronize()
    ms_per_frame = (time.perf_counter() - t0) * 1e3 / args.steps
    status = pipe.status(stream)

    # latency of single frames (one frame in flight, a synchronise between frames), outside the timed region
    lat = []
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    for _ in range(min(args.steps, 100)):
        with torch.cuda.stream(stream):
            ev[0].record(stream)
            pipe.enqueue(points, size, dense, stream)
            ev[1].record(stream)
        stream.synchronize()
        lat.append(ev[0].elapsed_time(ev[1]))
    lat_q = [round(float(v), 4) for v in np.percentile(lat, [50, 10, 90])]

    # throughput with two frames in flight: a second pipeline on a second stream, frames alternating.  Every
    # frame does all of its work; only the idle stretches of one frame (its launch-bound head, the narrow
    # layers) fill with the other's kernels.  Reported beside the headline, never as `value`.
    two_ms = None
    if not args.no_two_in_flight:
        pipe2 = api.Pipeline(layers, W, max_points, args.max_voxels, feature_dtype=args.dtype,
                             share_rulebooks=not args.no_share, skip_pad_rows=not args.pad_rows,
                             use_graph=not args.no_graph, overlap_streams=not args.no_overlap,
                             voxel_cap=args.voxel_cap, dense_size_xyz=B.DENSE_SIZE_XYZ)
        dense2 = pipe2.new_dense(dev)
        stream2 = torch.cuda.Stream()
        lanes = [(pipe, dense, stream), (pipe2, dense2, stream2)]

        def run_pairs(n):
            for i in range(n):
                pp, dd, ss = lanes[i & 1]
                with torch.cuda.stream(ss):
                    pp.enqueue(points, size, dd, ss)

        run_pairs(2 * max(2, args.warmup // 2))
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        run_pairs(args.steps)
        torch.cuda.synchronize()
        two_ms = (time.perf_counter() - t1) * 1e3 / args.steps
        same = bool(torch.equal(dense, dense2))
        del pipe2

    # per-layer active sites / rulebook pairs (small counting kernels, outside the timed region)
    n_vox, _ = pipe.layer_stats(-1, stream)
    stats, n_in = [], n_vox
    for l, layer in enumerate(layers):
        n_out, pairs = pipe.layer_stats(l, stream)
        stats.append((n_in, n_out, pairs))
        n_in = n_out

    # per-kernel durations: HIP events on the pipeline's stream around every segment, eager launches
    # (an event pair that brackets nothing still reads a few microseconds: that empty-segment time is
    # measured in the same pass and subtracted from every segment)
    seg, empty = None, 0.0
    with torch.cuda.stream(stream):
        for _ in range(5):
            pipe.enqueue_timed(points, size, dense, stream)
        for _ in range(args.profile_steps):
            s, e = pipe.enqueue_timed(points, size, dense, stream)
            s = np.asarray(s, np.float64)
            seg = s if seg is None else seg + s
            empty += e
    seg /= args.profile_steps
    empty /= args.profile_steps
    raw_sum = float(seg.sum())
    seg = np.maximum(seg - empty, 0.0)
    esize = 2 if args.dtype == "fp16" else 4
    per_layer = []
    tot_flops = tot_bytes = 0.0
    for l, layer in enumerate(layers):
        n_i, n_o, p = stats[l]
        fl, by = layer_work(layer, n_i, n_o, p, esize)
        tot_flops += fl
        tot_bytes += by
        per_layer.append({"name": layer.name, "n_in": n_i, "n_out": n_o, "pairs": p,
                          "build_us": round(seg[1 + 2 * l] * 1e3, 2), "gemm_us": round(seg[2 + 2 * l] * 1e3, 2),
                          "gemm_tflops": round(fl / (seg[2 + 2 * l] * 1e-3) / 1e12, 3) if seg[2 + 2 * l] > 0 else None,
                          "gemm_gbs": round(by / (seg[2 + 2 * l] * 1e-3) / 1e9, 1) if seg[2 + 2 * l] > 0 else None})
    # dominant kernel: the gather-GEMM instantiation for 64 -> 64 channels (six launches per frame)
    dom_c = 64 * preset["width"]
    dom = [l for l, layer in enumerate(layers) if layer.cin == dom_c and layer.cout == dom_c]
    dom_flops = sum(layer_work(layers[l], *stats[l], esize)[0] for l in dom) / len(dom)
    dom_bytes = sum(layer_work(layers[l], *stats[l], esize)[1] for l in dom) / len(dom)
    dom_ms = sum(seg[2 + 2 * l] for l in dom) / len(dom)
    peak_tf = PEAK_FP16_TFLOPS if args.dtype == "fp16" else PEAK_FP32_TFLOPS
    t_mfma = dom_flops / (peak_tf * 1e12)
    t_hbm = dom_bytes / (PEAK_HBM_GBS * 1e9)
    if t_mfma >= t_hbm:
        ach = dom_flops / (dom_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(ach, 3), "peak": peak_tf, "unit": "TFLOP/s",
                "frac": round(ach / peak_tf, 4), "traffic": None}
    else:
        ach = dom_bytes / (dom_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": None}
    tname = "__half" if args.dtype == "fp16" else "float"
    kname = "conv_mfma<%s, %d, %d, %s>" % (tname, dom_c, dom_c, tname)
    roof["traffic"] = profiled_traffic(kname, args.dtype) if args.config == 3 else None
    roof.update({"kernel": "gather-GEMM %d->%d (%s)" % (dom_c, dom_c, args.dtype), "launches_per_frame": len(dom),
                 "avg_launch_us": round(dom_ms * 1e3, 2), "algorithmic_flops_per_launch": dom_flops,
                 "algorithmic_bytes_per_launch": dom_bytes})
    # whole-frame algorithmic traffic: voxelizer + conv layers + sparse2dense (dense tensor written once)
    c_last, dsz = layers[-1].cout, B.DENSE_SIZE_XYZ
    frame_bytes = 16.0 * len(pts) + 32.0 * n_vox + tot_bytes + stats[-1][1] * (c_last * esize + 16) + \
        c_last * dsz[0] * dsz[1] * dsz[2] * esize
    out = {
        "metric": "ms/frame voxelize+3D sparse backbone @~17k voxels",
        "value": round(ms_per_frame, 4), "unit": "ms/frame", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_frame, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if args.dtype == "fp16" else "f32", "data": "synthetic",
        "config": {"workload": "config %d: %d-point seeded synthetic LiDAR frame (seed %d), %d voxels, reference 14-layer "
                               "SpMiddleFHD backbone (10 SubM + 4 SparseConv, channel widths x%d, BN folded + ReLU), "
                               "sparse2Dense to %dx200x176"
                               % (args.config, len(pts), args.seed, n_vox, preset["width"], layers[-1].cout * 2),
                   "max_voxels": args.max_voxels, "voxel_cap": args.voxel_cap, "graph": not args.no_graph, "overlap_streams": not args.no_overlap, "share_rulebooks": not args.no_share,
                   "pad_rows": args.pad_rows, "n_layers": len(layers)},
        "roofline": roof,
        "frame": {"frames_per_s": round(1e3 / ms_per_frame, 1), "algorithmic_gflop": round(tot_flops / 1e9, 3),
                  "algorithmic_mb": round(frame_bytes / 1e6, 2),
                  "hbm_roofline_frac": round(frame_bytes / (ms_per_frame * 1e-3) / (PEAK_HBM_GBS * 1e9), 4),
                  "single_frame_latency_ms_median_p10_p90": lat_q,
                  "two_frames_in_flight_ms_per_frame": None if two_ms is None else round(two_ms, 4),
                  "two_frames_in_flight_outputs_equal": None if two_ms is None else same,
                  "launches": pipe.num_launches(), "status": status,
                  "eager_segments_ms": {"voxelize": round(seg[0], 4), "sparse2dense": round(seg[-1], 4),
                                        "sum_raw": round(raw_sum, 4), "empty_segment": round(empty, 5)}},
        "layers": per_layer,
    }
    if args.calibrate_mb > 0:
        src = torch.full((args.calibrate_mb * (1 << 20) // 4,), 1.5, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration"] = {"copy_mib": args.calibrate_mb, "repeats": 3}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(pts, layers, W, args.max_voxels, args.voxel_cap)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
