#!/usr/bin/env python3
"""Benchmark of the 3-D front end on one MI355X: voxelGenerator -> SpMiddleFHD conv stack -> sparse2Dense.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3|4|5] [--seed 0]

A "step" is one frame: one pass of the whole path over one seeded synthetic LiDAR frame that is already
resident in device memory.  The timed region is exactly K pipeline enqueues bracketed by device
synchronisation.  One JSON line is printed:

  value / ms_per_step  ms per frame of the headline configuration (3: 20 000 points, FP32), one frame at a time,
                       back-to-back graph launches (the throughput with several frames in flight is reported beside it)
  roofline             the dominant kernel (the 64->64 channel gather-GEMM), timed live with HIP events on the
                       pipeline's stream, against the FP32 matrix peak
  parity               the timed configuration's tensors against the CPU oracle on the same frame (sites and their
                       numbering bit-exact, features per layer within 1e-4, end to end bounded by an FP64
                       recomputation); a mismatch makes the run exit non-zero
  other_configs        configurations 4 (60 000 points, voxel cap 40 000, FP16) and 5 (150 000 points over 360
                       degrees, voxel cap 60 000, doubled widths, FP16; p10/p50/p90 over seeded frames) and the
                       reference's first KITTI frame: ms/frame, dominant-kernel roofline, parity
  cpu_baseline         the CPU port (the parity oracle) on the same frame, on the host's cores
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "se-ssd-ai-trt_amd"))

PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
PEAK_FP32_TFLOPS = 157.3    # MI355X dense FP32 (vector and matrix)
PEAK_FP16_TFLOPS = 2500.0   # MI355X dense FP16 MFMA

PRESETS = {3: dict(points=20000, dtype="fp32", max_voxels=60000, voxel_cap=60000, width=1, full=False),
           4: dict(points=60000, dtype="fp16", max_voxels=100000, voxel_cap=40000, width=1, full=False),
           5: dict(points=150000, dtype="fp16", max_voxels=200000, voxel_cap=60000, width=2, full=True)}
KITTI_FRAME0 = os.path.join(ROOT, "tests", "golden", "kitti_000000.bin")


def layer_work(layer, n_in, n_out, pairs, esize):
    """Algorithmic work of one conv layer's gather-GEMM launch: flops = 2*P*Cin*Cout; bytes = gathered
    input rows + output rows written once + rulebook entries read + weights read once."""
    flops = 2.0 * pairs * layer.cin * layer.cout
    bytes_ = pairs * layer.cin * esize + n_out * layer.cout * esize + 8.0 * pairs + layer.kvol * layer.cin * layer.cout * esize
    return flops, bytes_


def kernel_source_hash():
    """Short hash of the gather-GEMM kernels' sources: the committed counter summaries carry the hash of the sources
    they were collected on, so a figure taken from them can be told from a stale one."""
    h = hashlib.sha256()
    for name in ("conv_mfma.hip", "conv_tall.hip", "conv_wide.hip"):
        with open(os.path.join(ROOT, "se-ssd-ai-trt_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def profiled_traffic(kernel, config, dtype):
    """HBM bytes per launch of the kernel whose name starts with `kernel`, from the committed rocprofv3 summary (FETCH_SIZE and WRITE_SIZE
    runs, scaled by a copy kernel of known size) -> (bytes or None, whether the summary was collected on the
    current kernel source)."""
    path = os.path.join(ROOT, "profiles", "frame_pipeline_config%d_%s.md" % (config, dtype))
    value, fresh = None, False
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("kernel source hash"):
                    fresh = kernel_source_hash() in line
                cells = [c.strip() for c in line.split("|")]
                if len(cells) >= 8 and cells[1].startswith(kernel) and cells[2].isdigit() and value is None:
                    value = float(round((float(cells[5]) + float(cells[6])) * 1e6))
    except (OSError, ValueError):
        pass
    return value, fresh


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


def host_threads():
    # a one-GPU machine of this pool gives a job 16 cores, whatever os.cpu_count() reports
    return max(1, min(16, os.cpu_count() or 1))


def cpu_baseline(pts, layers, W, voxel_cap, budget_s=20.0):
    """The CPU port (the parity oracle) on the same frame, a bounded number of frames: once on one thread and
    once with the pairs of every kernel offset split over the host's cores (same bits either way)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    from sessd3d import backbone as B
    vg = B.voxelgen_desc(max_voxels=voxel_cap)   # (oracle_frame has one capacity; it equals the layers' in config 3)
    dd = B.dense_desc(channel=layers[-1].cout)

    def median_ms(max_frames, budget):
        times, t_start = [], time.perf_counter()
        while len(times) < max_frames and (not times or (time.perf_counter() - t_start) < budget):
            t0 = time.perf_counter()
            O.frame(pts, vg, layers, W, dd)
            times.append((time.perf_counter() - t0) * 1e3)
        times.sort()
        return times[len(times) // 2], len(times)

    O.set_threads(1)
    O.frame(pts, vg, layers, W, dd)          # warm-up (allocates the dense index grids)
    one, n_one = median_ms(3, budget_s / 2)
    threads = host_threads()
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


def parity_gate(pipe, dense, pts, layers, W, voxel_cap, layer_cap, half):
    """The tensors of the frame the pipeline last ran against the CPU oracle (tests/gpu_util.py: every layer with the
    oracle fed the GPU's rows, the oracle's own chain, and an FP64 recomputation).  -> dict with ok = True/False."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    import gpu_util as G
    from sessd3d import backbone as B
    O.set_threads(host_threads())
    rep = {}
    try:
        G.check_frame_against_oracle(pipe, dense, pts, layers, W, voxel_cap, layer_cap, half, B.DENSE_SIZE_XYZ, rep)
        ok, why = True, None
    except AssertionError as e:
        ok, why = False, str(e)[:400] or "assertion failed"
    finally:
        O.set_threads(1)
    out = {"ok": ok, "checked": "voxel means, coordinates, counts, per-layer output sites + numbering and status words bit-exact; "
                                "features per layer <= %g relative to max(|value|, %g x the tensor's largest), elements whose terms "
                                "cancel admitted within %g x their sum of |terms| + 2 ulp (oracle fed the GPU's rows); GPU's RMS "
                                "distance from an FP64 recomputation <= 2x the oracle's, per layer"
                                % (G.RTOL_FP16 if half else G.RTOL_FP32, G.FLOOR_FRACTION, G.SUM_TOL)}
    if why:
        out["failure"] = why
    # worst over the layers: relative error among the elements above the floor, share of elements judged at the
    # floor, share admitted by the sum-of-terms bound only, largest |gpu - oracle| / sum of |terms|
    for k in ("worst_rel_error_above_floor", "share_judged_at_floor", "share_admitted_by_sum_bound", "worst_error_over_abs_sum",
              "gpu_over_oracle_rms_error", "last_layer_rms_error_gpu", "last_layer_rms_error_oracle",
              "last_layer_max_diff_gpu_vs_oracle"):
        if k in rep:
            out[k] = rep[k] if isinstance(rep[k], list) else float("%.3g" % rep[k])
    return out


def measure(config, args, torch, frames=None, points_override=None, deep=True, want_parity=True):
    """Build the pipeline of one configuration, time it, and (deep) take per-layer statistics, eager per-kernel
    durations and the dominant kernel's roofline position.  frames: list of point arrays timed one after the other
    in the same buffers (default: the one seeded frame of the preset)."""
    import numpy as np
    from sessd3d import api, backbone as B, frames as F
    preset = dict(PRESETS[config])
    dtype = args.dtype or preset["dtype"]
    max_voxels = args.max_voxels or preset["max_voxels"]
    voxel_cap = args.voxel_cap or preset["voxel_cap"]
    layers = B.reference_layers(width_mult=preset["width"])
    W = B.random_weights(layers, seed=1, w_std=0.05 if dtype == "fp16" else 0.1)
    half = dtype == "fp16"
    if half:       # FP16 configurations store weights in half: the library and the oracle get the rounded values
        W = B.Weights([w.astype(np.float16).astype(np.float32) for w in W.w], W.scale, W.shift)
    if frames is None:
        frames = [F.lidar_frame(points_override or preset["points"], args.seed, full_circle=preset["full"])]
    max_points = max(len(f) for f in frames)
    dev = "cuda:0"
    kw = dict(feature_dtype=dtype, share_rulebooks=not args.no_share, skip_pad_rows=not args.pad_rows,
              use_graph=not args.no_graph, overlap_streams=not args.no_overlap, voxel_cap=voxel_cap,
              dense_size_xyz=B.DENSE_SIZE_XYZ)
    pipe = api.Pipeline(layers, W, max_points, max_voxels, **kw)
    points = torch.zeros((max_points, 4), dtype=torch.float32, device=dev)
    size = torch.zeros((1,), dtype=torch.int32, device=dev)
    dense = pipe.new_dense(dev)
    stream = torch.cuda.Stream()

    def upload(pts):
        buf = np.zeros((max_points, 4), np.float32)
        buf[:len(pts)] = pts
        points.copy_(torch.as_tensor(buf))
        size.copy_(torch.tensor([len(pts)], dtype=torch.int32))
        torch.cuda.synchronize()

    def timed(steps, warmup):
        with torch.cuda.stream(stream):
            for _ in range(warmup):
                pipe.enqueue(points, size, dense, stream)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        with torch.cuda.stream(stream):
            for _ in range(steps):
                pipe.enqueue(points, size, dense, stream)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    per_frame_ms, status = [], 0
    for i, pts in enumerate(frames):
        upload(pts)
        per_frame_ms.append(timed(args.steps, args.warmup if i == 0 else 2))
        status |= pipe.status(stream)
    pts = frames[0]
    if len(frames) > 1:
        upload(pts)
        with torch.cuda.stream(stream):
            pipe.enqueue(points, size, dense, stream)
        torch.cuda.synchronize()
    ms_per_frame = float(np.median(per_frame_ms))

    # throughput with frames in flight: the library's replicas (frames_in_flight = R), frame t + 1 submitted before
    # frame t is joined.  Every frame does all of its work into a dense tensor of its own; the tensors must equal the
    # one-frame-at-a-time result bit for bit.
    fif_ms, fif_equal = None, None
    R = args.frames_in_flight
    if R >= 2 and not args.no_overlap:
        many = api.Pipeline(layers, W, max_points, max_voxels, frames_in_flight=R, **kw)
        outs = [many.new_dense(dev) for _ in range(R)]
        feeder = torch.cuda.Stream()     # the stream the frames are submitted from and joined on

        def run_many(steps):
            tickets = []
            for i in range(steps):
                tickets.append(many.submit(points, size, outs[i % R], feeder))
                if i >= R - 1:
                    many.join(tickets[i - (R - 1)], feeder)
            for t in tickets[-(R - 1):]:
                many.join(t, feeder)

        run_many(max(args.warmup, 2 * R))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_many(args.steps)
        torch.cuda.synchronize()
        fif_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        fif_equal = all(bool(torch.equal(o, dense)) for o in outs) and many.status(feeder) == status
        many.close()
        del outs
    res = {"config": config, "dtype": dtype, "points": len(pts), "max_voxels": max_voxels, "voxel_cap": voxel_cap,
           "ms_per_frame": round(ms_per_frame, 4), "status": status, "launches": pipe.num_launches(),
           "frames_in_flight": {"replicas": R, "ms_per_frame": None if fif_ms is None else round(fif_ms, 4),
                                "outputs_equal_one_at_a_time": fif_equal}}
    if len(frames) > 1:
        q = np.percentile(per_frame_ms, [10, 50, 90])
        res["ms_per_frame_p10_p50_p90"] = [round(float(v), 4) for v in q]
        res["seeded_frames"] = len(frames)
    res["parity"] = parity_gate(pipe, dense, pts, layers, W, voxel_cap, max_voxels, half) if want_parity else None

    # per-layer active sites / rulebook pairs (small counting kernels, outside the timed region)
    n_vox, _ = pipe.layer_stats(-1, stream)
    stats, n_in = [], n_vox
    for l, layer in enumerate(layers):
        n_out, pairs = pipe.layer_stats(l, stream)
        stats.append((n_in, n_out, pairs))
        n_in = n_out
    res["voxels"] = n_vox

    # per-kernel durations: HIP events recorded on the pipeline's stream right before and after every launch
    # (eager launches, one stream).  An event pair that brackets nothing reads a few microseconds on this stream
    # (`empty_segment`); rocprofv3's kernel trace reads the same few microseconds more than the events minus that
    # empty time, so the durations used for the roofline are the raw event figures, which agree with the trace.
    seg, empty = None, 0.0
    n_prof = max(1, args.profile_steps) if deep else max(5, args.profile_steps // 5)
    with torch.cuda.stream(stream):
        for _ in range(5):
            pipe.enqueue_timed(points, size, dense, stream)
        for _ in range(n_prof):
            s, e = pipe.enqueue_timed(points, size, dense, stream)
            s = np.asarray(s, np.float64)
            seg = s if seg is None else seg + s
            empty += e
    seg /= n_prof
    empty /= n_prof
    esize = 2 if half else 4
    per_layer = []
    tot_flops = tot_bytes = 0.0
    for l, layer in enumerate(layers):
        n_i, n_o, p = stats[l]
        fl, by = layer_work(layer, n_i, n_o, p, esize)
        tot_flops += fl
        tot_bytes += by
        g = seg[2 + 2 * l]
        per_layer.append({"name": layer.name, "n_in": n_i, "n_out": n_o, "pairs": p,
                          "build_us": round(seg[1 + 2 * l] * 1e3, 2), "gemm_us": round(g * 1e3, 2),
                          "gemm_tflops": round(fl / (g * 1e-3) / 1e12, 3) if g > 0 else None,
                          "gemm_gbs": round(by / (g * 1e-3) / 1e9, 1) if g > 0 else None})
    # dominant kernel: the gather-GEMM instantiation of the widest square layers (64 -> 64, or 128 -> 128)
    dom_c = 64 * preset["width"]
    dom = [l for l, layer in enumerate(layers) if layer.cin == dom_c and layer.cout == dom_c]
    dom_flops = sum(layer_work(layers[l], *stats[l], esize)[0] for l in dom) / len(dom)
    dom_bytes = sum(layer_work(layers[l], *stats[l], esize)[1] for l in dom) / len(dom)
    dom_ms = sum(seg[2 + 2 * l] for l in dom) / len(dom)
    peak_tf = PEAK_FP16_TFLOPS if half else PEAK_FP32_TFLOPS
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
    # (FP16 3x3x3 layers from 32 channels up run on the tall-tile kernel, FP32 64 -> 64 on the one-tile-per-unit
    # kernel, everything else on the split-K one)
    kname = ("conv_tall<%d, %d," if half else "conv_wide<%d, %d," if dom_c == 64 else "conv_mfma<float, %d, %d,") % (dom_c, dom_c)
    traffic, fresh = profiled_traffic(kname, config, dtype)
    roof["traffic"] = traffic
    roof.update({"traffic_source": "profiles/frame_pipeline_config%d_%s.md (rocprofv3 FETCH_SIZE/WRITE_SIZE), collected on %s"
                                   % (config, dtype, "this kernel source" if fresh else "an OLDER kernel source: stale"),
                 "kernel": "gather-GEMM %d->%d (%s)" % (dom_c, dom_c, dtype), "launches_per_frame": len(dom),
                 "avg_launch_us": round(dom_ms * 1e3, 2),
                 "avg_launch_us_less_empty_event_pair": round(max(dom_ms - empty, 0.0) * 1e3, 2),
                 "algorithmic_flops_per_launch": dom_flops, "algorithmic_bytes_per_launch": dom_bytes,
                 "other_bound_frac": round((dom_bytes / (dom_ms * 1e-3) / 1e9) / PEAK_HBM_GBS, 4) if roof["bound"] == "mfma"
                 else round((dom_flops / (dom_ms * 1e-3) / 1e12) / peak_tf, 4)})
    res["roofline"] = roof
    c_last, dsz = layers[-1].cout, B.DENSE_SIZE_XYZ
    frame_bytes = 16.0 * len(pts) + 32.0 * n_vox + tot_bytes + stats[-1][1] * (c_last * esize + 16) + \
        c_last * dsz[0] * dsz[1] * dsz[2] * esize
    res["frame"] = {"frames_per_s": round(1e3 / ms_per_frame, 1), "algorithmic_gflop": round(tot_flops / 1e9, 3),
                    "algorithmic_mb": round(frame_bytes / 1e6, 2),
                    "hbm_roofline_frac": round(frame_bytes / (ms_per_frame * 1e-3) / (PEAK_HBM_GBS * 1e9), 4),
                    "gemm_launches_sum_us": round(float(sum(seg[2 + 2 * l] for l in range(len(layers)))) * 1e3, 1),
                    "build_launches_sum_us": round(float(sum(seg[1 + 2 * l] for l in range(len(layers)))) * 1e3, 1),
                    "eager_segments_ms": {"voxelize": round(seg[0], 4), "sparse2dense": round(seg[-1], 4),
                                          "sum_raw": round(float(seg.sum()), 4), "empty_segment": round(empty, 5)}}
    if deep:
        # latency of single frames (one frame in flight, a synchronise between frames), outside the timed region
        lat = []
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        for _ in range(min(max(args.steps, 20), 100)):
            with torch.cuda.stream(stream):
                ev[0].record(stream)
                pipe.enqueue(points, size, dense, stream)
                ev[1].record(stream)
            stream.synchronize()
            lat.append(ev[0].elapsed_time(ev[1]))
        res["frame"]["single_frame_latency_ms_median_p10_p90"] = [round(float(v), 4) for v in np.percentile(lat, [50, 10, 90])]
        res["layers"] = per_layer
    else:
        res["layers"] = [{k: d[k] for k in ("name", "n_out", "pairs", "gemm_us")} for d in per_layer]
    res["_objects"] = (pts, layers, W, voxel_cap)
    pipe.close()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=[3, 4, 5],
                    help="configuration of the headline figure: 3 = 20k points FP32 (default, BASELINE's metric), 4 = 60k points, "
                         "voxel cap 40k, FP16, 5 = 150k points over 360 degrees, voxel cap 60k, doubled channel widths, FP16")
    ap.add_argument("--points", type=int, default=None)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--frame-file", default=None,
                    help="time this frame file (float32 x,y,z,intensity records, KITTI velodyne layout) instead of the "
                         "configuration's synthetic frame, e.g. tests/golden/kitti_000000.bin")
    ap.add_argument("--dtype", default=None, choices=["fp32", "fp16"])
    ap.add_argument("--max-voxels", type=int, default=None, help="rows of the conv layers' tensors")
    ap.add_argument("--voxel-cap", type=int, default=None, help="the voxelizer's max_voxels")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels directly instead of replaying a hipGraph")
    ap.add_argument("--no-share", action="store_true", help="every SubM layer rebuilds its rulebook (as the reference does)")
    ap.add_argument("--pad-rows", action="store_true", help="write rows >= voxel_num of every tensor (reference behaviour)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="single stream: do not run the rulebook builds concurrently with the GEMMs of earlier layers")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-parity", action="store_true", help="skip the comparison with the CPU oracle")
    ap.add_argument("--no-others", action="store_true", help="only the headline configuration")
    ap.add_argument("--frames-in-flight", type=int, default=2,
                    help="replicas of the pipeline for the throughput figure with frames in flight (sessd_pipeline_submit / "
                         "join); a replica runs on two streams and HIP has 4 hardware queues by default: 2 and 4 replicas "
                         "measured best, 3 worse than one frame at a time; 0 = skip")
    ap.add_argument("--config5-frames", type=int, default=100,
                    help="seeded frames of configuration 5 in other_configs (its stated repetition is 100; a pool of "
                         "threads generates them, ~0.1 s a frame)")
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
    from sessd3d import frames as F

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    want_parity = not args.no_parity
    own_frames = None
    if args.frame_file:
        own_frames = [np.fromfile(args.frame_file, np.float32).reshape(-1, 4)]
    head = measure(args.config, args, torch, frames=own_frames, points_override=args.points, deep=True, want_parity=want_parity)
    pts, layers, W, voxel_cap = head.pop("_objects")
    preset = PRESETS[args.config]
    fif = head["frames_in_flight"]
    # The headline is always one frame at a time (back-to-back graph launches on one stream): the figure with
    # frames in flight depends on how the replicas' streams fall onto the hardware queues and is reported beside
    # it (frame.frames_in_flight), never as `value`.
    value = head["ms_per_frame"]
    mode = "one frame at a time, back-to-back graph launches"
    out = {
        "metric": "ms/frame voxelize+3D sparse backbone @~17k voxels",
        "value": value, "unit": "ms/frame", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": value, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if head["dtype"] == "fp16" else "f32", "data": "synthetic",
        "config": {"workload": ("frame file %s through " % args.frame_file if args.frame_file else "") +
                               "config %d: %d-point seeded synthetic LiDAR frame (seed %d), %d voxels, reference 14-layer "
                               "SpMiddleFHD backbone (10 SubM + 4 SparseConv, channel widths x%d, BN folded + ReLU), "
                               "sparse2Dense to %dx200x176; value = %s (with frames in flight: "
                               "frame.frames_in_flight; single-frame latency: frame.single_frame_latency_ms_median_p10_p90)"
                               % (args.config, len(pts), args.seed, head["voxels"], preset["width"], layers[-1].cout * 2, mode),
                   "frames_in_flight": 1,
                   "data_file": args.frame_file,
                   "max_voxels": head["max_voxels"], "voxel_cap": head["voxel_cap"], "graph": not args.no_graph,
                   "overlap_streams": not args.no_overlap, "share_rulebooks": not args.no_share,
                   "pad_rows": args.pad_rows, "n_layers": len(layers)},
        "roofline": head["roofline"],
        "parity": head["parity"],
        "frame": dict(head["frame"], launches=head["launches"], status=head["status"],
                      one_frame_at_a_time_ms=head["ms_per_frame"], frames_in_flight=fif,
                      frames_per_s=round(1e3 / value, 1),
                      hbm_roofline_frac=round(head["frame"]["algorithmic_mb"] * 1e6 / (value * 1e-3) / (PEAK_HBM_GBS * 1e9), 4)),
        "layers": head["layers"],
    }
    ok = head["status"] == 0 if args.config == 3 else True   # (the voxel cap binds by design in configurations 4 and 5)
    ok = ok and (head["parity"] is None or head["parity"]["ok"])
    ok = ok and fif["outputs_equal_one_at_a_time"] is not False
    if not args.no_others:
        others = []
        for cfg in (3, 4, 5):
            if cfg == args.config:
                continue
            frames = None
            if cfg == 5:
                frames = list(F.lidar_frames(PRESETS[5]["points"], range(100, 100 + max(1, args.config5_frames)), full_circle=True))
            sub = argparse.Namespace(**vars(args))
            sub.dtype = sub.max_voxels = sub.voxel_cap = None
            sub.steps, sub.warmup = max(20, min(args.steps, 50)), 5
            r = measure(cfg, sub, torch, frames=frames, deep=False, want_parity=want_parity)
            r.pop("_objects")
            ok = ok and (r["parity"] is None or r["parity"]["ok"]) and r["frames_in_flight"]["outputs_equal_one_at_a_time"] is not False
            others.append(r)
        if os.path.exists(KITTI_FRAME0):
            kitti = np.fromfile(KITTI_FRAME0, np.float32).reshape(-1, 4)
            sub = argparse.Namespace(**vars(args))
            sub.dtype = sub.max_voxels = sub.voxel_cap = None
            sub.steps, sub.warmup = max(20, min(args.steps, 50)), 5
            r = measure(3, sub, torch, frames=[kitti], deep=False, want_parity=want_parity)
            r.pop("_objects")
            r["config"] = "the reference's first frame (KITTI 000000, 20 285 points) through configuration 3's pipeline"
            ok = ok and (r["parity"] is None or r["parity"]["ok"]) and r["status"] == 0
            others.append(r)
        out["other_configs"] = others
    if args.calibrate_mb > 0:
        src = torch.full((args.calibrate_mb * (1 << 20) // 4,), 1.5, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration"] = {"copy_mib": args.calibrate_mb, "repeats": 3}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(pts, layers, W, voxel_cap)
    print(json.dumps(out))
    if not ok:
        print("bench.py: parity or status check failed (see \"parity\" / \"status\" in the line above)", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
