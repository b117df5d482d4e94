"""Per-frame harness: a directory of LiDAR frame files through voxelize -> 3-D backbone -> dense BEV tensor.

    python se-ssd-ai-trt_amd/run_frames.py --data DIR [--frames 301] [--wts model.wts] [--dtype fp32]

Plays the role of the reference's inference loop (se-ssd-ai-trt.cpp:1824-1868) for the 3-D front end: frames
are DIR/000000.bin, 000001.bin, ... (float32 x,y,z,intensity), each is copied to the device and run through
the frame pipeline; one JSON line per frame (points, voxels, active sites after the last layer, ms with and
without the host-to-device copy) and a summary line (median / p10 / p90).  Without --wts the backbone gets
seeded random weights of the reference's shapes.  Needs a GPU.
"""
import argparse
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from sessd3d import api, backbone as B  # noqa: E402


def frame_path(data_dir, i):
    return os.path.join(data_dir, "%06d.bin" % i)  # six digits, zero padded (se-ssd-ai-trt.cpp:1834-1840)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--data", required=True, help="directory holding 000000.bin, 000001.bin, ...")
    ap.add_argument("--frames", type=int, default=301, help="frames 0 .. N-1 (the reference runs 301); missing files end the run")
    ap.add_argument("--wts", default=None, help="weight file in the reference's .wts format")
    ap.add_argument("--dtype", default="fp32", choices=["fp32", "fp16"])
    ap.add_argument("--max-points", type=int, default=B.MAX_POINTS)
    ap.add_argument("--max-voxels", type=int, default=B.MAX_VOXELS)
    ap.add_argument("--pad", action="store_true", help="write the dense tensor with the reference's 1-pixel zero border")
    ap.add_argument("--repeat", type=int, default=1, help="enqueue every frame this many times and report the last")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("run_frames.py needs a GPU")
    dev = torch.device("cuda:0")
    layers = B.reference_layers()
    weights = api.WeightFile(path=args.wts) if args.wts else B.random_weights(layers, seed=args.seed, w_std=0.05)
    pipe = api.Pipeline(layers, weights, args.max_points, args.max_voxels, feature_dtype=args.dtype,
                        share_rulebooks=True, skip_pad_rows=True, use_graph=True, overlap_streams=True,
                        dense_padding=(1, 1, 1, 1) if args.pad else (0, 0, 0, 0))
    host = torch.zeros((args.max_points, 4), dtype=torch.float32).pin_memory()
    host_n = torch.zeros((1,), dtype=torch.int32).pin_memory()
    points = torch.zeros((args.max_points, 4), dtype=torch.float32, device=dev)
    points_size = torch.zeros((1,), dtype=torch.int32, device=dev)
    dense = pipe.new_dense()
    stream = torch.cuda.Stream()
    e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    ms_gpu, ms_all, done = [], [], 0
    for i in range(args.frames):
        path = frame_path(args.data, i)
        if not os.path.exists(path):
            break
        _, n = api.load_frame(path, args.max_points, 4, out=host.numpy())
        host_n[0] = n
        with torch.cuda.stream(stream):
            for _ in range(max(args.repeat, 1)):
                e0.record(stream)
                # only the rows that hold points travel (the reference copies all MAX_POINTS rows, :1862)
                points[:n].copy_(host[:n], non_blocking=True)
                points_size.copy_(host_n, non_blocking=True)
                e1.record(stream)
                pipe.enqueue(points, points_size, dense, stream)
                e2.record(stream)
        stream.synchronize()
        n_vox, n_last = pipe.layer_count(-1), pipe.layer_count(len(layers) - 1)
        rec = {"frame": os.path.basename(path), "points": n, "voxels": int(n_vox), "sites_out": int(n_last),
               "status": pipe.status(), "ms_pipeline": round(e1.elapsed_time(e2), 4),
               "ms_with_h2d": round(e0.elapsed_time(e2), 4)}
        print(json.dumps(rec), flush=True)
        ms_gpu.append(rec["ms_pipeline"])
        ms_all.append(rec["ms_with_h2d"])
        done += 1
    if not done:
        raise SystemExit("no frame files found under %s" % args.data)
    q = lambda v: [round(float(x), 4) for x in np.percentile(v, [50, 10, 90])]  # noqa: E731
    print(json.dumps({"frames": done, "dtype": args.dtype, "weights": args.wts or "seeded random",
                      "ms_pipeline_median_p10_p90": q(ms_gpu), "ms_with_h2d_median_p10_p90": q(ms_all)}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
