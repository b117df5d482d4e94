"""GPU tests of the pieces either side of the hot path: a pipeline built from a `.wts` weight file and the
per-frame harness over a directory of frame files (synthetic frames written in the KITTI `.bin` layout; the
reference's own frames do not travel to the GPU machine)."""
import importlib.util
import json
import os

import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import points_input, to_np
from sessd3d import api, backbone as B, frames as F

pytestmark = pytest.mark.gpu


def run(pipe, pts, max_points):
    p, n = points_input(pts, max_points)
    dense = pipe.new_dense()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        pipe.enqueue(p, n, dense, stream)
    stream.synchronize()
    return dense


def test_pipeline_from_wts_equals_pipeline_from_arrays(tmp_path):
    layers = B.reference_layers()
    sd = B.random_state_dict(layers, seed=8, w_std=0.05)
    path = tmp_path / "sessd.wts"
    B.write_wts(path, sd)
    wf = api.WeightFile(path=str(path))
    pts = F.lidar_frame(3000, 4)
    kw = dict(share_rulebooks=True, skip_pad_rows=True)
    from_file = api.Pipeline(layers, wf, 4096, 12000, **kw)
    # the same numbers taken from the dict and folded on the Python side (FP32, as the reference folds)
    W = B.weights_from_blobs(layers, lambda k: sd[k])
    from_arrays = api.Pipeline(layers, W, 4096, 12000, **kw)
    a, b = run(from_file, pts, 4096), run(from_arrays, pts, 4096)
    assert float(a.abs().max()) > 0
    assert np.array_equal(to_np(a), to_np(b))
    # and the oracle agrees on what that file means
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=12000), layers, W, B.dense_desc())
    assert from_file.layer_count(-1) == ref["counts"][0] and from_file.layer_count(13) == ref["counts"][-1]
    # a file without the BatchNorm blobs of a layer is refused
    del sd["backbone.middle_conv.40.running_var"]
    B.write_wts(path, sd)
    with pytest.raises(api.SessdError, match="middle_conv.40.running_var"):
        api.Pipeline(layers, api.WeightFile(path=str(path)), 4096, 12000, **kw)


def test_frame_harness_over_a_directory(tmp_path, capsys):
    spec = importlib.util.spec_from_file_location(
        "run_frames", os.path.join(os.path.dirname(__file__), "..", "se-ssd-ai-trt_amd", "run_frames.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sizes = [2500, 1, 4000]
    frames = [F.lidar_frame(n, 30 + i) for i, n in enumerate(sizes)]
    for i, pts in enumerate(frames):
        np.ascontiguousarray(pts, np.float32).tofile(tmp_path / ("%06d.bin" % i))
    assert mod.main(["--data", str(tmp_path), "--frames", "10", "--max-points", "4096", "--max-voxels", "16384",
                     "--pad"]) == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.strip().split("\n")]
    assert len(lines) == 4 and lines[-1]["frames"] == 3
    for rec, pts in zip(lines, frames):
        _, _, n, _, _ = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, 16384)
        assert rec["points"] == len(pts) and rec["voxels"] == n and rec["status"] == 0
        assert rec["ms_with_h2d"] >= rec["ms_pipeline"] > 0


def test_c_host_program_matches_the_python_binding(tmp_path):
    """examples/run_frame.c -- a C99 program on the C-ABI and the HIP runtime API alone: frame file in, weight
    file in, dense tensor out -- against the ctypes binding on the same two files: same voxel count, same status,
    the same dense tensor bit for bit."""
    import subprocess
    exe = os.path.join(os.path.dirname(__file__), "..", "se-ssd-ai-trt_amd", "lib", "run_frame")
    if not os.path.exists(exe):
        pytest.skip("se-ssd-ai-trt_amd/lib/run_frame is not built (python se-ssd-ai-trt_amd/build.py)")
    layers = B.reference_layers()
    wts = tmp_path / "sessd.wts"
    B.write_wts(wts, B.random_state_dict(layers, seed=15, w_std=0.05))
    pts = F.lidar_frame(9000, 6)
    frame = tmp_path / "000000.bin"
    np.ascontiguousarray(pts, np.float32).tofile(frame)
    out = tmp_path / "dense.bin"
    r = subprocess.run([exe, str(frame), str(wts), str(out), "3"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    words = r.stdout.split()
    rec = dict(zip(words[::2], words[1::2]))
    pipe = api.Pipeline(layers, api.WeightFile(path=str(wts)), 80000, B.MAX_VOXELS, share_rulebooks=True,
                        skip_pad_rows=True, use_graph=True, overlap_streams=True)
    dense = run(pipe, pts, 80000)
    assert int(rec["points"]) == len(pts) and int(rec["voxels"]) == pipe.layer_count(-1)
    assert int(rec["status"]) == pipe.status() == 0 and float(rec["ms_per_frame"]) > 0
    got = np.fromfile(out, np.float32).reshape(tuple(dense.shape))
    assert got.any() and np.array_equal(got, to_np(dense))
