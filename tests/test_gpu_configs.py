"""The benchmark configurations at their stated workloads, on the GPU against the CPU oracle: configuration 3
(20 000 points, FP32), configuration 4 (60 000 points, voxel cap 40 000, FP16), configuration 5 (150 000 points over
360 degrees, voxel cap 60 000, doubled channel widths, FP16), the reference's own first frame (KITTI 000000), and the
wide FP32 kernels at a full-size row count.  Every frame runs on the benchmark's schedule (overlapped streams, captured
graph) with the benchmark's tensor capacities."""
import json
import os

import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import (RTOL_FP32, abs_sum_of, assert_features_close, check_frame_against_oracle, dev, points_input, to_np)
from sessd3d import api, backbone as B, ctypes_defs as D, frames as F
from test_gpu_pipeline import half_weights

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kitti_000000_counts.json")


@pytest.fixture(autouse=True)
def oracle_threads():
    O.set_threads(min(16, os.cpu_count() or 1))      # the oracle's results do not depend on the thread count
    yield
    O.set_threads(1)


def run_config(pts, layers, W, max_points, layer_cap, voxel_cap, dtype, replays=1):
    pipe = api.Pipeline(layers, W, max_points, layer_cap, feature_dtype=dtype, share_rulebooks=True,
                        skip_pad_rows=True, use_graph=True, overlap_streams=True, voxel_cap=voxel_cap)
    p, n = points_input(pts, max_points)
    dense = pipe.new_dense()
    stream = torch.cuda.Stream()
    first = None
    for _ in range(1 + replays):
        with torch.cuda.stream(stream):
            pipe.enqueue(p, n, dense, stream)
        stream.synchronize()
        if first is None:
            first = to_np(dense).copy()
        else:
            assert np.array_equal(to_np(dense), first), "a graph replay differs from the first run"
    return pipe, dense, (p, n, stream)


def test_config3_fp32_frame_against_oracle_and_fp64():
    pts = F.lidar_frame(20000, 0)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=1, w_std=0.05)
    pipe, dense, _ = run_config(pts, layers, W, 20000, 60000, 60000, "fp32")
    rep = {}
    ref = check_frame_against_oracle(pipe, dense, pts, layers, W, 60000, 60000, False, B.DENSE_SIZE_XYZ, rep)
    print("config 3:", json.dumps(rep))
    assert 15000 < ref["counts"][0] < 19000 and ref["status"] == 0
    # end to end against the oracle's own chain: the two FP32 computations differ by their rounding only, which
    # the FP64 recomputation bounds -- neither is further than 2e-6 of the tensor's scale (RMS) from it
    assert rep["last_layer_rms_error_gpu"] < 2e-6 and rep["last_layer_rms_error_oracle"] < 2e-6


def test_config4_fp16_frame_at_its_stated_workload():
    """60 000 points, voxel cap 40 000 (binds: overflow flag), FP16 features and weights, the reference's widths."""
    pts = F.lidar_frame(60000, 0)
    layers = B.reference_layers()
    W = half_weights(B.random_weights(layers, seed=1, w_std=0.05))
    pipe, dense, _ = run_config(pts, layers, W, 60000, 100000, 40000, "fp16")
    assert dense.dtype == torch.float16
    rep = {}
    ref = check_frame_against_oracle(pipe, dense, pts, layers, W, 40000, 100000, True, B.DENSE_SIZE_XYZ, rep)
    print("config 4:", json.dumps(rep))
    assert ref["counts"][0] == 40000 and ref["status"] & D.SESSD_STATUS_VOXEL_OVERFLOW
    assert max(ref["counts"]) <= 100000


def test_config5_stress_frame_at_its_stated_workload():
    """150 000 points over 360 degrees, voxel cap 60 000, channel widths doubled (8 -> 32 -> 64 -> 128 -> 128), FP16."""
    pts = F.lidar_frame(150000, 5, full_circle=True)
    layers = B.reference_layers(width_mult=2)
    W = half_weights(B.random_weights(layers, seed=4, w_std=0.03))
    pipe, dense, _ = run_config(pts, layers, W, 150000, 200000, 60000, "fp16")
    assert tuple(dense.shape) == (256, 200, 176)
    rep = {}
    ref = check_frame_against_oracle(pipe, dense, pts, layers, W, 60000, 200000, True, B.DENSE_SIZE_XYZ, rep)
    print("config 5:", json.dumps(rep))
    assert ref["counts"][0] == 60000 and ref["status"] & D.SESSD_STATUS_VOXEL_OVERFLOW
    assert ref["counts"][3] > 60000 and max(ref["counts"]) <= 200000      # the first strided layer grows the set


def test_config5_seeded_frames_keep_their_invariants():
    """The 100 seeded stress frames of the configuration through ONE pipeline (same buffers, same captured graph): voxelizer
    output against the oracle exactly, unique in-range sites, dense tensor = exact scatter of the last rows, finite
    values, identical bits on a second pass.  Stops at the first failure."""
    layers = B.reference_layers(width_mult=2)
    W = half_weights(B.random_weights(layers, seed=4, w_std=0.03))
    mp, cap = 150000, 60000
    pipe = api.Pipeline(layers, W, mp, 200000, feature_dtype="fp16", share_rulebooks=True, skip_pad_rows=True,
                        use_graph=True, overlap_streams=True, voxel_cap=cap)
    p, n = points_input(np.zeros((0, 4), np.float32), mp)
    dense, stream = pipe.new_dense(), torch.cuda.Stream()
    seeds = range(100, 200)
    for seed, pts in zip(seeds, F.lidar_frames(150000, seeds, full_circle=True)):
        hp, hn = points_input(pts, mp)
        outs = []
        for _ in range(2):
            with torch.cuda.stream(stream):
                p.copy_(hp)
                n.copy_(hn)
                pipe.enqueue(p, n, dense, stream)
            stream.synchronize()
            outs.append(to_np(dense).copy())
        assert np.array_equal(outs[0], outs[1]), seed
        vfeat, vcoors, vn = pipe.read_layer(-1)
        o = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, cap)
        assert vn == o[2] and np.array_equal(vcoors, o[1][:vn]), seed
        assert np.array_equal(vfeat.view(np.uint32), o[0][:vn].view(np.uint32)), seed
        assert pipe.status() == o[4], seed
        feat, coors, cnt = pipe.read_layer(len(layers) - 1)
        assert cnt > 0 and len(np.unique(coors[:, 1:] @ np.array([200 * 176, 176, 1]))) == cnt, seed
        assert coors.min() >= 0 and coors[:, 1].max() < 2 and coors[:, 2].max() < 200 and coors[:, 3].max() < 176, seed
        back = outs[0].reshape(128, 2, 200, 176)[:, coors[:, 1], coors[:, 2], coors[:, 3]].T
        assert np.array_equal(back.astype(np.float32), feat), seed
        assert np.isfinite(outs[0].astype(np.float32)).all(), seed
        assert np.count_nonzero(outs[0]) == np.count_nonzero(feat), seed


def test_reference_first_frame_kitti_000000(kitti_frame0):
    """The frame the reference's main loop reads first (se-ssd-ai-trt.cpp:1824-1868), with the reference's tensor
    shapes (80 000-row points tensor, 60 000 voxels): 16 825 voxels as the reference's comments say, the stage
    counts of the independent numpy recomputation, every layer against the oracle."""
    with open(GOLDEN) as f:
        golden = json.load(f)
    pts = kitti_frame0
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=2, w_std=0.05)
    pipe, dense, _ = run_config(pts, layers, W, B.MAX_POINTS, B.MAX_VOXELS, B.MAX_VOXELS, "fp32")
    rep = {}
    ref = check_frame_against_oracle(pipe, dense, pts, layers, W, B.MAX_VOXELS, B.MAX_VOXELS, False, B.DENSE_SIZE_XYZ, rep)
    print("KITTI 000000:", json.dumps(rep))
    assert ref["counts"][0] == golden["voxels"] == 16825
    stage_end = [0, 2, 5, 9, 13]                    # voxelizer, then the strided layers 6, 15, 27, 39
    assert [ref["counts"][i + 1] if i else ref["counts"][0] for i in stage_end] == golden["active_sites_after_stage"]
    assert ref["pairs"] == golden["pairs_per_layer"]
    assert [pipe.layer_stats(l)[1] for l in range(len(layers))] == golden["pairs_per_layer"]
    vfeat, vcoors, _ = pipe.read_layer(-1)
    first = np.floor((pts[0, :3] - np.float32([0, -40, -3])) / np.float32([0.05, 0.05, 0.1])).astype(int)[::-1]
    assert list(first) == golden["first_point_cell_zyx"] and list(vcoors[0, 1:]) == golden["first_point_cell_zyx"]


@pytest.mark.parametrize("cin,cout", [(64, 128), (128, 128)])
def test_wide_fp32_layers_against_the_oracle_at_full_row_count(cin, cout):
    """The 64->128 and 128->128 FP32 kernels (the doubled-width backbone in FP32) on the active sites of a
    60 000-point frame's second stage, ~50 000 rows in a 100 000-row tensor, against the oracle."""
    pts = F.lidar_frame(60000, 8)
    _, vco, vn, _, _ = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, 40000)
    mv = 100000
    _, _, coors, n, _ = O.sparse_rulebook(vco, vn, (704, 800, 21), (3, 3, 3), (2, 2, 2), (1, 1, 1), mv)
    assert 40000 < n <= mv
    rng = np.random.default_rng(cin + cout)
    feat = rng.uniform(-1, 1, (mv, cin)).astype(np.float32)
    w = rng.normal(0, 0.05, (27, cin, cout)).astype(np.float32)
    sc = rng.uniform(0.5, 1.5, cout).astype(np.float32)
    sh = rng.uniform(-0.2, 0.2, cout).astype(np.float32)
    conv = api.SubmConv3d(cin, cout, (704, 800, 21), w, mv)
    conv.set_epilogue(sc, sh, True)
    conv.set_flags(D.SESSD_FLAG_SKIP_PAD_ROWS)
    out = conv(dev(feat), dev(coors), dev(np.array([n], np.int32)))
    torch.cuda.synchronize()
    pairs, num, _ = O.subm_rulebook(coors, n, (704, 800, 21), mv)
    want = O.scale_shift_relu(O.gather_gemm_scatter(feat, w, pairs, num, mv), n, sc, sh, True)
    assert int(num.sum()) > 8 * n
    assert_features_close(to_np(out)[:n], want[:n], RTOL_FP32, "FP32 %d->%d at %d rows" % (cin, cout, n),
                          abs_sum=abs_sum_of(feat, w, pairs, num, mv, n, sc, sh)[:n])
    assert conv.status() == 0
