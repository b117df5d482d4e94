"""Pins the oracle's voxelizer (oracle_np_round, oracle_grid_size, oracle_voxelize) without running
any reference code: known answers recorded in the reference's own comments, an independent
numpy-float32 recomputation, brute-force grouping and FP32 boundary cases."""
import collections
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from sessd3d import backbone as B, frames as F

RANGE = B.POINT_CLOUD_RANGE
VSIZE = B.VOXEL_SIZE
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kitti_000000_counts.json")


def numpy_cells(points):
    """Independent float32 restatement of voxelGenerator.cu:363-378: mask + (z,y,x) cell per point."""
    p = points.astype(np.float32)
    lo = np.array(RANGE[:3], np.float32)
    hi = np.array(RANGE[3:], np.float32)
    vs = np.array(VSIZE, np.float32)
    inr = np.all((p[:, :3] >= lo) & (p[:, :3] < hi), axis=1)
    idx = np.floor((p[:, :3] - lo) / vs).astype(np.int64)   # float32 / float32 -> IEEE float32 division
    grid = np.array([1408, 1600, 40])
    ok = inr & np.all((idx >= 0) & (idx < grid), axis=1)
    return ok, idx[:, ::-1]  # z,y,x


def brute_force_voxelize(points, max_pts, max_voxels):
    ok, cells = numpy_cells(points)
    groups = collections.OrderedDict()
    for i in np.flatnonzero(ok):
        key = tuple(cells[i])
        if key not in groups:
            if len(groups) >= max_voxels:
                continue
            groups[key] = []
        groups[key].append(i)
    # cells first seen after the cap are dropped together with all their points
    coors = np.array([(0,) + k for k in groups], np.int32).reshape(-1, 4)
    feats = np.zeros((len(groups), 4), np.float32)
    for v, idxs in enumerate(groups.values()):
        kept = idxs[:max_pts]
        for c in range(4):
            s = np.float32(0)
            vals = [points[i, c] for i in kept] + [np.float32(0)] * (max_pts - len(kept))
            s = vals[0]
            for t in vals[1:]:
                s = np.float32(s + t)
            feats[v, c] = np.float32(s / np.float32(len(kept)))
    return feats, coors


def test_np_round_half_even():
    for x, want in [(0.5, 0), (1.5, 2), (2.5, 2), (2.4, 2), (2.6, 3), (3.5, 4), (1408.0, 1408)]:
        assert O.np_round(x) == want


def test_grid_size_closed_form():
    # voxelGenerator.cu:232-234 with params.h:27-35 -> 1408 x 1600 x 40
    assert O.grid_size(RANGE, VSIZE) == (1408, 1600, 40)


def test_kitti_known_answers(kitti_frame0):
    """submConv3dlayer.cu:254,618,739 record 16825 voxels for frame 000000 and :336,399,620 record the
    cell (38,800,366) for its first point."""
    pts = kitti_frame0
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    assert n == 16825 and st == 0
    assert tuple(coors[0]) == (0, 38, 800, 366)
    with open(GOLDEN) as f:
        gold = json.load(f)
    assert n == gold["voxels"]
    assert int(npts[:n].max()) == gold["max_points_in_voxel"]


def test_matches_numpy_float32(kitti_frame0):
    pts = kitti_frame0
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    ok, cells = numpy_cells(pts)
    _, first = np.unique(cells[ok] @ np.array([1600 * 1408, 1408, 1]), return_index=True)
    want = cells[ok][np.sort(first)]            # unique cells in first-appearance order
    assert n == len(want)
    assert np.array_equal(coors[:n, 1:], want)
    assert np.all(coors[:n, 0] == 0) and np.all(coors[n:] == 0) and np.all(vox[n:] == 0)


@pytest.mark.parametrize("seed", [0, 1])
def test_matches_brute_force_synthetic(seed):
    pts = F.lidar_frame(6000, seed)
    # crowd some voxels beyond 5 points and break the scan order
    rng = np.random.default_rng(seed)
    extra = pts[rng.integers(0, len(pts), 1500)] + rng.normal(0, 0.004, (1500, 4)).astype(np.float32)
    pts = np.concatenate([pts, extra.astype(np.float32)])[rng.permutation(7500)]
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    f2, c2 = brute_force_voxelize(pts, 5, 60000)
    assert n == len(c2) and np.array_equal(coors[:n], c2)
    assert np.array_equal(vox[:n].view(np.uint32), f2.view(np.uint32))   # bit-exact means
    assert npts[:n].max() == 5


def test_single_point_voxels_are_the_point():
    pts = F.lidar_frame(3000, 3)
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    ok, cells = numpy_cells(pts)
    single = np.flatnonzero(npts[:n] == 1)
    lin = cells @ np.array([1600 * 1408, 1408, 1])
    first_of = {int(l): i for i, l in reversed(list(enumerate(lin))) if ok[i]}
    for v in single[:200]:
        i = first_of[int(coors[v, 1:] @ np.array([1600 * 1408, 1408, 1]))]
        assert np.array_equal(vox[v].view(np.uint32), pts[i].view(np.uint32))


def test_cap_drops_new_cells_and_flags():
    pts = F.lidar_frame(5000, 5)
    full = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    cap = 1000
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, cap)
    assert n == cap and st & 1
    assert np.array_equal(coors[:cap], full[1][:cap])
    assert np.array_equal(vox[:cap].view(np.uint32), full[0][:cap].view(np.uint32))
    f2, c2 = brute_force_voxelize(pts, 5, cap)
    assert np.array_equal(coors[:cap], c2)


def test_fp32_boundaries():
    """Range test is [min,max); a point that passes it can still floor onto the grid size and is then
    dropped by the index check (voxelGenerator.cu:375)."""
    f = np.float32
    below = lambda v: np.nextafter(f(v), f(-np.inf))   # noqa: E731
    pts = np.array([
        [0.0, -40.0, -3.0, 0.1],               # all minima: kept -> (0,0,0)
        [70.4, 0.0, 0.0, 0.2],                 # x == xmax: rejected
        [10.0, 40.0, 0.0, 0.3],                # y == ymax: rejected
        [10.0, 0.0, 1.0, 0.4],                 # z == zmax: rejected
        [10.0, 0.0, below(1.0), 0.5],          # z = 0.99999994: iz = 40 -> dropped
        [10.0, below(40.0), 0.0, 0.6],         # y = 39.999996: iy = 1600 -> dropped
        [below(70.4), 0.0, 0.0, 0.7],          # x = 70.399994: ix = 1407 kept
        [-0.0, 0.0, 0.0, 0.8],                 # -0.0 >= 0.0: kept, ix = 0
    ], np.float32)
    vox, coors, n, npts, st = O.voxelize(pts, RANGE, VSIZE, 5, 100)
    assert n == 3
    assert coors[:3].tolist() == [[0, 0, 0, 0], [0, 30, 800, 1407], [0, 30, 800, 0]]


def test_point_features_stride():
    pts4 = F.lidar_frame(2000, 7)
    pts5 = np.concatenate([pts4, np.full((2000, 1), 9.0, np.float32)], axis=1)
    a = O.voxelize(pts4, RANGE, VSIZE, 5, 5000)
    b = O.voxelize(pts5, RANGE, VSIZE, 5, 5000)
    assert a[2] == b[2] and np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
