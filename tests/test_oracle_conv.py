"""Pins the oracle's rulebook builders, gather-GEMM-scatter, epilogue and sparse2dense by brute force,
invariants and reduction to torch's dense conv3d.  No reference code is executed."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import oracle_lib as O
from sessd3d import backbone as B, ctypes_defs as D, frames as F

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kitti_000000_counts.json")

SPARSE_CASES = [
    # ksize, stride, padding (z,y,x), in grid (z,y,x)
    ((3, 3, 3), (2, 2, 2), (1, 1, 1), (9, 12, 10)),
    ((3, 3, 3), (2, 2, 2), (0, 1, 1), (11, 12, 10)),
    ((3, 1, 1), (2, 1, 1), (0, 0, 0), (5, 8, 6)),
    ((3, 3, 3), (1, 1, 1), (1, 1, 1), (5, 6, 7)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1), (8, 11, 9)),
]


def out_grid(in_grid, k, s, p):
    return tuple(B.conv_out_size(in_grid[a], k[a], s[a], p[a]) for a in range(3))


def brute_triples(cells, k, s, p, og):
    """{(offset, in zyx, out zyx)}: out*s - p + kk == in on every axis, out inside the grid."""
    t = set()
    for c in map(tuple, cells):
        for kz, ky, kx in itertools.product(range(k[0]), range(k[1]), range(k[2])):
            kk = (kz, ky, kx)
            num = [c[a] + p[a] - kk[a] for a in range(3)]
            if all(num[a] % s[a] == 0 and 0 <= num[a] // s[a] < og[a] for a in range(3)):
                o = tuple(num[a] // s[a] for a in range(3))
                t.add((kz * k[1] * k[2] + ky * k[2] + kx,) + c + o)
    return t


def test_out_grid_formula_reproduces_params_h():
    g = (41, 1600, 1408)
    want = [(21, 800, 704), (11, 400, 352), (5, 200, 176), (2, 200, 176)]
    cfgs = [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
            ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((3, 1, 1), (2, 1, 1), (0, 0, 0))]
    for (k, s, p), w in zip(cfgs, want):
        g = out_grid(g, k, s, p)
        assert g == w
    # and the layer table carries the same shapes (x,y,z order)
    sp = [l for l in B.reference_layers() if l.type == D.SESSD_LAYER_SPARSE]
    assert [l.out_shape[::-1] for l in sp] == want


@pytest.mark.parametrize("k,s,p,ig", SPARSE_CASES)
def test_valid_out_pos_brute_force(k, s, p, ig):
    og = out_grid(ig, k, s, p)
    for c in itertools.product(range(ig[0]), range(ig[1]), range(ig[2])):
        got = O.valid_out_pos(c, k, s, p, og)
        want = brute_triples([c], k, s, p, og)
        assert {(r[3],) + tuple(c) + tuple(r[:3]) for r in got.tolist()} == want
        assert len(got) == len(want)          # no duplicates
        # enumeration order: (z,y,x) descending, x fastest
        keys = [tuple(r[:3]) for r in got.tolist()]
        assert keys == sorted(keys, reverse=True)


@pytest.mark.parametrize("seed", [0, 1])
def test_subm_rulebook_invariants_and_brute_force(seed):
    grid = (41, 160, 140)
    n = 2000
    coors = F.clustered_active_voxels(n, grid, seed)
    mv = 2500
    pairs, num, st = O.subm_rulebook(coors, n, grid[::-1], mv)
    assert st == 0
    # centre offset: every voxel pairs with itself
    assert num[13] == n
    assert np.array_equal(pairs[13, 0, :n], np.arange(n)) and np.array_equal(pairs[13, 1, :n], np.arange(n))
    assert np.all(pairs[13, :, n:] == -1)
    canon = O.canonical_rulebook(pairs, num, coors, coors)
    want = brute_triples(coors[:, 1:], (3, 3, 3), (1, 1, 1), (1, 1, 1), grid)
    # SubM keeps only outputs that are active inputs
    active = set(map(tuple, coors[:, 1:].tolist()))
    want = {t for t in want if t[4:] in active}
    assert set(map(tuple, canon.tolist())) == want and len(canon) == len(want)
    # symmetry (i,o,k) <-> (o,i,26-k)
    mirrored = {(26 - t[0],) + t[4:] + t[1:4] for t in want}
    assert mirrored == want
    assert len(want) > 3 * n   # the clustered input really has neighbours


def test_subm_rulebook_random_uniform_config1():
    """Benchmark configuration 1: 2000 uniform voxels in 41x160x140."""
    grid = (41, 160, 140)
    coors = F.random_active_voxels(2000, grid, 0)
    pairs, num, st = O.subm_rulebook(coors, 2000, grid[::-1], 2000)
    canon = O.canonical_rulebook(pairs, num, coors, coors)
    active = set(map(tuple, coors[:, 1:].tolist()))
    want = {t for t in brute_triples(coors[:, 1:], (3, 3, 3), (1, 1, 1), (1, 1, 1), grid) if t[4:] in active}
    assert set(map(tuple, canon.tolist())) == want


@pytest.mark.parametrize("k,s,p,ig", SPARSE_CASES)
def test_sparse_rulebook_brute_force(k, s, p, ig):
    og = out_grid(ig, k, s, p)
    n = min(150, ig[0] * ig[1] * ig[2] // 3)
    coors = F.random_active_voxels(n, ig, 3)
    mv = 4096
    pairs, num, oc, m, st = O.sparse_rulebook(coors, n, og[::-1], k, s, p, mv)
    assert st == 0
    want = brute_triples(coors[:, 1:], k, s, p, og)
    canon = O.canonical_rulebook(pairs, num, coors, oc)
    assert set(map(tuple, canon.tolist())) == want and len(canon) == len(want)
    outs = sorted({t[4:] for t in want})
    assert m == len(outs)
    assert sorted(map(tuple, oc[:m, 1:].tolist())) == outs
    assert np.all(oc[:m, 0] == 0) and np.all(oc[m:] == 0)
    # first-seen numbering: output ids appear in increasing order when walking inputs in order
    seen = []
    for v in range(n):
        for r in O.valid_out_pos(coors[v, 1:], k, s, p, og).tolist():
            if tuple(r[:3]) not in seen:
                seen.append(tuple(r[:3]))
    assert seen == list(map(tuple, oc[:m, 1:].tolist()))


def test_sparse_rulebook_cap():
    k, s, p, ig = SPARSE_CASES[0]
    og = out_grid(ig, k, s, p)
    coors = F.random_active_voxels(200, ig, 5)
    full = O.sparse_rulebook(coors, 200, og[::-1], k, s, p, 4096)
    cap = full[3] // 2
    pairs, num, oc, m, st = O.sparse_rulebook(coors, 200, og[::-1], k, s, p, cap)
    assert m == cap and st & D.SESSD_STATUS_VOXEL_OVERFLOW
    assert np.array_equal(oc[:cap], full[2][:cap])
    got = set(map(tuple, O.canonical_rulebook(pairs, num, coors, oc).tolist()))
    kept = set(map(tuple, oc[:cap, 1:].tolist()))
    want = {t for t in map(tuple, O.canonical_rulebook(full[0], full[1], coors, full[2]).tolist()) if t[4:] in kept}
    assert got == want


def test_kernel_offsets_stay_in_range_for_cells_on_the_grid_and_leave_it_for_negative_ones():
    """getValidOutPos' offset index lies in [0, K) for every non-negative cell coordinate, over kernel, stride and
    padding settings that include all of params.h's; a negative coordinate breaks that (C division truncates toward
    zero), which is why a strided layer refuses such rows (SESSD_STATUS_BAD_COORD) instead of indexing its rulebook
    with the result, as the reference would."""
    settings = [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((3, 1, 1), (2, 1, 1), (0, 0, 0)),
                ((3, 3, 3), (1, 1, 1), (1, 1, 1)), ((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (3, 3, 3), (2, 2, 2)),
                ((1, 3, 3), (1, 2, 2), (0, 1, 1)), ((3, 3, 3), (2, 2, 2), (2, 2, 2))]
    for k, s, p in settings:
        K = k[0] * k[1] * k[2]
        og = (9, 9, 9)
        for c in np.ndindex(6, 6, 6):
            vp = O.valid_out_pos(c, k, s, p, og)
            assert len(vp) <= 27 and (len(vp) == 0 or (vp[:, 3].min() >= 0 and vp[:, 3].max() < K)), (k, s, p, c)
    vp = O.valid_out_pos((-2, 0, 0), (3, 3, 3), (2, 2, 2), (1, 1, 1), (9, 9, 9))
    assert len(vp) and vp[:, 3].min() < 0                       # the reference's arithmetic, restated: out of range
    # the rulebook builder drops such rows: same result as without them, plus the status bit
    coors = np.array([[0, 2, 3, 4], [0, -2, 0, 0], [0, 4, 4, 4], [0, 1, -1, 1], [0, 0, 0, 0]], np.int32)
    good = coors[[0, 2, 4]]
    args = ((9, 9, 9), (3, 3, 3), (2, 2, 2), (1, 1, 1), 64)
    pairs, num, oc, on, st = O.sparse_rulebook(coors, len(coors), *args)
    g_pairs, g_num, g_oc, g_on, g_st = O.sparse_rulebook(good, len(good), *args)
    assert st == D.SESSD_STATUS_BAD_COORD and g_st == 0
    assert on == g_on and np.array_equal(oc, g_oc) and np.array_equal(num, g_num)
    assert np.array_equal(O.canonical_rulebook(pairs, num, coors, oc), O.canonical_rulebook(g_pairs, g_num, good, g_oc))


def test_kitti_stage_counts(kitti_frame0):
    with open(GOLDEN) as f:
        gold = json.load(f)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=1)
    r = O.frame(kitti_frame0, B.voxelgen_desc(), layers, W, B.dense_desc(), want_dense=False)
    stage_end = [0, 2, 5, 9, 13]   # counts index after voxelizer / sparse6 / 15 / 27 / 39 ... see below
    counts = r["counts"]
    sites = [int(counts[0]), int(counts[3]), int(counts[6]), int(counts[10]), int(counts[14])]
    assert sites == gold["active_sites_after_stage"]
    assert r["pairs"].tolist() == gold["pairs_per_layer"]
    assert r["status"] == 0 and stage_end


def dense_conv3d(coors, n, feat, w, k, s, p, ig):
    """Reference result through torch: scatter to a dense volume, conv3d, read every output cell."""
    cin, cout = w.shape[1], w.shape[2]
    vol = torch.zeros((1, cin) + tuple(ig), dtype=torch.float64)
    c = torch.as_tensor(coors[:n, 1:].astype(np.int64))
    vol[0, :, c[:, 0], c[:, 1], c[:, 2]] = torch.as_tensor(feat[:n].astype(np.float64)).T
    wt = torch.as_tensor(w.astype(np.float64)).reshape(k[0], k[1], k[2], cin, cout).permute(4, 3, 0, 1, 2)
    return torch.nn.functional.conv3d(vol, wt, stride=s, padding=p)[0].numpy()   # [cout, z, y, x]


@pytest.mark.parametrize("k,s,p,ig", SPARSE_CASES)
def test_sparse_conv_equals_dense_conv3d(k, s, p, ig):
    """Weight layout [K][Cin][Cout] with K = kz*k1*k2+ky*k2+kx, padding and stride per axis: on a small
    grid the sparse layer must reproduce torch's conv3d at every active output and the inactive
    outputs of conv3d must be exactly zero."""
    og = out_grid(ig, k, s, p)
    rng = np.random.default_rng(11)
    n = min(120, ig[0] * ig[1] * ig[2] // 3)
    coors = F.random_active_voxels(n, ig, 7)
    cin, cout = 5, 7
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.3, (k[0] * k[1] * k[2], cin, cout)).astype(np.float32)
    mv = 4096
    pairs, num, oc, m, st = O.sparse_rulebook(coors, n, og[::-1], k, s, p, mv)
    out = O.gather_gemm_scatter(feat, w, pairs, num, mv)
    ref = dense_conv3d(coors, n, feat, w, k, s, p, ig)
    got = np.zeros_like(ref)
    got[:, oc[:m, 1], oc[:m, 2], oc[:m, 3]] = out[:m].T
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)
    assert np.all(out[m:] == 0)


def test_subm_conv_equals_dense_conv3d_on_active_sites():
    ig = (6, 9, 8)
    rng = np.random.default_rng(2)
    n = 140
    coors = F.random_active_voxels(n, ig, 9)
    cin, cout = 4, 6
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.3, (27, cin, cout)).astype(np.float32)
    pairs, num, st = O.subm_rulebook(coors, n, ig[::-1], 256)
    out = O.gather_gemm_scatter(feat, w, pairs, num, 256)
    ref = dense_conv3d(coors, n, feat, w, (3, 3, 3), (1, 1, 1), (1, 1, 1), ig)
    assert np.allclose(out[:n].T, ref[:, coors[:, 1], coors[:, 2], coors[:, 3]], rtol=1e-5, atol=1e-5)


def test_gemm_counts_neighbours_and_is_linear():
    grid = (41, 160, 140)
    n = 1500
    coors = F.clustered_active_voxels(n, grid, 4)
    pairs, num, _ = O.subm_rulebook(coors, n, grid[::-1], n)
    ones = np.ones((n, 1), np.float32)
    out = O.gather_gemm_scatter(ones, np.ones((27, 1, 1), np.float32), pairs, num, n)
    cnt = np.zeros(n)
    for k in range(27):
        np.add.at(cnt, pairs[k, 1, :num[k]], 1)
    assert np.array_equal(out[:, 0], cnt) and int(cnt.sum()) == int(num.sum())
    rng = np.random.default_rng(0)
    a, b = rng.normal(size=(2, n, 3)).astype(np.float32)
    w = rng.normal(size=(27, 3, 4)).astype(np.float32)
    f = lambda x: O.gather_gemm_scatter(x, w, pairs, num, n).astype(np.float64)  # noqa: E731
    assert np.allclose(f(a + b), f(a) + f(b), atol=1e-4)
    assert np.all(O.gather_gemm_scatter(a, np.zeros_like(w), pairs, num, n) == 0)


def test_scale_shift_relu_and_fold_bn_closed_form():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(50, 8)).astype(np.float32)
    g, b, m = rng.normal(size=(3, 8)).astype(np.float32)
    v = rng.uniform(0.5, 2, 8).astype(np.float32)
    sc, sh = O.fold_bn(g, b, m, v, 1e-5)
    want = (x.astype(np.float64) - m) / np.sqrt(v.astype(np.float64) + 1e-5) * g + b
    got = O.scale_shift_relu(x, 50, sc, sh, True)
    assert np.allclose(got, np.maximum(want, 0), rtol=1e-5, atol=1e-6)
    assert np.array_equal(B.fold_bn(g, b, m, v)[0], sc) and np.array_equal(B.fold_bn(g, b, m, v)[1], sh)
    # identity statistics leave the input untouched
    one = np.ones(8, np.float32)
    sc, sh = O.fold_bn(one, 0 * one, 0 * one, one - np.float32(1e-5), 1e-5)
    assert np.allclose(sc, 1, atol=1e-7) and np.all(sh == 0)
    assert np.array_equal(O.scale_shift_relu(x, 50, None, None, False), x)
    # rows beyond `rows` are untouched
    y = O.scale_shift_relu(x, 10, sc, sh, True)
    assert np.array_equal(y[10:], x[10:])


def test_sparse2dense_closed_form():
    rng = np.random.default_rng(3)
    size = (176, 200, 2)
    n, c = 500, 64
    coors = F.random_active_voxels(n, size[::-1], 1)
    feat = rng.uniform(0.1, 1, (n, c)).astype(np.float32)
    dense = O.sparse2dense(feat, coors, n, size)
    assert dense.shape == (128, 200, 176)
    assert np.count_nonzero(dense) == n * c
    back = dense.reshape(c, 2, 200, 176)[:, coors[:, 1], coors[:, 2], coors[:, 3]].T
    assert np.array_equal(back, feat)
    v = 17
    assert dense[5 * 2 + coors[v, 1], coors[v, 2], coors[v, 3]] == feat[v, 5]


def test_gather_gemm_is_bit_identical_for_any_thread_count():
    layer = B.reference_layers()[3]                      # subm9, 32 -> 32
    rng = np.random.default_rng(6)
    n, mv = 3000, 4096
    coors = F.clustered_active_voxels(n, layer.out_shape[::-1], 5)
    n = len(coors)
    feat = rng.normal(size=(n, 32)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, 32, 32)).astype(np.float32)
    pairs, num, _ = O.subm_rulebook(coors, n, layer.out_shape, mv)
    assert int(num.sum()) > 3 * n
    one = O.gather_gemm_scatter(feat, w, pairs, num, mv)
    try:
        O.set_threads(4)
        four = O.gather_gemm_scatter(feat, w, pairs, num, mv)
    finally:
        O.set_threads(1)
    assert np.array_equal(one.view(np.uint32), four.view(np.uint32))


def test_zero_pad2d_equals_torch_pad():
    # zeroPad2d.cu:183-244 against the library routine, incl. asymmetric borders and the reference's 1,1,1,1
    import torch
    rng = np.random.default_rng(4)
    for (c, h, w), (t, b, l, r) in [((128, 200, 176), (1, 1, 1, 1)), ((3, 5, 7), (2, 0, 1, 3)), ((1, 1, 1), (0, 0, 0, 0)),
                                    ((4, 6, 2), (0, 3, 2, 0))]:
        x = rng.uniform(0.5, 1.5, (c, h, w)).astype(np.float32)
        want = torch.nn.functional.pad(torch.from_numpy(x), (l, r, t, b), mode="constant", value=0.0).numpy()
        got = O.zero_pad2d(x, t, b, l, r)
        assert got.shape == (c, h + t + b, w + l + r)
        assert np.array_equal(got, want)


def test_round_to_half_matches_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 1, 5000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
                        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6.1e-5, 5.96e-8, 2.98e-8, 2.99e-8]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    assert np.array_equal(O.round_to_half(x).view(np.uint32), want.view(np.uint32))


def test_frame_is_the_composition_of_its_parts():
    pts = F.lidar_frame(3000, 2)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=3, w_std=0.05)
    mv = 12000
    vg = B.voxelgen_desc(max_voxels=mv)
    r = O.frame(pts, vg, layers, W, B.dense_desc())
    vox, coors, n, _, _ = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, mv)
    feat = vox
    for i, l in enumerate(layers):
        feat, coors, n, pairs, num = O.conv_layer(feat, coors, n, l, W.w[i], W.scale[i], W.shift[i], mv)
        assert n == r["counts"][i + 1] and int(num.sum()) == r["pairs"][i]
    assert np.array_equal(feat[:n], r["feat"]) and np.array_equal(coors[:n], r["coors"])
    assert np.array_equal(O.sparse2dense(feat, coors, n, B.DENSE_SIZE_XYZ), r["dense"])
