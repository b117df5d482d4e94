"""GPU parity: every plugin of libsessd3d, called through the C-ABI, against the CPU oracle on the same
seeded inputs.  Integer results (voxel coordinates, active sites, rulebooks, counts) must be
bit-exact, after canonical sort where the numbering is free; FP32 features within 1e-4 relative."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import (DEV, RTOL_FP16, RTOL_FP32, abs_sum_of, assert_features_close, canonical, dev, points_input, to_np)
from sessd3d import api, backbone as B, ctypes_defs as D, frames as F

pytestmark = pytest.mark.gpu

RANGE, VSIZE = B.POINT_CLOUD_RANGE, B.VOXEL_SIZE


def run_voxelgen(pts, max_points, max_voxels, max_pts=5):
    vg = api.VoxelGenerator(max_voxels=max_voxels, max_num_points_per_voxel=max_pts)
    p, n = points_input(pts, max_points)
    vox, coors, num = vg(p, n)
    torch.cuda.synchronize()
    return to_np(vox), to_np(coors), int(to_np(num)[0]), vg.status()


def check_voxelgen(pts, max_points, max_voxels, max_pts=5):
    vox, coors, n, st = run_voxelgen(pts, max_points, max_voxels, max_pts)
    o_vox, o_coors, o_n, _, o_st = O.voxelize(pts[:max_points], RANGE, VSIZE, max_pts, max_voxels)
    assert n == o_n
    assert st == o_st
    # same numbering (first appearance) -> comparable row by row, and again after canonical sort
    assert np.array_equal(coors, o_coors)
    assert np.array_equal(vox.view(np.uint32), o_vox.view(np.uint32))      # bit-exact means
    a = canonical(coors, n, vox)
    b = canonical(o_coors, o_n, o_vox)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    return n


@pytest.mark.parametrize("seed", [0, 1])
def test_voxelgen_config2(seed):
    """Benchmark configuration 2: 20 000 points, voxel 0.05x0.05x0.1, <= 5 points/voxel, cap 20 000."""
    pts = F.lidar_frame(20000, seed)
    n = check_voxelgen(pts, 20000, 20000)
    assert 14000 < n <= 20000


def test_voxelgen_reference_shapes_and_padding():
    """MAX_POINTS 80000 / MAX_VOXELS 60000 as in params.h; rows past points_size are ignored even if
    they hold in-range garbage."""
    pts = F.lidar_frame(20000, 2)
    vg = api.VoxelGenerator(max_voxels=60000)
    buf = np.tile(pts[:100], (800, 1)).astype(np.float32)      # 80000 rows of valid-looking points
    buf[:20000] = pts
    vox, coors, num = vg(dev(buf), dev(np.array([20000], np.int32)))
    torch.cuda.synchronize()
    o = O.voxelize(pts, RANGE, VSIZE, 5, 60000)
    assert int(to_np(num)[0]) == o[2]
    assert np.array_equal(to_np(coors), o[1]) and np.array_equal(to_np(vox).view(np.uint32), o[0].view(np.uint32))
    assert vg.status() == 0


def test_voxelgen_crowded_voxels_and_shuffled_order():
    rng = np.random.default_rng(3)
    pts = F.lidar_frame(12000, 3)
    extra = pts[rng.integers(0, len(pts), 6000)] + rng.normal(0, 0.004, (6000, 4)).astype(np.float32)
    pts = np.concatenate([pts, extra.astype(np.float32)])[rng.permutation(18000)]
    check_voxelgen(pts, 18000, 20000)
    check_voxelgen(pts, 18000, 20000, max_pts=3)
    check_voxelgen(pts, 18000, 20000, max_pts=8)


def test_voxelgen_cap_overflow_and_edges():
    pts = F.lidar_frame(20000, 4)
    check_voxelgen(pts, 20000, 5000)                 # cap binds: first 5000 cells kept, flag raised
    vox, coors, n, st = run_voxelgen(pts, 20000, 5000)
    assert n == 5000 and st & D.SESSD_STATUS_VOXEL_OVERFLOW
    check_voxelgen(pts[:0], 1024, 1000)              # empty cloud
    check_voxelgen(pts[:1], 1024, 1000)
    # points_size larger than the tensor: clamped to max_points
    vox, coors, n, st = run_voxelgen(pts, 4096, 20000)
    assert n == O.voxelize(pts[:4096], RANGE, VSIZE, 5, 20000)[2]
    f = np.float32
    below = lambda v: np.nextafter(f(v), f(-np.inf))   # noqa: E731
    edge = np.array([[0.0, -40.0, -3.0, 0.1], [70.4, 0.0, 0.0, 0.2], [10.0, 40.0, 0.0, 0.3], [10.0, 0.0, 1.0, 0.4],
                     [10.0, 0.0, below(1.0), 0.5], [10.0, below(40.0), 0.0, 0.6], [below(70.4), 0.0, 0.0, 0.7],
                     [-0.0, 0.0, 0.0, 0.8], [np.nan, 0.0, 0.0, 0.9], [np.inf, 0.0, 0.0, 1.0]], np.float32)
    assert check_voxelgen(edge, 64, 100) == 3


def test_voxelgen_five_point_features():
    pts = F.lidar_frame(8000, 5)
    pts5 = np.concatenate([pts, np.full((8000, 1), 7.0, np.float32)], axis=1)
    check_voxelgen(pts5, 8192, 20000)


def run_subm(coors_np, n, feat_np, w, grid_zyx, max_voxels, scale=None, shift=None, relu=False):
    conv = api.SubmConv3d(w.shape[1], w.shape[2], grid_zyx[::-1], w, max_voxels)
    if scale is not None or relu:
        conv.set_epilogue(scale, shift, relu)
    cbuf = np.zeros((max_voxels, 4), np.int32)
    cbuf[:n] = coors_np[:n]
    fbuf = np.zeros((max_voxels, w.shape[1]), np.float32)
    fbuf[:n] = feat_np[:n]
    out = conv(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    pairs, num = conv.export_rulebook()
    torch.cuda.synchronize()
    return conv, to_np(out), to_np(pairs), to_np(num).astype(np.uint32), cbuf


def test_subm_config1_rulebook_and_features():
    """Benchmark configuration 1: one SubMConv3d 4->16 on 2000 uniform voxels in 41x160x140."""
    grid = (41, 160, 140)
    n, mv = 2000, 2000
    rng = np.random.default_rng(0)
    coors = F.random_active_voxels(n, grid, 0)
    feat = rng.uniform(0, 1, (n, 4)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, 4, 16)).astype(np.float32)
    conv, out, pairs, num, cbuf = run_subm(coors, n, feat, w, grid, mv)
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    assert np.array_equal(num, o_num)
    assert np.array_equal(O.canonical_rulebook(pairs, num, cbuf, cbuf), O.canonical_rulebook(o_pairs, o_num, coors, coors))
    o_out = O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)
    assert_features_close(out, o_out, RTOL_FP32, "subm config 1")
    assert conv.status() == 0


@pytest.mark.parametrize("cin,cout", [(4, 16), (16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128),
                                      (5, 7), (8, 32)])
def test_subm_clustered_with_epilogue_and_pad_rows(cin, cout):
    grid = (21, 200, 176)
    n, mv = 6000, 8192
    rng = np.random.default_rng(cin)
    coors = F.clustered_active_voxels(n, grid, 1, n_blobs=60)
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, cin, cout)).astype(np.float32)
    sc = rng.uniform(0.5, 1.5, cout).astype(np.float32)
    sh = rng.uniform(-0.2, 0.2, cout).astype(np.float32)
    conv, out, pairs, num, cbuf = run_subm(coors, n, feat, w, grid, mv, sc, sh, True)
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    assert int(o_num.sum()) > 4 * n
    assert np.array_equal(num, o_num)
    assert np.array_equal(O.canonical_rulebook(pairs, num, cbuf, cbuf), O.canonical_rulebook(o_pairs, o_num, coors, coors))
    # within an offset the exported pairs are in ascending output-row order, unused entries are -1
    for k in (0, 13, 26):
        assert np.all(np.diff(pairs[k, 1, :num[k]]) > 0) and np.all(pairs[k, :, num[k]:] == -1)
    o_out = O.scale_shift_relu(O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), mv, sc, sh, True)
    assert_features_close(out, o_out, RTOL_FP32, "subm %d->%d" % (cin, cout),   # incl. pad rows = relu(shift)
                          abs_sum=abs_sum_of(feat, w, o_pairs, o_num, mv, mv, sc, sh))


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_equal_work_tiles_with_dense_and_isolated_regions(dtype):
    """A fully dense block (27 pairs per row) followed by isolated voxels (1 pair per row): the equal-work tile
    cuts give the isolated stretch runs far longer than the kernel's tile capacity, which it walks in pieces.
    Shuffled row order as a second case (every tile mixes both kinds)."""
    grid = (21, 800, 704)
    rng = np.random.default_rng(31)
    z, y, x = np.meshgrid(np.arange(2, 14), np.arange(100, 114), np.arange(200, 214), indexing="ij")
    dense = np.stack([np.zeros(z.size, np.int64), z.ravel(), y.ravel(), x.ravel()], 1)
    iso = np.stack([np.zeros(4000, np.int64), rng.integers(0, 21, 4000) // 3 * 3, 300 + 3 * (np.arange(4000) // 60),
                    3 * (np.arange(4000) % 60)], 1)
    iso = np.unique(iso, axis=0)
    for order in ("blocked", "shuffled"):
        coors = np.concatenate([dense, iso]).astype(np.int32)
        if order == "shuffled":
            coors = coors[rng.permutation(len(coors))]
        n, mv = len(coors), 8192
        feat = rng.uniform(-1, 1, (n, 64)).astype(np.float32)
        w = rng.normal(0, 0.05, (27, 64, 64)).astype(np.float32)
        o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
        assert o_num[13] == n and int(o_num.sum()) > 20 * len(dense)
        if dtype == "fp32":
            conv, out, pairs, num, _ = run_subm(coors, n, feat, w, grid, mv)
            assert np.array_equal(num, o_num)
            assert_features_close(out[:n], O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)[:n], RTOL_FP32, order,
                                  abs_sum=abs_sum_of(feat, w, o_pairs, o_num, mv)[:n])
        else:
            conv = api.SubmConv3d(64, 64, grid[::-1], w, mv)
            cbuf = np.zeros((mv, 4), np.int32)
            cbuf[:n] = coors
            fbuf = np.zeros((mv, 64), np.float16)
            fbuf[:n] = feat
            out = to_np(conv(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32))).float())
            wh = w.astype(np.float16).astype(np.float32)
            want = O.gather_gemm_scatter(fbuf[:n].astype(np.float32), wh, o_pairs, o_num, mv)[:n]
            assert_features_close(out[:n], want, RTOL_FP16, order, half=True,
                                  abs_sum=abs_sum_of(fbuf[:n].astype(np.float32), wh, o_pairs, o_num, mv)[:n])
        assert conv.status() == 0


def test_mfma_and_valu_paths_agree():
    """The matrix-core kernel against the shape-agnostic VALU kernel on the same rulebook (both FP32)."""
    grid = (11, 120, 120)
    n, mv = 9000, 9001                      # a last tile that is only partly active
    rng = np.random.default_rng(7)
    coors = F.clustered_active_voxels(n, grid, 5, n_blobs=30, sigma=(1.5, 5.0, 5.0))
    feat = rng.uniform(-1, 1, (n, 64)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, 64, 64)).astype(np.float32)
    outs = []
    for flags in (0, D.SESSD_FLAG_FORCE_VALU):
        conv = api.SubmConv3d(64, 64, grid[::-1], w, mv)
        conv.set_flags(flags)
        cbuf = np.zeros((mv, 4), np.int32)
        cbuf[:n] = coors
        fbuf = np.zeros((mv, 64), np.float32)
        fbuf[:n] = feat
        outs.append(to_np(conv(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))))
    o_pairs, o_num, _ = O.subm_rulebook(cbuf, n, grid[::-1], mv)
    assert_features_close(outs[0], outs[1], RTOL_FP32, "mfma vs valu", abs_sum=abs_sum_of(feat, w, o_pairs, o_num, mv))


@pytest.mark.parametrize("cin,cout", [(4, 16), (16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128),
                                      (8, 32)])
def test_subm_fp16_features(cin, cout):
    """FP16 features and weights, FP32 accumulate (benchmark configurations 4-5).  The oracle runs in FP32 on the
    half-rounded inputs and weights and rounds its output to half: agreement within 1e-2 relative."""
    grid = (21, 200, 176)
    n, mv = 6000, 8192
    rng = np.random.default_rng(100 + cin)
    coors = F.clustered_active_voxels(n, grid, 2, n_blobs=60)
    in_half = cin != 4                               # the first layer reads the voxelizer's FP32 means
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    if in_half:
        feat = O.round_to_half(feat)
    w = O.round_to_half(rng.normal(0, 0.1, (27, cin, cout)).astype(np.float32))
    sc = rng.uniform(0.5, 1.5, cout).astype(np.float32)
    sh = rng.uniform(-0.2, 0.2, cout).astype(np.float32)
    conv = api.SubmConv3d(cin, cout, grid[::-1], w, mv)
    conv.set_epilogue(sc, sh, True)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n] = feat
    d_feat = dev(fbuf, torch.float16 if in_half else torch.float32)
    out = conv(d_feat, dev(cbuf), dev(np.array([n], np.int32)), out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    o_out = O.round_to_half(O.scale_shift_relu(O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), mv, sc, sh, True))
    assert_features_close(to_np(out.float()), o_out, RTOL_FP16, "fp16 subm %d->%d" % (cin, cout))
    # the MFMA and VALU FP16 paths agree much more tightly than the 1e-2 bound
    conv.set_flags(D.SESSD_FLAG_FORCE_VALU)
    out2 = conv(d_feat, dev(cbuf), dev(np.array([n], np.int32)), out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert_features_close(to_np(out.float()), to_np(out2.float()), 2e-3, "fp16 mfma vs valu %d->%d" % (cin, cout))


def test_sparse_fp16_features():
    layer = SPARSE_LAYERS[1]        # 32 -> 64, stride 2
    ig = sparse_input_grid(layer)
    n, mv = 5000, 30000
    rng = np.random.default_rng(77)
    coors = F.clustered_active_voxels(n, (ig[0], 300, 300), 3, n_blobs=50)
    feat = O.round_to_half(rng.uniform(-1, 1, (n, layer.cin)).astype(np.float32))
    w = O.round_to_half(rng.normal(0, 0.1, (layer.kvol, layer.cin, layer.cout)).astype(np.float32))
    conv = api.SparseConv3d(layer.cin, layer.cout, layer.out_shape, ig[::-1], layer.ksize, layer.stride,
                            layer.padding, w, mv)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, layer.cin), np.float32)
    fbuf[:n] = feat
    out, oc, on = conv(dev(fbuf, torch.float16), dev(cbuf), dev(np.array([n], np.int32)))
    torch.cuda.synchronize()
    o_pairs, o_num, o_oc, o_on, _ = O.sparse_rulebook(coors, n, layer.out_shape, layer.ksize, layer.stride,
                                                      layer.padding, mv)
    assert int(to_np(on)[0]) == o_on and np.array_equal(to_np(oc), o_oc)
    o_out = O.round_to_half(O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv))
    assert_features_close(to_np(out.float()), o_out, RTOL_FP16, "fp16 sparse15")


def test_sparse2dense_fp16():
    rng = np.random.default_rng(3)
    n, mv, c = 1500, 4096, 64
    coors = F.random_active_voxels(n, (2, 200, 176), 9)
    feat = O.round_to_half(rng.uniform(0.1, 1, (n, c)).astype(np.float32))
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, c), np.float32)
    fbuf[:n] = feat
    s2d = api.Sparse2Dense()
    dense = s2d(dev(fbuf, torch.float16), dev(cbuf), dev(np.array([n], np.int32)))
    torch.cuda.synchronize()
    assert dense.dtype == torch.float16
    assert np.array_equal(to_np(dense.float()), O.sparse2dense(feat, coors, n, B.DENSE_SIZE_XYZ))


def test_subm_shared_rulebook_skip_pad_and_empty():
    grid = (11, 100, 88)
    n, mv = 3000, 4096
    rng = np.random.default_rng(5)
    coors = F.clustered_active_voxels(n, grid, 2)
    feat = rng.uniform(-1, 1, (n, 16)).astype(np.float32)
    w1 = rng.normal(0, 0.1, (27, 16, 16)).astype(np.float32)
    w2 = rng.normal(0, 0.1, (27, 16, 32)).astype(np.float32)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, 16), np.float32)
    fbuf[:n] = feat
    a = api.SubmConv3d(16, 16, grid[::-1], w1, mv)
    b = api.SubmConv3d(16, 32, grid[::-1], w2, mv)
    b.set_flags(D.SESSD_FLAG_SKIP_PAD_ROWS)
    d_coors, d_num = dev(cbuf), dev(np.array([n], np.int32))
    y1 = a(dev(fbuf), d_coors, d_num)
    y2 = b(y1, d_coors, d_num, rulebook_from=a)           # GEMM only, on a's rulebook
    torch.cuda.synchronize()
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    o1 = O.gather_gemm_scatter(feat, w1, o_pairs, o_num, mv)
    o2 = O.gather_gemm_scatter(o1, w2, o_pairs, o_num, mv)
    assert_features_close(to_np(y1), o1, RTOL_FP32, "shared: layer 1")
    assert_features_close(to_np(y2)[:n], o2[:n], RTOL_FP32, "shared: layer 2")
    # empty input: nothing active, all rows are pad rows
    y0 = a(dev(fbuf), d_coors, dev(np.array([0], np.int32)))
    pairs, num = a.export_rulebook()
    torch.cuda.synchronize()
    assert np.all(to_np(y0) == 0) and np.all(to_np(num) == 0) and np.all(to_np(pairs) == -1)


@pytest.mark.parametrize("owner_cout,sharer_cout", [(64, 32), (32, 64)])
def test_shared_rulebook_between_layers_of_different_tile_capacity(owner_cout, sharer_cout):
    """Two FP16 3x3x3 layers of different widths on one rulebook.  Both run on the tall-tile kernel, which cuts
    its own tiles (a rulebook built by such a layer carries no equal-work cuts) and sums a row's offsets in
    ascending order whatever tile the row falls in: the sharer's output on the owner's rulebook must equal its
    output on its own bit for bit."""
    grid = (21, 400, 352)
    n, mv, cin = 15000, 16384, 32
    rng = np.random.default_rng(41)
    coors = F.clustered_active_voxels(n, grid, 2, n_blobs=120)
    feat = O.round_to_half(rng.uniform(-1, 1, (n, cin)).astype(np.float32))
    w1 = O.round_to_half(rng.normal(0, 0.1, (27, cin, owner_cout)).astype(np.float32))
    w2 = O.round_to_half(rng.normal(0, 0.1, (27, cin, sharer_cout)).astype(np.float32))
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n] = feat
    a = api.SubmConv3d(cin, owner_cout, grid[::-1], w1, mv)
    b = api.SubmConv3d(cin, sharer_cout, grid[::-1], w2, mv)
    d_feat, d_coors, d_num = dev(fbuf, torch.float16), dev(cbuf), dev(np.array([n], np.int32))
    y1 = a(d_feat, d_coors, d_num, out_dtype=torch.float16)
    y2 = b(d_feat, d_coors, d_num, out_dtype=torch.float16, rulebook_from=a)
    torch.cuda.synchronize()
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    o1 = O.round_to_half(O.gather_gemm_scatter(feat, w1, o_pairs, o_num, mv))
    o2 = O.round_to_half(O.gather_gemm_scatter(feat, w2, o_pairs, o_num, mv))
    assert_features_close(to_np(y1.float()), o1, RTOL_FP16, "owner %d" % owner_cout)
    assert_features_close(to_np(y2.float()), o2, RTOL_FP16, "sharer %d" % sharer_cout)
    y3 = b(d_feat, d_coors, d_num, out_dtype=torch.float16)      # the sharer on its own rulebook
    torch.cuda.synchronize()
    assert torch.equal(y2, y3)


@pytest.mark.parametrize("n", [1, 17, 300])
@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_fewer_rows_than_tiles_in_a_wide_layer(n, dtype):
    """A handful of active rows in a layer wide enough to get equal-work tile cuts: the rows weigh more than
    total / tiles, and every entry of the cut table up to the last tile must still be written."""
    grid = (3, 48, 15)
    mv, cin, cout = n + 225, 64, 64
    half = dtype == "fp16"
    rng = np.random.default_rng(n)
    coors = F.clustered_active_voxels(n, grid, 5, n_blobs=2)
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, cin, cout)).astype(np.float32)
    if half:
        feat, w = O.round_to_half(feat), O.round_to_half(w)
    conv = api.SubmConv3d(cin, cout, grid[::-1], w, mv)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n] = feat
    tdt = torch.float16 if half else torch.float32
    for _ in range(2):                                       # the second call finds the first one's table
        out = conv(dev(fbuf, tdt), dev(cbuf), dev(np.array([n], np.int32)), out_dtype=tdt)
        torch.cuda.synchronize()
        o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
        o_out = O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)
        terms = abs_sum_of(feat, w, o_pairs, o_num, mv)
        if half:
            assert_features_close(to_np(out.float()), O.round_to_half(o_out), RTOL_FP16, "few rows fp16", abs_sum=terms, half=True)
        else:
            assert_features_close(to_np(out), o_out, RTOL_FP32, "few rows fp32", abs_sum=terms)
        assert conv.status() == 0


def test_few_output_sites_in_a_wide_strided_layer():
    """36 input cells, kernel (3,3,1), stride (3,1,2): a few dozen output rows in a 32 -> 64 layer."""
    k, s, p, ig = (3, 3, 1), (3, 1, 2), (0, 1, 0), (3, 26, 7)
    og = tuple(B.conv_out_size(ig[a], k[a], s[a], p[a]) for a in range(3))
    layer = B.Layer("t", D.SESSD_LAYER_SPARSE, 32, 64, og[::-1], k, s, p)
    n, mv = 36, 86
    rng = np.random.default_rng(4)
    coors = F.random_active_voxels(n, ig, 11)
    feat = rng.uniform(-1, 1, (n, 32)).astype(np.float32)
    w = rng.normal(0, 0.1, (layer.kvol, 32, 64)).astype(np.float32)
    conv, out, oc, on, pairs, num = run_sparse(layer, coors, n, feat, w, mv, ig)
    o_pairs, o_num, o_oc, o_on, o_st = O.sparse_rulebook(coors, n, og[::-1], k, s, p, mv)
    assert on == o_on and conv.status() == o_st and np.array_equal(oc, o_oc) and np.array_equal(num, o_num)
    assert_features_close(out, O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), RTOL_FP32, "few output sites")


def test_subm_bad_coordinate_is_flagged_not_written():
    grid = (5, 20, 20)
    coors = np.array([[0, 1, 1, 1], [0, 1, 1, 2], [0, 7, 1, 1], [0, 1, 25, 1]], np.int32)   # rows 2,3 outside
    feat = np.ones((4, 4), np.float32)
    w = np.ones((27, 4, 4), np.float32)
    conv, out, pairs, num, _ = run_subm(coors, 4, feat, w, grid, 64)
    assert conv.status() & D.SESSD_STATUS_BAD_COORD
    o_pairs, o_num, o_st = O.subm_rulebook(coors, 4, grid[::-1], 64)
    assert o_st & D.SESSD_STATUS_BAD_COORD and np.array_equal(num, o_num)
    assert np.array_equal(out, O.gather_gemm_scatter(feat, w, o_pairs, o_num, 64))


SPARSE_LAYERS = [l for l in B.reference_layers() if l.type == D.SESSD_LAYER_SPARSE]


def sparse_input_grid(layer):
    """Input grid (z,y,x) of a reference sparse layer = out grid of the stage before it."""
    prev = {"sparse6": (41, 1600, 1408), "sparse15": (21, 800, 704), "sparse27": (11, 400, 352), "sparse39": (5, 200, 176)}
    return prev[layer.name]


def run_sparse(layer, coors, n, feat, w, mv, in_grid_zyx, **kw):
    conv = api.SparseConv3d(layer.cin, layer.cout, layer.out_shape, in_grid_zyx[::-1], layer.ksize, layer.stride,
                            layer.padding, w, mv)
    if kw.get("epilogue"):
        conv.set_epilogue(*kw["epilogue"])
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors[:n]
    fbuf = np.zeros((mv, layer.cin), np.float32)
    fbuf[:n] = feat[:n]
    out, oc, on = conv(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    pairs, num = conv.export_rulebook()
    torch.cuda.synchronize()
    return conv, to_np(out), to_np(oc), int(to_np(on)[0]), to_np(pairs), to_np(num).astype(np.uint32)


@pytest.mark.parametrize("layer", SPARSE_LAYERS, ids=[l.name for l in SPARSE_LAYERS])
def test_sparse_layers_of_the_backbone(layer):
    """Each strided layer shape of params.h on a neighbour-rich active set in its own input grid."""
    ig = sparse_input_grid(layer)
    n, mv = 5000, 30000
    rng = np.random.default_rng(len(layer.name))
    sub = (ig[0], min(ig[1], 300), min(ig[2], 300))
    coors = F.clustered_active_voxels(n, sub, 3, n_blobs=50)
    feat = rng.uniform(-1, 1, (n, layer.cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (layer.kvol, layer.cin, layer.cout)).astype(np.float32)
    conv, out, oc, on, pairs, num = run_sparse(layer, coors, n, feat, w, mv, ig)
    o_pairs, o_num, o_oc, o_on, o_st = O.sparse_rulebook(coors, n, layer.out_shape, layer.ksize, layer.stride,
                                                         layer.padding, mv)
    assert on == o_on and conv.status() == o_st == 0
    assert np.array_equal(oc, o_oc)                       # first-seen numbering reproduced row by row
    assert np.array_equal(canonical(oc, on)[0], canonical(o_oc, o_on)[0])
    assert np.array_equal(num, o_num)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    assert np.array_equal(O.canonical_rulebook(pairs, num, cbuf, oc), O.canonical_rulebook(o_pairs, o_num, coors, o_oc))
    o_out = O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)
    terms = abs_sum_of(feat, w, o_pairs, o_num, mv)
    assert_features_close(out, o_out, RTOL_FP32, layer.name, abs_sum=terms)
    a = canonical(oc, on, out)
    b = canonical(o_oc, o_on, o_out)
    assert_features_close(a[1], b[1], RTOL_FP32, layer.name + " (canonical order)", abs_sum=canonical(o_oc, o_on, terms)[1])


def test_sparse_cap_overflow_and_empty():
    layer = SPARSE_LAYERS[0]
    ig = sparse_input_grid(layer)
    n = 4000
    rng = np.random.default_rng(9)
    coors = F.random_active_voxels(n, (ig[0], 200, 200), 4)    # uncorrelated sites: the set grows ~8x
    feat = rng.uniform(-1, 1, (n, layer.cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (layer.kvol, layer.cin, layer.cout)).astype(np.float32)
    mv = 8192
    conv, out, oc, on, pairs, num = run_sparse(layer, coors, n, feat, w, mv, ig)
    o_pairs, o_num, o_oc, o_on, o_st = O.sparse_rulebook(coors, n, layer.out_shape, layer.ksize, layer.stride,
                                                         layer.padding, mv)
    assert o_st & D.SESSD_STATUS_VOXEL_OVERFLOW and conv.status() & D.SESSD_STATUS_VOXEL_OVERFLOW
    assert on == o_on == mv and np.array_equal(oc, o_oc) and np.array_equal(num, o_num)
    assert_features_close(out, O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), RTOL_FP32, "capped sparse layer")
    # an empty frame through the same plugin and workspace, which still hold the full frame's tickets and flags
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, layer.cin), np.float32)
    fbuf[:n] = feat
    out2, oc2, on2 = conv(dev(fbuf), dev(cbuf), dev(np.array([0], np.int32)))
    num2 = conv.export_rulebook()[1]
    torch.cuda.synchronize()
    assert int(to_np(on2)[0]) == 0 and not to_np(out2).any() and not to_np(oc2).any() and not to_np(num2).any()
    assert conv.status() == 0
    conv, out, oc, on, pairs, num = run_sparse(layer, coors, 0, feat, w, mv, ig)
    assert on == 0 and np.all(out == 0) and np.all(oc == 0) and np.all(num == 0)


def test_sparse_layer_refuses_negative_coordinates():
    """Rows with a negative coordinate (for which getValidOutPos' truncating divisions give kernel offsets outside
    the rulebook) contribute nothing and raise BAD_COORD; everything else equals the oracle, which drops them too."""
    layer = SPARSE_LAYERS[0]
    ig = sparse_input_grid(layer)
    n, mv = 3000, 16384
    rng = np.random.default_rng(12)
    coors = F.clustered_active_voxels(n, (ig[0], 200, 200), 8, n_blobs=30)
    bad = rng.choice(n, 40, replace=False)
    coors[bad[:15], 1] = -rng.integers(1, 4, 15)
    coors[bad[15:30], 2] = -rng.integers(1, 40, 15)
    coors[bad[30:], 3] = -2
    feat = rng.uniform(-1, 1, (n, layer.cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (layer.kvol, layer.cin, layer.cout)).astype(np.float32)
    conv, out, oc, on, pairs, num = run_sparse(layer, coors, n, feat, w, mv, ig)
    o_pairs, o_num, o_oc, o_on, o_st = O.sparse_rulebook(coors, n, layer.out_shape, layer.ksize, layer.stride,
                                                         layer.padding, mv)
    assert conv.status() == o_st == D.SESSD_STATUS_BAD_COORD
    assert on == o_on and np.array_equal(oc, o_oc) and np.array_equal(num, o_num)
    assert not np.isin(pairs[:, 0, :][pairs[:, 0, :] >= 0], bad).any()       # no pair names a refused row
    assert_features_close(out, O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), RTOL_FP32, "rows with negative coordinates")


def test_sparse_generic_stride1_and_corner_truncation():
    """stride 1 (27 candidates per input) and cells at coordinate 0 with padding 0 (C division
    truncates toward zero in getValidOutPos)."""
    cases = [((3, 3, 3), (1, 1, 1), (1, 1, 1), (6, 9, 8)), ((3, 3, 3), (2, 2, 2), (0, 0, 0), (9, 9, 9)),
             ((2, 2, 2), (2, 2, 2), (0, 0, 0), (8, 8, 8)), ((1, 3, 3), (1, 2, 2), (0, 1, 1), (4, 9, 9))]
    rng = np.random.default_rng(1)
    for k, s, p, ig in cases:
        og = tuple(B.conv_out_size(ig[a], k[a], s[a], p[a]) for a in range(3))
        layer = B.Layer("t", D.SESSD_LAYER_SPARSE, 8, 16, og[::-1], k, s, p)
        n = ig[0] * ig[1] * ig[2] // 2
        coors = F.random_active_voxels(n, ig, 6)
        feat = rng.uniform(-1, 1, (n, 8)).astype(np.float32)
        w = rng.normal(0, 0.1, (layer.kvol, 8, 16)).astype(np.float32)
        mv = 1024
        conv, out, oc, on, pairs, num = run_sparse(layer, coors, n, feat, w, mv, ig)
        o_pairs, o_num, o_oc, o_on, _ = O.sparse_rulebook(coors, n, og[::-1], k, s, p, mv)
        assert on == o_on and np.array_equal(oc, o_oc) and np.array_equal(num, o_num), (k, s, p)
        assert_features_close(out, O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), RTOL_FP32, str((k, s, p)))


def test_sparse2dense_with_folded_zero_pad():
    # sparse2Dense followed by ZeroPad2dPlugin (se-ssd-ai-trt.cpp:1253) in one scatter; a copy: bit-exact
    rng = np.random.default_rng(12)
    n, mv, c = 2739, 8192, 64
    coors = F.random_active_voxels(n, (2, 200, 176), 9)
    coors[:4] = [(0, 0, 0, 0), (0, 1, 199, 175), (0, 0, 199, 0), (0, 1, 0, 175)]      # the four corners
    coors = np.unique(coors, axis=0)
    n = len(coors)
    feat = rng.uniform(0.1, 1, (n, c)).astype(np.float32)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, c), np.float32)
    fbuf[:n] = feat
    for pad in [(1, 1, 1, 1), (2, 0, 1, 3)]:
        for dt in (torch.float32, torch.float16):
            s2d = api.Sparse2Dense(padding=pad)
            f = dev(fbuf).to(dt)
            dense = s2d(f, dev(cbuf), dev(np.array([n], np.int32)))
            torch.cuda.synchronize()
            want = O.zero_pad2d(O.sparse2dense(to_np(f[:n].float()), coors, n, B.DENSE_SIZE_XYZ), *pad)
            assert tuple(dense.shape) == want.shape
            assert np.array_equal(to_np(dense.float()), want), (pad, dt)
            assert s2d.status() == 0
    # the output descriptor must carry the padded shape
    s2d = api.Sparse2Dense(padding=(1, 1, 1, 1))
    bad = torch.empty((128, 200, 176), dtype=torch.float32, device="cuda")
    with pytest.raises(api.SessdError):
        s2d.configure([dev(fbuf), dev(cbuf), dev(np.array([n], np.int32))], [bad])


@pytest.mark.parametrize("size_xyz,channel,pad", [((1000, 12, 3), 40, (0, 0, 0, 0)), ((1000, 12, 3), 40, (1, 0, 3, 2)),
                                                  ((449, 9, 1), 5, (0, 1, 0, 0)), ((7, 5, 2), 3, (0, 0, 0, 0))])
def test_sparse2dense_long_lines_and_odd_shapes(size_xyz, channel, pad):
    """Lines longer than one LDS segment, widths no 16-byte run divides, fewer channels than a channel group."""
    rng = np.random.default_rng(5)
    W, H, Dz = size_xyz
    n, mv = min(3000, W * H * Dz // 3), 4000
    coors = F.random_active_voxels(n, (Dz, H, W), 8)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = rng.uniform(0.1, 1, (mv, channel)).astype(np.float32)
    for dt in (torch.float32, torch.float16):
        s2d = api.Sparse2Dense(size_xyz, channel, padding=pad)
        f = dev(fbuf).to(dt)
        dense = s2d(f, dev(cbuf), dev(np.array([n], np.int32)))
        torch.cuda.synchronize()
        want = O.zero_pad2d(O.sparse2dense(to_np(f[:n].float()), coors, n, size_xyz), *pad)
        assert tuple(dense.shape) == want.shape
        assert np.array_equal(to_np(dense.float()), want), dt
        assert s2d.status() == 0


def test_sparse2dense():
    rng = np.random.default_rng(2)
    n, mv, c = 2739, 60000, 64
    coors = F.random_active_voxels(n, (2, 200, 176), 8)
    feat = rng.uniform(0.1, 1, (n, c)).astype(np.float32)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = rng.uniform(5, 6, (mv, c)).astype(np.float32)      # rows >= n hold garbage that must not leak
    fbuf[:n] = feat
    s2d = api.Sparse2Dense()
    dense = s2d(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    torch.cuda.synchronize()
    want = O.sparse2dense(feat, coors, n, B.DENSE_SIZE_XYZ)
    assert dense.shape == (128, 200, 176)
    assert np.array_equal(to_np(dense), want)
    assert s2d.status() == 0
    # the workspace may hold anything: the cell map is never cleared, a stale or random entry must not leak a row
    ws = s2d.ws.clone()
    for fill in (lambda t: t.fill_(0), lambda t: t.fill_(0x7f), lambda t: t.copy_(torch.randint(0, 256, t.shape, dtype=torch.uint8))):
        fill(ws)
        dense.fill_(3.0)
        s2d.enqueue([dev(fbuf), dev(cbuf), dev(np.array([n], np.int32))], [dense], workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(dense), want)
    ws32 = ws.view(torch.int32)
    ws32.copy_(torch.randint(-3, 2 * n, ws32.shape, dtype=torch.int32))   # plausible row numbers everywhere
    s2d.enqueue([dev(fbuf), dev(cbuf), dev(np.array([n], np.int32))], [dense], workspace=ws)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(dense), want)
    assert int(ws32[0].item()) == 0
    # idempotent on a dirty output buffer, empty input gives all zeros
    dense.fill_(3.0)
    s2d.enqueue([dev(fbuf), dev(cbuf), dev(np.array([0], np.int32))], [dense])
    torch.cuda.synchronize()
    assert float(dense.abs().max()) == 0.0
    cbuf[5] = (0, 2, 0, 0)                                        # z outside D=2
    s2d(dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    assert s2d.status() & D.SESSD_STATUS_BAD_COORD


def test_conv_serialization_round_trip():
    rng = np.random.default_rng(4)
    w = rng.normal(0, 0.1, (27, 4, 16)).astype(np.float32)
    a = api.SubmConv3d(4, 16, (140, 160, 41), w, 2000)
    blob = a.serialize()
    assert len(blob) == 16 * 4 + w.size * 4                     # submConv3dlayer.cu:684-687
    head = np.frombuffer(blob[:64], np.int32)
    assert head.tolist() == [4, 16, 2000, 4, 140, 160, 41, 140, 160, 41, 3, 1, 1, 1, 0, w.size]
    assert np.array_equal(np.frombuffer(blob[64:], np.float32), w.ravel())
    a.set_epilogue(np.ones(16), np.zeros(16), True)
    blob2 = a.serialize()
    assert blob2[:len(blob)] == blob and len(blob2) > len(blob)
    b = api.SubmConv3d.deserialize(blob2)
    assert b.serialize() == blob2
    layer = SPARSE_LAYERS[2]
    ws = rng.normal(0, 0.1, (27, 64, 64)).astype(np.float32)
    s = api.SparseConv3d(64, 64, layer.out_shape, (352, 400, 11), layer.ksize, layer.stride, layer.padding, ws, 60000)
    sb = s.serialize()
    assert len(sb) == 22 * 4 + ws.size * 4                      # sparseConv3dlayer.cu:863-866
    assert np.frombuffer(sb[:88], np.int32).tolist() == [64, 64, 60000, 64, 176, 200, 5, 352, 400, 11, 3, 3, 3,
                                                          2, 2, 2, 0, 1, 1, 1, 0, ws.size]
    assert api.SparseConv3d.deserialize(sb).serialize() == sb


def test_conv_plugins_by_name_and_their_clones():
    """createPlugin(name, fields) and clone() of the reference's plugin surface for the two conv plugins: the plugin
    built from named fields, and its clone (own device weights, epilogue and flags carried over), give the bits of the
    plugin built from the descriptor."""
    grid = (21, 200, 176)
    n, mv = 3000, 4096
    rng = np.random.default_rng(77)
    coors = F.clustered_active_voxels(n, grid, 2, n_blobs=30)
    feat = rng.uniform(-1, 1, (n, 16)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, 16, 32)).astype(np.float32)
    sc, sh = rng.uniform(0.5, 1.5, 32).astype(np.float32), rng.uniform(-0.2, 0.2, 32).astype(np.float32)
    i32 = lambda *v: np.array(v, np.int32)  # noqa: E731
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, 16), np.float32)
    fbuf[:n] = feat
    ins = (dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    # SubM
    base = api.SubmConv3d(16, 32, grid[::-1], w, mv)
    named = api.create_plugin("SubmConv3dLayerPlugin", dict(
        in_channel=i32(16), out_channel=i32(32), max_voxels=i32(mv), feature_num=i32(16), out_shape=i32(*grid[::-1]),
        spatial_shape=i32(*grid[::-1]), ksize=i32(3), stride=i32(1), padding=i32(1), dilation=i32(1), out_padding=i32(0),
        weights=w))
    assert named.serialize() == base.serialize()
    for p in (base, named):
        p.set_epilogue(sc, sh, True)
        p.set_flags(D.SESSD_FLAG_SKIP_PAD_ROWS)
    twin = named.clone()
    assert twin.serialize() == named.serialize()
    named.close()                                         # the clone owns its own copies
    outs = [to_np(p(*ins))[:n] for p in (base, twin)]
    torch.cuda.synchronize()
    assert np.array_equal(outs[0], outs[1]) and np.abs(outs[0]).max() > 0
    # SparseConv
    layer = SPARSE_LAYERS[1]
    ig = sparse_input_grid(layer)
    coors = F.clustered_active_voxels(n, (ig[0], 200, 176), 4, n_blobs=30)
    cbuf[:n] = coors
    feat = rng.uniform(-1, 1, (n, layer.cin)).astype(np.float32)
    fbuf = np.zeros((mv, layer.cin), np.float32)
    fbuf[:n] = feat
    w = rng.normal(0, 0.1, (layer.kvol, layer.cin, layer.cout)).astype(np.float32)
    ins = (dev(fbuf), dev(cbuf), dev(np.array([n], np.int32)))
    base = api.SparseConv3d(layer.cin, layer.cout, layer.out_shape, ig[::-1], layer.ksize, layer.stride, layer.padding, w, mv)
    named = api.create_plugin("SparseConv3dLayerPlugin", dict(
        in_channel=i32(layer.cin), out_channel=i32(layer.cout), max_voxels=i32(mv), feature_num=i32(layer.cin),
        out_shape=i32(*layer.out_shape), spatial_shape=i32(*ig[::-1]), ksize=i32(*layer.ksize), stride=i32(*layer.stride),
        padding=i32(*layer.padding), dilation=i32(1), out_padding=i32(0), weights=w))
    assert named.serialize() == base.serialize()
    twin = named.clone()
    a, b = base(*ins), twin(*ins)
    torch.cuda.synchronize()
    na = int(to_np(a[2])[0])
    assert na == int(to_np(b[2])[0]) > 0 and np.array_equal(to_np(a[1]), to_np(b[1]))
    assert np.array_equal(to_np(a[0])[:na], to_np(b[0])[:na])


# ---------------------------------------------------------------------------------------------
# the tall-tile FP16 kernel (3x3x3 layers from 32 channels up): tile edges and both tile heights
# ---------------------------------------------------------------------------------------------
def _fp16_subm_against_oracle(cin, cout, n, mv, grid, seed, clustered=True, epilogue=True):
    rng = np.random.default_rng(seed)
    coors = (F.clustered_active_voxels(n, grid, seed, n_blobs=max(4, n // 100)) if clustered
             else F.random_active_voxels(n, grid, seed))
    feat = O.round_to_half(rng.uniform(-1, 1, (n, cin)).astype(np.float32))
    w = O.round_to_half(rng.normal(0, 0.1, (27, cin, cout)).astype(np.float32))
    sc = rng.uniform(0.5, 1.5, cout).astype(np.float32) if epilogue else None
    sh = rng.uniform(-0.2, 0.2, cout).astype(np.float32) if epilogue else None
    conv = api.SubmConv3d(cin, cout, grid[::-1], w, mv)
    if epilogue:
        conv.set_epilogue(sc, sh, True)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n] = feat
    out = conv(dev(fbuf, torch.float16), dev(cbuf), dev(np.array([n], np.int32)), out_dtype=torch.float16)
    torch.cuda.synchronize()
    o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
    o_out = O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)
    if epilogue:
        o_out = O.scale_shift_relu(o_out, mv, sc, sh, True)
    # every row of the tensor: rows >= n are the epilogue of zero (the reference zero-fills, then BN + ReLU)
    assert_features_close(to_np(out.float()), O.round_to_half(o_out), RTOL_FP16, "tall fp16 %d->%d, %d rows" % (cin, cout, n))
    conv.close()


@pytest.mark.parametrize("cin,cout", [(32, 32), (64, 64), (128, 128)])
@pytest.mark.parametrize("n", [1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 300])
def test_tall_fp16_kernel_row_counts_around_its_tiles(cin, cout, n):
    """A tile of the tall-tile kernel is 64 rows, 16 per wave: row counts on either side of a block, a wave's
    share and a tile, down to a single row, against the oracle (pad rows included)."""
    _fp16_subm_against_oracle(cin, cout, n, 512, (5, 40, 40), 900 + n, epilogue=(n % 2 == 1))


@pytest.mark.parametrize("cin,cout,n", [(32, 32, 66000), (64, 64, 40000), (64, 128, 66000), (128, 128, 40000), (128, 128, 66000)])
def test_tall_fp16_kernel_with_two_row_blocks_per_wave(cin, cout, n):
    """Beyond 64 rows x the workgroups resident at a time, tiles at the head of the grid take two 16-row blocks per
    wave (128 rows): a launch with short and tall tiles side by side (40 000 rows) and one with tall tiles only
    (66 000 rows, the last tile partly filled), against the oracle on 16 threads."""
    O.set_threads(16)
    try:
        _fp16_subm_against_oracle(cin, cout, n, 66560, (21, 400, 352), 4000 + cin + cout)
    finally:
        O.set_threads(1)


# ---------------------------------------------------------------------------------------------
# the FP32 kernel with one tall tile per compute unit (conv_wide.hip: 64 -> 64 and 32 -> 64)
# ---------------------------------------------------------------------------------------------
def _fp32_subm_wide_against_oracle(n, mv, grid, seed, clustered=True, epilogue=True, threads=1, cin=64):
    rng = np.random.default_rng(seed)
    coors = (F.clustered_active_voxels(n, grid, seed, n_blobs=max(4, n // 100)) if clustered
             else F.random_active_voxels(n, grid, seed))
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, cin, 64)).astype(np.float32)
    sc = rng.uniform(0.5, 1.5, 64).astype(np.float32) if epilogue else None
    sh = rng.uniform(-0.2, 0.2, 64).astype(np.float32) if epilogue else None
    conv, out, pairs, num, cbuf = run_subm(coors, n, feat, w, grid, mv, sc, sh, epilogue)
    O.set_threads(threads)
    try:
        o_pairs, o_num, _ = O.subm_rulebook(coors, n, grid[::-1], mv)
        o_out = O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv)
    finally:
        O.set_threads(1)
    assert np.array_equal(num, o_num)
    if epilogue:
        o_out = O.scale_shift_relu(o_out, mv, sc, sh, True)
    # every row of the tensor: rows >= n are the epilogue of zero (the reference zero-fills, then BN + ReLU)
    assert_features_close(out, o_out, RTOL_FP32, "wide fp32 %d->64, %d rows" % (cin, n),
                          abs_sum=abs_sum_of(feat, w, o_pairs, o_num, mv, mv, sc, sh))
    assert conv.status() == 0
    conv.close()


@pytest.mark.parametrize("cin", [64, 32])
@pytest.mark.parametrize("n", [1, 15, 16, 17, 63, 64, 65, 95, 96, 97, 255, 256, 257, 1000])
def test_wide_fp32_kernel_row_counts_around_its_tiles(n, cin):
    """One workgroup per compute unit walks tiles of up to 96 rows whose neighbour lists are staged in two halves
    of 64 rows: row counts on either side of a 16-pair block, the staging halves, the tile capacity and the number
    of compute units (256 rows: one row per tile), against the oracle (pad rows included)."""
    _fp32_subm_wide_against_oracle(n, n + 200, (5, 40, 40), 700 + n, epilogue=(n % 2 == 1), cin=cin)


@pytest.mark.parametrize("n,clustered,cin", [(20000, True, 64), (20000, True, 32), (24577, False, 64), (50000, True, 64)])
def test_wide_fp32_kernel_tall_tiles_and_two_tiles_per_workgroup(n, clustered, cin):
    """~78-row tiles (20 000 rows: both staging halves in use), the first row count past one 96-row tile per
    compute unit (24 577 rows of scattered voxels: every workgroup walks two tiles), and 50 000 clustered rows
    (tiles of uneven length from the equal-work cuts, two or three per workgroup), against the oracle on 16
    threads."""
    _fp32_subm_wide_against_oracle(n, 51200, (21, 400, 352), 5000 + n, clustered=clustered, threads=16, cin=cin)
