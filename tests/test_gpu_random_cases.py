"""Seeded random cases, GPU against the oracle: layer shapes, grids, kernel / stride / padding triples, row counts
around the tile and wave sizes, capacities that bind, and random layer stacks through the pipeline.  The fixed
cases of the other files follow the reference's network; these look for what nobody thought of."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import RTOL_FP16, RTOL_FP32, abs_sum_of, assert_end_to_end_close, assert_features_close, dev, points_input, to_np
from sessd3d import api, backbone as B, ctypes_defs as D, frames as F

pytestmark = pytest.mark.gpu

SHAPES = [(4, 16), (4, 32), (16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128), (8, 24), (24, 8),
          (3, 5)]
ROW_COUNTS = [1, 15, 16, 17, 47, 48, 49, 63, 64, 65, 255, 256, 257, 12287, 12288, 12289, 16383, 16385]


@pytest.mark.parametrize("seed", range(30))
def test_random_subm_layer(seed):
    rng = np.random.default_rng(1000 + seed)
    cin, cout = SHAPES[rng.integers(len(SHAPES))]
    half = bool(rng.integers(2)) and cin not in (3, 8, 24)
    grid = (int(rng.integers(1, 12)), int(rng.integers(4, 120)), int(rng.integers(4, 120)))
    cells = grid[0] * grid[1] * grid[2]
    n = int(ROW_COUNTS[rng.integers(len(ROW_COUNTS))]) if rng.integers(3) == 0 else int(rng.integers(1, 20000))
    n = max(1, min(n, cells * 3 // 4))
    mv = n + int(rng.integers(0, 300))
    clustered = bool(rng.integers(2)) and n < cells // 4
    coors = (F.clustered_active_voxels(n, grid, seed, n_blobs=max(2, n // 100)) if clustered
             else F.random_active_voxels(n, grid, seed))
    feat = rng.uniform(-1, 1, (n, cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (27, cin, cout)).astype(np.float32)
    in_half = half and cin != 4                      # a 4-channel layer reads the voxelizer's FP32 means
    if half:
        w = O.round_to_half(w)
        if in_half:
            feat = O.round_to_half(feat)
    sc = rng.uniform(0.5, 1.5, cout).astype(np.float32)
    sh = rng.uniform(-0.2, 0.2, cout).astype(np.float32)
    relu = bool(rng.integers(2))
    conv = api.SubmConv3d(cin, cout, grid[::-1], w, mv)
    conv.set_epilogue(sc, sh, relu)
    if rng.integers(2):
        conv.set_flags(D.SESSD_FLAG_SKIP_PAD_ROWS)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n] = feat
    out = conv(dev(fbuf, torch.float16 if in_half else torch.float32), dev(cbuf), dev(np.array([n], np.int32)),
               out_dtype=torch.float16 if half else torch.float32)
    pairs, num = conv.export_rulebook()
    torch.cuda.synchronize()
    o_pairs, o_num, o_st = O.subm_rulebook(coors, n, grid[::-1], mv)
    o_out = O.scale_shift_relu(O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), mv, sc, sh, relu)
    what = "subm %d->%d %s n=%d grid=%s" % (cin, cout, "fp16" if half else "fp32", n, grid)
    assert conv.status() == o_st, what
    assert np.array_equal(to_np(num).astype(np.uint32), o_num), what
    terms = abs_sum_of(feat, w, o_pairs, o_num, mv, mv, sc, sh)[:n]
    if half:
        assert_features_close(to_np(out.float())[:n], O.round_to_half(o_out)[:n], RTOL_FP16, what, abs_sum=terms, half=True)
    else:
        assert_features_close(to_np(out)[:n], o_out[:n], RTOL_FP32, what, abs_sum=terms)


@pytest.mark.parametrize("seed", range(30))
def test_random_strided_layer(seed):
    rng = np.random.default_rng(2000 + seed)
    while True:
        k = tuple(int(v) for v in rng.integers(1, 4, 3))
        s = tuple(int(v) for v in rng.integers(1, 4, 3))
        p = tuple(int(min(v, kk - 1)) for v, kk in zip(rng.integers(0, 2, 3), k))
        ig = (int(rng.integers(3, 12)), int(rng.integers(6, 60)), int(rng.integers(6, 60)))
        og = tuple(B.conv_out_size(ig[a], k[a], s[a], p[a]) for a in range(3))
        if min(og) >= 1:
            break
    cin, cout = [(16, 32), (32, 64), (64, 64), (8, 16), (4, 16)][rng.integers(5)]
    n = int(rng.integers(1, max(2, ig[0] * ig[1] * ig[2] // 2)))
    mv = int(rng.integers(max(1, n // 2), 4 * n + 64))           # may bind on the input or the output side
    n_in = min(n, mv)
    layer = B.Layer("t", D.SESSD_LAYER_SPARSE, cin, cout, og[::-1], k, s, p)
    coors = F.random_active_voxels(n, ig, seed)[:n_in]
    feat = rng.uniform(-1, 1, (n_in, cin)).astype(np.float32)
    w = rng.normal(0, 0.1, (layer.kvol, cin, cout)).astype(np.float32)
    conv = api.SparseConv3d(cin, cout, layer.out_shape, ig[::-1], k, s, p, w, mv)
    cbuf = np.zeros((mv, 4), np.int32)
    cbuf[:n_in] = coors
    fbuf = np.zeros((mv, cin), np.float32)
    fbuf[:n_in] = feat
    out, oc, on = conv(dev(fbuf), dev(cbuf), dev(np.array([n_in], np.int32)))
    pairs, num = conv.export_rulebook()
    torch.cuda.synchronize()
    o_pairs, o_num, o_oc, o_on, o_st = O.sparse_rulebook(coors, n_in, og[::-1], k, s, p, mv)
    what = "strided k=%s s=%s p=%s in=%s %d->%d n=%d mv=%d" % (k, s, p, ig, cin, cout, n_in, mv)
    assert int(to_np(on)[0]) == o_on and conv.status() == o_st, what
    assert np.array_equal(to_np(oc), o_oc) and np.array_equal(to_np(num).astype(np.uint32), o_num), what
    assert_features_close(to_np(out), O.gather_gemm_scatter(feat, w, o_pairs, o_num, mv), RTOL_FP32, what,
                          abs_sum=abs_sum_of(feat, w, o_pairs, o_num, mv))


def random_stack(rng):
    """A random stack in the reference's style: SubM runs (kernel 3 or 1) between strided layers, on the
    voxelizer's grid.  -> layers, last grid (z,y,x), last channel count"""
    S, P = D.SESSD_LAYER_SUBM, D.SESSD_LAYER_SPARSE
    grid, c, layers = (41, 1600, 1408), 4, []
    for st in range(int(rng.integers(3, 6))):
        for j in range(int(rng.integers(0, 4))):
            co = c if (rng.integers(2) and c != 4) else int(rng.choice([16, 32, 64, 128, 8, 24]))
            k = 3 if rng.integers(4) else 1
            layers.append(B.Layer("subm%d_%d" % (st, j), S, c, co, grid[::-1], (k, k, k), (1, 1, 1), ((k - 1) // 2,) * 3))
            c = co
        k, s, p = ((3, 1, 1), (2, 1, 1), (0, 0, 0)) if rng.integers(3) == 0 else ((3, 3, 3), (2, 2, 2), (int(rng.integers(2)), 1, 1))
        og = tuple(B.conv_out_size(grid[a], k[a], s[a], p[a]) for a in range(3))
        if min(og) < 1:
            break
        co = int(rng.choice([16, 32, 64, 128, 8, 24]))
        layers.append(B.Layer("sparse%d" % st, P, c, co, og[::-1], k, s, p))
        c, grid = co, og
    return layers, grid, c


@pytest.mark.parametrize("seed", range(16))
def test_random_layer_stack_through_the_pipeline(seed):
    rng = np.random.default_rng(3000 + seed)
    while True:
        layers, grid, c = random_stack(rng)
        if layers and c * grid[0] * grid[1] * grid[2] <= 40_000_000:     # keep the dense tensor small
            break
    half, graph, share, skip = (bool(rng.integers(2)) for _ in range(4))
    overlap = graph or bool(rng.integers(2))
    npts = int(rng.integers(1, 5000))
    mv = int(rng.integers(max(64, npts // 4), 3 * npts + 4096))           # one capacity for every tensor; may bind
    W = B.random_weights(layers, seed=seed, w_std=0.05)
    if half:
        W = B.Weights([O.round_to_half(w) for w in W.w], W.scale, W.shift)
    pts = F.lidar_frame(npts, seed)
    dsize = (grid[2], grid[1], grid[0])
    pad = (1, 1, 1, 1) if rng.integers(2) else (0, 0, 0, 0)
    pipe = api.Pipeline(layers, W, npts, mv, feature_dtype="fp16" if half else "fp32", share_rulebooks=share,
                        skip_pad_rows=skip, use_graph=graph, overlap_streams=overlap, dense_size_xyz=dsize,
                        dense_padding=pad)
    p, n = points_input(pts, npts)
    dense, stream = pipe.new_dense(), torch.cuda.Stream()
    for _ in range(2):
        with torch.cuda.stream(stream):
            pipe.enqueue(p, n, dense, stream)
        stream.synchronize()
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=mv), layers, W, B.dense_desc(dsize, c), round_half=half)
    want = np.pad(ref["dense"], ((0, 0), (1, 1), (1, 1))) if any(pad) else ref["dense"]
    what = "%s graph=%s overlap=%s share=%s: %s" % ("fp16" if half else "fp32", graph, overlap, share,
                                                   [(l.name, l.cin, l.cout) for l in layers])
    assert pipe.status() == ref["status"], what
    assert [pipe.layer_count(l) for l in range(-1, len(layers))] == list(ref["counts"]), what
    assert np.array_equal(pipe.read_layer(len(layers) - 1)[1], ref["coors"]), what
    assert_end_to_end_close(to_np(dense).astype(np.float32), want, half, what)
    pipe.close()
