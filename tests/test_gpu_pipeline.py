"""GPU parity of the whole frame pipeline (voxelGenerator -> 14 conv layers with folded BN + ReLU ->
sparse2Dense) against oracle_frame, plus size-independent properties at the full benchmark size."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import (RTOL_FP16, RTOL_FP32, assert_end_to_end_close, assert_features_close, canonical, layer_abs_sum,
                      points_input, to_np)
from sessd3d import api, backbone as B, ctypes_defs as D, frames as F

pytestmark = pytest.mark.gpu


def run_pipeline(pts, layers, W, max_points, max_voxels, **kw):
    pipe = api.Pipeline(layers, W, max_points, max_voxels, **kw)
    p, n = points_input(pts, max_points)
    dense = pipe.new_dense()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        pipe.enqueue(p, n, dense, stream)
    stream.synchronize()
    return pipe, dense, (p, n, stream)


def compare_with_oracle(pipe, dense, pts, layers, W, max_voxels, rtol_layer):
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=max_voxels), layers, W, B.dense_desc())
    feat, coors, n = pipe.read_layer(-1)
    assert n == ref["counts"][0]
    for l, layer in enumerate(layers):
        fbuf = np.zeros((max_voxels, layer.cin), np.float32)
        fbuf[:n] = feat
        cbuf = np.zeros((max_voxels, 4), np.int32)
        cbuf[:n] = coors
        o_out, o_coors, o_n, _, _ = O.conv_layer(fbuf, cbuf, n, layer, W.w[l], W.scale[l], W.shift[l], max_voxels)
        terms = layer_abs_sum(fbuf, cbuf, n, layer, W.w[l], W.scale[l], W.shift[l], max_voxels)
        feat, g_coors, g_n = pipe.read_layer(l)
        assert g_n == o_n == ref["counts"][l + 1], layer.name
        assert np.array_equal(g_coors, o_coors[:o_n]), layer.name          # same numbering, row by row
        assert_features_close(feat, o_out[:o_n], rtol_layer, layer.name, abs_sum=terms[:o_n])
        coors, n = g_coors, g_n
    assert np.array_equal(coors, ref["coors"])
    a, b = canonical(coors, n, feat), canonical(ref["coors"], n, ref["feat"])
    assert np.array_equal(a[0], b[0])
    assert_end_to_end_close(a[1], b[1], False, "last layer features (end to end)")
    assert_end_to_end_close(to_np(dense).astype(np.float32), ref["dense"], False, "dense BEV tensor (end to end)")
    # the dense tensor is an exact scatter of the last layer's rows
    assert np.array_equal(to_np(dense).astype(np.float32), O.sparse2dense(feat, coors, n, B.DENSE_SIZE_XYZ))
    assert pipe.status() == ref["status"]
    return ref


@pytest.mark.parametrize("share,skip_pad", [(True, True), (False, False)])
def test_full_backbone_small_frame(share, skip_pad):
    pts = F.lidar_frame(5000, 11)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=5, w_std=0.05)
    pipe, dense, _ = run_pipeline(pts, layers, W, 8192, 16384, share_rulebooks=share, skip_pad_rows=skip_pad)
    compare_with_oracle(pipe, dense, pts, layers, W, 16384, RTOL_FP32)


@pytest.mark.parametrize("overlap", [False, True])
def test_pipeline_writes_the_zero_padded_dense_tensor(overlap):
    """dense_padding = the reference's ZeroPad2dPlugin (params.h:200-203: 1,1,1,1) folded into the last scatter:
    the padded tensor must equal the oracle's sparse2dense -> zero_pad2d of the same rows, and its interior
    the unpadded pipeline's output, bit for bit."""
    pts = F.lidar_frame(4000, 21)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=6, w_std=0.05)
    kw = dict(share_rulebooks=True, skip_pad_rows=True, overlap_streams=overlap, use_graph=overlap)
    plain, dense, _ = run_pipeline(pts, layers, W, 4096, 16384, **kw)
    pad = (1, 1, 1, 1)
    pipe, padded, (p, n, stream) = run_pipeline(pts, layers, W, 4096, 16384, dense_padding=pad, **kw)
    assert tuple(padded.shape) == (128, 202, 178)
    feat, coors, m = pipe.read_layer(len(layers) - 1)
    want = O.zero_pad2d(O.sparse2dense(feat, coors, m, B.DENSE_SIZE_XYZ), *pad)
    assert np.array_equal(to_np(padded), want)
    assert np.array_equal(to_np(padded)[:, 1:-1, 1:-1], to_np(dense))
    # a second enqueue into a dirty buffer restores the zero border
    padded.fill_(7.0)
    with torch.cuda.stream(stream):
        pipe.enqueue(p, n, padded, stream)
    stream.synchronize()
    assert np.array_equal(to_np(padded), want)


def test_capacity_binds_in_the_voxelizer_and_in_a_strided_layer():
    """One capacity for every tensor (as in the reference), small enough that the voxelizer drops cells and the
    first strided layer drops output sites.  The overlapped schedule -- where SubM layers probe the cell table
    the voxelizer / strided layer left behind, dropped cells included -- must agree with the single-stream run
    bit for bit, and both with the oracle."""
    pts = F.lidar_frame(6000, 13)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=9, w_std=0.05)
    cap = 3000
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=cap), layers, W, B.dense_desc())
    assert ref["status"] & D.SESSD_STATUS_VOXEL_OVERFLOW and ref["counts"][0] == cap and ref["counts"][3] == cap
    plain, dense, _ = run_pipeline(pts, layers, W, 6000, cap, share_rulebooks=True, skip_pad_rows=True)
    fast, fdense, (p, n, stream) = run_pipeline(pts, layers, W, 6000, cap, share_rulebooks=True, skip_pad_rows=True,
                                                overlap_streams=True, use_graph=True)
    with torch.cuda.stream(stream):
        fast.enqueue(p, n, fdense, stream)                      # a replay of the captured graph
    stream.synchronize()
    assert np.array_equal(to_np(fdense), to_np(dense))
    for pipe in (plain, fast):
        assert pipe.status() == ref["status"]
        assert [pipe.layer_count(l) for l in range(-1, len(layers))] == list(ref["counts"])
        feat, coors, cnt = pipe.read_layer(len(layers) - 1)
        assert np.array_equal(coors, ref["coors"])
        assert_end_to_end_close(feat, ref["feat"], False, "last layer features with binding capacities")
    assert_end_to_end_close(to_np(dense), ref["dense"], False, "dense tensor with binding capacities")


def test_overlapped_graph_schedule_with_reference_pad_rows():
    """Reference behaviour for rows past the active count (every output tensor is zero-filled, then BN + ReLU
    runs over all rows: rows >= n hold relu(shift)) under the overlapped schedule and its captured graph: dense
    tensor, active rows and pad rows must equal the single-stream run bit for bit, frame after frame."""
    pts = F.lidar_frame(3000, 17)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=12, w_std=0.05)
    mv = 8192
    plain, dense, _ = run_pipeline(pts, layers, W, 4096, mv, share_rulebooks=True, skip_pad_rows=False)
    fast, fdense, (p, n, stream) = run_pipeline(pts, layers, W, 4096, mv, share_rulebooks=True, skip_pad_rows=False,
                                                overlap_streams=True, use_graph=True)
    for _ in range(2):                                               # graph replays
        with torch.cuda.stream(stream):
            fast.enqueue(p, n, fdense, stream)
        stream.synchronize()
        assert np.array_equal(to_np(fdense), to_np(dense))
    assert fast.status() == plain.status() == 0
    for l in (0, 5, len(layers) - 1):
        rows = []
        for pipe in (plain, fast):
            f, _, _, _, ch = pipe.layer_io(l)
            full = np.zeros((mv, ch), np.float32)
            api._hip_d2h(full, f)
            rows.append((full, 0))
        assert np.array_equal(rows[0][0], rows[1][0]), layers[l].name
        cnt = plain.layer_count(l)
        want_pad = np.maximum(W.shift[l], 0.0).astype(np.float32)    # relu(0 * scale + shift)
        assert np.array_equal(rows[0][0][cnt:], np.broadcast_to(want_pad, (mv - cnt, len(want_pad)))), layers[l].name


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_tiny_frames_through_the_pipeline(dtype):
    """Frames of 0, 1, 7, 40 and 150 points through one pipeline (overlapped schedule, captured graph): the wide
    layers then see far fewer rows than they have tiles.  Site counts exact, dense tensor against the oracle."""
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=3, w_std=0.05)
    half = dtype == "fp16"
    if half:
        W = half_weights(W)
    mp, mv = 1024, 4096
    pipe = api.Pipeline(layers, W, mp, mv, feature_dtype=dtype, share_rulebooks=True, skip_pad_rows=True,
                        use_graph=True, overlap_streams=True)
    p, n = points_input(np.zeros((0, 4), np.float32), mp)
    dense, stream = pipe.new_dense(), torch.cuda.Stream()
    for npts in (150, 0, 1, 40, 7):
        pts = F.lidar_frame(npts, 100 + npts) if npts else np.zeros((0, 4), np.float32)
        hp, hn = points_input(pts, mp)
        with torch.cuda.stream(stream):
            p.copy_(hp)
            n.copy_(hn)
            pipe.enqueue(p, n, dense, stream)
        stream.synchronize()
        ref = O.frame(pts, B.voxelgen_desc(max_voxels=mv), layers, W, B.dense_desc(), round_half=half)
        assert pipe.status() == ref["status"] == 0
        for l in range(-1, len(layers)):
            assert pipe.layer_count(l) == ref["counts"][l + 1], (npts, l)
        assert_end_to_end_close(to_np(dense).astype(np.float32), ref["dense"], half, "dense, %d points" % npts)


def test_full_backbone_config3_frame_and_graph_replay():
    """Benchmark configuration 3: the 20 000-point frame (~17 k voxels) through the reference's 14 conv layers.
    The eager enqueue and repeated replays of the captured graph must give identical bits."""
    pts = F.lidar_frame(20000, 0)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=1, w_std=0.05)
    pipe, dense, _ = run_pipeline(pts, layers, W, 20000, 60000, share_rulebooks=True, skip_pad_rows=True)
    ref = compare_with_oracle(pipe, dense, pts, layers, W, 60000, RTOL_FP32)
    assert 15000 < ref["counts"][0] < 19000
    eager = to_np(dense).copy()

    # two-stream schedule, eager: same bits as the single-stream run
    opipe, odense, _ = run_pipeline(pts, layers, W, 20000, 60000, share_rulebooks=True, skip_pad_rows=True,
                                    overlap_streams=True)
    assert np.array_equal(to_np(odense), eager), "two-stream schedule differs from the single-stream result"
    assert opipe.status() == 0

    gpipe = api.Pipeline(layers, W, 20000, 60000, share_rulebooks=True, skip_pad_rows=True, use_graph=True,
                         overlap_streams=True)
    p, n = points_input(pts, 20000)
    gd = gpipe.new_dense()
    stream = torch.cuda.Stream()
    for rep in range(3):
        gd.fill_(float(rep + 1))                        # eager work between replays
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            gpipe.enqueue(p, n, gd, stream)
        stream.synchronize()
        assert np.array_equal(to_np(gd), eager), "graph replay %d differs from the eager result" % rep
    assert gpipe.num_launches() > 0
    # a different frame in the same buffers: the replayed graph reads the new data
    pts2 = F.lidar_frame(18000, 1)
    p2, n2 = points_input(pts2, 20000)
    p.copy_(p2)
    n.copy_(n2)
    with torch.cuda.stream(stream):
        gpipe.enqueue(p, n, gd, stream)
    stream.synchronize()
    ref2 = O.frame(pts2, B.voxelgen_desc(max_voxels=60000), layers, W, B.dense_desc())
    assert_end_to_end_close(to_np(gd), ref2["dense"], False, "graph replay on a new frame")


def half_weights(W):
    """The FP16 configurations store weights in half: round once, hand the same values to both sides."""
    return B.Weights([O.round_to_half(w) for w in W.w], W.scale, W.shift)


def test_fp16_backbone_against_half_rounding_oracle():
    """FP16 features/weights with FP32 accumulate through all 14 layers.  The oracle keeps FP32 arithmetic
    but rounds every layer's output to half, as the FP16 pipeline stores it.  Sites are bit-exact; features
    within 1e-2 relative per layer (oracle fed the GPU's rows) and end to end."""
    pts = F.lidar_frame(12000, 21)
    layers = B.reference_layers()
    W = half_weights(B.random_weights(layers, seed=9, w_std=0.05))
    mv = 40000
    pipe, dense, _ = run_pipeline(pts, layers, W, 12000, mv, feature_dtype="fp16", share_rulebooks=True,
                                  skip_pad_rows=True, overlap_streams=True)
    assert dense.dtype == torch.float16
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=mv), layers, W, B.dense_desc(), round_half=True)
    feat, coors, n = pipe.read_layer(-1)
    for l, layer in enumerate(layers):
        fbuf = np.zeros((mv, layer.cin), np.float32)
        fbuf[:n] = feat
        cbuf = np.zeros((mv, 4), np.int32)
        cbuf[:n] = coors
        o_out, o_coors, o_n, _, _ = O.conv_layer(fbuf, cbuf, n, layer, W.w[l], W.scale[l], W.shift[l], mv)
        terms = layer_abs_sum(fbuf, cbuf, n, layer, W.w[l], W.scale[l], W.shift[l], mv)
        feat, g_coors, g_n = pipe.read_layer(l)
        assert g_n == o_n == ref["counts"][l + 1] and np.array_equal(g_coors, o_coors[:o_n]), layer.name
        assert_features_close(feat, O.round_to_half(o_out[:o_n]), RTOL_FP16, "fp16 " + layer.name, abs_sum=terms[:o_n], half=True)
        coors, n = g_coors, g_n
    assert np.array_equal(coors, ref["coors"])
    # end to end a half-rounding that falls the other way in an early layer is carried on by the layers after
    # it (gpu_util.END_TO_END_RMS / END_TO_END_MAX say how far, measured); in the L2 norm the error must stay within 1e-2
    assert_end_to_end_close(feat, ref["feat"], True, "fp16 last layer (end to end)")
    d = to_np(dense.float())
    assert_end_to_end_close(d, ref["dense"], True, "fp16 dense (end to end)")
    assert np.linalg.norm(d - ref["dense"]) <= RTOL_FP16 * np.linalg.norm(ref["dense"])
    assert pipe.status() == ref["status"]


def test_properties_at_full_size():
    """Size-independent checks on a frame too large to push through the CPU oracle quickly:
    determinism, active-site bookkeeping and dense/sparse consistency."""
    pts = F.lidar_frame(60000, 7)
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=2, w_std=0.05)
    pipe, dense, (p, n, stream) = run_pipeline(pts, layers, W, 60000, 60000, skip_pad_rows=True)
    first = to_np(dense).copy()
    with torch.cuda.stream(stream):
        pipe.enqueue(p, n, dense, stream)
    stream.synchronize()
    assert np.array_equal(to_np(dense), first)                     # run-to-run bit identical
    feat, coors, cnt = pipe.read_layer(len(layers) - 1)
    assert len(np.unique(coors[:, 1:] @ np.array([200 * 176, 176, 1]))) == cnt     # unique sites
    assert coors[:, 1].max() < 2 and coors[:, 2].max() < 200 and coors[:, 3].max() < 176 and coors.min() >= 0
    back = first.reshape(64, 2, 200, 176)[:, coors[:, 1], coors[:, 2], coors[:, 3]].T
    assert np.array_equal(back, feat)                               # dense holds exactly the sparse rows
    assert np.count_nonzero(first) == np.count_nonzero(feat)
    # voxelizer output is independent of everything downstream: compare with the oracle's voxelizer
    vfeat, vcoors, vn = pipe.read_layer(-1)
    o = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, 60000)
    assert vn == o[2] and np.array_equal(vcoors, o[1][:vn]) and np.array_equal(vfeat.view(np.uint32), o[0][:vn].view(np.uint32))


def test_stress_configuration_properties():
    """Benchmark configuration 5: 150 000 points over 360 degrees (cropped to range), voxel cap 60 000, doubled
    channel widths, FP16 features.  Too heavy for the scalar oracle's conv layers, so: the voxelizer part
    is compared with the oracle exactly (the cap binds -> overflow flag), the rest through properties."""
    pts = F.lidar_frame(150000, 5, full_circle=True)
    layers = B.reference_layers(width_mult=2)
    W = half_weights(B.random_weights(layers, seed=4, w_std=0.03))
    pipe, dense, (p, n, stream) = run_pipeline(pts, layers, W, 150000, 200000, feature_dtype="fp16",
                                               skip_pad_rows=True, overlap_streams=True, use_graph=True,
                                               voxel_cap=60000)
    assert tuple(dense.shape) == (256, 200, 176)
    first = to_np(dense).copy()
    for _ in range(2):                                               # graph replays are bit identical
        with torch.cuda.stream(stream):
            pipe.enqueue(p, n, dense, stream)
        stream.synchronize()
        assert np.array_equal(to_np(dense), first)
    vfeat, vcoors, vn = pipe.read_layer(-1)
    o = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, 60000)
    assert vn == o[2] == 60000 and o[4] & D.SESSD_STATUS_VOXEL_OVERFLOW
    assert np.array_equal(vcoors, o[1][:vn]) and np.array_equal(vfeat.view(np.uint32), o[0][:vn].view(np.uint32))
    assert pipe.status() & D.SESSD_STATUS_VOXEL_OVERFLOW
    counts = [pipe.layer_stats(l)[0] for l in range(len(layers))]
    assert counts[0] == counts[1] == 60000 and max(counts) <= 200000
    assert counts[2] > 60000                                         # the first strided layer grows the set
    feat, coors, cnt = pipe.read_layer(len(layers) - 1)
    assert cnt == counts[-1] and len(np.unique(coors[:, 1:] @ np.array([200 * 176, 176, 1]))) == cnt
    back = first.reshape(128, 2, 200, 176)[:, coors[:, 1], coors[:, 2], coors[:, 3]].T
    assert np.array_equal(back.astype(np.float32), feat)
    assert np.isfinite(first.astype(np.float32)).all()


def test_frames_in_flight_give_the_bits_of_one_frame_at_a_time():
    """frames_in_flight = 3: three replicas of the pipeline, successive frames on successive replicas (submit / join).
    A sequence of DIFFERENT frames, submitted ahead of their joins, must give exactly the dense tensors, statuses and
    layer counts of the one-frame-at-a-time pipeline; enqueue() on the same object is submit + join."""
    layers = B.reference_layers()
    W = B.random_weights(layers, seed=8, w_std=0.05)
    mp, mv, R = 8192, 16384, 3
    kw = dict(share_rulebooks=True, skip_pad_rows=True, use_graph=True, overlap_streams=True)
    one = api.Pipeline(layers, W, mp, mv, **kw)
    many = api.Pipeline(layers, W, mp, mv, frames_in_flight=R, **kw)
    frames = [F.lidar_frame(npts, 40 + i) for i, npts in enumerate((6000, 2500, 8000, 50, 7000, 3000, 6500))]
    stream = torch.cuda.Stream()
    want, counts = [], []
    p, n = points_input(frames[0], mp)
    dense = one.new_dense()
    for pts in frames:
        hp, hn = points_input(pts, mp)
        with torch.cuda.stream(stream):
            p.copy_(hp)
            n.copy_(hn)
            one.enqueue(p, n, dense, stream)
        stream.synchronize()
        want.append(to_np(dense).copy())
        counts.append([one.layer_count(l) for l in range(-1, len(layers))])
    # every frame in flight has its own input and output buffers (they must stay untouched until its join)
    ins = [points_input(pts, mp) for pts in frames]
    outs = [many.new_dense() for _ in frames]
    tickets = []
    with torch.cuda.stream(stream):
        for i in range(len(frames)):
            tickets.append(many.submit(ins[i][0], ins[i][1], outs[i], stream))
            if i >= R - 1:
                many.join(tickets[i - (R - 1)], stream)
        for t in tickets[-(R - 1):]:
            many.join(t, stream)
    stream.synchronize()
    assert tickets == list(range(len(frames)))
    for i in range(len(frames)):
        assert np.array_equal(to_np(outs[i]), want[i]), "frame %d differs with frames in flight" % i
    assert [many.layer_count(l) for l in range(-1, len(layers))] == counts[-1]        # queries: the frame submitted last
    assert many.status() == one.status() == 0 and many.num_launches() == one.num_launches()
    # enqueue = submit + join, again and again into the same buffers
    for rep in range(4):
        outs[0].fill_(3.0)
        with torch.cuda.stream(stream):
            many.enqueue(ins[2][0], ins[2][1], outs[0], stream)
        stream.synchronize()
        assert np.array_equal(to_np(outs[0]), want[2]), rep
    # host-driven loop: the inputs are resident (synchronised above), nothing is ordered after a stream, the host
    # blocks on the oldest frame in flight
    for o in outs:
        o.fill_(5.0)
    torch.cuda.synchronize()
    tickets = []
    for i in range(len(frames)):
        tickets.append(many.submit(ins[i][0], ins[i][1], outs[i], api.STREAM_NONE))
        if i >= R - 1:
            many.wait(tickets[i - (R - 1)])
            j = i - (R - 1)
            assert np.array_equal(to_np(outs[j]), want[j]), "frame %d differs after a host-side wait" % j
    for t in tickets[-(R - 1):]:
        many.wait(t)
    for i in range(len(frames)):
        assert np.array_equal(to_np(outs[i]), want[i]), i
    with pytest.raises(api.SessdError, match="no frame with ticket"):
        many.join(10 ** 6, stream)
    with pytest.raises(api.SessdError, match="no frame with ticket"):
        many.wait(10 ** 6)
    with pytest.raises(api.SessdError, match="STREAM_NONE needs frames_in_flight"):
        one.submit(p, n, dense, api.STREAM_NONE)
    with pytest.raises(api.SessdError, match="runs its frames on the caller's stream"):
        one.wait(one.submit(p, n, dense, stream))
    stream.synchronize()


def test_fp16_stack_ending_in_a_3x3x3_layer_scatters_from_the_tall_tile_kernel():
    """A stack whose LAST layer is a 3x3x3 FP16 layer of 32+ channels: in the overlapped schedule that layer's
    kernel (the tall-tile one) also writes the dense tensor.  Dense tensor, sites and status against the oracle,
    and equal to the single-stream schedule's separate scatter bit for bit."""
    S, P = D.SESSD_LAYER_SUBM, D.SESSD_LAYER_SPARSE
    layers = [B.Layer("subm0", S, 4, 32, (1408, 1600, 41), (3, 3, 3), (1, 1, 1), (1, 1, 1)),
              B.Layer("sparse1", P, 32, 64, (704, 800, 21), (3, 3, 3), (2, 2, 2), (1, 1, 1)),
              B.Layer("sparse2", P, 64, 64, (352, 400, 11), (3, 3, 3), (2, 2, 2), (1, 1, 1)),
              B.Layer("sparse3", P, 64, 32, (176, 200, 5), (3, 3, 3), (2, 2, 2), (0, 1, 1)),
              B.Layer("subm4", S, 32, 32, (176, 200, 5), (3, 3, 3), (1, 1, 1), (1, 1, 1))]
    W = half_weights(B.random_weights(layers, seed=12, w_std=0.08))
    pts = F.lidar_frame(9000, 33)
    mv = 16384
    dsize = (176, 200, 5)
    kw = dict(feature_dtype="fp16", share_rulebooks=True, skip_pad_rows=True, dense_size_xyz=dsize, dense_padding=(1, 1, 1, 1))
    fused, d_fused, _ = run_pipeline(pts, layers, W, 9000, mv, use_graph=True, overlap_streams=True, **kw)
    plain, d_plain, _ = run_pipeline(pts, layers, W, 9000, mv, use_graph=False, overlap_streams=False, **kw)
    ref = O.frame(pts, B.voxelgen_desc(max_voxels=mv), layers, W, B.dense_desc(dsize, 32), round_half=True)
    want = np.pad(ref["dense"], ((0, 0), (1, 1), (1, 1)))
    assert fused.status() == plain.status() == ref["status"] == 0
    assert [fused.layer_count(l) for l in range(-1, len(layers))] == list(ref["counts"])
    assert np.array_equal(fused.read_layer(len(layers) - 1)[1], ref["coors"])
    assert_end_to_end_close(to_np(d_fused).astype(np.float32), want, True, "dense from the tall-tile kernel")
    assert torch.equal(d_fused, d_plain)
