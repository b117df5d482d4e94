"""Helpers for the GPU parity tests: device upload, canonical comparisons, tolerances."""
import numpy as np
import torch

import oracle_lib as O

DEV = "cuda:0"

# Per layer, FP32 features: |gpu - oracle| <= 1e-4 * max(|oracle|, floor), FP16: 1e-2, the floor being 1e-3 of the
# tensor's largest magnitude.  An element that is small because its terms cancel cannot meet a bound relative to
# itself, in any arithmetic: the two sides add the same FP32 products in different orders, and the error of a sum
# of n terms is bounded by n * u * A, A = sum of |terms|, u = 2^-24, and behaves like sqrt(n) * u * A.  Such an
# element is admitted when it is within SUM_TOL * A plus the rounding of the stored value (2 ulp: the sides may
# round to neighbouring values) -- a bound from the sum's own terms, not a fraction of some other element.
# SUM_TOL = 2e-6: n <= 27 * 128 terms give sqrt(n) * u = 3.5e-6 per side if every addition rounded independently;
# the matrix cores add 4 (FP32) or 32 (FP16) products per instruction and the largest |gpu - oracle| / A seen,
# beyond the stored value's own rounding, is 3.2e-7 in FP32 and 5e-8 in FP16 over this suite and the benchmark
# configurations (pytest prints the session's figures at the end, bench.py those of its frames).  The benchmark
# configurations pass on the floor criterion alone; the sum bound admits at most 1.2e-4 of a tensor's elements, in
# the unit tests whose inputs are centred on zero.
RTOL_FP32 = 1e-4
RTOL_FP16 = 1e-2
FLOOR_FRACTION = 1e-3
SUM_TOL = 2e-6
# End to end the rounding differences of 14 stacked layers compound, and in FP16 a value near a rounding boundary
# falls to different sides in the two chains; the layers after it carry the difference on.  An FP64 recomputation
# of the frame (check_frame_against_oracle, run at the benchmark configurations in test_gpu_configs.py) puts both
# chains 2.0e-8 (FP32) and 2.3e-5 .. 2.9e-5 (FP16) of the last tensor's largest magnitude from the exact result in
# RMS, and their largest element-wise difference at 7.9e-7 (FP32) and 9.3e-4 (FP16: two units in the last place of
# a half near the top of the range) of it.  The whole-frame comparison is therefore stated in those terms: RMS
# difference and largest difference, both relative to the tensor's largest magnitude, each with about fourfold
# room over what was measured.
END_TO_END_RMS = {False: 1e-7, True: 1.5e-4}
END_TO_END_MAX = {False: 4e-6, True: 8 * 2.0 ** -11}


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def points_input(pts, max_points):
    """-> points tensor [max_points,F] (zero padded, as the reference's loader does) and size tensor."""
    buf = np.zeros((max_points, pts.shape[1]), np.float32)
    n = min(len(pts), max_points)
    buf[:n] = pts[:n]
    return dev(buf), dev(np.array([len(pts)], np.int32))


WORST_SEEN = {}   # over the session: what the comparisons saw, by (figure, half)


def assert_features_close(got, want, rtol, what="", abs_sum=None, half=False, floor_fraction=None, report=None):
    """|got - want| <= rtol * max(|want|, floor), floor = FLOOR_FRACTION of the tensor's largest magnitude; with
    abs_sum (the sum of |terms| behind every element, same shape) an element is also admitted within
    SUM_TOL * abs_sum + 2 ulp of the stored value (see the note at the top of this file).  report (a dict)
    receives what the comparison saw: the worst relative error among the elements above the floor, the share of
    the non-zero elements that were judged at the floor, the share admitted by the sum bound alone, and the
    largest error beyond the stored value's rounding in units of the sum of |terms|."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.size == 0:
        return
    top = float(np.abs(want).max())
    floor = (FLOOR_FRACTION if floor_fraction is None else floor_fraction) * top
    mag = np.abs(want)
    bound = rtol * np.maximum(mag, floor)
    err = np.abs(got - want)
    bad = err > bound
    by_sum = np.zeros_like(bad)
    if abs_sum is not None:
        A = np.asarray(abs_sum, np.float64)
        assert A.shape == want.shape, (what, A.shape, want.shape)
        sum_bound = SUM_TOL * A + (2.0 ** -10 if half else 2.0 ** -22) * mag + (2.0 ** -24 if half else 0.0)
        by_sum = bad & (err <= sum_bound)
        bad = bad & ~by_sum
    held = (want != 0) | (got != 0)     # (what the ReLU zeroed on both sides is not judged by anything)
    above = mag >= floor
    seen = {"worst_rel_error_above_floor": float((err[above] / mag[above]).max()) if above.any() and floor > 0 else 0.0,
            "share_judged_at_floor": float((held & ~above).sum() / max(1, held.sum())),
            "share_admitted_by_sum_bound": float(by_sum.sum() / max(1, held.sum()))}
    if abs_sum is not None:
        pos = A > 0
        excess = np.maximum(err - (2.0 ** -10 if half else 2.0 ** -22) * mag - (2.0 ** -24 if half else 0.0), 0.0)
        seen["worst_error_over_abs_sum"] = float((excess[pos] / A[pos]).max()) if pos.any() else 0.0
    for k, v in seen.items():
        WORST_SEEN[(k, half)] = max(WORST_SEEN.get((k, half), 0.0), v)
    if report is not None:
        report.update(seen)
    assert not bad.any(), "%s: %d of %d elements off, worst %.3g x the bound (rtol %.3g, floor %.3g of the largest) at %s" % (
        what, int(bad.sum()), bad.size, float((err / np.maximum(bound, 1e-300))[bad].max()), rtol,
        FLOOR_FRACTION if floor_fraction is None else floor_fraction,
        np.unravel_index(np.argmax(np.where(bad, err / np.maximum(bound, 1e-300), 0)), err.shape))


def assert_end_to_end_close(got, want, half, what=""):
    """Whole-frame comparison of two chains that round independently: RMS and largest difference relative to the
    tensor's largest magnitude (END_TO_END_RMS / END_TO_END_MAX above)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.size == 0:
        return
    top = max(float(np.abs(want).max()), 1e-300)
    # RMS over the elements either side holds (a dense tensor is mostly structural zeros)
    held = (got != 0) | (want != 0)
    if not held.any():
        return
    d = (got - want)[held]
    r, m = float(np.sqrt(np.mean(d * d))) / top, float(np.abs(d).max()) / top
    assert r <= END_TO_END_RMS[half] and m <= END_TO_END_MAX[half], \
        "%s: RMS difference %.3g (bound %.3g), largest %.3g (bound %.3g) of the largest magnitude" % (
            what, r, END_TO_END_RMS[half], m, END_TO_END_MAX[half])


def abs_sum_of(feat_in, w, pairs, num, max_voxels, rows=None, scale=None, shift=None):
    """Sum of |terms| behind every element of gather_gemm_scatter(feat_in, w, pairs, num) (and of the scale/shift
    epilogue over the first `rows` rows, where given).  -> [max_voxels, cout]"""
    f = np.zeros((max_voxels, w.shape[1]), np.float32)
    f[:len(feat_in)] = np.abs(np.asarray(feat_in, np.float32))[:max_voxels]
    a = O.gather_gemm_scatter(f, np.abs(w).astype(np.float32), pairs, num, max_voxels)
    if scale is not None:
        a = O.scale_shift_relu(a, max_voxels if rows is None else rows, np.abs(scale).astype(np.float32),
                               np.abs(shift).astype(np.float32), False)
    return a


def layer_abs_sum(feat_in, coors, n, layer, w, scale, shift, max_voxels):
    """Sum of |terms| behind every output element of a conv layer: the layer itself on |rows|, |W|, |scale|, |shift|
    without the ReLU.  -> [max_voxels, cout]"""
    return O.conv_layer(np.abs(feat_in), coors, n, layer, np.abs(w), np.abs(scale), np.abs(shift), max_voxels, relu=False)[0]


def canonical(coors, n, *arrays):
    return O.sort_by_zyx(coors, n, *arrays)


def to_np(t):
    return t.detach().cpu().numpy()


# ---------------------------------------------------------------------------------------------
# whole-frame comparison with two capacities (the voxelizer's cap and the conv layers' row count) and an
# FP64 recomputation that says how much of a difference is rounding
# ---------------------------------------------------------------------------------------------
def fp64_layer(x64, w, pairs, num, n_out, scale, shift, relu=True):
    """One conv layer in float64 over a given rulebook: out[o] = sum_k x[i] @ W[k] for the pairs (i, o) of
    offset k (an output row appears at most once per offset), then scale/shift/ReLU."""
    out = np.zeros((n_out, w.shape[2]), np.float64)
    for k in range(w.shape[0]):
        m = int(num[k])
        if m:
            out[pairs[k, 1, :m]] += x64[pairs[k, 0, :m]] @ w[k].astype(np.float64)
    out = out * np.asarray(scale, np.float64) + np.asarray(shift, np.float64)
    return np.maximum(out, 0.0) if relu else out


def rms(a):
    a = np.asarray(a, np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


def check_frame_against_oracle(pipe, dense, pts, layers, W, voxel_cap, layer_cap, half, dense_size_xyz, report=None):
    """Every tensor of the frame the pipeline just ran against three CPU chains over the same points:
      (a) the oracle layer by layer, each layer fed the GPU's own input rows: output sites and their numbering
          bit-exact, features within the per-layer tolerance (1e-4 FP32, 1e-2 FP16 relative, floor 1e-3 of the largest
          magnitude, cancelling sums by their own terms: assert_features_close);
      (b) the oracle fed its own rows from the voxelizer on (what oracle_frame computes, here with separate
          capacities for the voxelizer and the layers): status words and final sites bit-exact;
      (c) the same layers in float64 with exact products and no rounding of stored rows.
    (c) is what tells rounding from defects end to end: the GPU's distance from it must stay within twice
    the oracle's own distance from it (RMS over each layer's tensor).  Returns the oracle chain's results."""
    import oracle_lib as O
    from sessd3d import backbone as B, ctypes_defs as D
    rtol = RTOL_FP16 if half else RTOL_FP32
    rnd = O.round_to_half if half else (lambda a: a)
    vox, vco, vn, _, status = O.voxelize(pts, B.POINT_CLOUD_RANGE, B.VOXEL_SIZE, 5, voxel_cap)
    g_feat, g_coors, g_n = pipe.read_layer(-1)
    assert g_n == vn and np.array_equal(g_coors, vco[:vn])
    assert np.array_equal(g_feat.view(np.uint32), vox[:vn].view(np.uint32))
    o_feat, f64 = vox[:vn], vox[:vn].astype(np.float64)
    coors, n = vco[:vn], vn
    counts, npairs, ratios, per_layer = [vn], [], [], []

    def padded(a, rows, cols, dtype):
        buf = np.zeros((rows, cols), dtype)
        buf[:len(a)] = a
        return buf

    for l, layer in enumerate(layers):
        cbuf = padded(coors, layer_cap, 4, np.int32)
        if layer.type == D.SESSD_LAYER_SUBM:
            pairs, num, st = O.subm_rulebook(cbuf, n, layer.out_shape, layer_cap)
            oc, on = cbuf, n
        else:
            pairs, num, oc, on, st = O.sparse_rulebook(cbuf, n, layer.out_shape, layer.ksize, layer.stride,
                                                       layer.padding, layer_cap)
        status |= st
        sc, sh = W.scale[l], W.shift[l]
        out_a = O.scale_shift_relu(O.gather_gemm_scatter(padded(g_feat, layer_cap, layer.cin, np.float32), W.w[l],
                                                         pairs, num, layer_cap), on, sc, sh, True)[:on]
        out_b = O.scale_shift_relu(O.gather_gemm_scatter(padded(o_feat, layer_cap, layer.cin, np.float32), W.w[l],
                                                         pairs, num, layer_cap), on, sc, sh, True)[:on]
        f64 = fp64_layer(f64, W.w[l], pairs, num, on, sc, sh)
        abs_a = O.scale_shift_relu(O.gather_gemm_scatter(np.abs(padded(g_feat, layer_cap, layer.cin, np.float32)), np.abs(W.w[l]),
                                                         pairs, num, layer_cap), on, np.abs(sc), np.abs(sh), False)[:on]
        g_feat, g_coors, g_n = pipe.read_layer(l)
        assert g_n == on, (layer.name, g_n, on)
        assert np.array_equal(g_coors, oc[:on]), layer.name               # same sites, same numbering
        seen = {}
        assert_features_close(g_feat, rnd(out_a), rtol, layer.name + " (oracle fed the GPU's rows)", abs_sum=abs_a, half=half, report=seen)
        per_layer.append(seen)
        o_feat = rnd(out_b)
        err_g, err_o = rms(g_feat - f64), rms(o_feat - f64)
        ratios.append(err_g / err_o if err_o > 0 else (0.0 if err_g == 0 else np.inf))
        assert err_g <= 2.0 * err_o + 1e-30, "%s: GPU is %.3g from the FP64 result, the oracle %.3g" % (layer.name, err_g, err_o)
        coors, n = oc[:on], on
        counts.append(on)
        npairs.append(int(num.sum()))
    got = to_np(dense).astype(np.float32)
    assert np.array_equal(got, O.sparse2dense(g_feat, coors, n, dense_size_xyz))   # exact scatter of the last rows
    assert pipe.status() == status
    if report is not None:
        scale = max(float(np.abs(f64).max()), 1e-30)
        for k in ("worst_rel_error_above_floor", "share_judged_at_floor", "share_admitted_by_sum_bound", "worst_error_over_abs_sum"):
            report[k] = max(d.get(k, 0.0) for d in per_layer) if per_layer else 0.0
        report.update(counts=counts, pairs=npairs, gpu_over_oracle_rms_error=[round(r, 3) for r in ratios],
                      last_layer_rms_error_gpu=rms(g_feat - f64) / scale, last_layer_rms_error_oracle=rms(o_feat - f64) / scale,
                      last_layer_max_diff_gpu_vs_oracle=float(np.abs(g_feat - o_feat).max()) / scale)
    return dict(counts=counts, pairs=npairs, feat=o_feat, coors=coors, status=status, f64=f64)
