"""Helpers for the GPU parity tests: device upload, canonical comparisons, tolerances."""
import numpy as np
import torch

import oracle_lib as O

DEV = "cuda:0"

# FP32 features: |gpu - oracle| <= 1e-4 * max(|oracle|, floor), FP16: 1e-2.  The floor (1 % of the
# tensor's largest magnitude) keeps elements that are tiny through cancellation from being judged by a
# relative error against ~0.
RTOL_FP32 = 1e-4
RTOL_FP16 = 1e-2
# End to end the FP32 rounding differences of 14 stacked layers compound.  How far: an FP64 recomputation of the
# frame (gpu_util.check_frame_against_oracle, run at the benchmark configurations in test_gpu_configs.py) puts
# the oracle 2.0e-8 and the GPU 1.9e-8 of the last tensor's largest magnitude (RMS) from the exact result, and the
# largest element-wise difference between the two at 7.9e-7 of it -- 0.8 of the per-layer bound at its floor.
# The whole-frame comparison therefore uses 3e-4; the 1e-4 bound is checked layer by layer, each layer of the
# oracle being fed the GPU's own input rows.
RTOL_END_TO_END = 3e-4
# FP16 end to end: the GPU and the oracle round every layer's output to half independently, so a value that sits
# near a rounding boundary falls to different sides in the two chains and the layers after it carry the
# difference on.  Measured at configurations 4 and 5 (same FP64 recomputation): both are 2.3e-5 .. 2.9e-5 of the
# last tensor's largest magnitude (RMS) from the exact result, equal to each other within 1 % at every layer, and
# their largest element-wise difference is 9.3e-4 of that magnitude (two units in the last place of a half near
# the top of the range) -- 0.93 of this bound at its floor.  The 1e-2 bound is checked layer by layer.
RTOL_END_TO_END_FP16 = 1e-1


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


def assert_features_close(got, want, rtol, what=""):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.size == 0:
        return
    floor = 1e-2 * float(np.abs(want).max())
    bound = rtol * np.maximum(np.abs(want), floor)
    err = np.abs(got - want)
    bad = err > bound
    assert not bad.any(), "%s: %d of %d elements off, worst %.3g (bound %.3g) at %s" % (
        what, int(bad.sum()), bad.size, float((err / np.maximum(bound, 1e-300)).max()), rtol,
        np.unravel_index(np.argmax(err / np.maximum(bound, 1e-300)), err.shape))


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
          bit-exact, features within the per-layer tolerance (1e-4 FP32, 1e-2 FP16);
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
    counts, npairs, ratios = [vn], [], []

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
        g_feat, g_coors, g_n = pipe.read_layer(l)
        assert g_n == on, (layer.name, g_n, on)
        assert np.array_equal(g_coors, oc[:on]), layer.name               # same sites, same numbering
        assert_features_close(g_feat, rnd(out_a), rtol, layer.name + " (oracle fed the GPU's rows)")
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
        report.update(counts=counts, pairs=npairs, gpu_over_oracle_rms_error=[round(r, 3) for r in ratios],
                      last_layer_rms_error_gpu=rms(g_feat - f64) / scale, last_layer_rms_error_oracle=rms(o_feat - f64) / scale,
                      last_layer_max_diff_gpu_vs_oracle=float(np.abs(g_feat - o_feat).max()) / scale)
    return dict(counts=counts, pairs=npairs, feat=o_feat, coors=coors, status=status, f64=f64)
