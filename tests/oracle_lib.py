"""ctypes front end of the CPU oracle (oracle/sessd_oracle.cpp).  Test infrastructure only."""
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "se-ssd-ai-trt_amd"))
from sessd3d import ctypes_defs as D  # noqa: E402

_SO = os.path.join(ROOT, "oracle", "_build", "libsessd_oracle.so")


def _load():
    if not os.path.exists(_SO):
        spec = importlib.util.spec_from_file_location("oracle_build", os.path.join(ROOT, "oracle", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    return C.CDLL(_SO)


lib = _load()
_f = C.POINTER(C.c_float)
_i = C.POINTER(C.c_int32)
_u = C.POINTER(C.c_uint32)


def _p(a, t):
    return a.ctypes.data_as(t)


lib.oracle_np_round.argtypes = [C.c_float]
lib.oracle_np_round.restype = C.c_int
lib.oracle_round_to_half.argtypes = [_f, C.c_int64]
lib.oracle_round_to_half.restype = None
lib.oracle_frame.restype = C.c_int


def np_round(x):
    return lib.oracle_np_round(float(np.float32(x)))


def grid_size(pc_range, voxel_size):
    r = np.asarray(pc_range, np.float32)
    v = np.asarray(voxel_size, np.float32)
    g = np.zeros(3, np.int32)
    lib.oracle_grid_size(_p(r, _f), _p(v, _f), _p(g, _i))
    return tuple(int(x) for x in g)


def round_to_half(x):
    y = np.ascontiguousarray(x, np.float32).copy()
    lib.oracle_round_to_half(_p(y, _f), C.c_int64(y.size))
    return y


def voxelize(points, pc_range, voxel_size, max_pts, max_voxels):
    """-> voxels[max_voxels,4], coors[max_voxels,4], voxel_num, num_points[max_voxels], status"""
    pts = np.ascontiguousarray(points, np.float32)
    r = np.asarray(pc_range, np.float32)
    v = np.asarray(voxel_size, np.float32)
    vox = np.zeros((max_voxels, 4), np.float32)
    coors = np.zeros((max_voxels, 4), np.int32)
    num = np.zeros(1, np.int32)
    npts = np.zeros(max_voxels, np.int32)
    st = lib.oracle_voxelize(_p(pts, _f), C.c_int32(pts.shape[0]), C.c_int32(pts.shape[1]), _p(r, _f),
                             _p(v, _f), C.c_int32(max_pts), C.c_int32(max_voxels), _p(vox, _f),
                             _p(coors, _i), _p(num, _i), _p(npts, _i))
    return vox, coors, int(num[0]), npts, st


def valid_out_pos(c_zyx, ksize, stride, padding, out_shape_zyx, dilation=1):
    c = np.asarray(c_zyx, np.int32)
    k = np.asarray(ksize, np.int32)
    s = np.asarray(stride, np.int32)
    p = np.asarray(padding, np.int32)
    o = np.asarray(out_shape_zyx, np.int32)
    out = np.zeros((27, 4), np.int32)
    n = lib.oracle_valid_out_pos(_p(c, _i), _p(k, _i), _p(s, _i), _p(p, _i), C.c_int32(dilation),
                                 _p(o, _i), _p(out, _i))
    return out[:n].copy()


def subm_rulebook(coors, n, out_shape_xyz, max_voxels, ksize=3, stride=1, padding=1, dilation=1):
    """-> indice_pairs[K,2,max_voxels], indice_num[K], status"""
    co = np.ascontiguousarray(coors, np.int32)
    os_ = np.asarray(out_shape_xyz, np.int32)
    K = ksize ** 3
    pairs = np.empty((K, 2, max_voxels), np.int32)
    num = np.zeros(K, np.uint32)
    st = lib.oracle_subm_rulebook(_p(co, _i), C.c_int32(n), _p(os_, _i), C.c_int32(ksize),
                                  C.c_int32(stride), C.c_int32(padding), C.c_int32(dilation),
                                  C.c_int32(max_voxels), _p(pairs, _i), _p(num, _u))
    return pairs, num, st


def sparse_rulebook(coors, n, out_shape_xyz, ksize, stride, padding, max_voxels, dilation=1):
    """-> indice_pairs[K,2,max_voxels], indice_num[K], out_coors[max_voxels,4], out_num, status"""
    co = np.ascontiguousarray(coors, np.int32)
    os_ = np.asarray(out_shape_xyz, np.int32)
    k = np.asarray(ksize, np.int32)
    s = np.asarray(stride, np.int32)
    p = np.asarray(padding, np.int32)
    K = int(k[0] * k[1] * k[2])
    pairs = np.empty((K, 2, max_voxels), np.int32)
    num = np.zeros(K, np.uint32)
    oc = np.zeros((max_voxels, 4), np.int32)
    on = np.zeros(1, np.int32)
    st = lib.oracle_sparse_rulebook(_p(co, _i), C.c_int32(n), _p(os_, _i), _p(k, _i), _p(s, _i),
                                    _p(p, _i), C.c_int32(dilation), C.c_int32(max_voxels),
                                    _p(pairs, _i), _p(num, _u), _p(oc, _i), _p(on, _i))
    return pairs, num, oc, int(on[0]), st


def gather_gemm_scatter(in_feat, weights, pairs, num, max_voxels):
    x = np.ascontiguousarray(in_feat, np.float32)
    w = np.ascontiguousarray(weights, np.float32)
    K, cin, cout = w.shape
    out = np.empty((max_voxels, cout), np.float32)
    pr = np.ascontiguousarray(pairs, np.int32)
    nm = np.ascontiguousarray(num, np.uint32)
    lib.oracle_gather_gemm_scatter(_p(x, _f), _p(w, _f), _p(pr, _i), _p(nm, _u), C.c_int32(K),
                                   C.c_int32(max_voxels), C.c_int32(cin), C.c_int32(cout), _p(out, _f))
    return out


def fold_bn(gamma, beta, mean, var, eps=1e-5):
    g, b, m, v = (np.ascontiguousarray(a, np.float32) for a in (gamma, beta, mean, var))
    sc = np.empty_like(g)
    sh = np.empty_like(g)
    lib.oracle_fold_bn(_p(g, _f), _p(b, _f), _p(m, _f), _p(v, _f), C.c_float(eps), C.c_int32(g.size),
                       _p(sc, _f), _p(sh, _f))
    return sc, sh


def scale_shift_relu(x, rows, scale, shift, relu=True):
    y = np.ascontiguousarray(x, np.float32).copy()
    c = y.shape[1]
    sc = None if scale is None else _p(np.ascontiguousarray(scale, np.float32), _f)
    sh = None if shift is None else _p(np.ascontiguousarray(shift, np.float32), _f)
    lib.oracle_scale_shift_relu(_p(y, _f), C.c_int32(rows), C.c_int32(c), sc, sh, C.c_int32(int(relu)))
    return y


def sparse2dense(feat, coors, n, size_xyz):
    f = np.ascontiguousarray(feat, np.float32)
    co = np.ascontiguousarray(coors, np.int32)
    c = f.shape[1]
    sz = np.asarray(size_xyz, np.int32)
    dense = np.empty((c * int(sz[2]), int(sz[1]), int(sz[0])), np.float32)
    lib.oracle_sparse2dense(_p(f, _f), _p(co, _i), C.c_int32(n), C.c_int32(c), _p(sz, _i), _p(dense, _f))
    return dense



def set_threads(n):
    """Threads the gather-GEMM of the oracle may use (results do not depend on it)."""
    lib.oracle_set_threads(C.c_int32(n))


def zero_pad2d(x, top, bottom, left, right):
    """x f32[channels, height, width] -> zero-bordered copy (the reference's ZeroPad2dPlugin)."""
    a = np.ascontiguousarray(x, np.float32)
    c, h, w = a.shape
    out = np.empty((c, h + top + bottom, w + left + right), np.float32)
    lib.oracle_zero_pad2d(_p(a, _f), C.c_int32(c), C.c_int32(h), C.c_int32(w), C.c_int32(top), C.c_int32(bottom),
                          C.c_int32(left), C.c_int32(right), _p(out, _f))
    return out

def conv_layer(feat, coors, n, layer, w, scale, shift, max_voxels, relu=True):
    """One backbone layer through the oracle: rulebook, gather-GEMM-scatter, epilogue.
    -> out_feat[max_voxels,Cout], out_coors, out_n, pairs, num"""
    if layer.type == D.SESSD_LAYER_SUBM:
        pairs, num, _ = subm_rulebook(coors, n, layer.out_shape, max_voxels)
        oc, on = coors, n
    else:
        pairs, num, oc, on, _ = sparse_rulebook(coors, n, layer.out_shape, layer.ksize, layer.stride,
                                                layer.padding, max_voxels)
    out = gather_gemm_scatter(feat, w, pairs, num, max_voxels)
    out = scale_shift_relu(out, on, scale, shift, relu)
    return out, oc, on, pairs, num


def frame(points, vg_desc, layers, weights, dense_desc, relu=True, round_half=False, want_dense=True):
    """Whole frame through oracle_frame.  -> dict(dense, counts, pairs, feat, coors, status)"""
    from sessd3d import backbone as B
    pts = np.ascontiguousarray(points, np.float32)
    nl = len(layers)
    specs = B.layer_specs(layers)
    wl = [np.ascontiguousarray(w, np.float32) for w in weights.w]
    sl = [np.ascontiguousarray(s, np.float32) for s in weights.scale]
    bl = [np.ascontiguousarray(s, np.float32) for s in weights.shift]
    PP = _f * max(nl, 1)
    wp = PP(*[_p(a, _f) for a in wl])
    sp = PP(*[_p(a, _f) for a in sl])
    bp = PP(*[_p(a, _f) for a in bl])
    mv = vg_desc.max_voxels
    ch = dense_desc.feature_map_channel
    sz = dense_desc.feature_map_size
    dense = np.empty((ch * sz[2], sz[1], sz[0]), np.float32) if want_dense else None
    counts = np.zeros(nl + 1, np.int32)
    npairs = np.zeros(max(nl, 1), np.int64)
    c_last = layers[-1].cout if nl else 4
    feat = np.zeros((mv, c_last), np.float32)
    coors = np.zeros((mv, 4), np.int32)
    st = lib.oracle_frame(_p(pts, _f), C.c_int32(pts.shape[0]), C.c_int32(pts.shape[1]), C.byref(vg_desc),
                          C.c_int32(nl), specs, wp, sp, bp, C.c_int32(int(relu)),
                          C.c_int32(int(round_half)), C.byref(dense_desc),
                          _p(dense, _f) if want_dense else None, _p(counts, _i),
                          npairs.ctypes.data_as(C.POINTER(C.c_int64)), _p(feat, _f), _p(coors, _i))
    n = int(counts[-1])
    return dict(dense=dense, counts=counts, pairs=npairs, feat=feat[:n], coors=coors[:n], status=st)


def canonical_rulebook(pairs, num, in_coors, out_coors):
    """Rulebook as a sorted array of rows (offset, in z,y,x, out z,y,x): independent of how input and
    output rows are numbered and of the order of pairs inside an offset."""
    rows = []
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n == 0:
            continue
        i = pairs[k, 0, :n]
        o = pairs[k, 1, :n]
        rows.append(np.concatenate([np.full((n, 1), k, np.int64), in_coors[i, 1:4].astype(np.int64),
                                    out_coors[o, 1:4].astype(np.int64)], axis=1))
    if not rows:
        return np.zeros((0, 7), np.int64)
    r = np.concatenate(rows, axis=0)
    order = np.lexsort(r.T[::-1])
    return r[order]


def sort_by_zyx(coors, n, *arrays):
    """Canonical order: rows sorted by (z,y,x).  -> sorted coors[:n] and each array[:n] permuted."""
    c = np.asarray(coors)[:n]
    order = np.lexsort((c[:, 3], c[:, 2], c[:, 1]))
    return (c[order],) + tuple(np.asarray(a)[:n][order] for a in arrays)
