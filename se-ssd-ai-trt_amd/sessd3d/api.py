"""ctypes binding of libsessd3d.so plus thin per-plugin wrappers.

torch is used only to own device memory and streams; every compute call goes through the C-ABI
declared in include/sessd3d.h.  There is no fallback: if the library is missing the import of
`lib()` raises.
"""
import ctypes as C
import os
import re

import numpy as np

from . import backbone as B
from . import ctypes_defs as D

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SESSD3D_LIB") or os.path.join(os.path.dirname(_HERE), "lib", "libsessd3d.so")
HEADER_PATH = os.path.join(os.path.dirname(os.path.dirname(_HERE)), "include", "sessd3d.h")
_lib = None


class SessdError(RuntimeError):
    pass


def declared_symbols():
    """Names of all functions declared in include/sessd3d.h."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sessd_[a-z0-9_]+)\s*\(", text)))


def lib():
    """Load libsessd3d.so (built by se-ssd-ai-trt_amd/build.py).  Never falls back to anything else."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SessdError("libsessd3d.so is not built: run `python se-ssd-ai-trt_amd/build.py` (%s)" % LIB_PATH)
    # torch bundles its own HIP runtime under the same soname as the system one.  A process must hold
    # exactly one: import torch first so that the library binds to the runtime torch's tensors live in.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int32
    TD = C.POINTER(D.TensorDesc)
    VPP = C.POINTER(C.c_void_p)
    L.sessd_last_error.restype = C.c_char_p
    L.sessd_version.restype = C.c_char_p
    for name in ("voxelgen", "submconv3d", "sparseconv3d", "sparse2dense"):
        getattr(L, "sessd_%s_serialization_size" % name).restype = sz
        getattr(L, "sessd_%s_serialization_size" % name).argtypes = [vp]
        getattr(L, "sessd_%s_serialize" % name).argtypes = [vp, vp]
        getattr(L, "sessd_%s_deserialize" % name).argtypes = [vp, sz, VPP]
        getattr(L, "sessd_%s_configure" % name).argtypes = [vp, TD, C.c_int, TD, C.c_int]
        getattr(L, "sessd_%s_workspace_size" % name).restype = sz
        getattr(L, "sessd_%s_workspace_size" % name).argtypes = [vp, TD, C.c_int, TD, C.c_int]
        getattr(L, "sessd_%s_enqueue" % name).argtypes = [vp, TD, TD, VPP, VPP, vp, vp]
        getattr(L, "sessd_%s_destroy" % name).argtypes = [vp]
        getattr(L, "sessd_%s_destroy" % name).restype = None
    for name in ("voxelgen", "submconv3d", "sparseconv3d"):
        getattr(L, "sessd_%s_status" % name).argtypes = [vp, vp, vp, C.POINTER(i32)]
        getattr(L, "sessd_%s_set_flags" % name).argtypes = [vp, i32]
    for name in ("submconv3d", "sparseconv3d"):
        getattr(L, "sessd_%s_set_epilogue" % name).argtypes = [vp, vp, vp, C.c_int]
        getattr(L, "sessd_%s_export_rulebook" % name).argtypes = [vp, vp, vp, vp, vp]
    L.sessd_voxelgen_create.argtypes = [C.POINTER(D.VoxelGenDesc), VPP]
    L.sessd_voxelgen_grid_size.argtypes = [vp, C.POINTER(i32)]
    L.sessd_voxelgen_enqueue_static.argtypes = [vp, TD, TD, VPP, VPP, vp]
    L.sessd_submconv3d_create.argtypes = [C.POINTER(D.SubmConv3dDesc), vp, VPP]
    L.sessd_submconv3d_enqueue_shared.argtypes = [vp, TD, TD, VPP, VPP, vp, vp]
    L.sessd_sparseconv3d_create.argtypes = [C.POINTER(D.SparseConv3dDesc), vp, VPP]
    L.sessd_sparse2dense_create.argtypes = [C.POINTER(D.Sparse2DenseDesc), VPP]
    L.sessd_sparse2dense_set_padding.argtypes = [C.c_void_p] + [C.c_int32] * 4
    L.sessd_sparse2dense_set_padding.restype = C.c_int
    FPP = C.POINTER(C.POINTER(C.c_float))
    L.sessd_wts_load.argtypes = [C.c_char_p, VPP]
    L.sessd_wts_parse.argtypes = [C.c_char_p, sz, VPP]
    L.sessd_wts_count.argtypes = [vp]
    L.sessd_wts_name.argtypes = [vp, C.c_int, C.POINTER(C.c_char_p)]
    L.sessd_wts_find.argtypes = [vp, C.c_char_p, FPP, C.POINTER(C.c_int64)]
    L.sessd_wts_destroy.argtypes = [vp]
    L.sessd_wts_destroy.restype = None
    FP1 = C.POINTER(C.c_float)
    L.sessd_fold_batchnorm.argtypes = [FP1, FP1, FP1, FP1, i32, C.c_float, FP1, FP1]
    L.sessd_pipeline_create_from_wts.argtypes = [C.POINTER(D.PipelineDesc), vp, C.c_char_p, C.POINTER(i32), C.c_float, VPP]
    L.sessd_load_frame.argtypes = [C.c_char_p, FP1, i32, i32, C.POINTER(i32)]
    L.sessd_reference_backbone.argtypes = [C.POINTER(D.LayerSpec), C.c_int, C.POINTER(D.VoxelGenDesc),
                                           C.POINTER(D.Sparse2DenseDesc)]
    L.sessd_pipeline_create.argtypes = [C.POINTER(D.PipelineDesc), VPP]
    L.sessd_pipeline_enqueue.argtypes = [vp, vp, vp, vp, vp]
    L.sessd_pipeline_submit.argtypes = [vp, vp, vp, vp, vp, C.POINTER(C.c_int64)]
    L.sessd_pipeline_join.argtypes = [vp, C.c_int64, vp]
    L.sessd_pipeline_wait.argtypes = [vp, C.c_int64]
    L.sessd_pipeline_layer_io.argtypes = [vp, C.c_int, VPP, VPP, VPP, VPP, C.POINTER(i32)]
    L.sessd_pipeline_status.argtypes = [vp, vp, C.POINTER(i32)]
    L.sessd_pipeline_enqueue_timed.argtypes = [vp, vp, vp, vp, vp, C.POINTER(C.c_float), C.c_int, C.POINTER(C.c_int)]
    L.sessd_pipeline_layer_stats.argtypes = [vp, C.c_int, vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    L.sessd_pipeline_device_bytes.restype = sz
    L.sessd_pipeline_device_bytes.argtypes = [vp]
    L.sessd_pipeline_num_launches.argtypes = [vp]
    L.sessd_pipeline_destroy.argtypes = [vp]
    L.sessd_pipeline_destroy.restype = None
    L.sessd_copy_to_host.argtypes = [vp, vp, sz, vp]
    L.sessd_plugin_field_names.restype = C.POINTER(D.PluginFieldCollection)
    L.sessd_plugin_field_names.argtypes = [C.c_char_p]
    L.sessd_plugin_create.argtypes = [C.c_char_p, C.POINTER(D.PluginFieldCollection), VPP]
    for name in ("voxelgen", "submconv3d", "sparseconv3d", "sparse2dense"):
        getattr(L, "sessd_%s_clone" % name).argtypes = [vp, VPP]
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise SessdError("sessd3d error %d: %s" % (rc, lib().sessd_last_error().decode()))


def _torch():
    import torch
    return torch


class _NoStream:
    """SESSD_STREAM_NONE of the header: Pipeline.submit orders the frame after no stream (the inputs are ready)."""
    cuda_stream = -1


STREAM_NONE = _NoStream()


def _stream_ptr(stream=None):
    torch = _torch()
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _np_f32_ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else C.c_void_p(0)


def _dtype_code(t):
    torch = _torch()
    return {torch.float32: D.SESSD_FLOAT, torch.float16: D.SESSD_HALF, torch.int32: D.SESSD_INT32}[t.dtype]


def _descs(tensors):
    arr = (D.TensorDesc * len(tensors))()
    for i, t in enumerate(tensors):
        dims = [1] + list(t.shape) if t.dim() >= 2 else list(t.shape)
        arr[i] = D.TensorDesc.make(dims, _dtype_code(t))
    return arr


def _voidpp(tensors):
    return (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


class _Plugin:
    """Life cycle shared by the four plugin wrappers; `kind` is the symbol infix."""
    kind = ""

    def __init__(self, handle):
        self.h = handle
        self.ws = None

    def _fn(self, name):
        return getattr(lib(), "sessd_%s_%s" % (self.kind, name))

    def serialize(self) -> bytes:
        n = self._fn("serialization_size")(self.h)
        buf = C.create_string_buffer(n)
        check(self._fn("serialize")(self.h, buf))
        return buf.raw

    @classmethod
    def deserialize(cls, blob: bytes):
        h = C.c_void_p()
        check(getattr(lib(), "sessd_%s_deserialize" % cls.kind)(blob, len(blob), C.byref(h)))
        obj = cls.__new__(cls)
        _Plugin.__init__(obj, h)
        return obj

    def clone(self):
        """An independent copy (own device weights, same epilogue / flags / configured types): clone() of the reference."""
        h = C.c_void_p()
        check(self._fn("clone")(self.h, C.byref(h)))
        obj = self.__class__.__new__(self.__class__)
        obj.__dict__.update({k: v for k, v in self.__dict__.items() if k not in ("h", "ws")})
        _Plugin.__init__(obj, h)
        return obj

    def configure(self, inputs, outputs):
        check(self._fn("configure")(self.h, _descs(inputs), len(inputs), _descs(outputs), len(outputs)))

    def workspace_size(self, inputs, outputs) -> int:
        return self._fn("workspace_size")(self.h, _descs(inputs), len(inputs), _descs(outputs), len(outputs))

    def _workspace(self, inputs, outputs):
        torch = _torch()
        n = self.workspace_size(inputs, outputs)
        if self.ws is None or self.ws.numel() < n:
            self.ws = torch.empty(max(n, 256), dtype=torch.uint8, device=inputs[0].device)
        return self.ws

    def enqueue(self, inputs, outputs, stream=None, workspace=None):
        """inputs/outputs: lists of torch device tensors without the batch dimension."""
        ws = workspace if workspace is not None else self._workspace(inputs, outputs)
        check(self._fn("enqueue")(self.h, _descs(inputs), _descs(outputs), _voidpp(inputs), _voidpp(outputs),
                                  _ptr(ws), _stream_ptr(stream)))
        return ws

    def status(self, stream=None) -> int:
        s = C.c_int32(0)
        check(self._fn("status")(self.h, _ptr(self.ws), _stream_ptr(stream), C.byref(s)))
        return s.value

    def set_flags(self, flags):
        check(self._fn("set_flags")(self.h, flags))

    def close(self):
        if self.h:
            self._fn("destroy")(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class VoxelGenerator(_Plugin):
    kind = "voxelgen"

    def __init__(self, max_voxels=B.MAX_VOXELS, max_num_points_per_voxel=B.MAX_NUM_POINTS_PER_VOXEL,
                 point_cloud_range=B.POINT_CLOUD_RANGE, voxel_size=B.VOXEL_SIZE):
        d = B.voxelgen_desc(max_voxels, max_num_points_per_voxel, point_cloud_range, voxel_size)
        h = C.c_void_p()
        check(lib().sessd_voxelgen_create(C.byref(d), C.byref(h)))
        super().__init__(h)
        self.max_voxels = max_voxels

    def grid_size(self):
        g = (C.c_int32 * 3)()
        check(lib().sessd_voxelgen_grid_size(self.h, g))
        return tuple(g)

    def enqueue_static(self, inputs, outputs, stream=None):
        """enqueue() on the library's static scratch array: no workspace, no allocation (sessd_voxelgen_enqueue_static)."""
        check(lib().sessd_voxelgen_enqueue_static(self.h, _descs(inputs), _descs(outputs), _voidpp(inputs),
                                                  _voidpp(outputs), _stream_ptr(stream)))

    def status_static(self, stream=None) -> int:
        s = C.c_int32(0)
        check(lib().sessd_voxelgen_status(self.h, None, _stream_ptr(stream), C.byref(s)))
        return s.value

    def __call__(self, points, points_size, stream=None):
        """points f32[max_points,F], points_size i32[1] (device) -> voxels, coors, voxel_num (device)"""
        torch = _torch()
        dev = points.device
        voxels = torch.empty((self.max_voxels, 4), dtype=torch.float32, device=dev)
        coors = torch.empty((self.max_voxels, 4), dtype=torch.int32, device=dev)
        num = torch.empty((1,), dtype=torch.int32, device=dev)
        self.configure([points, points_size], [voxels, coors, num])
        self.enqueue([points, points_size], [voxels, coors, num], stream)
        return voxels, coors, num


class _Conv(_Plugin):
    def set_epilogue(self, scale=None, shift=None, relu=True):
        sc = None if scale is None else np.ascontiguousarray(scale, np.float32)
        sh = None if shift is None else np.ascontiguousarray(shift, np.float32)
        check(self._fn("set_epilogue")(self.h, _np_f32_ptr(sc), _np_f32_ptr(sh), int(relu)))

    def export_rulebook(self, stream=None, workspace=None):
        """-> indice_pairs i32[K,2,max_voxels], indice_num i32[K] (device tensors)"""
        torch = _torch()
        ws = workspace if workspace is not None else self.ws
        pairs = torch.empty((self.kvol, 2, self.max_voxels), dtype=torch.int32, device=ws.device)
        num = torch.empty((self.kvol,), dtype=torch.int32, device=ws.device)
        check(self._fn("export_rulebook")(self.h, _ptr(ws), _ptr(pairs), _ptr(num), _stream_ptr(stream)))
        return pairs, num


class SubmConv3d(_Conv):
    kind = "submconv3d"

    def __init__(self, in_channel, out_channel, out_shape_xyz, weights, max_voxels=B.MAX_VOXELS, ksize=3,
                 stride=1, padding=1, dilation=1):
        d = D.SubmConv3dDesc()
        d.in_channel, d.out_channel, d.max_voxels, d.feature_num = in_channel, out_channel, max_voxels, in_channel
        for a in range(3):
            d.out_shape[a] = out_shape_xyz[a]
            d.spatial_shape[a] = out_shape_xyz[a]
        d.ksize, d.stride, d.padding, d.dilation, d.out_padding = ksize, stride, padding, dilation, 0
        w = np.ascontiguousarray(weights, np.float32)
        assert w.shape == (ksize ** 3, in_channel, out_channel)
        h = C.c_void_p()
        check(lib().sessd_submconv3d_create(C.byref(d), _np_f32_ptr(w), C.byref(h)))
        super().__init__(h)
        self.max_voxels, self.cout, self.kvol = max_voxels, out_channel, ksize ** 3

    def __call__(self, feat, coors, voxel_num, out_dtype=None, stream=None, rulebook_from=None):
        torch = _torch()
        out = torch.empty((self.max_voxels, self.cout), dtype=out_dtype or feat.dtype, device=feat.device)
        ins = [feat, coors, voxel_num]
        self.configure(ins, [out])
        if rulebook_from is None:
            self.enqueue(ins, [out], stream)
        else:
            check(lib().sessd_submconv3d_enqueue_shared(self.h, _descs(ins), _descs([out]), _voidpp(ins),
                                                        _voidpp([out]), _ptr(rulebook_from.ws),
                                                        _stream_ptr(stream)))
        return out


class SparseConv3d(_Conv):
    kind = "sparseconv3d"

    def __init__(self, in_channel, out_channel, out_shape_xyz, spatial_shape_xyz, ksize, stride, padding, weights,
                 max_voxels=B.MAX_VOXELS, dilation=1):
        d = D.SparseConv3dDesc()
        d.in_channel, d.out_channel, d.max_voxels, d.feature_num = in_channel, out_channel, max_voxels, in_channel
        for a in range(3):
            d.out_shape[a] = out_shape_xyz[a]
            d.spatial_shape[a] = spatial_shape_xyz[a]
            d.ksize[a], d.stride[a], d.padding[a] = ksize[a], stride[a], padding[a]
        d.dilation, d.out_padding = dilation, 0
        w = np.ascontiguousarray(weights, np.float32)
        self.kvol = ksize[0] * ksize[1] * ksize[2]
        assert w.shape == (self.kvol, in_channel, out_channel)
        h = C.c_void_p()
        check(lib().sessd_sparseconv3d_create(C.byref(d), _np_f32_ptr(w), C.byref(h)))
        super().__init__(h)
        self.max_voxels, self.cout = max_voxels, out_channel

    def __call__(self, feat, coors, voxel_num, out_dtype=None, stream=None):
        torch = _torch()
        dev = feat.device
        out = torch.empty((self.max_voxels, self.cout), dtype=out_dtype or feat.dtype, device=dev)
        ocoors = torch.empty((self.max_voxels, 4), dtype=torch.int32, device=dev)
        onum = torch.empty((1,), dtype=torch.int32, device=dev)
        ins = [feat, coors, voxel_num]
        self.configure(ins, [out, ocoors, onum])
        self.enqueue(ins, [out, ocoors, onum], stream)
        return out, ocoors, onum


class Sparse2Dense(_Plugin):
    kind = "sparse2dense"

    def __init__(self, feature_map_size_xyz=B.DENSE_SIZE_XYZ, feature_map_channel=B.DENSE_CHANNEL,
                 padding=(0, 0, 0, 0)):
        d = B.dense_desc(feature_map_size_xyz, feature_map_channel)
        h = C.c_void_p()
        check(lib().sessd_sparse2dense_create(C.byref(d), C.byref(h)))
        super().__init__(h)
        self.size, self.channel = tuple(feature_map_size_xyz), feature_map_channel
        self.padding = tuple(int(v) for v in padding)  # top, bottom, left, right
        if any(self.padding):
            check(lib().sessd_sparse2dense_set_padding(self.h, *self.padding))

    def __call__(self, feat, coors, voxel_num, out_dtype=None, stream=None):
        torch = _torch()
        W, H, Dz = self.size
        top, bottom, left, right = self.padding
        dense = torch.empty((self.channel * Dz, H + top + bottom, W + left + right),
                            dtype=out_dtype or feat.dtype, device=feat.device)
        ins = [feat, coors, voxel_num]
        self.configure(ins, [dense])
        self.enqueue(ins, [dense], stream)
        return dense

    def status(self, stream=None):
        torch = _torch()
        torch.cuda.synchronize()
        return int(self.ws[:4].view(torch.int32)[0].item())


PLUGIN_CLASSES = {}


def plugin_field_names(plugin_name):
    """-> [(name, type, length)] the creator of `plugin_name` reads (getFieldNames of the reference's creators)."""
    fc = lib().sessd_plugin_field_names(plugin_name.encode())
    if not fc:
        raise SessdError(lib().sessd_last_error().decode())
    return [(fc.contents.fields[i].name.decode(), fc.contents.fields[i].type, fc.contents.fields[i].length)
            for i in range(fc.contents.nbFields)]


def create_plugin(plugin_name, fields):
    """createPlugin(name, PluginFieldCollection) of the reference's creators: `fields` maps field names to numpy
    arrays (int32 or float32).  -> the wrapper object of that plugin type."""
    keep = []
    arr = (D.PluginField * max(len(fields), 1))()
    for i, (k, v) in enumerate(fields.items()):
        a = np.ascontiguousarray(v)
        keep.append(a)
        arr[i].name = k.encode()
        arr[i].data = a.ctypes.data
        arr[i].type = D.SESSD_FIELD_FLOAT32 if a.dtype == np.float32 else D.SESSD_FIELD_INT32
        arr[i].length = a.size
    fc = D.PluginFieldCollection(len(fields), arr)
    h = C.c_void_p()
    check(lib().sessd_plugin_create(plugin_name.encode(), C.byref(fc), C.byref(h)))
    cls = {"VoxelGeneratorPlugin": VoxelGenerator, "SubmConv3dLayerPlugin": SubmConv3d,
           "SparseConv3dLayerPlugin": SparseConv3d, "Sparse2DensePlugin": Sparse2Dense}[plugin_name]
    obj = cls.__new__(cls)
    _Plugin.__init__(obj, h)
    g = lambda k: np.asarray(fields[k]).reshape(-1)  # noqa: E731
    if cls is VoxelGenerator:
        obj.max_voxels = int(g("max_voxels")[0])
    elif cls is Sparse2Dense:
        obj.size, obj.channel, obj.padding = tuple(int(v) for v in g("feature_map_size")), int(g("feature_map_channel")[0]), (0, 0, 0, 0)
    else:
        obj.max_voxels, obj.cout = int(g("max_voxels")[0]), int(g("out_channel")[0])
        k = g("ksize")
        obj.kvol = int(k[0]) ** 3 if cls is SubmConv3d else int(k[0] * k[1] * k[2])
    return obj


def make_conv(layer: B.Layer, weights, prev_grid_xyz, max_voxels, scale=None, shift=None, relu=True):
    """Plugin for one entry of the backbone table, with its folded BatchNorm + ReLU epilogue."""
    if layer.type == D.SESSD_LAYER_SUBM:
        p = SubmConv3d(layer.cin, layer.cout, layer.out_shape, weights, max_voxels, layer.ksize[0],
                       layer.stride[0], layer.padding[0])
    else:
        p = SparseConv3d(layer.cin, layer.cout, layer.out_shape, prev_grid_xyz, layer.ksize, layer.stride,
                         layer.padding, weights, max_voxels)
    if scale is not None or shift is not None or relu:
        p.set_epilogue(scale, shift, relu)
    return p


class WeightFile:
    """A parsed `.wts` file (the reference's text weight format, se-ssd-ai-trt.cpp:276-314)."""

    def __init__(self, path=None, text=None):
        self.h = C.c_void_p()
        if path is not None:
            check(lib().sessd_wts_load(os.fsencode(path), C.byref(self.h)))
        else:
            data = text.encode() if isinstance(text, str) else bytes(text)
            check(lib().sessd_wts_parse(data, len(data), C.byref(self.h)))

    def __del__(self):
        if getattr(self, "h", None):
            lib().sessd_wts_destroy(self.h)
            self.h = None

    def names(self):
        out = []
        for i in range(lib().sessd_wts_count(self.h)):
            s = C.c_char_p()
            check(lib().sessd_wts_name(self.h, i, C.byref(s)))
            out.append(s.value.decode())
        return out

    def __getitem__(self, name):
        p = C.POINTER(C.c_float)()
        n = C.c_int64()
        check(lib().sessd_wts_find(self.h, name.encode(), C.byref(p), C.byref(n)))
        if n.value == 0:
            return np.zeros(0, np.float32)
        return np.ctypeslib.as_array(p, shape=(n.value,)).copy()


def load_frame(path, max_points, point_features=4, out=None):
    """One frame file -> (points float32[max_points, point_features] host array, number of points); see
    sessd_load_frame.  `out` may be a pinned torch tensor's numpy view to read straight into it."""
    pts = out if out is not None else np.empty((max_points, point_features), np.float32)
    assert pts.dtype == np.float32 and pts.flags["C_CONTIGUOUS"] and pts.shape == (max_points, point_features)
    n = C.c_int32()
    check(lib().sessd_load_frame(os.fsencode(path), pts.ctypes.data_as(C.POINTER(C.c_float)), max_points,
                                 point_features, C.byref(n)))
    return pts, n.value


def fold_batchnorm(gamma, beta, mean, var, eps=1e-5):
    """The library's BatchNorm folding (se-ssd-ai-trt.cpp:808-824) -> (scale, shift)."""
    g, b, m, v = (np.ascontiguousarray(a, np.float32) for a in (gamma, beta, mean, var))
    sc, sh = np.empty_like(g), np.empty_like(g)
    FP = C.POINTER(C.c_float)
    check(lib().sessd_fold_batchnorm(*[a.ctypes.data_as(FP) for a in (g, b, m, v)], g.size, C.c_float(eps),
                                     sc.ctypes.data_as(FP), sh.ctypes.data_as(FP)))
    return sc, sh


class Pipeline:
    """voxelGenerator -> conv stack -> sparse2Dense, owned and run by the library (C++)."""

    def __init__(self, layers, weights: B.Weights, max_points, max_voxels=B.MAX_VOXELS, point_features=4,
                 feature_dtype="fp32", relu=True, share_rulebooks=True, skip_pad_rows=False, use_graph=False,
                 dense_size_xyz=B.DENSE_SIZE_XYZ, max_pts_per_voxel=B.MAX_NUM_POINTS_PER_VOXEL,
                 use_epilogue=True, overlap_streams=False, voxel_cap=None, dense_padding=(0, 0, 0, 0),
                 force_valu=False, frames_in_flight=0):
        """max_voxels = rows of every conv-layer tensor; voxel_cap (default: max_voxels) = the voxelizer's
        own limit.  force_valu: every gather-GEMM on the shape-agnostic VALU kernel (cross-checks)."""
        torch = _torch()
        self.layers = list(layers)
        self.max_points, self.max_voxels = max_points, max_voxels
        self.voxel_cap = voxel_cap or max_voxels
        self.dtype = torch.float16 if feature_dtype in ("fp16", "half", torch.float16) else torch.float32
        n = len(self.layers)
        self._specs = B.layer_specs(self.layers)
        from_file = isinstance(weights, WeightFile)
        if from_file:
            self._w = self._s = self._b = []
        else:
            self._w = [np.ascontiguousarray(w, np.float32) for w in weights.w]
            self._s = [np.ascontiguousarray(s, np.float32) for s in weights.scale]
            self._b = [np.ascontiguousarray(s, np.float32) for s in weights.shift]
        FP = C.POINTER(C.c_float)
        arr = lambda xs: (FP * max(n, 1))(*[x.ctypes.data_as(FP) for x in xs])  # noqa: E731
        d = D.PipelineDesc()
        d.voxelgen = B.voxelgen_desc(voxel_cap or max_voxels, max_pts_per_voxel)
        d.layer_max_voxels = max_voxels
        d.max_points, d.point_features, d.n_layers = max_points, point_features, n
        d.layers = self._specs
        if not from_file:
            d.weights = arr(self._w)
            if use_epilogue:
                d.scale = arr(self._s)
                d.shift = arr(self._b)
        d.relu = int(relu)
        d.feature_dtype = D.SESSD_HALF if self.dtype == torch.float16 else D.SESSD_FLOAT
        c_last = self.layers[-1].cout if n else 4
        d.dense = B.dense_desc(dense_size_xyz, c_last)
        d.share_rulebooks = int(share_rulebooks)
        d.flags = (D.SESSD_FLAG_SKIP_PAD_ROWS if skip_pad_rows else 0) | (D.SESSD_FLAG_FORCE_VALU if force_valu else 0)
        d.use_graph = int(use_graph)
        d.overlap_streams = int(overlap_streams)
        d.frames_in_flight = int(frames_in_flight)
        top, bottom, left, right = (int(v) for v in dense_padding)
        d.dense_padding = (C.c_int32 * 4)(top, bottom, left, right)
        self.dense_shape = (c_last * dense_size_xyz[2], dense_size_xyz[1] + top + bottom,
                            dense_size_xyz[0] + left + right)
        self.h = C.c_void_p()
        if from_file:  # conv weights and BatchNorm statistics by the reference's blob names, folded by the library
            idx = (C.c_int32 * n)(*[B.conv_index(l) for l in self.layers])
            check(lib().sessd_pipeline_create_from_wts(C.byref(d), weights.h, None, idx, C.c_float(1e-5),
                                                       C.byref(self.h)))
        else:
            check(lib().sessd_pipeline_create(C.byref(d), C.byref(self.h)))

    def new_dense(self, device="cuda"):
        torch = _torch()
        return torch.empty(self.dense_shape, dtype=self.dtype, device=device)

    def enqueue(self, points, points_size, dense, stream=None):
        check(lib().sessd_pipeline_enqueue(self.h, _ptr(points), _ptr(points_size), _ptr(dense), _stream_ptr(stream)))

    def submit(self, points, points_size, dense, stream=None):
        """Start a frame without making `stream` wait for it -> ticket for join() / wait() (sessd_pipeline_submit).
        stream = STREAM_NONE (frames in flight only): the inputs are ready, the frame waits for nothing."""
        t = C.c_int64(0)
        check(lib().sessd_pipeline_submit(self.h, _ptr(points), _ptr(points_size), _ptr(dense), _stream_ptr(stream), C.byref(t)))
        return t.value

    def join(self, ticket, stream=None):
        """Make `stream` wait until the frame of `ticket` is complete (sessd_pipeline_join)."""
        check(lib().sessd_pipeline_join(self.h, ticket, _stream_ptr(stream)))

    def wait(self, ticket):
        """Block the calling thread until the frame of `ticket` is complete (sessd_pipeline_wait)."""
        check(lib().sessd_pipeline_wait(self.h, ticket))

    def layer_io(self, layer):
        """-> (feat ptr, coors ptr, voxel_num ptr, workspace ptr, channels) of layer (or -1 = voxelizer)"""
        f, c, n, w = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
        ch = C.c_int32()
        check(lib().sessd_pipeline_layer_io(self.h, layer, C.byref(f), C.byref(c), C.byref(n), C.byref(w), C.byref(ch)))
        return f.value, c.value, n.value, w.value, ch.value

    def layer_count(self, layer):
        """Active rows a layer produced in the last enqueue (layer = -1: the voxelizer)."""
        _torch().cuda.synchronize()
        num = np.zeros(1, np.int32)
        _hip_d2h(num, self.layer_io(layer)[2])
        return int(num[0])

    def read_layer(self, layer):
        """Copy a layer's output of the last enqueue to the host: feat[n,C] float32, coors[n,4], n."""
        torch = _torch()
        torch.cuda.synchronize()
        f, c, n, _, ch = self.layer_io(layer)
        num = np.zeros(1, np.int32)
        _hip_d2h(num, n)
        cnt = int(num[0])
        es = 4 if (layer < 0 or self.dtype == torch.float32) else 2
        rows = self.voxel_cap if layer < 0 else self.max_voxels
        feat = np.zeros((rows, ch), np.float32 if es == 4 else np.float16)
        coors = np.zeros((rows, 4), np.int32)
        _hip_d2h(feat, f)
        _hip_d2h(coors, c)
        return feat[:cnt].astype(np.float32), coors[:cnt], cnt

    def status(self, stream=None):
        s = C.c_int32(0)
        check(lib().sessd_pipeline_status(self.h, _stream_ptr(stream), C.byref(s)))
        return s.value

    def enqueue_timed(self, points, points_size, dense, stream=None):
        """-> (segment durations in ms: [voxelizer, (build, gemm) per layer ..., sparse2dense],
              duration of an empty segment = what the event pair itself measures)"""
        nseg = 2 * len(self.layers) + 2
        ms = (C.c_float * (nseg + 1))()
        got = C.c_int(0)
        check(lib().sessd_pipeline_enqueue_timed(self.h, _ptr(points), _ptr(points_size), _ptr(dense),
                                                 _stream_ptr(stream), ms, nseg + 1, C.byref(got)))
        return list(ms)[:got.value], float(ms[got.value])

    def layer_stats(self, layer, stream=None):
        """-> (active output rows, rulebook pairs) of `layer` in the last enqueue"""
        n, p = C.c_int64(0), C.c_int64(0)
        check(lib().sessd_pipeline_layer_stats(self.h, layer, _stream_ptr(stream), C.byref(n), C.byref(p)))
        return n.value, p.value

    def device_bytes(self):
        return lib().sessd_pipeline_device_bytes(self.h)

    def num_launches(self):
        return lib().sessd_pipeline_num_launches(self.h)

    def close(self):
        if self.h:
            lib().sessd_pipeline_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _hip_d2h(dst_np, src_ptr):
    """Synchronous device->host copy into a numpy array (for pointers owned by the library)."""
    check(lib().sessd_copy_to_host(dst_np.ctypes.data_as(C.c_void_p), C.c_void_p(src_ptr), dst_np.nbytes, None))
