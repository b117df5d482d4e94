"""ctypes mirrors of the structs declared in include/sessd3d.h (field order must match)."""
import ctypes as C

SESSD_FLOAT = 0
SESSD_HALF = 1
SESSD_INT32 = 3

SESSD_OK = 0
SESSD_E_INVALID = 1
SESSD_E_UNSUPPORTED = 2
SESSD_E_HIP = 3
SESSD_E_NOMEM = 4

SESSD_STATUS_VOXEL_OVERFLOW = 1
SESSD_STATUS_HASH_FULL = 2
SESSD_STATUS_BAD_COORD = 4

SESSD_FLAG_SKIP_PAD_ROWS = 1
SESSD_FLAG_FORCE_VALU = 2

SESSD_LAYER_SUBM = 0
SESSD_LAYER_SPARSE = 1


class TensorDesc(C.Structure):
    _fields_ = [("nbDims", C.c_int32), ("d", C.c_int32 * 8), ("type", C.c_int32),
                ("format", C.c_int32), ("scale", C.c_float)]

    @staticmethod
    def make(dims, dtype):
        t = TensorDesc()
        t.nbDims = len(dims)
        for i, v in enumerate(dims):
            t.d[i] = int(v)
        t.type = dtype
        t.format = 0
        t.scale = 1.0
        return t


class VoxelGenDesc(C.Structure):
    _fields_ = [("max_num_points_per_voxel", C.c_int32), ("max_voxels", C.c_int32),
                ("point_cloud_range", C.c_float * 6), ("voxel_feature_num", C.c_int32),
                ("voxel_size", C.c_float * 3)]


class SubmConv3dDesc(C.Structure):
    _fields_ = [("in_channel", C.c_int32), ("out_channel", C.c_int32), ("max_voxels", C.c_int32),
                ("feature_num", C.c_int32), ("out_shape", C.c_int32 * 3),
                ("spatial_shape", C.c_int32 * 3), ("ksize", C.c_int32), ("stride", C.c_int32),
                ("padding", C.c_int32), ("dilation", C.c_int32), ("out_padding", C.c_int32)]


class SparseConv3dDesc(C.Structure):
    _fields_ = [("in_channel", C.c_int32), ("out_channel", C.c_int32), ("max_voxels", C.c_int32),
                ("feature_num", C.c_int32), ("out_shape", C.c_int32 * 3),
                ("spatial_shape", C.c_int32 * 3), ("ksize", C.c_int32 * 3),
                ("stride", C.c_int32 * 3), ("padding", C.c_int32 * 3), ("dilation", C.c_int32),
                ("out_padding", C.c_int32)]


class Sparse2DenseDesc(C.Structure):
    _fields_ = [("feature_map_size", C.c_int32 * 3), ("feature_map_channel", C.c_int32)]


class LayerSpec(C.Structure):
    _fields_ = [("type", C.c_int32), ("in_channel", C.c_int32), ("out_channel", C.c_int32),
                ("ksize", C.c_int32 * 3), ("stride", C.c_int32 * 3), ("padding", C.c_int32 * 3),
                ("out_shape", C.c_int32 * 3)]


SESSD_FIELD_FLOAT32 = 1
SESSD_FIELD_INT32 = 5


class PluginField(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("type", C.c_int32), ("length", C.c_int32)]


class PluginFieldCollection(C.Structure):
    _fields_ = [("nbFields", C.c_int32), ("fields", C.POINTER(PluginField))]


FloatPP = C.POINTER(C.POINTER(C.c_float))


class PipelineDesc(C.Structure):
    _fields_ = [("voxelgen", VoxelGenDesc), ("max_points", C.c_int32),
                ("point_features", C.c_int32), ("n_layers", C.c_int32),
                ("layers", C.POINTER(LayerSpec)), ("weights", FloatPP), ("scale", FloatPP),
                ("shift", FloatPP), ("relu", C.c_int32), ("feature_dtype", C.c_int32),
                ("dense", Sparse2DenseDesc), ("share_rulebooks", C.c_int32), ("flags", C.c_int32),
                ("use_graph", C.c_int32), ("layer_max_voxels", C.c_int32), ("overlap_streams", C.c_int32),
                ("dense_padding", C.c_int32 * 4), ("frames_in_flight", C.c_int32)]
