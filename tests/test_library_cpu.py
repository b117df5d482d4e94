"""CPU-only checks of the C-ABI library: it loads, exports every declared symbol, and the host logic
that needs no GPU (descriptors, serialisation, grid derivation, argument checking) behaves like the
reference plugins.  No kernel is launched here."""
import ctypes as C
import struct

import numpy as np
import pytest

from sessd3d import api, backbone as B, ctypes_defs as D


def test_library_exports_every_declared_symbol():
    L = api.lib()
    names = api.declared_symbols()
    assert len(names) >= 50
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    assert b"gfx950" in L.sessd_version()


def test_struct_layouts_match_header_sizes():
    assert C.sizeof(D.TensorDesc) == 4 + 32 + 4 + 4 + 4
    assert C.sizeof(D.VoxelGenDesc) == 4 + 4 + 24 + 4 + 12
    assert C.sizeof(D.SubmConv3dDesc) == 4 * 4 + 12 + 12 + 5 * 4
    assert C.sizeof(D.SparseConv3dDesc) == 4 * 4 + 12 * 5 + 2 * 4
    assert C.sizeof(D.Sparse2DenseDesc) == 16
    assert C.sizeof(D.LayerSpec) == 12 + 12 * 4


def test_header_compiles_as_c_and_the_ctypes_mirror_matches_it(tmp_path):
    """include/sessd3d.h is a C header (C99, -pedantic): a C program built against it prints the size of every
    struct and the offset of every field, and the ctypes mirror the tests and the benchmark bind with must
    agree field by field."""
    import os
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pairs = [("sessd_tensor_desc", D.TensorDesc), ("sessd_voxelgen_desc", D.VoxelGenDesc),
             ("sessd_submconv3d_desc", D.SubmConv3dDesc), ("sessd_sparseconv3d_desc", D.SparseConv3dDesc),
             ("sessd_sparse2dense_desc", D.Sparse2DenseDesc), ("sessd_layer_spec", D.LayerSpec),
             ("sessd_pipeline_desc", D.PipelineDesc)]
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "sessd3d.h"', 'int main(void) {']
    for cname, mirror in pairs:
        lines.append('    printf("%s %%zu\\n", sizeof(%s));' % (cname, cname))
        for fname, _ in mirror._fields_:
            lines.append('    printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (cname, fname, cname, fname))
    lines += ['    return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                    str(src), "-o", str(exe)], check=True)
    out = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, mirror in pairs:
        assert int(out[cname]) == C.sizeof(mirror), cname
        for fname, _ in mirror._fields_:
            assert int(out["%s.%s" % (cname, fname)]) == getattr(mirror, fname).offset, (cname, fname)


def test_reference_backbone_table_matches_python_table():
    L = api.lib()
    specs = (D.LayerSpec * 14)()
    vg, dd = D.VoxelGenDesc(), D.Sparse2DenseDesc()
    assert L.sessd_reference_backbone(specs, 14, C.byref(vg), C.byref(dd)) == 14
    for s, l in zip(specs, B.reference_layers()):
        assert (s.type, s.in_channel, s.out_channel) == (l.type, l.cin, l.cout)
        assert tuple(s.ksize) == l.ksize and tuple(s.stride) == l.stride and tuple(s.padding) == l.padding
        assert tuple(s.out_shape) == l.out_shape
    assert vg.max_voxels == 60000 and vg.max_num_points_per_voxel == 5
    assert np.allclose(list(vg.point_cloud_range), B.POINT_CLOUD_RANGE) and np.allclose(list(vg.voxel_size), B.VOXEL_SIZE)
    assert tuple(dd.feature_map_size) == (176, 200, 2) and dd.feature_map_channel == 64
    # each sparse layer's out grid follows from the previous grid (spconv formula)
    g = (1408, 1600, 41)
    for l in B.reference_layers():
        if l.type == D.SESSD_LAYER_SPARSE:
            g = tuple(B.conv_out_size(g[a], l.ksize[2 - a], l.stride[2 - a], l.padding[2 - a]) for a in range(3))
        assert l.out_shape == g


def test_voxelgen_host_side():
    vg = api.VoxelGenerator(max_voxels=20000)
    blob = vg.serialize()
    # voxelGenerator.cu:584-599: 3 ints, 9 floats, 4 ints
    assert len(blob) == 7 * 4 + 9 * 4
    f = struct.unpack("<3i9f4i", blob)
    assert f[:3] == (20000, 5, 4)
    assert np.allclose(f[3:12], [0.0, 70.4, -40.0, 40.0, -3.0, 1.0, 0.05, 0.05, 0.1])
    assert f[13:] == (1408, 1600, 40)          # grid derived at create, as configurePlugin would
    assert vg.grid_size() == (1408, 1600, 40)
    vg2 = api.VoxelGenerator.deserialize(blob)
    assert vg2.serialize() == blob
    ind = (D.TensorDesc * 2)(D.TensorDesc.make([1, 80000, 4], D.SESSD_FLOAT), D.TensorDesc.make([1], D.SESSD_INT32))
    outd = (D.TensorDesc * 3)(D.TensorDesc.make([1, 20000, 4], D.SESSD_FLOAT),
                              D.TensorDesc.make([1, 20000, 4], D.SESSD_INT32), D.TensorDesc.make([1], D.SESSD_INT32))
    L = api.lib()
    assert L.sessd_voxelgen_configure(vg.h, ind, 2, outd, 3) == 0
    ws = L.sessd_voxelgen_workspace_size(vg.h, ind, 2, outd, 3)
    # hash table instead of the reference's 721 MB dense slot table
    assert 0 < ws < 16 * 2 ** 20
    # enqueue argument checking happens before any launch
    assert L.sessd_voxelgen_enqueue(vg.h, ind, outd, None, None, None, None) == D.SESSD_E_INVALID
    assert b"null" in L.sessd_last_error()


def test_voxelgen_static_enqueue_rejects_oversize_before_any_gpu_call():
    """sessd_voxelgen_enqueue_static: a points tensor whose scratch layout exceeds the library's static 8 MiB array
    is refused with a message that names both sizes, before any runtime call (so it is testable without a GPU)."""
    vg = api.VoxelGenerator(max_voxels=60000)
    L = api.lib()
    ind = (D.TensorDesc * 2)(D.TensorDesc.make([1, 150000, 4], D.SESSD_FLOAT), D.TensorDesc.make([1], D.SESSD_INT32))
    outd = (D.TensorDesc * 3)(D.TensorDesc.make([1, 60000, 4], D.SESSD_FLOAT),
                              D.TensorDesc.make([1, 60000, 4], D.SESSD_INT32), D.TensorDesc.make([1], D.SESSD_INT32))
    fake = (C.c_void_p * 3)(16, 32, 48)                       # never dereferenced: the call fails first
    assert L.sessd_voxelgen_workspace_size(vg.h, ind, 2, outd, 3) > 8 * 2 ** 20
    assert L.sessd_voxelgen_enqueue_static(vg.h, ind, outd, fake, fake, None) == D.SESSD_E_INVALID
    msg = L.sessd_last_error()
    assert b"static buffer holds 8388608" in msg and b"150000" in msg
    ind[0] = D.TensorDesc.make([1, 80000, 4], D.SESSD_FLOAT)  # the reference's shape fits
    assert L.sessd_voxelgen_workspace_size(vg.h, ind, 2, outd, 3) <= 8 * 2 ** 20
    assert L.sessd_voxelgen_enqueue_static(None, ind, outd, fake, fake, None) == D.SESSD_E_INVALID


def test_voxelgen_create_rejects_bad_fields():
    L = api.lib()
    d = B.voxelgen_desc()
    d.voxel_size[1] = 0.0
    h = C.c_void_p()
    assert L.sessd_voxelgen_create(C.byref(d), C.byref(h)) == D.SESSD_E_INVALID
    d = B.voxelgen_desc()
    d.voxel_feature_num = 5
    assert L.sessd_voxelgen_create(C.byref(d), C.byref(h)) == D.SESSD_E_UNSUPPORTED
    assert L.sessd_voxelgen_deserialize(b"\0" * 10, 10, C.byref(h)) == D.SESSD_E_INVALID


def test_sparse2dense_host_side():
    s = api.Sparse2Dense()
    blob = s.serialize()
    assert struct.unpack("<4i", blob) == (176, 200, 2, 64)   # sparse2Dense.cu:288-295
    assert api.Sparse2Dense.deserialize(blob).serialize() == blob
    L = api.lib()
    d = B.dense_desc((176, 0, 2), 64)
    h = C.c_void_p()
    assert L.sessd_sparse2dense_create(C.byref(d), C.byref(h)) == D.SESSD_E_INVALID
    # with a border the blob grows by a tagged trailer in the order of zeroPad2d.cu:283-290
    p = api.Sparse2Dense(padding=(1, 2, 3, 4))
    blob = p.serialize()
    assert struct.unpack("<4i", blob[:16]) == (176, 200, 2, 64) and struct.unpack("<4i", blob[20:]) == (1, 2, 3, 4)
    assert api.Sparse2Dense.deserialize(blob).serialize() == blob
    assert L.sessd_sparse2dense_set_padding(p.h, -1, 0, 0, 0) == D.SESSD_E_INVALID
    # the workspace: status block, one word per 256 rows, the cell -> row map; an enqueue without one is refused
    # before any runtime call (the reference's plugin needs none, sparse2Dense.cu:175-179)
    ind = (D.TensorDesc * 3)(D.TensorDesc.make([1, 60000, 64], D.SESSD_FLOAT), D.TensorDesc.make([1, 60000, 4], D.SESSD_INT32),
                             D.TensorDesc.make([1], D.SESSD_INT32))
    outd = (D.TensorDesc * 1)(D.TensorDesc.make([1, 128, 200, 176], D.SESSD_FLOAT))
    assert L.sessd_sparse2dense_configure(s.h, ind, 3, outd, 1) == D.SESSD_OK
    assert L.sessd_sparse2dense_workspace_size(s.h, ind, 3, outd, 1) == 256 + 1024 + 2 * 200 * 176 * 4
    fake = (C.c_void_p * 3)(4096, 8192, 12288)                # never dereferenced: the call fails first
    assert L.sessd_sparse2dense_enqueue(s.h, ind, outd, fake, fake, None, None) == D.SESSD_E_INVALID
    assert b"workspace" in L.sessd_last_error()


def test_conv_create_validates_before_touching_the_gpu():
    L = api.lib()
    h = C.c_void_p()
    w = np.zeros((27, 4, 16), np.float32)
    d = D.SubmConv3dDesc()
    d.in_channel, d.out_channel, d.max_voxels, d.feature_num = 4, 16, 1000, 4
    for a, v in enumerate((140, 160, 41)):
        d.out_shape[a] = d.spatial_shape[a] = v
    d.ksize, d.stride, d.padding, d.dilation = 5, 1, 2, 1      # 125 offsets: beyond the rulebook's 27
    assert L.sessd_submconv3d_create(C.byref(d), w.ctypes.data_as(C.c_void_p), C.byref(h)) == D.SESSD_E_UNSUPPORTED
    d.ksize, d.padding, d.stride = 3, 1, 2
    assert L.sessd_submconv3d_create(C.byref(d), w.ctypes.data_as(C.c_void_p), C.byref(h)) == D.SESSD_E_UNSUPPORTED
    sd = D.SparseConv3dDesc()
    sd.in_channel, sd.out_channel, sd.max_voxels = 4, 16, 1000
    for a in range(3):
        sd.out_shape[a] = sd.spatial_shape[a] = 10
        sd.ksize[a], sd.stride[a], sd.padding[a] = 3, 0, 1      # zero stride
    sd.dilation = 1
    assert L.sessd_sparseconv3d_create(C.byref(sd), w.ctypes.data_as(C.c_void_p), C.byref(h)) == D.SESSD_E_INVALID
    assert L.sessd_submconv3d_create(None, None, None) == D.SESSD_E_INVALID


def test_creators_by_name_list_and_read_the_reference_fields():
    """sessd_plugin_field_names / sessd_plugin_create: the reference's creators by PLUGIN_NAME, fields picked by name."""
    names = dict((n, [f[0] for f in api.plugin_field_names(n)]) for n in
                 ("VoxelGeneratorPlugin", "SubmConv3dLayerPlugin", "SparseConv3dLayerPlugin", "Sparse2DensePlugin"))
    assert names["VoxelGeneratorPlugin"] == ["max_num_points_per_voxel", "max_voxels", "point_cloud_range",
                                             "voxel_feature_num", "voxel_size"]            # voxelGenerator.cu:624-628
    conv = ["in_channel", "out_channel", "max_voxels", "feature_num", "out_shape", "spatial_shape", "ksize", "stride",
            "padding", "dilation", "out_padding", "weights"]                                 # submConv3dlayer.cu:737-748
    assert names["SubmConv3dLayerPlugin"] == conv and names["SparseConv3dLayerPlugin"] == conv
    assert names["Sparse2DensePlugin"] == ["feature_map_size", "feature_map_channel"]      # sparse2Dense.cu:321-322
    assert dict((f[0], f[2]) for f in api.plugin_field_names("SparseConv3dLayerPlugin"))["ksize"] == 3
    assert dict((f[0], f[2]) for f in api.plugin_field_names("SubmConv3dLayerPlugin"))["ksize"] == 1
    with pytest.raises(api.SessdError, match="no plugin named"):
        api.plugin_field_names("ZeroPad2dPlugin")
    # the voxelizer and sparse2Dense need no GPU to be created: by name == by descriptor, field order free
    i32, f32 = (lambda *v: np.array(v, np.int32)), (lambda *v: np.array(v, np.float32))
    vg = api.create_plugin("VoxelGeneratorPlugin", {
        "voxel_size": f32(*B.VOXEL_SIZE), "max_voxels": i32(20000), "ignored_extra_field": i32(7),
        "point_cloud_range": f32(*B.POINT_CLOUD_RANGE), "voxel_feature_num": i32(4), "max_num_points_per_voxel": i32(5)})
    assert vg.serialize() == api.VoxelGenerator(max_voxels=20000).serialize() and vg.grid_size() == (1408, 1600, 40)
    s2d = api.create_plugin("Sparse2DensePlugin", {"feature_map_channel": i32(64), "feature_map_size": i32(176, 200, 2)})
    assert s2d.serialize() == api.Sparse2Dense().serialize()
    with pytest.raises(api.SessdError, match="field 'voxel_size' is missing"):
        api.create_plugin("VoxelGeneratorPlugin", {"max_voxels": i32(1), "max_num_points_per_voxel": i32(5),
                                                   "point_cloud_range": f32(*B.POINT_CLOUD_RANGE), "voxel_feature_num": i32(4)})
    with pytest.raises(api.SessdError, match="has type 5, the creator reads type 1"):
        api.create_plugin("VoxelGeneratorPlugin", {"max_voxels": i32(1), "max_num_points_per_voxel": i32(5), "voxel_size": i32(1, 1, 1),
                                                   "point_cloud_range": f32(*B.POINT_CLOUD_RANGE), "voxel_feature_num": i32(4)})
    # a vector field declared shorter than what the creator reads is refused (read out of bounds otherwise); the
    # reference's own declaration -- length 1 on every field -- is accepted
    with pytest.raises(api.SessdError, match="field 'point_cloud_range' declares 2 elements, the creator reads 6"):
        api.create_plugin("VoxelGeneratorPlugin", {"max_voxels": i32(1), "max_num_points_per_voxel": i32(5), "voxel_size": f32(*B.VOXEL_SIZE),
                                                   "point_cloud_range": f32(0, 1), "voxel_feature_num": i32(4)})
    with pytest.raises(api.SessdError, match="field 'feature_map_size' declares 2 elements, the creator reads 3"):
        api.create_plugin("Sparse2DensePlugin", {"feature_map_channel": i32(64), "feature_map_size": i32(176, 200)})
    keep = [np.ascontiguousarray(v) for v in (i32(64), i32(176, 200, 2))]
    arr = (D.PluginField * 2)()
    for i, (k, a) in enumerate(zip((b"feature_map_channel", b"feature_map_size"), keep)):
        arr[i].name, arr[i].data, arr[i].type, arr[i].length = k, a.ctypes.data, D.SESSD_FIELD_INT32, 1
    h = C.c_void_p()
    assert api.lib().sessd_plugin_create(b"Sparse2DensePlugin", C.byref(D.PluginFieldCollection(2, arr)), C.byref(h)) == 0
    api.lib().sessd_sparse2dense_destroy(h)
    with pytest.raises(api.SessdError, match="field 'weights' is missing"):      # checked before any GPU call
        api.create_plugin("SubmConv3dLayerPlugin", {k: i32(*([3] * (3 if "shape" in k else 1))) for k in conv[:-1]})
    with pytest.raises(api.SessdError, match="holds 5 values"):
        api.create_plugin("SubmConv3dLayerPlugin", dict({k: i32(*([3] * (3 if "shape" in k else 1))) for k in conv[:-1]},
                                                        weights=f32(1, 2, 3, 4, 5)))


def test_clone_of_the_gpu_free_plugins():
    vg = api.VoxelGenerator(max_voxels=1234)
    vg.set_flags(D.SESSD_FLAG_SKIP_PAD_ROWS)
    c = vg.clone()
    assert c.h.value != vg.h.value and c.serialize() == vg.serialize() and c.max_voxels == 1234
    p = api.Sparse2Dense(padding=(1, 1, 2, 2))
    c = p.clone()
    assert c.serialize() == p.serialize() and c.padding == (1, 1, 2, 2)
    assert api.lib().sessd_voxelgen_clone(None, None) == D.SESSD_E_INVALID


def test_pipeline_frames_in_flight_is_validated_before_anything_is_built():
    L = api.lib()
    specs = (D.LayerSpec * 14)()
    d = D.PipelineDesc()
    assert L.sessd_reference_backbone(specs, 14, C.byref(d.voxelgen), C.byref(d.dense)) == 14
    d.max_points, d.point_features, d.n_layers, d.layers = 1000, 4, 14, specs
    h = C.c_void_p()
    d.frames_in_flight, d.overlap_streams = 9, 1
    assert L.sessd_pipeline_create(C.byref(d), C.byref(h)) == D.SESSD_E_INVALID and b"at most 8" in L.sessd_last_error()
    d.frames_in_flight, d.overlap_streams = 3, 0
    assert L.sessd_pipeline_create(C.byref(d), C.byref(h)) == D.SESSD_E_INVALID and b"overlap_streams" in L.sessd_last_error()
    assert L.sessd_pipeline_submit(None, None, None, None, None, None) == D.SESSD_E_INVALID
    assert L.sessd_pipeline_join(None, 0, None) == D.SESSD_E_INVALID
