// c_api.hip -- extern "C" surface of libsessd3d (declared in include/sessd3d.h): thin forwarding
// to the plugin classes; only plain pointers and sizes cross the boundary.
#include "plugins.h"

namespace sessd {
const char* last_error_cstr();
}

using namespace sessd;

#define H_VG(h) reinterpret_cast<VoxelGeneratorPlugin*>(h)
#define H_SUBM(h) reinterpret_cast<SubmConv3dLayerPlugin*>(h)
#define H_SP(h) reinterpret_cast<SparseConv3dLayerPlugin*>(h)
#define H_S2D(h) reinterpret_cast<Sparse2DensePlugin*>(h)
#define CH_VG(h) reinterpret_cast<const VoxelGeneratorPlugin*>(h)
#define CH_SUBM(h) reinterpret_cast<const SubmConv3dLayerPlugin*>(h)
#define CH_SP(h) reinterpret_cast<const SparseConv3dLayerPlugin*>(h)
#define CH_S2D(h) reinterpret_cast<const Sparse2DensePlugin*>(h)
#define NEED(cond, what)                                                  \
    do {                                                                  \
        if (!(cond)) return fail(SESSD_E_INVALID, "%s: %s", __func__, what); \
    } while (0)

extern "C" {

const char* sessd_last_error(void) { return last_error_cstr(); }
const char* sessd_version(void) { return "sessd3d 0.1 (gfx950)"; }
int sessd_copy_to_host(void* dst_host, const void* src_device, size_t bytes, sessd_stream_t stream_) {
    NEED(dst_host && src_device, "null argument");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    SESSD_HIP_TRY(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, stream));
    SESSD_HIP_TRY(hipStreamSynchronize(stream));
    return SESSD_OK;
}

// ------------------------------------------------------------------ voxelgen
int sessd_voxelgen_create(const sessd_voxelgen_desc* desc, sessd_voxelgen** out) {
    NEED(desc && out, "null argument");
    return guarded(__func__, [&]() -> int {
        VoxelGeneratorPlugin* p = nullptr;
        SESSD_TRY(VoxelGeneratorPlugin::create(*desc, &p));
        *out = reinterpret_cast<sessd_voxelgen*>(p);
        return SESSD_OK;
    });
}
int sessd_voxelgen_deserialize(const void* bytes, size_t n, sessd_voxelgen** out) {
    NEED(out, "null argument");
    return guarded(__func__, [&]() -> int {
        VoxelGeneratorPlugin* p = nullptr;
        SESSD_TRY(VoxelGeneratorPlugin::deserialize(bytes, n, &p));
        *out = reinterpret_cast<sessd_voxelgen*>(p);
        return SESSD_OK;
    });
}
size_t sessd_voxelgen_serialization_size(const sessd_voxelgen* h) { return h ? CH_VG(h)->getSerializationSize() : 0; }
int sessd_voxelgen_serialize(const sessd_voxelgen* h, void* buf) {
    NEED(h && buf, "null argument");
    CH_VG(h)->serialize(buf);
    return SESSD_OK;
}
int sessd_voxelgen_configure(sessd_voxelgen* h, const sessd_tensor_desc* in, int nIn, const sessd_tensor_desc* out,
                             int nOut) {
    NEED(h, "null handle");
    return H_VG(h)->configurePlugin(in, nIn, out, nOut);
}
int sessd_voxelgen_grid_size(const sessd_voxelgen* h, int32_t grid_xyz[3]) {
    NEED(h && grid_xyz, "null argument");
    grid_xyz[0] = CH_VG(h)->grid_x_size_;
    grid_xyz[1] = CH_VG(h)->grid_y_size_;
    grid_xyz[2] = CH_VG(h)->grid_z_size_;
    return SESSD_OK;
}
size_t sessd_voxelgen_workspace_size(const sessd_voxelgen* h, const sessd_tensor_desc* in, int nIn,
                                     const sessd_tensor_desc* out, int nOut) {
    return h ? CH_VG(h)->getWorkspaceSize(in, nIn, out, nOut) : 0;
}
int sessd_voxelgen_enqueue(sessd_voxelgen* h, const sessd_tensor_desc* inDesc, const sessd_tensor_desc* outDesc,
                           const void* const* inputs, void* const* outputs, void* workspace, sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_VG(h)->enqueue(inDesc, outDesc, inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}
int sessd_voxelgen_enqueue_static(sessd_voxelgen* h, const sessd_tensor_desc* inDesc, const sessd_tensor_desc* outDesc,
                                  const void* const* inputs, void* const* outputs, sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_VG(h)->enqueueStatic(inDesc, outDesc, inputs, outputs, static_cast<hipStream_t>(stream));
}
int sessd_voxelgen_status(const sessd_voxelgen* h, const void* workspace, sessd_stream_t stream, int32_t* status) {
    NEED(h && status, "null argument");
    NEED(CH_VG(h)->lastMaxPoints_ > 0, "configure or enqueue must run first (the layout depends on max_points)");
    void* own = nullptr;
    if (!workspace) {  // the static scratch of sessd_voxelgen_enqueue_static on the current device
        SESSD_TRY(voxelgen_static_scratch(&own));
        workspace = own;
    }
    return read_status_word(workspace, CH_VG(h)->statusOffset(CH_VG(h)->lastMaxPoints_),
                            static_cast<hipStream_t>(stream), status);
}
int sessd_voxelgen_set_flags(sessd_voxelgen* h, int32_t flags) {
    NEED(h, "null handle");
    H_VG(h)->flags_ = flags;
    return SESSD_OK;
}
void sessd_voxelgen_destroy(sessd_voxelgen* h) { delete H_VG(h); }

// ------------------------------------------------------------------ submconv3d
int sessd_submconv3d_create(const sessd_submconv3d_desc* desc, const float* weights, sessd_submconv3d** out) {
    NEED(desc && weights && out, "null argument");
    return guarded(__func__, [&]() -> int {
        SubmConv3dLayerPlugin* p = nullptr;
        SESSD_TRY(SubmConv3dLayerPlugin::create(*desc, weights, &p));
        *out = reinterpret_cast<sessd_submconv3d*>(p);
        return SESSD_OK;
    });
}
int sessd_submconv3d_deserialize(const void* bytes, size_t n, sessd_submconv3d** out) {
    NEED(out, "null argument");
    return guarded(__func__, [&]() -> int {
        SubmConv3dLayerPlugin* p = nullptr;
        SESSD_TRY(SubmConv3dLayerPlugin::deserialize(bytes, n, &p));
        *out = reinterpret_cast<sessd_submconv3d*>(p);
        return SESSD_OK;
    });
}
size_t sessd_submconv3d_serialization_size(const sessd_submconv3d* h) {
    return h ? CH_SUBM(h)->getSerializationSize() : 0;
}
int sessd_submconv3d_serialize(const sessd_submconv3d* h, void* buf) {
    NEED(h && buf, "null argument");
    CH_SUBM(h)->serialize(buf);
    return SESSD_OK;
}
int sessd_submconv3d_configure(sessd_submconv3d* h, const sessd_tensor_desc* in, int nIn,
                               const sessd_tensor_desc* out, int nOut) {
    NEED(h, "null handle");
    return guarded(__func__, [&]() -> int { return H_SUBM(h)->configurePlugin(in, nIn, out, nOut); });
}
size_t sessd_submconv3d_workspace_size(const sessd_submconv3d* h, const sessd_tensor_desc* in, int nIn,
                                       const sessd_tensor_desc* out, int nOut) {
    return h ? CH_SUBM(h)->getWorkspaceSize(in, nIn, out, nOut) : 0;
}
int sessd_submconv3d_enqueue(sessd_submconv3d* h, const sessd_tensor_desc* inDesc, const sessd_tensor_desc* outDesc,
                             const void* const* inputs, void* const* outputs, void* workspace,
                             sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_SUBM(h)->enqueue(inDesc, outDesc, inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}
int sessd_submconv3d_enqueue_shared(sessd_submconv3d* h, const sessd_tensor_desc* inDesc,
                                    const sessd_tensor_desc* outDesc, const void* const* inputs,
                                    void* const* outputs, const void* rulebook_workspace, sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_SUBM(h)->enqueueShared(inDesc, outDesc, inputs, outputs, rulebook_workspace,
                                    static_cast<hipStream_t>(stream));
}
int sessd_submconv3d_export_rulebook(const sessd_submconv3d* h, const void* workspace, int32_t* indice_pairs,
                                     uint32_t* indice_num, sessd_stream_t stream) {
    NEED(h, "null handle");
    return CH_SUBM(h)->exportRulebook(workspace, indice_pairs, indice_num, static_cast<hipStream_t>(stream));
}
int sessd_submconv3d_set_epilogue(sessd_submconv3d* h, const float* scale, const float* shift, int relu) {
    NEED(h, "null handle");
    return guarded(__func__, [&]() -> int {
        return H_SUBM(h)->setEpilogue(scale, shift, relu);
    });
}
int sessd_submconv3d_set_flags(sessd_submconv3d* h, int32_t flags) {
    NEED(h, "null handle");
    H_SUBM(h)->flags_ = flags;
    return SESSD_OK;
}
int sessd_submconv3d_status(const sessd_submconv3d* h, const void* workspace, sessd_stream_t stream,
                            int32_t* status) {
    NEED(h && workspace && status, "null argument");
    return read_status_word(workspace, CH_SUBM(h)->statusOffset(), static_cast<hipStream_t>(stream), status);
}
void sessd_submconv3d_destroy(sessd_submconv3d* h) { delete H_SUBM(h); }

// ------------------------------------------------------------------ sparseconv3d
int sessd_sparseconv3d_create(const sessd_sparseconv3d_desc* desc, const float* weights, sessd_sparseconv3d** out) {
    NEED(desc && weights && out, "null argument");
    return guarded(__func__, [&]() -> int {
        SparseConv3dLayerPlugin* p = nullptr;
        SESSD_TRY(SparseConv3dLayerPlugin::create(*desc, weights, &p));
        *out = reinterpret_cast<sessd_sparseconv3d*>(p);
        return SESSD_OK;
    });
}
int sessd_sparseconv3d_deserialize(const void* bytes, size_t n, sessd_sparseconv3d** out) {
    NEED(out, "null argument");
    return guarded(__func__, [&]() -> int {
        SparseConv3dLayerPlugin* p = nullptr;
        SESSD_TRY(SparseConv3dLayerPlugin::deserialize(bytes, n, &p));
        *out = reinterpret_cast<sessd_sparseconv3d*>(p);
        return SESSD_OK;
    });
}
size_t sessd_sparseconv3d_serialization_size(const sessd_sparseconv3d* h) {
    return h ? CH_SP(h)->getSerializationSize() : 0;
}
int sessd_sparseconv3d_serialize(const sessd_sparseconv3d* h, void* buf) {
    NEED(h && buf, "null argument");
    CH_SP(h)->serialize(buf);
    return SESSD_OK;
}
int sessd_sparseconv3d_configure(sessd_sparseconv3d* h, const sessd_tensor_desc* in, int nIn,
                                 const sessd_tensor_desc* out, int nOut) {
    NEED(h, "null handle");
    return guarded(__func__, [&]() -> int { return H_SP(h)->configurePlugin(in, nIn, out, nOut); });
}
size_t sessd_sparseconv3d_workspace_size(const sessd_sparseconv3d* h, const sessd_tensor_desc* in, int nIn,
                                         const sessd_tensor_desc* out, int nOut) {
    return h ? CH_SP(h)->getWorkspaceSize(in, nIn, out, nOut) : 0;
}
int sessd_sparseconv3d_enqueue(sessd_sparseconv3d* h, const sessd_tensor_desc* inDesc,
                               const sessd_tensor_desc* outDesc, const void* const* inputs, void* const* outputs,
                               void* workspace, sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_SP(h)->enqueue(inDesc, outDesc, inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}
int sessd_sparseconv3d_export_rulebook(const sessd_sparseconv3d* h, const void* workspace, int32_t* indice_pairs,
                                       uint32_t* indice_num, sessd_stream_t stream) {
    NEED(h, "null handle");
    return CH_SP(h)->exportRulebook(workspace, indice_pairs, indice_num, static_cast<hipStream_t>(stream));
}
int sessd_sparseconv3d_set_epilogue(sessd_sparseconv3d* h, const float* scale, const float* shift, int relu) {
    NEED(h, "null handle");
    return guarded(__func__, [&]() -> int {
        return H_SP(h)->setEpilogue(scale, shift, relu);
    });
}
int sessd_sparseconv3d_set_flags(sessd_sparseconv3d* h, int32_t flags) {
    NEED(h, "null handle");
    H_SP(h)->flags_ = flags;
    return SESSD_OK;
}
int sessd_sparseconv3d_status(const sessd_sparseconv3d* h, const void* workspace, sessd_stream_t stream,
                              int32_t* status) {
    NEED(h && workspace && status, "null argument");
    return read_status_word(workspace, CH_SP(h)->statusOffset(), static_cast<hipStream_t>(stream), status);
}
void sessd_sparseconv3d_destroy(sessd_sparseconv3d* h) { delete H_SP(h); }

// ------------------------------------------------------------------ sparse2dense
int sessd_sparse2dense_create(const sessd_sparse2dense_desc* desc, sessd_sparse2dense** out) {
    NEED(desc && out, "null argument");
    return guarded(__func__, [&]() -> int {
        Sparse2DensePlugin* p = nullptr;
        SESSD_TRY(Sparse2DensePlugin::create(*desc, &p));
        *out = reinterpret_cast<sessd_sparse2dense*>(p);
        return SESSD_OK;
    });
}
int sessd_sparse2dense_deserialize(const void* bytes, size_t n, sessd_sparse2dense** out) {
    NEED(out, "null argument");
    return guarded(__func__, [&]() -> int {
        Sparse2DensePlugin* p = nullptr;
        SESSD_TRY(Sparse2DensePlugin::deserialize(bytes, n, &p));
        *out = reinterpret_cast<sessd_sparse2dense*>(p);
        return SESSD_OK;
    });
}
size_t sessd_sparse2dense_serialization_size(const sessd_sparse2dense* h) {
    return h ? CH_S2D(h)->getSerializationSize() : 0;
}
int sessd_sparse2dense_serialize(const sessd_sparse2dense* h, void* buf) {
    NEED(h && buf, "null argument");
    CH_S2D(h)->serialize(buf);
    return SESSD_OK;
}
int sessd_sparse2dense_configure(sessd_sparse2dense* h, const sessd_tensor_desc* in, int nIn,
                                 const sessd_tensor_desc* out, int nOut) {
    NEED(h, "null handle");
    return H_S2D(h)->configurePlugin(in, nIn, out, nOut);
}
size_t sessd_sparse2dense_workspace_size(const sessd_sparse2dense* h, const sessd_tensor_desc* in, int nIn,
                                         const sessd_tensor_desc* out, int nOut) {
    return h ? CH_S2D(h)->getWorkspaceSize(in, nIn, out, nOut) : 0;
}
int sessd_sparse2dense_enqueue(sessd_sparse2dense* h, const sessd_tensor_desc* inDesc,
                               const sessd_tensor_desc* outDesc, const void* const* inputs, void* const* outputs,
                               void* workspace, sessd_stream_t stream) {
    NEED(h, "null handle");
    return H_S2D(h)->enqueue(inDesc, outDesc, inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}
int sessd_sparse2dense_set_padding(sessd_sparse2dense* h, int32_t top, int32_t bottom, int32_t left, int32_t right) {
    NEED(h, "null handle");
    return H_S2D(h)->setPadding(top, bottom, left, right);
}
void sessd_sparse2dense_destroy(sessd_sparse2dense* h) { delete H_S2D(h); }

}  // extern "C"
