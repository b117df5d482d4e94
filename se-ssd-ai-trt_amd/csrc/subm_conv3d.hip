// subm_conv3d.hip -- SubmConv3dLayerPlugin: submanifold 3-D convolution.
//
// Replaces submConv3dlayer.cu:271-641.  The reference memsets a dense int grid over the whole volume
// (369 MB at 41x1600x1408), materialises 27 candidate positions per voxel, appends rulebook pairs
// with atomicAdd and then launches the GEMM kernel 27 times.  Here:
//
//   subm_insert      one thread per active voxel: cell key -> hash table (value = voxel row)
//   subm_neighbours  one thread per (offset k, output row o): look up cell o - padding + k and
//                    write nbr[k][o] (coalesced, one 4-byte store per thread)
//   gather-GEMM      conv_gemm.hip, one launch for all offsets
//
// nbr[k][o] is the rulebook: the pair (i, o) is in the reference's list of offset k exactly when
// nbr[k][o] == i.  sessd_submconv3d_export_rulebook compacts it into the reference's layout.
#include "kernels.h"
#include "plugins.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;

struct Grid3 {
    int X, Y, Z;
};

__device__ __forceinline__ int clamp_count(const int32_t* p, int cap) {
    int n = *p;
    return n < 0 ? 0 : (n > cap ? cap : n);
}

// submConv3dlayer.cu:441-459 (prepareSubMGridKernel) with the dense grid replaced by a hash
__global__ void __launch_bounds__(kBlock)
subm_insert(const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num, int max_voxels,
            Grid3 g, HashTable t, int32_t* meta) {
    const int v = blockIdx.x * kBlock + threadIdx.x;
    const int n = clamp_count(voxel_num, max_voxels);
    if (v == 0) meta[1] = n;
    if (v >= n) return;
    const int4 c = reinterpret_cast<const int4*>(coors)[v];  // (b,z,y,x)
    if (c.y < 0 || c.y >= g.Z || c.z < 0 || c.z >= g.Y || c.w < 0 || c.w >= g.X) {
        atomicOr(&meta[0], SESSD_STATUS_BAD_COORD);  // the reference would write outside its grid
        return;
    }
    const uint32_t key = ((uint32_t)c.y * (uint32_t)g.Y + (uint32_t)c.z) * (uint32_t)g.X + (uint32_t)c.w;
    const int32_t slot = hash_insert(t, key);
    if (slot < 0) {
        atomicOr(&meta[0], SESSD_STATUS_HASH_FULL);
        return;
    }
    atomicMin(&t.vals[slot], (uint32_t)v);
}

// submConv3dlayer.cu:271-358 + 376-424: the pair (i, o) exists at offset (kz,ky,kx) iff the active
// cell i sits at o - padding + k on every axis (stride 1, dilation 1).
__global__ void __launch_bounds__(kBlock)
subm_neighbours(const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num, int max_voxels,
                Grid3 g, int ksize, int padding, HashTable t, int32_t* __restrict__ nbr, int32_t* meta) {
    const int v = blockIdx.x * kBlock + threadIdx.x;
    const int k = blockIdx.y;
    const int n = clamp_count(voxel_num, max_voxels);
    if (meta && v == 0 && k == 0) meta[1] = n;  // (subm_insert's job when that pass runs)
    if (v >= n) return;
    const int4 c = reinterpret_cast<const int4*>(coors)[v];
    const int kz = k / (ksize * ksize), ky = (k / ksize) % ksize, kx = k % ksize;
    const int z = c.y - padding + kz, y = c.z - padding + ky, x = c.w - padding + kx;
    int32_t res = -1;
    const bool self_ok = c.y >= 0 && c.y < g.Z && c.z >= 0 && c.z < g.Y && c.w >= 0 && c.w < g.X;
    if (self_ok && z >= 0 && z < g.Z && y >= 0 && y < g.Y && x >= 0 && x < g.X) {
        const uint32_t key = ((uint32_t)z * (uint32_t)g.Y + (uint32_t)y) * (uint32_t)g.X + (uint32_t)x;
        const int32_t slot = hash_find(t, key);
        if (slot >= 0) res = (int32_t)t.vals[slot];
    }
    nbr[(size_t)k * max_voxels + v] = res;
}

// The same lookup for a 3x3x3 kernel over a table whose rows are unique (coordinates made by the voxelizer or a
// strided layer of this library): the pair (i, o) at offset k is the pair (o, i) at offset 26 - k, so a thread
// probes only the 13 offsets below the centre and writes both directions of a hit; the centre is the row itself.
// Entries 14..26 of the active rows must hold -1 before the launch (MirrorInit: the kernel that created the rows
// wrote them), because only hits are written there.  Half the probes of subm_neighbours.
__global__ void __launch_bounds__(kBlock)
subm_neighbours_mirrored(const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num, int max_voxels,
                         Grid3 g, HashTable t, int32_t* __restrict__ nbr, int32_t* meta) {
    const int v = blockIdx.x * kBlock + threadIdx.x;
    const int k = blockIdx.y;  // 0 .. 13
    const int n = clamp_count(voxel_num, max_voxels);
    if (meta && v == 0 && k == 0) meta[1] = n;
    if (v >= n) return;
    if (k == 13) {
        nbr[(size_t)13 * max_voxels + v] = v;
        return;
    }
    const int4 c = reinterpret_cast<const int4*>(coors)[v];
    const int z = c.y - 1 + k / 9, y = c.z - 1 + (k / 3) % 3, x = c.w - 1 + k % 3;
    int32_t res = -1;
    if (z >= 0 && z < g.Z && y >= 0 && y < g.Y && x >= 0 && x < g.X) {
        const uint32_t key = ((uint32_t)z * (uint32_t)g.Y + (uint32_t)y) * (uint32_t)g.X + (uint32_t)x;
        const int32_t slot = hash_find(t, key);
        if (slot >= 0) res = (int32_t)t.vals[slot];  // (-1 for a cell that was dropped at the capacity)
    }
    nbr[(size_t)k * max_voxels + v] = res;
    if (res >= 0 && res < max_voxels) nbr[(size_t)(26 - k) * max_voxels + res] = v;
}

}  // namespace

struct SubmConv3dLayerPlugin::Layout {
    uint32_t* keys;
    uint32_t* vals;
    int32_t* nbr;
    void* export_scratch;
    int32_t* tiles;  // equal-work tile cuts of the rulebook (tile_cut.hip); first word 0 = none
    int32_t* meta;  // [0] status word, [1] active rows of the last enqueue
    uint32_t cap;
    size_t meta_offset;
    size_t total;
};

SubmConv3dLayerPlugin::Layout SubmConv3dLayerPlugin::carve(void* workspace) const {
    Layout L;
    WorkspaceCarver c(workspace);
    L.cap = next_pow2((uint64_t)(max_voxels_ < 32 ? 32 : max_voxels_) * 2);
    L.keys = c.take<uint32_t>((size_t)L.cap * 2);  // keys then vals: one fill region
    L.vals = L.keys ? L.keys + L.cap : nullptr;
    L.nbr = c.take<int32_t>((size_t)kernel_volume_ * max_voxels_);
    L.export_scratch = c.take<uint8_t>(export_scratch_bytes(kernel_volume_, max_voxels_));
    L.tiles = reinterpret_cast<int32_t*>(c.take<uint8_t>(tile_cut_bytes(max_voxels_)));
    L.meta_offset = c.offset;
    L.meta = c.take<int32_t>(4);
    L.total = c.total();
    return L;
}

int SubmConv3dLayerPlugin::validate() const {
    if (in_channel_ <= 0 || out_channel_ <= 0 || max_voxels_ <= 0)
        return fail(SESSD_E_INVALID, "submconv3d: channels/max_voxels must be positive");
    if (ksize_ != 1 && ksize_ != 3)
        return fail(SESSD_E_UNSUPPORTED, "submconv3d: ksize %d (the rulebook holds at most 27 offsets)", ksize_);
    if (stride_ != 1 || dilation_ != 1)
        return fail(SESSD_E_UNSUPPORTED, "submconv3d: stride and dilation must be 1");
    if (padding_ != ksize_ / 2)
        return fail(SESSD_E_UNSUPPORTED, "submconv3d: padding must be ksize/2 (output sites == input sites)");
    if (out_shape_x_ <= 0 || out_shape_y_ <= 0 || out_shape_z_ <= 0 ||
        (int64_t)out_shape_x_ * out_shape_y_ * out_shape_z_ >= (int64_t)kEmpty)
        return fail(SESSD_E_UNSUPPORTED, "submconv3d: out_shape volume must fit a 32-bit cell key");
    return SESSD_OK;
}

int SubmConv3dLayerPlugin::create(const sessd_submconv3d_desc& d, const float* weights,
                                  SubmConv3dLayerPlugin** out) {
    auto* p = new SubmConv3dLayerPlugin();
    p->in_channel_ = d.in_channel;
    p->out_channel_ = d.out_channel;
    p->max_voxels_ = d.max_voxels;
    p->feature_num_ = d.feature_num;
    p->out_shape_x_ = d.out_shape[0];
    p->out_shape_y_ = d.out_shape[1];
    p->out_shape_z_ = d.out_shape[2];
    p->spatial_shape_x_ = d.spatial_shape[0];
    p->spatial_shape_y_ = d.spatial_shape[1];
    p->spatial_shape_z_ = d.spatial_shape[2];
    p->ksize_ = d.ksize;
    p->stride_ = d.stride;
    p->padding_ = d.padding;
    p->dilation_ = d.dilation;
    p->out_padding_ = d.out_padding;
    p->kernel_volume_ = d.ksize * d.ksize * d.ksize;
    int rc = p->validate();
    if (rc == SESSD_OK)
        rc = p->uploadWeights(weights, (size_t)p->kernel_volume_ * d.in_channel * d.out_channel);
    if (rc != SESSD_OK) {
        delete p;
        return rc;
    }
    *out = p;
    return SESSD_OK;
}

// 16 ints + FP32 weights, submConv3dlayer.cu:684-714 (+ optional epilogue trailer, conv_base.hip)
size_t SubmConv3dLayerPlugin::getSerializationSize() const {
    return (size_t)weights_size_ * sizeof(float) + 16 * sizeof(int) + conv_epilogue_trailer_size(epi_);
}

void SubmConv3dLayerPlugin::serialize(void* buffer) const {
    char* d = static_cast<char*>(buffer);
    writeToBuffer<int>(d, in_channel_);
    writeToBuffer<int>(d, out_channel_);
    writeToBuffer<int>(d, max_voxels_);
    writeToBuffer<int>(d, feature_num_);
    writeToBuffer<int>(d, out_shape_x_);
    writeToBuffer<int>(d, out_shape_y_);
    writeToBuffer<int>(d, out_shape_z_);
    writeToBuffer<int>(d, spatial_shape_x_);
    writeToBuffer<int>(d, spatial_shape_y_);
    writeToBuffer<int>(d, spatial_shape_z_);
    writeToBuffer<int>(d, ksize_);
    writeToBuffer<int>(d, stride_);
    writeToBuffer<int>(d, padding_);
    writeToBuffer<int>(d, dilation_);
    writeToBuffer<int>(d, out_padding_);
    writeToBuffer<int>(d, weights_size_);
    for (int i = 0; i < weights_size_; ++i) writeToBuffer<float>(d, weights_data_[i]);
    conv_write_epilogue_trailer(d, epi_);
}

// The reference's deserialising ctor leaves the device weights unset and relies on TensorRT calling
// clone() (submConv3dlayer.cu:154-196); here the plugin is usable right away.
int SubmConv3dLayerPlugin::deserialize(const void* data, size_t length, SubmConv3dLayerPlugin** out) {
    if (!data || length < 16 * sizeof(int)) return fail(SESSD_E_INVALID, "submconv3d: blob too short");
    const char* d = static_cast<const char*>(data);
    sessd_submconv3d_desc desc;
    desc.in_channel = readFromBuffer<int>(d);
    desc.out_channel = readFromBuffer<int>(d);
    desc.max_voxels = readFromBuffer<int>(d);
    desc.feature_num = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.out_shape[a] = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.spatial_shape[a] = readFromBuffer<int>(d);
    desc.ksize = readFromBuffer<int>(d);
    desc.stride = readFromBuffer<int>(d);
    desc.padding = readFromBuffer<int>(d);
    desc.dilation = readFromBuffer<int>(d);
    desc.out_padding = readFromBuffer<int>(d);
    const int wsize = readFromBuffer<int>(d);
    const int64_t expect = (int64_t)desc.ksize * desc.ksize * desc.ksize * desc.in_channel * desc.out_channel;
    if (wsize < 0 || wsize != expect || length < 16 * sizeof(int) + (size_t)wsize * sizeof(float))
        return fail(SESSD_E_INVALID, "submconv3d: weights_size %d does not match the layer shape", wsize);
    std::vector<float> w((size_t)wsize);
    std::memcpy(w.data(), d, (size_t)wsize * sizeof(float));
    d += (size_t)wsize * sizeof(float);
    SubmConv3dLayerPlugin* p = nullptr;
    SESSD_TRY(create(desc, w.data(), &p));
    const int rc = read_epilogue_trailer(d, length - 16 * sizeof(int) - (size_t)wsize * sizeof(float), p);
    if (rc != SESSD_OK) {
        delete p;
        return rc;
    }
    *out = p;
    return SESSD_OK;
}

int SubmConv3dLayerPlugin::configurePlugin(const sessd_tensor_desc* in, int nbInputs,
                                           const sessd_tensor_desc* out, int nbOutputs) {
    return configureTypes(in, nbInputs, out, nbOutputs);
}

size_t SubmConv3dLayerPlugin::getWorkspaceSize(const sessd_tensor_desc*, int, const sessd_tensor_desc*,
                                               int) const {
    return carve(nullptr).total;
}

size_t SubmConv3dLayerPlugin::statusOffset() const { return carve(nullptr).meta_offset; }

// The two halves of enqueue.  The rulebook depends only on the coordinates, the GEMM only on the
// rulebook and the features: a pipeline may run the halves of different layers on different streams.
// what enqueueBuild clears before it launches anything: a caller that batches the clears of many layers
// into one launch collects them with this and passes prefilled = true
void SubmConv3dLayerPlugin::collectFill(void* workspace, FillArgs& f, bool own_table) const {
    const Layout L = carve(workspace);
    if (own_table) f.add(L.keys, (uint64_t)L.cap * 2, kEmpty);  // (not when the build probes another table)
    f.add(L.tiles, 4, 0);
    f.add(L.meta, 4, 0);
}

int SubmConv3dLayerPlugin::enqueueBuild(const int32_t* coors, const int32_t* voxel_num, void* workspace,
                                        hipStream_t stream, bool prefilled, const HashTable* cells, bool mirrored) {
    if (!coors || !voxel_num || !workspace) return fail(SESSD_E_INVALID, "submconv3d.build: null pointer");
    const Layout L = carve(workspace);
    const HashTable t = make_hash(L.keys, L.vals, L.cap);
    const Grid3 g{out_shape_x_, out_shape_y_, out_shape_z_};
    if (!prefilled) {
        FillArgs f;
        collectFill(workspace, f);
        SESSD_TRY(launch_fill(f, stream));
    }
    const int row_blocks = ceil_div(max_voxels_, kBlock);
    if (!cells)
        hipLaunchKernelGGL(subm_insert, dim3(row_blocks), dim3(kBlock), 0, stream, coors, voxel_num, max_voxels_,
                           g, t, L.meta);
    if (mirrored && cells && kernel_volume_ == 27)
        hipLaunchKernelGGL(subm_neighbours_mirrored, dim3(row_blocks, 14), dim3(kBlock), 0, stream, coors, voxel_num,
                           max_voxels_, g, *cells, L.nbr, L.meta);
    else
        hipLaunchKernelGGL(subm_neighbours, dim3(row_blocks, kernel_volume_), dim3(kBlock), 0, stream, coors,
                           voxel_num, max_voxels_, g, ksize_, padding_, cells ? *cells : t, L.nbr,
                           cells ? L.meta : nullptr);
    SESSD_HIP_TRY(hipGetLastError());
    if (wantTileCuts()) SESSD_TRY(launch_tile_cuts(L.nbr, voxel_num, kernel_volume_, max_voxels_, tileRows(), tileRowWeight(), L.tiles, stream));
    return SESSD_OK;
}

MirrorInit SubmConv3dLayerPlugin::mirrorInit(void* workspace) const {
    MirrorInit m;
    if (kernel_volume_ != 27 || !workspace) return m;
    m.nbr = carve(workspace).nbr;
    m.stride = max_voxels_;
    m.first_offset = 14;
    m.K = 27;
    return m;
}

int SubmConv3dLayerPlugin::enqueueGemm(const void* in_feat, void* out_feat, const int32_t* voxel_num,
                                       const void* rulebook_workspace, hipStream_t stream,
                                       const DenseTarget* dense) {
    if (!in_feat || !out_feat || !voxel_num || !rulebook_workspace)
        return fail(SESSD_E_INVALID, "submconv3d.gemm: null pointer");
    const Layout L = carve(const_cast<void*>(rulebook_workspace));
    return runGemm(in_feat, out_feat, L.nbr, L.tiles, voxel_num, stream, dense);
}

int SubmConv3dLayerPlugin::enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                                   const void* const* inputs, void* const* outputs, void* workspace,
                                   hipStream_t stream) {
    SESSD_TRY(conv_check_io(inputDesc, outputDesc, inputs, outputs, in_type_, out_type_, max_voxels_,
                            in_channel_, out_channel_, "submconv3d.enqueue"));
    if (!workspace) return fail(SESSD_E_INVALID, "submconv3d.enqueue: workspace is null");
    const int32_t* voxel_num = static_cast<const int32_t*>(inputs[2]);
    SESSD_TRY(enqueueBuild(static_cast<const int32_t*>(inputs[1]), voxel_num, workspace, stream));
    return enqueueGemm(inputs[0], outputs[0], voxel_num, workspace, stream);
}

int SubmConv3dLayerPlugin::enqueueShared(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                                         const void* const* inputs, void* const* outputs,
                                         const void* rulebook_workspace, hipStream_t stream) {
    SESSD_TRY(conv_check_io(inputDesc, outputDesc, inputs, outputs, in_type_, out_type_, max_voxels_,
                            in_channel_, out_channel_, "submconv3d.enqueue_shared"));
    if (!rulebook_workspace) return fail(SESSD_E_INVALID, "submconv3d.enqueue_shared: rulebook workspace is null");
    return enqueueGemm(inputs[0], outputs[0], static_cast<const int32_t*>(inputs[2]), rulebook_workspace, stream);
}

int SubmConv3dLayerPlugin::exportRulebook(const void* workspace, int32_t* indice_pairs, uint32_t* indice_num,
                                          hipStream_t stream) const {
    if (!workspace) return fail(SESSD_E_INVALID, "submconv3d.export_rulebook: workspace is null");
    const Layout L = carve(const_cast<void*>(workspace));
    return ConvPluginBase::exportRulebook(L.nbr, L.meta + 1, L.export_scratch, indice_pairs, indice_num, stream);
}

int SubmConv3dLayerPlugin::countPairs(const void* workspace, uint32_t* indice_num, hipStream_t stream) const {
    if (!workspace) return fail(SESSD_E_INVALID, "submconv3d.count_pairs: workspace is null");
    const Layout L = carve(const_cast<void*>(workspace));
    return launch_count_pairs(L.nbr, L.meta + 1, kernel_volume_, max_voxels_, L.export_scratch, indice_num, stream);
}

}  // namespace sessd
