// sparse2dense.hip -- Sparse2DensePlugin: scatter [N,C] voxel features into a dense BEV tensor.
//
// Replaces sparse2Dense.cu:182-249.  Output layout [1, C*D, H, W] with channel index c*D + z
// (sparse2Dense.cu:200-206).  Two launches: a fill of the whole dense tensor (it must be defined
// everywhere; this 18 MB write is the kernel's HBM floor) and a scatter with one thread per
// (voxel, channel) so that the feature reads are coalesced; the 4-byte stores are strided by H*W*D
// by construction of the layout.
//
// Optional border (setPadding): the reference pads the dense tensor right afterwards with its
// ZeroPad2dPlugin (zeroPad2d.cu:183-244: memset of the padded tensor, then a copy of every element to
// (y + top, x + left)).  With a border set, the scatter writes straight into the padded tensor
// [1, C*D, H + top + bottom, W + left + right]; the unpadded tensor is never materialised.
#include "plugins.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;

template <typename T> __device__ __forceinline__ float ld_f32(const T* p);
template <> __device__ __forceinline__ float ld_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f32<__half>(const __half* p) { return __half2float(*p); }
template <typename T> __device__ __forceinline__ void st_f32(T* p, float v);
template <> __device__ __forceinline__ void st_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f32<__half>(__half* p, float v) { *p = __float2half_rn(v); }

template <typename Tin, typename Tout>
__global__ void __launch_bounds__(kBlock)
s2d_scatter(const Tin* __restrict__ feat, const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num,
            int max_voxels, int C, int D, int H, int W, int pad_top, int pad_left, int Hp, int Wp,
            Tout* __restrict__ dense, int32_t* status) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int v = (int)(e / C);
    const int c = (int)(e - (int64_t)v * C);
    int n = *voxel_num;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    if (v >= n) return;
    const int4 cc = reinterpret_cast<const int4*>(coors)[v];  // (b,z,y,x)
    if (cc.x != 0 || cc.y < 0 || cc.y >= D || cc.z < 0 || cc.z >= H || cc.w < 0 || cc.w >= W) {
        if (status && c == 0) atomicOr(status, SESSD_STATUS_BAD_COORD);  // the reference writes out of bounds
        return;
    }
    st_f32(dense + ((size_t)(c * D + cc.y) * Hp + cc.z + pad_top) * Wp + cc.w + pad_left, ld_f32(feat + e));
}

}  // namespace

int Sparse2DensePlugin::create(const sessd_sparse2dense_desc& d, Sparse2DensePlugin** out) {
    if (d.feature_map_size[0] <= 0 || d.feature_map_size[1] <= 0 || d.feature_map_size[2] <= 0 ||
        d.feature_map_channel <= 0)
        return fail(SESSD_E_INVALID, "sparse2dense: feature map size and channel must be positive");
    auto* p = new Sparse2DensePlugin();
    p->feature_map_size_x_ = d.feature_map_size[0];
    p->feature_map_size_y_ = d.feature_map_size[1];
    p->feature_map_size_z_ = d.feature_map_size[2];
    p->feature_map_channel_ = d.feature_map_channel;
    *out = p;
    return SESSD_OK;
}

int Sparse2DensePlugin::setPadding(int top, int bottom, int left, int right) {
    if (top < 0 || bottom < 0 || left < 0 || right < 0)
        return fail(SESSD_E_INVALID, "sparse2dense.set_padding: the border widths must not be negative");
    zero_padding_2d_top_ = top;
    zero_padding_2d_bottom_ = bottom;
    zero_padding_2d_left_ = left;
    zero_padding_2d_right_ = right;
    return SESSD_OK;
}

// Without a border the blob is the reference's four ints (sparse2Dense.cu:288-295).  With one, a tagged
// trailer follows: the tag, then top, bottom, left, right in the order of zeroPad2d.cu:283-290.
constexpr uint32_t kPadTag = 0x44415053u;  // "SPAD"

size_t Sparse2DensePlugin::getSerializationSize() const { return (padded() ? 9 : 4) * sizeof(int); }

void Sparse2DensePlugin::serialize(void* buffer) const {
    char* d = static_cast<char*>(buffer);
    writeToBuffer<int>(d, feature_map_size_x_);
    writeToBuffer<int>(d, feature_map_size_y_);
    writeToBuffer<int>(d, feature_map_size_z_);
    writeToBuffer<int>(d, feature_map_channel_);
    if (padded()) {
        writeToBuffer<uint32_t>(d, kPadTag);
        writeToBuffer<int>(d, zero_padding_2d_top_);
        writeToBuffer<int>(d, zero_padding_2d_bottom_);
        writeToBuffer<int>(d, zero_padding_2d_left_);
        writeToBuffer<int>(d, zero_padding_2d_right_);
    }
}

int Sparse2DensePlugin::deserialize(const void* data, size_t length, Sparse2DensePlugin** out) {
    if (!data || length < 4 * sizeof(int)) return fail(SESSD_E_INVALID, "sparse2dense: blob too short");
    const char* d = static_cast<const char*>(data);
    sessd_sparse2dense_desc desc;
    desc.feature_map_size[0] = readFromBuffer<int>(d);
    desc.feature_map_size[1] = readFromBuffer<int>(d);
    desc.feature_map_size[2] = readFromBuffer<int>(d);
    desc.feature_map_channel = readFromBuffer<int>(d);
    SESSD_TRY(create(desc, out));
    if (length >= 9 * sizeof(int) && readFromBuffer<uint32_t>(d) == kPadTag) {
        const int t = readFromBuffer<int>(d), b = readFromBuffer<int>(d), l = readFromBuffer<int>(d),
                  r = readFromBuffer<int>(d);
        const int rc = (*out)->setPadding(t, b, l, r);
        if (rc != SESSD_OK) {
            delete *out;
            *out = nullptr;
            return rc;
        }
    }
    return SESSD_OK;
}

int Sparse2DensePlugin::configurePlugin(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                                        int nbOutputs) {
    if (!in || !out || nbInputs < 3 || nbOutputs < 1)
        return fail(SESSD_E_INVALID, "sparse2dense.configure: expected 3 inputs and 1 output");
    for (const sessd_tensor_desc* d : {&in[0], &out[0]})
        if (d->type != SESSD_FLOAT && d->type != SESSD_HALF)
            return fail(SESSD_E_UNSUPPORTED, "sparse2dense.configure: features must be FP32 or FP16");
    if (in[0].nbDims != 3 || in[0].d[2] != feature_map_channel_)
        return fail(SESSD_E_INVALID, "sparse2dense.configure: features must be [1,max_voxels,%d]", feature_map_channel_);
    const int nd = out[0].nbDims;
    if (nd >= 3 && (out[0].d[nd - 3] != feature_map_channel_ * feature_map_size_z_ ||
                    out[0].d[nd - 2] != outHeight() || out[0].d[nd - 1] != outWidth()))
        return fail(SESSD_E_INVALID, "sparse2dense.configure: output must be [1,%d,%d,%d]",
                    feature_map_channel_ * feature_map_size_z_, outHeight(), outWidth());
    in_type_ = in[0].type;
    out_type_ = out[0].type;
    return SESSD_OK;
}

// The reference needs no workspace (sparse2Dense.cu:175-179); one 256-byte block carries the status word.
size_t Sparse2DensePlugin::getWorkspaceSize(const sessd_tensor_desc*, int, const sessd_tensor_desc*, int) const {
    return kWorkspaceAlign;
}

void Sparse2DensePlugin::collectFill(void* dense, void* workspace, FillArgs& f) const {
    const uint64_t elems = (uint64_t)feature_map_channel_ * feature_map_size_z_ * outHeight() * outWidth();
    f.add(dense, elems * dtype_size(out_type_) / 4, 0);  // sparse2Dense.cu:242, zeroPad2d.cu:230
    if (workspace) f.add(workspace, 4, 0);
}

DenseTarget Sparse2DensePlugin::denseTarget(void* dense, const int32_t* coors, void* workspace) const {
    DenseTarget t;
    t.dense = dense;
    t.coors = coors;
    t.D = feature_map_size_z_;
    t.H = feature_map_size_y_;
    t.W = feature_map_size_x_;
    t.Hp = outHeight();
    t.Wp = outWidth();
    t.pad_top = zero_padding_2d_top_;
    t.pad_left = zero_padding_2d_left_;
    t.status = static_cast<int32_t*>(workspace);
    return t;
}

int Sparse2DensePlugin::enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                                const void* const* inputs, void* const* outputs, void* workspace,
                                hipStream_t stream, bool prefilled) {
    if (!inputDesc || !outputDesc || !inputs || !outputs || !inputs[0] || !inputs[1] || !inputs[2] || !outputs[0])
        return fail(SESSD_E_INVALID, "sparse2dense.enqueue: null argument");
    if (inputDesc[0].d[0] != 1) return fail(SESSD_E_UNSUPPORTED, "sparse2dense.enqueue: batch size must be 1");
    if (inputDesc[0].type != in_type_ || outputDesc[0].type != out_type_)
        return fail(SESSD_E_INVALID, "sparse2dense.enqueue: tensor dtypes differ from the configured ones");
    if (inputDesc[0].d[2] != feature_map_channel_)
        return fail(SESSD_E_INVALID, "sparse2dense.enqueue: feature channels do not match");
    const int max_voxels = inputDesc[0].d[1];
    const int C = feature_map_channel_, D = feature_map_size_z_, H = feature_map_size_y_, W = feature_map_size_x_;
    const int Hp = outHeight(), Wp = outWidth();
    const uint64_t elems = (uint64_t)C * D * Hp * Wp;
    const uint64_t bytes = elems * dtype_size(out_type_);
    if (bytes % 4) return fail(SESSD_E_UNSUPPORTED, "sparse2dense.enqueue: dense tensor size must be a multiple of 4 bytes");
    if ((reinterpret_cast<uintptr_t>(outputs[0]) | reinterpret_cast<uintptr_t>(inputs[1])) & 15)
        return fail(SESSD_E_INVALID, "sparse2dense.enqueue: tensors must be 16-byte aligned");
    int32_t* status = static_cast<int32_t*>(workspace);

    if (!prefilled) {
        FillArgs f;
        collectFill(outputs[0], workspace, f);
        SESSD_TRY(launch_fill(f, stream));
    }
    const unsigned blocks = (unsigned)(((uint64_t)max_voxels * C + kBlock - 1) / kBlock);
    const int32_t* coors = static_cast<const int32_t*>(inputs[1]);
    const int32_t* num = static_cast<const int32_t*>(inputs[2]);
#define SESSD_S2D(TI, TO)                                                                              \
    hipLaunchKernelGGL((s2d_scatter<TI, TO>), dim3(blocks), dim3(kBlock), 0, stream,                   \
                       static_cast<const TI*>(inputs[0]), coors, num, max_voxels, C, D, H, W,          \
                       zero_padding_2d_top_, zero_padding_2d_left_, Hp, Wp, static_cast<TO*>(outputs[0]), status)
    if (in_type_ == SESSD_FLOAT && out_type_ == SESSD_FLOAT) SESSD_S2D(float, float);
    else if (in_type_ == SESSD_HALF && out_type_ == SESSD_HALF) SESSD_S2D(__half, __half);
    else if (in_type_ == SESSD_HALF && out_type_ == SESSD_FLOAT) SESSD_S2D(__half, float);
    else SESSD_S2D(float, __half);
#undef SESSD_S2D
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
