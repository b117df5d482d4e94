// sparse2dense.hip -- Sparse2DensePlugin: [N,C] voxel features into a dense BEV tensor, written once.
//
// Replaces sparse2Dense.cu:182-249.  Output layout [1, C*D, H, W] with channel index c*D + z
// (sparse2Dense.cu:200-206).  The reference clears the tensor and then scatters one element per (voxel, channel):
// 2- or 4-byte stores D*H*W elements apart, every one of which dirties a whole memory sector on top of the fill
// (measured: 6x the tensor's bytes written in FP32, 15x in FP16).  Here the tensor is produced cell-major instead:
//
//   s2d_index   one thread per voxel: row -> map[cell], a D*H*W map in the workspace (288 KB for the 2x200x176 grid)
//   s2d_dense   one block per (z, y) line: the line's rows from the map, their features through LDS (read along
//               the channels, written along x), every element of the line stored exactly once -- the feature or
//               zero -- in 16-byte runs along x
//
// so the tensor's bytes are written once (its HBM floor) and no separate fill of it exists.  The map is never
// cleared either: an entry counts only if it names an active row whose coordinates are this very cell, which no
// stale or uninitialised entry can do wrongly.  Where two rows name the same cell one of them wins, as in the
// reference, whose threads race there.
//
// Optional border (setPadding): the reference pads the dense tensor right afterwards with its
// ZeroPad2dPlugin (zeroPad2d.cu:183-244: memset of the padded tensor, then a copy of every element to
// (y + top, x + left)).  With a border set, the lines are written straight into the padded tensor
// [1, C*D, H + top + bottom, W + left + right], border included; the unpadded tensor is never materialised.
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

// row -> map[cell] for every active voxel.  Rows with coordinates outside the grid are skipped (the reference
// writes out of bounds there); each block reports whether it met one in its own word of `bad`.
__global__ void __launch_bounds__(kBlock)
s2d_index(const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num, int max_voxels, int D, int H, int W,
          int32_t* __restrict__ map, int32_t* __restrict__ bad) {
    const int v = blockIdx.x * kBlock + threadIdx.x;
    int n = *voxel_num;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    bool outside = false;
    if (v < n) {
        const int4 cc = reinterpret_cast<const int4*>(coors)[v];  // (b,z,y,x)
        outside = cc.x != 0 || cc.y < 0 || cc.y >= D || cc.z < 0 || cc.z >= H || cc.w < 0 || cc.w >= W;
        if (!outside) map[(cc.y * H + cc.z) * W + cc.w] = v;
    }
    const int any = __syncthreads_or(outside);
    if (threadIdx.x == 0) bad[blockIdx.x] = any;
}

template <typename T, int VW> struct StoreVec;
template <> struct StoreVec<float, 4> { using type = float4; };
template <> struct StoreVec<__half, 8> { using type = uint4; };
template <> struct StoreVec<float, 1> { using type = float; };
template <> struct StoreVec<__half, 1> { using type = __half; };

// One (z, padded y) line per block -- a segment of `seg` padded cells of it where the line is longer (blockIdx.z)
// -- CC channels at a time: blockIdx.x = z * Hp + yp; the channel groups blockIdx.y, blockIdx.y + gridDim.y, ... are
// this block's.  The segment's active cells are compacted first (few cells of a line are active), their rows read
// along the channels into the LDS tile [CC][cells + 1], and the segment is then stored VW elements per lane along
// x.  VW > 1 needs Wp % VW == 0, seg % VW == 0 and a 16-byte aligned tensor.
template <typename Tin, typename Tout, int CC, int VW>
__global__ void __launch_bounds__(kBlock)
s2d_dense(const Tin* __restrict__ feat, const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num,
          int max_voxels, const int32_t* __restrict__ map, const int32_t* __restrict__ bad, int bad_words, int C, int D,
          int H, int W, int pad_top, int pad_left, int Hp, int Wp, int seg, Tout* __restrict__ dense, int32_t* status) {
    extern __shared__ int32_t lds[];
    // slot[i]: position of padded cell xp0 + i among the segment's active cells, -1 = empty or border;
    // rows[k]: row of the k-th active cell
    int32_t* slot = lds;
    int32_t* rows = lds + seg;
    float* tile = reinterpret_cast<float*>(lds + 2 * seg);
    __shared__ int wave_count[kBlock / 64];
    const int z = blockIdx.x / Hp, yp = blockIdx.x - z * Hp;
    const int y = yp - pad_top;
    const int xp0 = blockIdx.z * seg;
    const int len = Wp - xp0 < seg ? Wp - xp0 : seg;
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {   // the status word: has s2d_index met a row off the grid
        int any = 0;
        for (int i = threadIdx.x; i < bad_words; i += kBlock) any |= bad[i];
        any = __syncthreads_or(any);
        if (threadIdx.x == 0) *status = any ? SESSD_STATUS_BAD_COORD : 0;
    }
    int n = *voxel_num;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    int cells = 0;
    if (y >= 0 && y < H) {
        const int32_t* line = map + (size_t)(z * H + y) * W;
        for (int i0 = 0; i0 < len; i0 += kBlock) {   // (one round for segments of up to 256 cells)
            const int i = i0 + threadIdx.x;
            const int x = xp0 + i - pad_left;
            int32_t row = -1;
            if (i < len && x >= 0 && x < W) {
                row = line[x];
                // an entry counts if it names an active row that lies in this cell
                if (row >= 0 && row < n) {
                    const int4 cc = reinterpret_cast<const int4*>(coors)[row];
                    if (cc.x != 0 || cc.y != z || cc.z != y || cc.w != x) row = -1;
                } else {
                    row = -1;
                }
            }
            const uint64_t m = __ballot(row >= 0);
            if ((threadIdx.x & 63) == 0) wave_count[threadIdx.x >> 6] = __popcll(m);
            __syncthreads();
            int base = cells;
            for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) base += wave_count[w];
            int total = cells;
            for (int w = 0; w < kBlock / 64; ++w) total += wave_count[w];
            if (i < len) {
                const int k = row >= 0 ? base + rank_in_wave(m) : -1;
                slot[i] = k;
                if (k >= 0) rows[k] = row;
            }
            cells = total;
            __syncthreads();
        }
    }
    const int pitch = cells + 1;
    // a lane keeps its VW cells of the segment and walks down the channels: the cells' slots are looked up once,
    // and an empty group of cells costs no further LDS read
    using V = typename StoreVec<Tout, VW>::type;
    const int groups = len / VW;   // VW divides len
    const int gl = groups < kBlock ? groups : kBlock;
    const int lanes_j = kBlock / gl;
    const int g_first = (int)threadIdx.x % gl, jl = (int)threadIdx.x / gl;
    const size_t step = (size_t)D * Hp * Wp;   // one channel further
    for (int c0 = blockIdx.y * CC; c0 < C; c0 += gridDim.y * CC) {
        if (cells > 0) {
            __syncthreads();   // (the tile of the channels before is read out)
            const int j = threadIdx.x % CC, sub = threadIdx.x / CC;
            for (int k = sub; k < cells; k += kBlock / CC)
                tile[j * pitch + k] = c0 + j < C ? ld_f32(feat + (size_t)rows[k] * C + c0 + j) : 0.0f;
            __syncthreads();
        }
        if (jl >= lanes_j) continue;
        for (int g = g_first; g < groups; g += kBlock) {   // (one round unless the segment has more than 256 groups)
            int k[VW];
            bool some = false;
#pragma unroll
            for (int i = 0; i < VW; ++i) {
                k[i] = cells > 0 ? slot[g * VW + i] : -1;
                some |= k[i] >= 0;
            }
            Tout* dst = dense + ((size_t)(c0 * D + z) * Hp + yp) * Wp + xp0 + g * VW;
            for (int j = jl; j < CC && c0 + j < C; j += lanes_j) {
                alignas(16) Tout out[VW];
#pragma unroll
                for (int i = 0; i < VW; ++i) st_f32(&out[i], some && k[i] >= 0 ? tile[j * pitch + k[i]] : 0.0f);
                *reinterpret_cast<V*>(dst + j * step) = *reinterpret_cast<const V*>(out);
            }
        }
    }
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

// The reference needs no workspace (sparse2Dense.cu:175-179).  Here: one 256-byte block with the status word, one
// word per block of s2d_index, the cell map.
static size_t s2d_bad_words(int max_voxels) { return (size_t)(max_voxels + kBlock - 1) / kBlock; }
static size_t round_ws(size_t b) { return (b + kWorkspaceAlign - 1) / kWorkspaceAlign * kWorkspaceAlign; }

size_t Sparse2DensePlugin::getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs, const sessd_tensor_desc*, int) const {
    const int max_voxels = inputs && nbInputs > 0 && inputs[0].nbDims >= 2 ? inputs[0].d[1] : 0;
    const size_t map = (size_t)feature_map_size_z_ * feature_map_size_y_ * feature_map_size_x_ * sizeof(int32_t);
    return kWorkspaceAlign + round_ws(s2d_bad_words(max_voxels) * sizeof(int32_t)) + round_ws(map);
}

// what must be cleared before the last gather-GEMM scatters into the dense tensor through denseTarget(): the
// tensor and the status word.  (enqueue() itself needs nothing cleared.)
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
                                hipStream_t stream) {
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
    if ((reinterpret_cast<uintptr_t>(outputs[0]) | reinterpret_cast<uintptr_t>(inputs[1])) & 15)
        return fail(SESSD_E_INVALID, "sparse2dense.enqueue: tensors must be 16-byte aligned");
    if (!workspace) return fail(SESSD_E_INVALID, "sparse2dense.enqueue: the workspace carries the cell map and is required");
    int32_t* status = static_cast<int32_t*>(workspace);
    const int bad_words = (int)s2d_bad_words(max_voxels);
    int32_t* bad = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + kWorkspaceAlign);
    int32_t* map = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + kWorkspaceAlign +
                                              round_ws((size_t)bad_words * sizeof(int32_t)));
    const int32_t* coors = static_cast<const int32_t*>(inputs[1]);
    const int32_t* num = static_cast<const int32_t*>(inputs[2]);
    if (bad_words > 0)
        hipLaunchKernelGGL(s2d_index, dim3((unsigned)bad_words), dim3(kBlock), 0, stream, coors, num, max_voxels, D, H, W,
                           map, bad);
    SESSD_HIP_TRY(hipGetLastError());
    const int CC = 32;  // channels per block: 128 bytes of an FP32 row, 64 of an FP16 one
    const int vw = 16 / (int)dtype_size(out_type_);
    const bool wide = Wp % vw == 0;  // (the tensor's 16-byte alignment is checked above)
    // a line goes through LDS whole up to 448 padded cells (60 KB), in segments of 448 beyond
    const int seg = Wp <= 448 ? Wp : 448;   // (a multiple of every vw)
    const int segments = (Wp + seg - 1) / seg;
    // about a thousand blocks: a block takes several channel groups of its line where there are more
    const int cgroups = (C + CC - 1) / CC;
    int split = 1024 / (D * Hp * segments);
    split = split < 1 ? 1 : (split > cgroups ? cgroups : split);
    const dim3 grid((unsigned)(D * Hp), (unsigned)split, (unsigned)segments);
    const size_t lds = (size_t)(2 * seg + CC * (seg + 1)) * sizeof(float);
#define SESSD_S2D(TI, TO, CCV, VWV)                                                                                   \
    hipLaunchKernelGGL((s2d_dense<TI, TO, CCV, VWV>), grid, dim3(kBlock), lds, stream,                                \
                       static_cast<const TI*>(inputs[0]), coors, num, max_voxels, map, bad, bad_words, C, D, H, W,   \
                       zero_padding_2d_top_, zero_padding_2d_left_, Hp, Wp, seg, static_cast<TO*>(outputs[0]), status)
    if (in_type_ == SESSD_FLOAT && out_type_ == SESSD_FLOAT) { if (wide) SESSD_S2D(float, float, 32, 4); else SESSD_S2D(float, float, 32, 1); }
    else if (in_type_ == SESSD_HALF && out_type_ == SESSD_HALF) { if (wide) SESSD_S2D(__half, __half, 32, 8); else SESSD_S2D(__half, __half, 32, 1); }
    else if (in_type_ == SESSD_HALF && out_type_ == SESSD_FLOAT) { if (wide) SESSD_S2D(__half, float, 32, 4); else SESSD_S2D(__half, float, 32, 1); }
    else { if (wide) SESSD_S2D(float, __half, 32, 8); else SESSD_S2D(float, __half, 32, 1); }
#undef SESSD_S2D
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
