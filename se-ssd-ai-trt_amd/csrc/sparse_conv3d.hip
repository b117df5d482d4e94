// sparse_conv3d.hip -- SparseConv3dLayerPlugin: strided sparse 3-D convolution.
//
// Replaces sparseConv3dlayer.cu:310-813.  The reference marks candidate output cells in a dense
// grid, numbers them by scanning the WHOLE grid with atomicAdd (fillGridKernel2: 46 200 blocks at
// 21x800x704) and appends rulebook pairs with atomics.  Here every (input row, candidate) pair is
// a "ticket" t = row*Kc + e, e being the position in getValidOutPos' enumeration order:
//
//   sp_insert   one thread per ticket: output cell key -> hash, value = min ticket that names it
//   sp_flags    one thread per ticket: "am I the first ticket of my cell" -> wave64 ballot words
//   sp_number   exclusive prefix over the ballot words = output row in first-seen order (the order
//               of a sequential walk, sparseConv3dlayer.cu:738-757); writes out coors + voxel_num
//   sp_scatter  one thread per ticket: nbr[offset][out row] = input row
//   gather-GEMM conv_gemm.hip
//
// No pass touches anything larger than O(active sites); numbering is deterministic.
#include "kernels.h"
#include "plugins.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;
constexpr uint32_t kSlotBits = 26;
constexpr uint32_t kSlotMask = (1u << kSlotBits) - 1u;

struct SpParams {
    int k[3], s[3], p[3], os[3];  // z,y,x
    int Kc;                       // enumeration slots per input row
    int max_voxels;
    int dilation;
};

__device__ __forceinline__ int clamp_count(const int32_t* p, int cap) {
    int n = *p;
    return n < 0 ? 0 : (n > cap ? cap : n);
}

// getValidOutPosKernel (sparseConv3dlayer.cu:310-386), one enumeration step: candidate `e` of the
// input cell c.  Integer divisions truncate toward zero exactly as in the reference.
// -> false when e is past the enumeration or the output cell is outside the grid
__device__ __forceinline__ bool sp_candidate(const int c[3], const SpParams& P, int e, int o[3], int& offset) {
    int lo[3], up[3], cs[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        lo[a] = (c[a] - (P.k[a] - 1) * P.dilation - 1 + P.s[a] + P.p[a]) / P.s[a];
        up[a] = (c[a] + P.p[a]) / P.s[a];
        cs[a] = (up[a] - lo[a]) / P.dilation + 1;
    }
    if (cs[0] <= 0 || cs[1] <= 0 || cs[2] <= 0 || e >= cs[0] * cs[1] * cs[2]) return false;
    const int cnt[3] = {e / (cs[2] * cs[1]), (e / cs[2]) % cs[1], e % cs[2]};  // x fastest
    bool valid = true;
    int m = 1;
    offset = 0;
#pragma unroll
    for (int a = 2; a >= 0; --a) {
        o[a] = up[a] - cnt[a] * P.dilation;
        if (o[a] < 0 || o[a] > P.os[a] - 1) valid = false;
        offset += m * (c[a] - o[a] * P.s[a] + P.p[a]) / P.dilation;
        m *= P.k[a];
    }
    return valid;
}

// Rows that follow each other name the same output cells again and again (eight input cells share an output cell
// of a 3x3x3 stride-2 layer, and neighbours in space are mostly neighbours in the row order), and device-wide
// atomics are what this pass is made of.  A block therefore gathers the cells its 256 tickets name in an LDS table
// first (cell -> smallest ticket of the block), and one thread per distinct cell goes to the table in memory.
constexpr int kLocalBits = 9, kLocalSlots = 1 << kLocalBits;  // twice the block's tickets

__global__ void __launch_bounds__(kBlock)
sp_insert(const int32_t* __restrict__ coors, const int32_t* __restrict__ voxel_num, SpParams P, HashTable t,
          uint32_t* __restrict__ cand, int32_t* meta) {
    __shared__ uint32_t s_key[kLocalSlots], s_val[kLocalSlots];
    const uint32_t tk = blockIdx.x * kBlock + threadIdx.x;
    const int v = tk / P.Kc, e = tk % P.Kc;
    const int n = clamp_count(voxel_num, P.max_voxels);
    if ((int64_t)blockIdx.x * kBlock >= (int64_t)n * P.Kc) return;  // (the whole block is beyond the active rows)
    for (int i = threadIdx.x; i < kLocalSlots; i += kBlock) {
        s_key[i] = kEmpty;
        s_val[i] = kEmpty;
    }
    __syncthreads();
    uint32_t key = kEmpty;
    int offset = 0, local = -1;
    bool owner = false;
    if (v < n) {
        const int4 cc = reinterpret_cast<const int4*>(coors)[v];
        const int c[3] = {cc.y, cc.z, cc.w};
        int o[3];
        // A negative coordinate makes the truncating divisions of getValidOutPos yield kernel offsets outside [0, K)
        // (c = -2, k = 3, s = 2, p = 1: o = 0, offset term -1), with which the reference indexes its rulebook.  Such a
        // row contributes nothing here and raises BAD_COORD; the offset is checked as well, so that nothing a caller
        // passes can make sp_scatter store outside the neighbour table.
        const bool bad = c[0] < 0 || c[1] < 0 || c[2] < 0;
        if (bad && e == 0) atomicOr(&meta[0], SESSD_STATUS_BAD_COORD);
        if (!bad && sp_candidate(c, P, e, o, offset) && offset >= 0 && offset < P.k[0] * P.k[1] * P.k[2]) {
            key = ((uint32_t)o[0] * (uint32_t)P.os[1] + (uint32_t)o[1]) * (uint32_t)P.os[2] + (uint32_t)o[2];
            uint32_t ls = (key * 2654435769u) >> (32 - kLocalBits);
            for (;;) {  // (at most kBlock keys in 2 * kBlock slots: room is always found)
                const uint32_t prev = atomicCAS(&s_key[ls], kEmpty, key);
                if (prev == kEmpty || prev == key) {
                    owner = prev == kEmpty;
                    break;
                }
                ls = (ls + 1) & (kLocalSlots - 1);
            }
            local = (int)ls;
            atomicMin(&s_val[ls], tk);
        }
    }
    __syncthreads();
    if (owner) {  // this thread claimed the cell's LDS entry: it carries the block's smallest ticket to memory
        const int32_t slot = hash_insert(t, key);
        if (slot < 0) {
            atomicOr(&meta[0], SESSD_STATUS_HASH_FULL);
            s_key[local] = kEmpty;  // (read below as "no slot")
        } else {
            atomicMin(&t.vals[slot], s_val[local]);
            s_val[local] = (uint32_t)slot;
        }
    }
    __syncthreads();
    if (v >= n) return;
    cand[tk] = (local >= 0 && s_key[local] != kEmpty) ? (((uint32_t)offset << kSlotBits) | s_val[local]) : kEmpty;
}

__global__ void __launch_bounds__(kBlock)
sp_flags(const int32_t* __restrict__ voxel_num, SpParams P, HashTable t, const uint32_t* __restrict__ cand,
         uint64_t* __restrict__ first_words, uint32_t* __restrict__ block_counts) {
    __shared__ uint32_t lds4[4];
    const uint32_t tk = blockIdx.x * kBlock + threadIdx.x;
    const int v = tk / P.Kc;
    const int n = clamp_count(voxel_num, P.max_voxels);
    // the grid covers the capacity; a block beyond the tickets of the active rows has nothing to say, and
    // sp_number reads no word of it
    if ((int64_t)blockIdx.x * kBlock >= (int64_t)n * P.Kc) return;
    bool first = false;
    if (v < n) {
        const uint32_t c = cand[tk];
        first = c != kEmpty && t.vals[c & kSlotMask] == tk;
    }
    const uint64_t m = __ballot(first);
    if ((threadIdx.x & 63) == 0) {
        first_words[tk >> 6] = m;
        lds4[threadIdx.x >> 6] = __popcll(m);
    }
    __syncthreads();
    if (threadIdx.x == 0) block_counts[blockIdx.x] = lds4[0] + lds4[1] + lds4[2] + lds4[3];
}

__global__ void __launch_bounds__(kBlock)
sp_number(const int32_t* __restrict__ voxel_num, SpParams P, HashTable t, const uint32_t* __restrict__ cand,
          const uint64_t* __restrict__ first_words, const uint32_t* __restrict__ block_counts, int n_blocks,
          int32_t* __restrict__ out_coors, int32_t* __restrict__ out_num, int32_t* __restrict__ nbr, int K, int32_t* meta,
          MirrorInit mi) {
    __shared__ uint32_t lds4[4];
    const int b = blockIdx.x;
    // Only the blocks that hold tickets of active input rows carry anything (at a capacity of 100 000 rows and
    // 26 000 active ones, three blocks in four would each add up thousands of counts to find nothing to number).
    int active = (int)(((int64_t)clamp_count(voxel_num, P.max_voxels) * P.Kc + kBlock - 1) / kBlock);
    active = active < n_blocks ? active : n_blocks;
    if (b >= active) {
        // (no active input row at all: block 0 still owes the count; the words sp_flags left unwritten are not read)
        if (b == 0 && threadIdx.x == 0) {
            *out_num = 0;
            meta[1] = 0;
        }
        return;
    }
    const int upto = b == 0 ? active : b;  // block 0 computes the total
    uint32_t part = 0;
    for (int j = threadIdx.x; j < upto; j += kBlock) part += block_counts[j];
    for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off, 64);
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = part;
    __syncthreads();
    const uint32_t sum = lds4[0] + lds4[1] + lds4[2] + lds4[3];
    if (b == 0 && threadIdx.x == 0) {
        const uint32_t m = sum > (uint32_t)P.max_voxels ? (uint32_t)P.max_voxels : sum;
        *out_num = (int32_t)m;
        meta[1] = (int32_t)m;
        if (sum > (uint32_t)P.max_voxels) atomicOr(&meta[0], SESSD_STATUS_VOXEL_OVERFLOW);
    }
    uint32_t base = b == 0 ? 0u : sum;
    const int wave = threadIdx.x >> 6;
    for (int w = 0; w < wave; ++w) base += __popcll(first_words[b * 4 + w]);
    const uint64_t m = first_words[b * 4 + wave];
    if (!((m >> (threadIdx.x & 63)) & 1ull)) return;
    const uint32_t id = base + rank_in_wave(m);
    const uint32_t tk = b * kBlock + threadIdx.x;
    const uint32_t slot = cand[tk] & kSlotMask;
    if (id >= (uint32_t)P.max_voxels) {  // the reference overflows its buffers; the site is dropped
        t.vals[slot] = kEmpty;
        return;
    }
    t.vals[slot] = id;  // from here on the table maps cell -> output row
    const uint32_t key = t.keys[slot];
    const uint32_t plane = (uint32_t)(P.os[1] * P.os[2]);
    const int z = key / plane;
    const int rem = key - z * plane;
    const int y = rem / P.os[2];
    reinterpret_cast<int4*>(out_coors)[id] = make_int4(0, z, y, rem - y * P.os[2]);  // sparseConv3dlayer.cu:438-441
    // the new row's neighbour entries start empty (sp_scatter fills in the pairs): clearing them here, row by
    // row, instead of the whole K x max_voxels table before the frame touches only the rows that exist
    for (int k = 0; k < K; ++k) nbr[(size_t)k * P.max_voxels + id] = -1;
    // ... and so do the mirrored entries of this row in the table of the SubM layer that follows
    if (mi.nbr && (int)id < mi.stride)
        for (int k = mi.first_offset; k < mi.K; ++k) mi.nbr[(size_t)k * mi.stride + id] = -1;
}

__global__ void __launch_bounds__(kBlock)
sp_scatter(const int32_t* __restrict__ voxel_num, SpParams P, HashTable t, const uint32_t* __restrict__ cand,
           int32_t* __restrict__ nbr) {
    const uint32_t tk = blockIdx.x * kBlock + threadIdx.x;
    const int v = tk / P.Kc;
    const int n = clamp_count(voxel_num, P.max_voxels);
    if (v >= n) return;
    const uint32_t c = cand[tk];
    if (c == kEmpty) return;
    const uint32_t id = t.vals[c & kSlotMask];
    if (id == kEmpty) return;
    nbr[(size_t)(c >> kSlotBits) * P.max_voxels + id] = v;  // unique (offset, out row): plain store
}

}  // namespace

struct SparseConv3dLayerPlugin::Layout {
    uint32_t* keys;
    uint32_t* vals;
    int32_t* nbr;
    uint32_t* cand;
    uint64_t* first_words;
    uint32_t* block_counts;
    void* export_scratch;
    int32_t* tiles;  // equal-work tile cuts of the rulebook (tile_cut.hip); first word 0 = none
    int32_t* meta;
    uint32_t cap;
    int Kc;
    int n_blocks;
    size_t meta_offset;
    size_t total;
};

// slots of the candidate hash beyond the worst-case number of distinct candidates: 1/kHashSlack of it
constexpr uint64_t kHashSlack = 16;

int SparseConv3dLayerPlugin::maxCandidates() const {
    const int k[3] = {ksize0_, ksize1_, ksize2_}, s[3] = {stride0_, stride1_, stride2_};
    int kc = 1;
    for (int a = 0; a < 3; ++a) kc *= (k[a] + s[a] - 1) / s[a];
    return kc;
}

SparseConv3dLayerPlugin::Layout SparseConv3dLayerPlugin::carve(void* workspace) const {
    Layout L;
    WorkspaceCarver c(workspace);
    L.Kc = maxCandidates();
    const uint64_t volume = (uint64_t)out_shape_x_ * out_shape_y_ * out_shape_z_;
    uint64_t distinct = (uint64_t)L.Kc * max_voxels_;  // upper bound on distinct candidate cells
    if (distinct > volume) distinct = volume;
    if (distinct < 32) distinct = 32;
    // every distinct candidate cell gets a slot (the cap on output rows applies after numbering).  The bound is
    // the worst case -- every input row with Kc candidates of its own -- of which a real frame uses a few per
    // cent, so the table is sized just above it rather than at twice it: half the bytes to clear per frame.
    L.cap = next_pow2(distinct + distinct / kHashSlack);
    const int64_t tickets = (int64_t)L.Kc * max_voxels_;
    L.n_blocks = ceil_div(tickets, kBlock);
    L.keys = c.take<uint32_t>((size_t)L.cap * 2);
    L.vals = L.keys ? L.keys + L.cap : nullptr;
    L.nbr = c.take<int32_t>((size_t)kernel_volume_ * max_voxels_);
    L.cand = c.take<uint32_t>((size_t)L.n_blocks * kBlock);
    L.first_words = c.take<uint64_t>((size_t)L.n_blocks * 4);
    L.block_counts = c.take<uint32_t>((size_t)L.n_blocks);
    L.export_scratch = c.take<uint8_t>(export_scratch_bytes(kernel_volume_, max_voxels_));
    L.tiles = reinterpret_cast<int32_t*>(c.take<uint8_t>(tile_cut_bytes(max_voxels_)));
    L.meta_offset = c.offset;
    L.meta = c.take<int32_t>(4);
    L.total = c.total();
    return L;
}

int SparseConv3dLayerPlugin::validate() const {
    if (in_channel_ <= 0 || out_channel_ <= 0 || max_voxels_ <= 0)
        return fail(SESSD_E_INVALID, "sparseconv3d: channels/max_voxels must be positive");
    const int k[3] = {ksize0_, ksize1_, ksize2_}, s[3] = {stride0_, stride1_, stride2_},
              p[3] = {padding0_, padding1_, padding2_};
    for (int a = 0; a < 3; ++a)
        if (k[a] <= 0 || s[a] <= 0 || p[a] < 0)
            return fail(SESSD_E_INVALID, "sparseconv3d: bad ksize/stride/padding on axis %d", a);
    if (kernel_volume_ > 27 || maxCandidates() > 27)
        return fail(SESSD_E_UNSUPPORTED, "sparseconv3d: more than 27 kernel offsets (the reference's limit)");
    if (dilation_ != 1) return fail(SESSD_E_UNSUPPORTED, "sparseconv3d: dilation must be 1");
    if (out_shape_x_ <= 0 || out_shape_y_ <= 0 || out_shape_z_ <= 0 ||
        (int64_t)out_shape_x_ * out_shape_y_ * out_shape_z_ >= (int64_t)kEmpty)
        return fail(SESSD_E_UNSUPPORTED, "sparseconv3d: out_shape volume must fit a 32-bit cell key");
    if ((uint64_t)next_pow2((uint64_t)maxCandidates() * max_voxels_ * 2) > (1ull << kSlotBits))
        return fail(SESSD_E_UNSUPPORTED, "sparseconv3d: max_voxels too large for the candidate table");
    if ((int64_t)maxCandidates() * max_voxels_ >= (int64_t)kEmpty)
        return fail(SESSD_E_UNSUPPORTED, "sparseconv3d: ticket space exceeds 32 bits");
    return SESSD_OK;
}

int SparseConv3dLayerPlugin::create(const sessd_sparseconv3d_desc& d, const float* weights,
                                    SparseConv3dLayerPlugin** out) {
    auto* p = new SparseConv3dLayerPlugin();
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
    p->ksize0_ = d.ksize[0]; p->ksize1_ = d.ksize[1]; p->ksize2_ = d.ksize[2];
    p->stride0_ = d.stride[0]; p->stride1_ = d.stride[1]; p->stride2_ = d.stride[2];
    p->padding0_ = d.padding[0]; p->padding1_ = d.padding[1]; p->padding2_ = d.padding[2];
    p->dilation_ = d.dilation;
    p->out_padding_ = d.out_padding;
    p->kernel_volume_ = d.ksize[0] * d.ksize[1] * d.ksize[2];
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

// 22 ints + FP32 weights, sparseConv3dlayer.cu:863-899 (+ optional epilogue trailer)
size_t SparseConv3dLayerPlugin::getSerializationSize() const {
    return (size_t)weights_size_ * sizeof(float) + 22 * sizeof(int) + conv_epilogue_trailer_size(epi_);
}

void SparseConv3dLayerPlugin::serialize(void* buffer) const {
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
    writeToBuffer<int>(d, ksize0_);
    writeToBuffer<int>(d, ksize1_);
    writeToBuffer<int>(d, ksize2_);
    writeToBuffer<int>(d, stride0_);
    writeToBuffer<int>(d, stride1_);
    writeToBuffer<int>(d, stride2_);
    writeToBuffer<int>(d, padding0_);
    writeToBuffer<int>(d, padding1_);
    writeToBuffer<int>(d, padding2_);
    writeToBuffer<int>(d, dilation_);
    writeToBuffer<int>(d, out_padding_);
    writeToBuffer<int>(d, weights_size_);
    for (int i = 0; i < weights_size_; ++i) writeToBuffer<float>(d, weights_data_[i]);
    conv_write_epilogue_trailer(d, epi_);
}

int SparseConv3dLayerPlugin::deserialize(const void* data, size_t length, SparseConv3dLayerPlugin** out) {
    if (!data || length < 22 * sizeof(int)) return fail(SESSD_E_INVALID, "sparseconv3d: blob too short");
    const char* d = static_cast<const char*>(data);
    sessd_sparseconv3d_desc desc;
    desc.in_channel = readFromBuffer<int>(d);
    desc.out_channel = readFromBuffer<int>(d);
    desc.max_voxels = readFromBuffer<int>(d);
    desc.feature_num = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.out_shape[a] = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.spatial_shape[a] = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.ksize[a] = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.stride[a] = readFromBuffer<int>(d);
    for (int a = 0; a < 3; ++a) desc.padding[a] = readFromBuffer<int>(d);
    desc.dilation = readFromBuffer<int>(d);
    desc.out_padding = readFromBuffer<int>(d);
    const int wsize = readFromBuffer<int>(d);
    const int64_t expect = (int64_t)desc.ksize[0] * desc.ksize[1] * desc.ksize[2] * desc.in_channel * desc.out_channel;
    if (wsize < 0 || wsize != expect || length < 22 * sizeof(int) + (size_t)wsize * sizeof(float))
        return fail(SESSD_E_INVALID, "sparseconv3d: weights_size %d does not match the layer shape", wsize);
    std::vector<float> w((size_t)wsize);
    std::memcpy(w.data(), d, (size_t)wsize * sizeof(float));
    d += (size_t)wsize * sizeof(float);
    SparseConv3dLayerPlugin* p = nullptr;
    SESSD_TRY(create(desc, w.data(), &p));
    const int rc = read_epilogue_trailer(d, length - 22 * sizeof(int) - (size_t)wsize * sizeof(float), p);
    if (rc != SESSD_OK) {
        delete p;
        return rc;
    }
    *out = p;
    return SESSD_OK;
}

int SparseConv3dLayerPlugin::configurePlugin(const sessd_tensor_desc* in, int nbInputs,
                                             const sessd_tensor_desc* out, int nbOutputs) {
    if (nbOutputs < 3) return fail(SESSD_E_INVALID, "sparseconv3d.configure: expected 3 outputs");
    return configureTypes(in, nbInputs, out, nbOutputs);
}

size_t SparseConv3dLayerPlugin::getWorkspaceSize(const sessd_tensor_desc*, int, const sessd_tensor_desc*,
                                                 int) const {
    return carve(nullptr).total;
}

size_t SparseConv3dLayerPlugin::statusOffset() const { return carve(nullptr).meta_offset; }

// The two halves of enqueue (see SubmConv3dLayerPlugin::enqueueBuild): output sites + rulebook from the
// coordinates, then the GEMM over the features.
void SparseConv3dLayerPlugin::collectFill(void* workspace, int32_t* out_coors, FillArgs& f) const {
    const Layout L = carve(workspace);
    f.add(L.keys, (uint64_t)L.cap * 2, kEmpty);
    f.add(L.tiles, 4, 0);
    f.add(L.meta, 4, 0);
    if (!(flags_ & SESSD_FLAG_SKIP_PAD_ROWS)) f.add(out_coors, (uint64_t)max_voxels_ * 4, 0);  // :668
}

int SparseConv3dLayerPlugin::enqueueBuild(const int32_t* coors, const int32_t* voxel_num, int32_t* out_coors,
                                          int32_t* out_num, void* workspace, hipStream_t stream, bool prefilled,
                                          const MirrorInit* mirror) {
    if (!coors || !voxel_num || !out_coors || !out_num || !workspace)
        return fail(SESSD_E_INVALID, "sparseconv3d.build: null pointer");
    if (reinterpret_cast<uintptr_t>(out_coors) & 15)
        return fail(SESSD_E_INVALID, "sparseconv3d.build: output coors must be 16-byte aligned");
    const Layout L = carve(workspace);
    const HashTable t = make_hash(L.keys, L.vals, L.cap);
    SpParams P;
    P.k[0] = ksize0_; P.k[1] = ksize1_; P.k[2] = ksize2_;
    P.s[0] = stride0_; P.s[1] = stride1_; P.s[2] = stride2_;
    P.p[0] = padding0_; P.p[1] = padding1_; P.p[2] = padding2_;
    P.os[0] = out_shape_z_; P.os[1] = out_shape_y_; P.os[2] = out_shape_x_;
    P.Kc = L.Kc;
    P.max_voxels = max_voxels_;
    P.dilation = dilation_;

    if (!prefilled) {
        FillArgs f;
        collectFill(workspace, out_coors, f);
        SESSD_TRY(launch_fill(f, stream));
    }
    const dim3 grid(L.n_blocks), block(kBlock);
    hipLaunchKernelGGL(sp_insert, grid, block, 0, stream, coors, voxel_num, P, t, L.cand, L.meta);
    hipLaunchKernelGGL(sp_flags, grid, block, 0, stream, voxel_num, P, t, L.cand, L.first_words, L.block_counts);
    hipLaunchKernelGGL(sp_number, grid, block, 0, stream, voxel_num, P, t, L.cand, L.first_words, L.block_counts,
                       L.n_blocks, out_coors, out_num, L.nbr, kernel_volume_, L.meta, mirror ? *mirror : MirrorInit());
    hipLaunchKernelGGL(sp_scatter, grid, block, 0, stream, voxel_num, P, t, L.cand, L.nbr);
    SESSD_HIP_TRY(hipGetLastError());
    if (wantTileCuts()) SESSD_TRY(launch_tile_cuts(L.nbr, out_num, kernel_volume_, max_voxels_, tileRows(), tileRowWeight(), L.tiles, stream));
    return SESSD_OK;
}

HashTable SparseConv3dLayerPlugin::cellTable(void* workspace) const {
    const Layout L = carve(workspace);
    return make_hash(L.keys, L.vals, L.cap);
}

int SparseConv3dLayerPlugin::enqueueGemm(const void* in_feat, void* out_feat, const int32_t* out_num,
                                         const void* workspace, hipStream_t stream, const DenseTarget* dense) {
    if (!in_feat || !out_feat || !out_num || !workspace) return fail(SESSD_E_INVALID, "sparseconv3d.gemm: null pointer");
    const Layout L = carve(const_cast<void*>(workspace));
    return runGemm(in_feat, out_feat, L.nbr, L.tiles, out_num, stream, dense);
}

int SparseConv3dLayerPlugin::enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                                     const void* const* inputs, void* const* outputs, void* workspace,
                                     hipStream_t stream) {
    SESSD_TRY(conv_check_io(inputDesc, outputDesc, inputs, outputs, in_type_, out_type_, max_voxels_,
                            in_channel_, out_channel_, "sparseconv3d.enqueue"));
    if (!workspace || !outputs[1] || !outputs[2]) return fail(SESSD_E_INVALID, "sparseconv3d.enqueue: null pointer");
    int32_t* out_num = static_cast<int32_t*>(outputs[2]);
    SESSD_TRY(enqueueBuild(static_cast<const int32_t*>(inputs[1]), static_cast<const int32_t*>(inputs[2]),
                           static_cast<int32_t*>(outputs[1]), out_num, workspace, stream));
    return enqueueGemm(inputs[0], outputs[0], out_num, workspace, stream);
}

int SparseConv3dLayerPlugin::exportRulebook(const void* workspace, int32_t* indice_pairs, uint32_t* indice_num,
                                            hipStream_t stream) const {
    if (!workspace) return fail(SESSD_E_INVALID, "sparseconv3d.export_rulebook: workspace is null");
    const Layout L = carve(const_cast<void*>(workspace));
    return ConvPluginBase::exportRulebook(L.nbr, L.meta + 1, L.export_scratch, indice_pairs, indice_num, stream);
}

int SparseConv3dLayerPlugin::countPairs(const void* workspace, uint32_t* indice_num, hipStream_t stream) const {
    if (!workspace) return fail(SESSD_E_INVALID, "sparseconv3d.count_pairs: workspace is null");
    const Layout L = carve(const_cast<void*>(workspace));
    return launch_count_pairs(L.nbr, L.meta + 1, kernel_volume_, max_voxels_, L.export_scratch, indice_num, stream);
}

}  // namespace sessd
