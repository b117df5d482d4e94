// voxel_generator.hip -- VoxelGeneratorPlugin: points -> voxels with mean VFE.
//
// Replaces voxelGenerator.cu:255-542 of the reference.  The reference keeps a dense
// [Z*Y*X][2] slot table (721 MB, memset every frame) and hands out voxel ids and point slots with
// atomicAdd, so which points are kept and how voxels are numbered depends on scheduling.  Here:
//
//   vg_insert    one thread per point: cell key -> open-addressing hash (a few MB, L2 resident);
//                each entry keeps the S smallest point indices of its cell, maintained with a
//                chain of atomicMin "comparators" whose final state is independent of the order
//                in which threads arrive
//   vg_flags     one thread per point: "am I the lowest-index point of my cell" -> wave64 ballot
//                words + per-block counts
//   vg_finalize  exclusive prefix over the ballot words = voxel id in first-appearance order;
//                that thread writes the coordinate and the mean of the (<= S) kept points
//
// The result equals a sequential walk over the points: ids in first-appearance order, the first S
// points of a cell kept, cells first seen after max_voxels dropped.  All traffic is O(points):
// 16 B/point read + 32 B/voxel written, plus the hash clear.
#include <mutex>

#include "plugins.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;

struct VgParams {
    float min_x, max_x, min_y, max_y, min_z, max_z;
    float vx, vy, vz;
    int gx, gy, gz;
    int max_voxels;
    int max_pts;  // S
};

__device__ __forceinline__ int clamp_count(const int32_t* p, int cap) {
    int n = *p;
    return n < 0 ? 0 : (n > cap ? cap : n);
}

// sum of v over the block (blockDim.x == kBlock), returned to every thread
__device__ __forceinline__ uint32_t block_sum(uint32_t v, uint32_t* lds4) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    return lds4[0] + lds4[1] + lds4[2] + lds4[3];
}

__global__ void __launch_bounds__(kBlock)
vg_insert(const float* __restrict__ points, const int32_t* __restrict__ points_size, int max_points,
          int pf, VgParams p, HashTable t, uint32_t* __restrict__ slots, int32_t* __restrict__ pt_slot,
          int32_t* status) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    const int n = clamp_count(points_size, max_points);
    if (i >= n) return;
    const float* pt = points + (size_t)i * pf;
    const float x = pt[0], y = pt[1], z = pt[2];
    int32_t slot = -1;
    // voxelGenerator.cu:363-367: half-open range test
    if (x >= p.min_x && x < p.max_x && y >= p.min_y && y < p.max_y && z >= p.min_z && z < p.max_z) {
        // voxelGenerator.cu:369-371: IEEE FP32 division (never a reciprocal multiply)
        const int ix = (int)floorf((x - p.min_x) / p.vx);
        const int iy = (int)floorf((y - p.min_y) / p.vy);
        const int iz = (int)floorf((z - p.min_z) / p.vz);
        // voxelGenerator.cu:375: a value just below max can still land on the grid size
        if (ix >= 0 && ix < p.gx && iy >= 0 && iy < p.gy && iz >= 0 && iz < p.gz) {
            const uint32_t key = (uint32_t)iz * (uint32_t)(p.gy * p.gx) + (uint32_t)iy * (uint32_t)p.gx + (uint32_t)ix;
            slot = hash_insert(t, key);
            if (slot < 0) {
                atomicOr(status, SESSD_STATUS_HASH_FULL);
            } else {
                // keep the S smallest point indices of the cell, ascending: slot q ends up with
                // the minimum of everything offered to it and passes the rest on
                uint32_t* s = slots + (size_t)slot * p.max_pts;
                uint32_t cur = (uint32_t)i;
                for (int q = 0; q < p.max_pts; ++q) {
                    const uint32_t old = atomicMin(&s[q], cur);
                    if (old == kEmpty) break;
                    cur = old > cur ? old : cur;
                }
            }
        }
    }
    pt_slot[i] = slot;
}

__global__ void __launch_bounds__(kBlock)
vg_flags(const int32_t* __restrict__ points_size, int max_points, int max_pts,
         const uint32_t* __restrict__ slots, const int32_t* __restrict__ pt_slot,
         uint64_t* __restrict__ first_words, uint32_t* __restrict__ block_counts) {
    __shared__ uint32_t lds4[4];
    const int i = blockIdx.x * kBlock + threadIdx.x;
    const int n = clamp_count(points_size, max_points);
    bool first = false;
    if (i < n) {
        const int32_t slot = pt_slot[i];
        first = slot >= 0 && slots[(size_t)slot * max_pts] == (uint32_t)i;
    }
    const uint64_t m = __ballot(first);
    if ((threadIdx.x & 63) == 0) {
        first_words[i >> 6] = m;
        lds4[threadIdx.x >> 6] = __popcll(m);
    }
    __syncthreads();
    if (threadIdx.x == 0) block_counts[blockIdx.x] = lds4[0] + lds4[1] + lds4[2] + lds4[3];
}

__global__ void __launch_bounds__(kBlock)
vg_finalize(const float* __restrict__ points, int pf, VgParams p, HashTable t,
            const uint32_t* __restrict__ slots, const int32_t* __restrict__ pt_slot,
            const uint64_t* __restrict__ first_words, const uint32_t* __restrict__ block_counts,
            int n_blocks, float* __restrict__ voxels, int32_t* __restrict__ coors,
            int32_t* __restrict__ voxel_num, int32_t* status, MirrorInit mi) {
    __shared__ uint32_t lds4[4];
    const int b = blockIdx.x;
    // block 0 sums every block's count (the total); the others sum the blocks before them
    const int upto = b == 0 ? n_blocks : b;
    uint32_t part = 0;
    for (int j = threadIdx.x; j < upto; j += kBlock) part += block_counts[j];
    const uint32_t sum = block_sum(part, lds4);
    if (b == 0 && threadIdx.x == 0) {
        *voxel_num = (int32_t)(sum > (uint32_t)p.max_voxels ? (uint32_t)p.max_voxels : sum);
        if (sum > (uint32_t)p.max_voxels) atomicOr(status, SESSD_STATUS_VOXEL_OVERFLOW);
    }
    uint32_t base = b == 0 ? 0u : sum;
    const int i = b * kBlock + threadIdx.x;
    const int wave = threadIdx.x >> 6;
    for (int w = 0; w < wave; ++w) base += __popcll(first_words[b * 4 + w]);
    const uint64_t m = first_words[b * 4 + wave];
    if (!((m >> (threadIdx.x & 63)) & 1ull)) return;
    const uint32_t vid = base + rank_in_wave(m);
    if (vid >= (uint32_t)p.max_voxels) return;  // cells first seen beyond the cap are dropped

    const int32_t slot = pt_slot[i];
    const uint32_t key = t.keys[slot];
    const uint32_t plane = (uint32_t)(p.gy * p.gx);
    const int iz = key / plane;
    const int rem = key - iz * plane;
    const int iy = rem / p.gx;
    const int ix = rem - iy * p.gx;
    reinterpret_cast<int4*>(coors)[vid] = make_int4(0, iz, iy, ix);  // voxelGenerator.cu:404-405
    t.vals[slot] = vid;  // the table now maps cell -> voxel row (VoxelGeneratorPlugin::cellTable)
    if (mi.nbr && (int)vid < mi.stride)  // the next SubM layer's mirrored neighbour entries of this row start empty
        for (int k = mi.first_offset; k < mi.K; ++k) mi.nbr[(size_t)k * mi.stride + vid] = -1;

    // voxelGenerator.cu:274-296: all S slots are summed left to right, unfilled slots count as 0
    const uint32_t* s = slots + (size_t)slot * p.max_pts;
    float sx = 0.f, sy = 0.f, sz = 0.f, sw = 0.f;
    int cnt = 0;
    for (int q = 0; q < p.max_pts; ++q) {
        const uint32_t idx = s[q];
        float ax = 0.f, ay = 0.f, az = 0.f, aw = 0.f;
        if (idx != kEmpty) {
            const float* pt = points + (size_t)idx * pf;
            ax = pt[0]; ay = pt[1]; az = pt[2]; aw = pt[3];
            ++cnt;
        }
        if (q == 0) { sx = ax; sy = ay; sz = az; sw = aw; }
        else { sx = sx + ax; sy = sy + ay; sz = sz + az; sw = sw + aw; }
    }
    const float c = (float)cnt;
    reinterpret_cast<float4*>(voxels)[vid] = make_float4(sx / c, sy / c, sz / c, sw / c);
}

// np.round as in spconv's voxel generator (voxelGenerator.cu:61-68): half to even
int np_round(float x) {
    int x2 = int(x * 2.0f);
    if (x != int(x) && x2 == x * 2.0f) return int(x / 2.0f + 0.5f) * 2;
    return int(x + 0.5f);
}

}  // namespace

struct VoxelGeneratorPlugin::Layout {
    uint32_t* keys;
    uint32_t* vals;  // voxel row of the cell (written by vg_finalize; kEmpty for dropped cells)
    uint32_t* slots;
    int32_t* pt_slot;
    uint64_t* first_words;
    uint32_t* block_counts;
    int32_t* status;
    uint32_t cap;
    int n_blocks;
    size_t status_offset;
    size_t total;
};

VoxelGeneratorPlugin::Layout VoxelGeneratorPlugin::carve(void* workspace, int max_points) const {
    Layout L;
    WorkspaceCarver c(workspace);
    L.cap = next_pow2((uint64_t)(max_points < 32 ? 32 : max_points) * 2);
    L.n_blocks = ceil_div(max_points, kBlock);
    // keys, vals and slots are adjacent so that one fill region clears all three
    const size_t cap_words = align_up((size_t)L.cap * 4) / 4;
    const size_t table_words = 2 * cap_words + (size_t)L.cap * pointNum_;
    L.keys = c.take<uint32_t>(table_words);
    L.vals = L.keys ? L.keys + cap_words : nullptr;
    L.slots = L.keys ? L.keys + 2 * cap_words : nullptr;
    L.pt_slot = c.take<int32_t>((size_t)L.n_blocks * kBlock);
    L.first_words = c.take<uint64_t>((size_t)L.n_blocks * 4);
    L.block_counts = c.take<uint32_t>((size_t)L.n_blocks);
    L.status_offset = c.offset;
    L.status = c.take<int32_t>(4);
    L.total = c.total();
    return L;
}

HashTable VoxelGeneratorPlugin::cellTable(void* workspace, int max_points) const {
    const Layout L = carve(workspace, max_points);
    return make_hash(L.keys, L.vals, L.cap);
}

void VoxelGeneratorPlugin::deriveGrid() {
    // voxelGenerator.cu:232-234
    grid_x_size_ = np_round((max_x_range_ - min_x_range_) / voxel_x_size_);
    grid_y_size_ = np_round((max_y_range_ - min_y_range_) / voxel_y_size_);
    grid_z_size_ = np_round((max_z_range_ - min_z_range_) / voxel_z_size_);
}

int VoxelGeneratorPlugin::create(const sessd_voxelgen_desc& d, VoxelGeneratorPlugin** out) {
    if (d.max_voxels <= 0 || d.max_num_points_per_voxel <= 0 || d.max_num_points_per_voxel > 64)
        return fail(SESSD_E_INVALID, "voxelgen: max_voxels=%d max_num_points_per_voxel=%d", d.max_voxels,
                    d.max_num_points_per_voxel);
    if (d.voxel_feature_num != 4)
        return fail(SESSD_E_UNSUPPORTED, "voxelgen: voxel_feature_num must be 4 (x,y,z,i), got %d",
                    d.voxel_feature_num);
    for (int a = 0; a < 3; ++a)
        if (!(d.voxel_size[a] > 0.f) || !(d.point_cloud_range[a + 3] > d.point_cloud_range[a]))
            return fail(SESSD_E_INVALID, "voxelgen: empty range or non-positive voxel size on axis %d", a);
    auto* p = new VoxelGeneratorPlugin();
    // argument order of the reference creator call (voxelGenerator.cu:697-699)
    p->voxelNum_ = d.max_voxels;
    p->pointNum_ = d.max_num_points_per_voxel;
    p->featureNum_ = d.voxel_feature_num;
    p->min_x_range_ = d.point_cloud_range[0];
    p->max_x_range_ = d.point_cloud_range[3];
    p->min_y_range_ = d.point_cloud_range[1];
    p->max_y_range_ = d.point_cloud_range[4];
    p->min_z_range_ = d.point_cloud_range[2];
    p->max_z_range_ = d.point_cloud_range[5];
    p->voxel_x_size_ = d.voxel_size[0];
    p->voxel_y_size_ = d.voxel_size[1];
    p->voxel_z_size_ = d.voxel_size[2];
    p->deriveGrid();
    if ((int64_t)p->grid_x_size_ * p->grid_y_size_ * p->grid_z_size_ >= (int64_t)kEmpty) {
        delete p;
        return fail(SESSD_E_UNSUPPORTED, "voxelgen: grid volume does not fit a 32-bit cell key");
    }
    *out = p;
    return SESSD_OK;
}

size_t VoxelGeneratorPlugin::getSerializationSize() const { return 9 * sizeof(float) + 7 * sizeof(int); }

void VoxelGeneratorPlugin::serialize(void* buffer) const {
    char* d = static_cast<char*>(buffer);
    writeToBuffer<int>(d, voxelNum_);
    writeToBuffer<int>(d, pointNum_);
    writeToBuffer<int>(d, featureNum_);
    writeToBuffer<float>(d, min_x_range_);
    writeToBuffer<float>(d, max_x_range_);
    writeToBuffer<float>(d, min_y_range_);
    writeToBuffer<float>(d, max_y_range_);
    writeToBuffer<float>(d, min_z_range_);
    writeToBuffer<float>(d, max_z_range_);
    writeToBuffer<float>(d, voxel_x_size_);
    writeToBuffer<float>(d, voxel_y_size_);
    writeToBuffer<float>(d, voxel_z_size_);
    writeToBuffer<int>(d, pointFeatureNum_);
    writeToBuffer<int>(d, grid_x_size_);
    writeToBuffer<int>(d, grid_y_size_);
    writeToBuffer<int>(d, grid_z_size_);
}

int VoxelGeneratorPlugin::deserialize(const void* data, size_t length, VoxelGeneratorPlugin** out) {
    if (!data || length < 9 * sizeof(float) + 7 * sizeof(int))
        return fail(SESSD_E_INVALID, "voxelgen: serialized blob too short (%zu bytes)", length);
    const char* d = static_cast<const char*>(data);
    auto* p = new VoxelGeneratorPlugin();
    p->voxelNum_ = readFromBuffer<int>(d);
    p->pointNum_ = readFromBuffer<int>(d);
    p->featureNum_ = readFromBuffer<int>(d);
    p->min_x_range_ = readFromBuffer<float>(d);
    p->max_x_range_ = readFromBuffer<float>(d);
    p->min_y_range_ = readFromBuffer<float>(d);
    p->max_y_range_ = readFromBuffer<float>(d);
    p->min_z_range_ = readFromBuffer<float>(d);
    p->max_z_range_ = readFromBuffer<float>(d);
    p->voxel_x_size_ = readFromBuffer<float>(d);
    p->voxel_y_size_ = readFromBuffer<float>(d);
    p->voxel_z_size_ = readFromBuffer<float>(d);
    p->pointFeatureNum_ = readFromBuffer<int>(d);
    p->grid_x_size_ = readFromBuffer<int>(d);
    p->grid_y_size_ = readFromBuffer<int>(d);
    p->grid_z_size_ = readFromBuffer<int>(d);
    if (p->voxelNum_ <= 0 || p->pointNum_ <= 0 || p->pointNum_ > 64 || p->featureNum_ != 4) {
        delete p;
        return fail(SESSD_E_INVALID, "voxelgen: serialized fields out of range");
    }
    *out = p;
    return SESSD_OK;
}

int VoxelGeneratorPlugin::configurePlugin(const sessd_tensor_desc* in, int nbInputs,
                                          const sessd_tensor_desc*, int) {
    if (!in || nbInputs < 1 || in[0].nbDims != 3)
        return fail(SESSD_E_INVALID, "voxelgen.configure: expected points desc [1,max_points,F]");
    if (in[0].d[2] < 4) return fail(SESSD_E_INVALID, "voxelgen.configure: need >= 4 point features");
    pointFeatureNum_ = in[0].d[2];  // voxelGenerator.cu:231
    lastMaxPoints_ = in[0].d[1];
    deriveGrid();
    return SESSD_OK;
}

size_t VoxelGeneratorPlugin::getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs,
                                              const sessd_tensor_desc*, int) const {
    if (!inputs || nbInputs < 1 || inputs[0].nbDims != 3 || inputs[0].d[1] <= 0) return 0;
    return carve(nullptr, inputs[0].d[1]).total;
}

size_t VoxelGeneratorPlugin::statusOffset(int max_points) const {
    return carve(nullptr, max_points).status_offset;
}

int VoxelGeneratorPlugin::enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc*,
                                  const void* const* inputs, void* const* outputs, void* workspace,
                                  hipStream_t stream, const MirrorInit* mirror, const FillArgs* also_clear) {
    if (!inputDesc || !inputs || !outputs || !workspace)
        return fail(SESSD_E_INVALID, "voxelgen.enqueue: null argument");
    if (inputDesc[0].nbDims != 3 || inputDesc[0].d[0] != 1)
        return fail(SESSD_E_UNSUPPORTED, "voxelgen.enqueue: points must be [1,max_points,F]");
    if (inputDesc[0].type != SESSD_FLOAT) return fail(SESSD_E_UNSUPPORTED, "voxelgen.enqueue: points must be FP32");
    const int max_points = inputDesc[0].d[1];
    const int pf = inputDesc[0].d[2];
    if (max_points <= 0 || pf < 4) return fail(SESSD_E_INVALID, "voxelgen.enqueue: bad points shape");
    if (grid_x_size_ <= 0) return fail(SESSD_E_INVALID, "voxelgen.enqueue: configure() was not called");
    const float* points = static_cast<const float*>(inputs[0]);
    const int32_t* points_size = static_cast<const int32_t*>(inputs[1]);
    float* voxels = static_cast<float*>(outputs[0]);
    int32_t* coors = static_cast<int32_t*>(outputs[1]);
    int32_t* voxel_num = static_cast<int32_t*>(outputs[2]);
    if (!points || !points_size || !voxels || !coors || !voxel_num)
        return fail(SESSD_E_INVALID, "voxelgen.enqueue: null tensor pointer");
    if ((reinterpret_cast<uintptr_t>(voxels) | reinterpret_cast<uintptr_t>(coors)) & 15)
        return fail(SESSD_E_INVALID, "voxelgen.enqueue: outputs must be 16-byte aligned");

    lastMaxPoints_ = max_points;
    const Layout L = carve(workspace, max_points);
    HashTable t = make_hash(L.keys, L.vals, L.cap);
    VgParams p{min_x_range_, max_x_range_, min_y_range_, max_y_range_, min_z_range_, max_z_range_,
               voxel_x_size_, voxel_y_size_, voxel_z_size_, grid_x_size_, grid_y_size_, grid_z_size_,
               voxelNum_, pointNum_};

    FillArgs f;
    f.add(L.keys, (uint64_t)(L.slots - L.keys) + (uint64_t)L.cap * pointNum_, kEmpty);
    f.add(L.status, 4, 0);
    if (!(flags_ & SESSD_FLAG_SKIP_PAD_ROWS)) {  // voxelGenerator.cu:524-525
        f.add(voxels, (uint64_t)voxelNum_ * 4, 0);
        f.add(coors, (uint64_t)voxelNum_ * 4, 0);
    }
    if (also_clear) {  // a pipeline's small clears ride along in the launch that heads the frame anyway
        if (f.n + also_clear->n > FillArgs::kMaxRegions) return fail(SESSD_E_INVALID, "voxelgen.enqueue: too many regions to clear");
        for (int i = 0; i < also_clear->n; ++i) f.r[f.n++] = also_clear->r[i];
    }
    SESSD_TRY(launch_fill(f, stream));

    const dim3 grid(L.n_blocks), block(kBlock);
    hipLaunchKernelGGL(vg_insert, grid, block, 0, stream, points, points_size, max_points, pf, p, t,
                       L.slots, L.pt_slot, L.status);
    hipLaunchKernelGGL(vg_flags, grid, block, 0, stream, points_size, max_points, pointNum_, L.slots,
                       L.pt_slot, L.first_words, L.block_counts);
    hipLaunchKernelGGL(vg_finalize, grid, block, 0, stream, points, pf, p, t, L.slots, L.pt_slot,
                       L.first_words, L.block_counts, L.n_blocks, voxels, coors, voxel_num, L.status,
                       mirror ? *mirror : MirrorInit());
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

int read_status_word(const void* workspace, size_t offset, hipStream_t stream, int32_t* status) {
    if (!workspace || !status) return fail(SESSD_E_INVALID, "status: null argument");
    SESSD_HIP_TRY(hipMemcpyAsync(status, static_cast<const uint8_t*>(workspace) + offset, sizeof(int32_t),
                                 hipMemcpyDeviceToHost, stream));
    SESSD_HIP_TRY(hipStreamSynchronize(stream));
    return SESSD_OK;
}

// ---------------------------------------------------------------------------------------------
// The enqueue that allocates nothing and takes no workspace: its scratch memory is a file-scope device
// array.  Every GPU the library runs on holds its own copy of the array (8 MiB, until the process ends)
// at its own address; `scratch` below is only the host-side name of the symbol, never a device pointer,
// so host code asks the runtime for the address once per device and hands THAT to the kernels.
// ---------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = 8u << 20;  // fits the reference's 80000-point tensor (7.7 MB)
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};  // device address of `scratch`, per device
}  // namespace

// -> address of the current device's copy of `scratch` (resolved on the first call per device)
int voxelgen_static_scratch(void** out) {
    int dev = -1;
    SESSD_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(SESSD_E_UNSUPPORTED, "voxelgen: device index %d is beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        SESSD_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(SESSD_E_HIP, "voxelgen: the static scratch array has no address on device %d", dev);
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return SESSD_OK;
}

int VoxelGeneratorPlugin::enqueueStatic(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                                        const void* const* inputs, void* const* outputs, hipStream_t stream) {
    if (!inputDesc || inputDesc[0].nbDims != 3 || inputDesc[0].d[1] <= 0)
        return fail(SESSD_E_INVALID, "voxelgen.enqueue_static: points must be [1,max_points,F]");
    // the size check comes before any runtime call: a request that does not fit touches nothing
    const size_t need = carve(nullptr, inputDesc[0].d[1]).total;
    if (need > kStaticScratchBytes)
        return fail(SESSD_E_INVALID,
                    "voxelgen.enqueue_static: a points tensor of %d rows with %d points per voxel needs %zu bytes of "
                    "scratch, the static buffer holds %zu; use sessd_voxelgen_enqueue with a workspace of your own",
                    inputDesc[0].d[1], pointNum_, need, kStaticScratchBytes);
    void* ws = nullptr;
    SESSD_TRY(voxelgen_static_scratch(&ws));
    return enqueue(inputDesc, outputDesc, inputs, outputs, ws, stream);
}

}  // namespace sessd
