// common.h -- helpers shared by every translation unit of libsessd3d.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <new>
#include <stdexcept>
#include <string>

#include "../../include/sessd3d.h"

namespace sessd {

// ---------------------------------------------------------------------------------------------
// error reporting: no abort(), a thread-local message and an error code instead
// (the reference's checkCudaErrors prints and aborts, voxelGenerator.cu:8-19)
// ---------------------------------------------------------------------------------------------
void set_last_error(const std::string& msg);
int fail(int code, const char* fmt, ...);

#define SESSD_HIP_TRY(expr)                                                                      \
    do {                                                                                         \
        hipError_t e__ = (expr);                                                                 \
        if (e__ != hipSuccess)                                                                   \
            return ::sessd::fail(SESSD_E_HIP, "%s:%d: %s -> %s", __FILE__, __LINE__, #expr,      \
                                 hipGetErrorString(e__));                                        \
    } while (0)

// The body of an extern "C" entry point that can allocate on the host (new, std::vector, std::string): no C++
// exception may cross the C boundary, so what the body throws becomes an error code and a message.
template <typename F>
inline int guarded(const char* who, F&& body) noexcept {
    try {
        return body();
    } catch (const std::bad_alloc&) {
        return fail(SESSD_E_NOMEM, "%s: out of host memory", who);
    } catch (const std::length_error&) {
        return fail(SESSD_E_NOMEM, "%s: a size beyond what host memory can hold", who);
    } catch (const std::exception& e) {
        return fail(SESSD_E_INVALID, "%s: %s", who, e.what());
    } catch (...) {
        return fail(SESSD_E_INVALID, "%s: unknown C++ exception", who);
    }
}

#define SESSD_TRY(expr)                  \
    do {                                 \
        int rc__ = (expr);               \
        if (rc__ != SESSD_OK) return rc__; \
    } while (0)

// ---------------------------------------------------------------------------------------------
// workspace carving: 256-byte aligned bump allocation, the same rule the reference uses
// (alignPtr / nextWorkspacePtr / calculateTotalWorkspaceSize, submConv3dlayer.cu:93-124)
// ---------------------------------------------------------------------------------------------
constexpr size_t kWorkspaceAlign = 256;

inline size_t align_up(size_t n, size_t a = kWorkspaceAlign) { return (n + a - 1) / a * a; }

struct WorkspaceCarver {
    uint8_t* base;
    size_t offset = 0;
    explicit WorkspaceCarver(void* p) : base(static_cast<uint8_t*>(p)) {}
    template <typename T>
    T* take(size_t count) {
        T* p = base ? reinterpret_cast<T*>(base + offset) : nullptr;
        offset += align_up(count * sizeof(T));
        return p;
    }
    size_t total() const { return offset; }
};

inline uint32_t next_pow2(uint64_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}
inline int ilog2(uint32_t pow2) {
    int l = 0;
    while ((1u << l) < pow2) ++l;
    return l;
}
inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

inline size_t dtype_size(int32_t t) { return t == SESSD_HALF ? 2 : 4; }

constexpr uint32_t kEmpty = 0xFFFFFFFFu;

// ---------------------------------------------------------------------------------------------
// device side: open-addressing hash over linearised cell keys
// ---------------------------------------------------------------------------------------------
// keys[cap] (cap a power of two) start as kEmpty.  Multiplicative hashing spreads the strongly
// correlated keys of neighbouring cells; linear probing keeps a probe sequence inside one or two
// cache lines.  Every loop is bounded by the capacity: a full table is reported, never spun on.
struct HashTable {
    uint32_t* keys;
    uint32_t* vals;
    uint32_t mask;   // cap - 1
    int32_t shift;   // 32 - log2(cap)
};

#ifdef __HIPCC__
__device__ __forceinline__ uint32_t hash_slot0(const HashTable& t, uint32_t key) {
    return (key * 2654435769u) >> t.shift;
}

// -> slot holding `key` (claimed now or earlier), or -1 when the table is full
__device__ __forceinline__ int32_t hash_insert(const HashTable& t, uint32_t key) {
    uint32_t slot = hash_slot0(t, key);
    for (uint32_t probe = 0; probe <= t.mask; ++probe) {
        uint32_t prev = atomicCAS(&t.keys[slot], kEmpty, key);
        if (prev == kEmpty || prev == key) return (int32_t)slot;
        slot = (slot + 1) & t.mask;
    }
    return -1;
}

// -> slot holding `key`, or -1 when absent
__device__ __forceinline__ int32_t hash_find(const HashTable& t, uint32_t key) {
    uint32_t slot = hash_slot0(t, key);
    for (uint32_t probe = 0; probe <= t.mask; ++probe) {
        uint32_t k = t.keys[slot];
        if (k == key) return (int32_t)slot;
        if (k == kEmpty) return -1;
        slot = (slot + 1) & t.mask;
    }
    return -1;
}

__device__ __forceinline__ uint32_t lane_id() { return __lane_id(); }

// number of set bits of `m` below this lane (wave64)
__device__ __forceinline__ uint32_t rank_in_wave(uint64_t m) {
    return __popcll(m & ((1ull << lane_id()) - 1ull));
}
#endif

inline HashTable make_hash(uint32_t* keys, uint32_t* vals, uint32_t cap) {
    HashTable t;
    t.keys = keys;
    t.vals = vals;
    t.mask = cap - 1;
    t.shift = 32 - ilog2(cap);
    return t;
}

// The neighbour table of the SubM layer that comes next on a coors tensor, as the kernel that CREATES the rows
// of that tensor sees it: it writes "no neighbour" into entries [first_offset, K) of every row it creates, so
// that the SubM build can run its symmetric lookup (which writes those entries only where a neighbour exists)
// without the whole K x max_voxels table being cleared per frame.
struct MirrorInit {
    int32_t* nbr = nullptr;  // [K][stride]
    int stride = 0;          // max_voxels of the SubM layer
    int first_offset = 0;    // 14 for a 3x3x3 kernel: offsets 14..26 are the mirrored ones
    int K = 0;
};

// Optional second destination of a gather-GEMM's epilogue: the dense tensor of the sparse2Dense step that
// would follow (sparse2Dense.cu:182-207: dense[(c*D + z)][y][x] = feat[row][c], here with the zero border of
// Sparse2DensePlugin::setPadding).  The tensor must already be cleared; its element type is the output
// rows' type.
struct DenseTarget {
    void* dense = nullptr;
    const int32_t* coors = nullptr;  // (b,z,y,x) of every output row
    int D = 0, H = 0, W = 0;         // feature map extent the coordinates are checked against
    int Hp = 0, Wp = 0;              // padded plane size
    int pad_top = 0, pad_left = 0;
    int32_t* status = nullptr;       // SESSD_STATUS_BAD_COORD is raised here
};

// ---------------------------------------------------------------------------------------------
// fill: the only way memory is cleared (a kernel, so an enqueue can be captured in a hipGraph)
// ---------------------------------------------------------------------------------------------
struct FillRegion {
    uint32_t* ptr;     // 16-byte aligned
    uint64_t words;    // 32-bit words
    uint32_t value;
};
struct FillArgs {
    static constexpr int kMaxRegions = 48;
    FillRegion r[kMaxRegions];
    int n = 0;
    bool full() const { return n >= kMaxRegions; }
    void add(void* p, uint64_t words, uint32_t value) {
        if (!p || !words || n >= kMaxRegions) return;
        r[n].ptr = static_cast<uint32_t*>(p);
        r[n].words = words;
        r[n].value = value;
        ++n;
    }
};
int launch_fill(const FillArgs& a, hipStream_t stream);

}  // namespace sessd
