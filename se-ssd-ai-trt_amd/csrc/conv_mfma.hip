// conv_mfma.hip -- gather-GEMM on the matrix cores (gfx950 MFMA), FP32 or FP16 features, FP32 accumulate.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// One workgroup (4 wave64) owns a tile of consecutive output rows and all Cout columns.  The number of
// tiles is chosen per launch from the device-side row count so that every CU gets the same number of
// tiles (tile_plan()); where the rulebook carries equal-work cuts (tile_cut.hip) the tiles follow them,
// otherwise all tiles have the same length.
//   * The tile's neighbour lists nbr[k][row0 .. row0+rows) are staged in LDS and compacted per offset
//     with wave64 ballot + popcount: pair list k = the (input row, local output row) pairs of the rows
//     that really have a neighbour at offset k.  Only those rows enter an MFMA block, so the matrix
//     cores do not multiply the zero rows a dense [rows x K*Cin] gather matrix would be half full of.
//   * Non-empty offsets are dealt to the four waves (split-K over offsets), ranked by their number of
//     16-pair blocks and dealt back and forth (0 1 2 3 3 2 1 0 ...): tiles x 4 waves is what fills 256 CUs
//     with a ~17k-row problem.
//   * A wave gathers 16 pairs per MFMA block straight into operand registers: lane (i = lane%16,
//     q = lane/16) loads 16 bytes of pair i's input row per K-chunk (FP32: channels 16g+4q..+3, FP16:
//     channels 32g+8q..+7), i.e. every row is read as 64-byte segments.  The weights were reordered on
//     the host so that the other operand of the same MFMA steps is one 16-byte load per lane as well;
//     one pass over W[k] serves all blocks of the offset.  The next offset's rows are loaded at the top
//     of the current one, and the weight registers of chunk g are refilled with the next offset's chunk g
//     as soon as the MFMAs that read them have issued.  The FP32 kernels issue all of these as buffer loads
//     outside any branch (a request with nothing to fetch points out of range), so that the waits the
//     compiler inserts cover exactly the operands about to be used.
//   * FP32: v_mfma_f32_16x16x4_f32; FP16: v_mfma_f32_16x16x32_f16 (16x16x16 for Cin = 16).  The weights
//     are the MFMA's A operand and the gathered rows its B operand, so a lane ends up with four
//     consecutive output channels of one pair; the block is then added into the wave's private partial
//     tile in LDS at the pairs' output rows with 16-byte read-modify-writes (only this wave touches its
//     partial and LDS keeps a wave's operations in order, so the sum order is fixed; LDS float atomics
//     measured several times slower).
//   * The four partial tiles are summed in a fixed order, scale/shift/ReLU is applied in FP32 and each
//     output row is written once, coalesced.  No global atomics; results are bit-identical run to run.
//     A caller may name a dense tensor (DenseTarget): the epilogue then also stores every row at its voxel's
//     place there, which is the sparse2Dense step that follows the last layer.
#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kWaves = 4;           // wave64s per workgroup
constexpr int kTileRowsBase = 48;   // tile capacity of most kernel instantiations
constexpr int kTileRowsWideF16 = 64;  // ... and of the wide FP16 ones
constexpr int kMaxK = kGemmMaxOffsets;

// Tile capacity: most output rows a workgroup can own (<= 64: one wave stages a neighbour list).  The rows
// of all blocks of two offsets live in registers, so the capacity is what the register file allows: 48 rows
// for FP32 (64 spill in the 64-wide layers), 64 for the wide FP16 layers, whose rows take half the registers
// and whose launches are short enough for one tile per CU less to show.  The narrow FP16 layers and
// Cin = 128 measured slower with 64.
constexpr int tile_rows(bool half_operands, int cin, int cout) {
    return half_operands && cin <= 64 && cin * cout >= 32 * 64 ? kTileRowsWideF16 : kTileRowsBase;
}

// Per-dtype shape of one K-chunk: how many channels it spans, what a lane holds of it, and the MFMA
// sequence that consumes it (w = weights fragment -> A operand, x = gathered-row fragment -> B operand).
template <typename T, int CIN>
struct Chunk;

template <int CIN>
struct Chunk<float, CIN> {
    using Vec = float4;  // 4 channels
    static constexpr int kChannels = 16, kLaneElems = 4;
    static __device__ __forceinline__ Vec zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ void mma(const Vec& w, const Vec& x, v4f& acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, x.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, x.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, x.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, x.w, acc, 0, 0, 0);
    }
};

// Cin = 4 (the voxel means entering the first layer): the whole inner dimension of an offset is one MFMA
// K-step, a lane holds a single channel
template <>
struct Chunk<float, 4> {
    using Vec = float;
    static constexpr int kChannels = 4, kLaneElems = 1;
    static __device__ __forceinline__ Vec zero() { return 0.f; }
    static __device__ __forceinline__ void mma(const Vec& w, const Vec& x, v4f& acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w, x, acc, 0, 0, 0);
    }
};

template <int CIN>
struct Chunk<__half, CIN> {
    using Vec = float4;  // 8 halfs = channels 32g+8q .. +7
    static constexpr int kChannels = 32, kLaneElems = 8;
    static __device__ __forceinline__ Vec zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ void mma(const Vec& w, const Vec& x, v4f& acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const v8h*>(&w),
                                                     *reinterpret_cast<const v8h*>(&x), acc, 0, 0, 0);
    }
};

template <>
struct Chunk<__half, 16> {
    using Vec = float2;  // 4 halfs = channels 4q .. +3
    static constexpr int kChannels = 16, kLaneElems = 4;
    static __device__ __forceinline__ Vec zero() { return make_float2(0.f, 0.f); }
    static __device__ __forceinline__ void mma(const Vec& w, const Vec& x, v4f& acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(*reinterpret_cast<const v4h*>(&w),
                                                    *reinterpret_cast<const v4h*>(&x), acc, 0, 0, 0);
    }
};

// Buffer loads (FP32 kernels): a lane whose offset lies beyond the buffer gets zeros and no memory is touched,
// so a request that has nothing to fetch needs no branch around it.
typedef unsigned int v4u32 __attribute__((__vector_size__(16)));
constexpr unsigned kOutOfRange = 0x80000000u;   // beyond any buffer the kernel is given (launch() checks)
constexpr int kRawBuffer = 0x00020000;          // descriptor word 3: raw 32-bit data format, no swizzle
template <typename Vec>
__device__ __forceinline__ Vec buffer_load(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {
    if constexpr (sizeof(Vec) == 16) {
        v4u32 v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, 0);
        return *reinterpret_cast<Vec*>(&v);
    } else {
        static_assert(sizeof(Vec) == 4, "FP32 operands are 16 bytes per lane, or 4 when Cin = 4");
        unsigned v = __builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, 0);
        return *reinterpret_cast<Vec*>(&v);
    }
}

__device__ __forceinline__ void store1(float* dst, float v) { *dst = v; }
__device__ __forceinline__ void store1(__half* dst, float v) { *dst = __float2half_rn(v); }

// four consecutive output channels -> memory
__device__ __forceinline__ void store4(float* dst, const float (&o)[4]) {
    *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void store4(__half* dst, const float (&o)[4]) {
    union {
        __half2 h[2];
        uint2 u;
    } p;
    p.h[0] = __floats2half2_rn(o[0], o[1]);
    p.h[1] = __floats2half2_rn(o[2], o[3]);
    *reinterpret_cast<uint2*>(dst) = p.u;
}

// waves per SIMD the register allocation must leave room for: two workgroups per CU in the wide layers
// (whose tiles come two to a CU), more in the narrow ones
constexpr int min_waves_per_simd(int cin, int cout) {
    return cin * cout >= 32 * 64 ? 2 : (cin * cout >= 32 * 32 ? 3 : 4);
}

// T = type of the input features and of the arithmetic's operands, TO = type the output rows are stored
// in (differs only for the first layer of an FP16 pipeline: FP32 voxel means in, FP16 features out)
template <typename T, int CIN, int COUT, typename TO = T>
__global__ void __launch_bounds__(kWaves * 64, min_waves_per_simd(CIN, COUT))
conv_mfma(const T* __restrict__ in, TO* __restrict__ out, const void* __restrict__ Wp,
          const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
          const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad,
          int num_cu, const int32_t* __restrict__ tiles, DenseTarget dt) {
    using C = Chunk<T, CIN>;
    using Vec = typename C::Vec;
    constexpr int G = CIN / C::kChannels;  // K-chunks of the inner dimension
    constexpr int NBT = COUT / 16;         // 16-column blocks of the layer
    // 128 output columns: the waves pair up, each wave of a pair takes half of the columns of the offsets
    // dealt to the pair.  Weight registers, accumulators and the wave's partial tile then have the size of
    // the 64-column case (two workgroups per CU instead of one wave per SIMD and 100 KB of LDS); the price
    // is that both waves of a pair gather the rows of their offsets.
    constexpr int CS = COUT >= 128 ? 2 : 1;  // waves sharing an offset (column split)
    constexpr int KG = kWaves / CS;          // groups the offsets are dealt to
    constexpr int NB = NBT / CS;             // column blocks of one wave
    constexpr int CW = COUT / CS;            // columns of one wave
    constexpr int LDP = CW + 4;              // padded row stride of the partial tiles in LDS
    static_assert(CIN % C::kChannels == 0 && COUT % 16 == 0, "channel counts must fill whole MFMA chunks");
    constexpr int kTileRows = tile_rows(sizeof(T) == 2, CIN, COUT);
    constexpr int kMaxBlk = (kTileRows + 15) / 16;  // MFMA row blocks an offset can need
    static_assert(kGemmMinTileRows <= kTileRows && kTileRows <= 64, "capacity: at least the bound the grid is sized with, at most one wave");
    __shared__ int32_t s_in[kMaxK * kTileRows];   // compacted pair lists: input row ...
    __shared__ uint8_t s_row[kMaxK * kTileRows];  // ... and local output row of pair j of offset k
    __shared__ int32_t s_cnt[kMaxK + 5];          // pairs per offset
    __shared__ float s_part[kWaves * kTileRows * LDP];

    // the row count and the tile cuts are independent loads: request them together (the grid is sized for
    // the smallest tile height any rulebook is cut for and never indexes past the cut table)
    int n = *num_out;
    const int cut_count = tiles ? tiles[0] : 0;
    const int cut_begin = tiles ? tiles[4 + blockIdx.x] : 0;
    const int cut_end = tiles ? tiles[5 + blockIdx.x] : 0;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int kgrp = wave / CS;   // offsets are dealt to this group ...
    const int chalf = wave % CS;  // ... and this wave computes this part of their columns
    constexpr int kVecPerRow = COUT / 4;
    // scale/shift are requested now and parked in LDS (below, once the first piece's list loads are out as
    // well, so that the workgroup waits once for all of them): the epilogue does not wait for global memory
    __shared__ float s_epi[2 * COUT];
    static_assert(COUT <= kWaves * 64, "one thread per output channel fetches the epilogue constants");
    float epi_scale = 1.f, epi_shift = 0.f;
    if (tid < COUT) {
        if (scale) epi_scale = scale[tid];
        if (shift) epi_shift = shift[tid];
    }
    const int ec4 = (tid % kVecPerRow) * 4;  // this thread's epilogue columns, the same for every row it stores
    static_assert((kWaves * 64) % kVecPerRow == 0, "a thread must keep its columns from row to row");

    // rows >= n: the reference zero-fills them (then BN+ReLU): epilogue(0), spread over all workgroups
    if (write_pad) {
        const int chunks = (max_voxels - n + kTileRows - 1) / kTileRows;
        for (int c = blockIdx.x; c < chunks; c += gridDim.x)
            for (int v = tid; v < kTileRows * kVecPerRow; v += kWaves * 64) {
                const int row = n + c * kTileRows + v / kVecPerRow, c4 = (v % kVecPerRow) * 4;
                if (row >= max_voxels) continue;
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float s = 0.f;
                    if (scale) s = s * scale[c4 + e];
                    if (shift) s = s + shift[c4 + e];
                    if (relu) s = s > 0.f ? s : 0.f;
                    o[e] = s;
                }
                store4(out + (size_t)row * COUT + c4, o);
            }
    }
    // this workgroup's run of rows: from the rulebook's equal-work cuts, or equal lengths
    int run_begin, run_end;
    if (cut_count > 0) {
        if ((int)blockIdx.x >= cut_count) return;
        run_begin = cut_begin;
        run_end = cut_end;
    } else {
        const int R = tile_plan(n, num_cu, kTileRows).height;
        run_begin = blockIdx.x * R;
        run_end = run_begin + R < n ? run_begin + R : n;
    }
    const int i = lane & 15;  // pair inside a 16-pair block
    const int q = lane >> 4;  // channel group inside a K-chunk
    const Vec* wp = reinterpret_cast<const Vec*>(Wp) + lane;
    // a run longer than the tile capacity (sparse stretches under equal-work cuts) is walked in pieces
    for (int row0 = run_begin; row0 < run_end; row0 += kTileRows) {
    const int rows = run_end - row0 < kTileRows ? run_end - row0 : kTileRows;

    // ---- stage + compact: a wave turns one offset's neighbour list into a pair list per step ----
    // (all of a wave's list loads are requested before the first one is consumed)
    constexpr int kListsPerWave = (kMaxK + kWaves - 1) / kWaves;
    int staged[kListsPerWave];
#pragma unroll
    for (int s = 0; s < kListsPerWave; ++s) {
        const int k = wave + s * kWaves;
        staged[s] = (k < K && lane < rows) ? nbr[(size_t)k * max_voxels + row0 + lane] : -1;
    }
    if (row0 == run_begin && tid < COUT) {
        s_epi[tid] = epi_scale;
        s_epi[COUT + tid] = epi_shift;
    }
#pragma unroll
    for (int s = 0; s < kListsPerWave; ++s) {
        const int k = wave + s * kWaves;
        if (k >= K) break;
        const int v = staged[s];
        const uint64_t m = __ballot(v >= 0);
        if (v >= 0) {
            const int j = __popcll(m & ((1ull << lane) - 1ull));
            s_in[k * kTileRows + j] = v;
            s_row[k * kTileRows + j] = (uint8_t)lane;
        }
        if (lane == 0) s_cnt[k] = __popcll(m);
    }
    // zero this wave's partial tile
    float* part = s_part + wave * kTileRows * LDP;
    for (int t = lane; t < rows * LDP / 4; t += 64) reinterpret_cast<float4*>(part)[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();

    // offsets this wave handles.  An offset costs one MFMA pass per 16 pairs, so the offsets are ranked by
    // pass count (ballots: lane k holds offset k) and dealt in that order back and forth over the waves
    // (0 1 2 3 3 2 1 0 ...): plain round-robin left the busiest wave ~13 % above the mean, this ~8 %.
    uint32_t my_mask;
    {
        const int c = lane < K ? s_cnt[lane] : 0;
        const int b = (c + 15) >> 4;
        const uint64_t below = (1ull << lane) - 1ull;
        int rank = 0, ahead = 0;
#pragma unroll
        for (int size = kMaxBlk; size >= 1; --size) {
            const uint64_t m = __ballot(b == size);
            if (b == size) rank = ahead + __popcll(m & below);
            ahead += __popcll(m);
        }
        const int r8 = rank % (2 * KG);
        const int w = r8 < KG ? r8 : 2 * KG - 1 - r8;
        my_mask = (uint32_t)__ballot(b > 0 && w == kgrp);
    }

    // FP32: every load of the main loop is a buffer load outside any branch -- padding lanes, absent blocks and
    // the requests behind the last offset get an out-of-range offset.  Straight-line requests are what lets
    // the compiler count the loads in flight exactly (s_waitcnt vmcnt counts in issue order; one load under a
    // branch and every later wait becomes a wait for nearly everything, the operands just requested
    // included).  64->64: 37 -> 33 us.  FP16 measured 1-2 % slower this way and keeps plain loads.
    constexpr bool kBuf = sizeof(T) == 4;
    __amdgpu_buffer_rsrc_t rs_in, rs_w;
    if constexpr (kBuf) {
        rs_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(in), 0, (int)((size_t)max_voxels * CIN * sizeof(T)),
                                                  kRawBuffer);
        rs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(Wp), 0,
                                                 (int)((size_t)K * G * NBT * 64 * sizeof(Vec)), kRawBuffer);
    }
    // gathered rows of all blocks of offset k -> operand registers (zeros for the padding pairs); cnt = 0:
    // nothing to fetch
    auto load_a_block = [&](int k, int cnt, int blk, Vec (&a)[kMaxBlk][G]) {
        const int j = blk * 16 + i;
        const bool live = j < cnt;
        if constexpr (kBuf) {
            const int idx = s_in[k * kTileRows + (live ? j : 0)];
            const unsigned at = live ? (unsigned)((idx * CIN + q * C::kLaneElems) * (int)sizeof(T)) : kOutOfRange;
#pragma unroll
            for (int g = 0; g < G; ++g) a[blk][g] = buffer_load<Vec>(rs_in, at + g * C::kChannels * (unsigned)sizeof(T));
        } else {
            const int idx = live ? s_in[k * kTileRows + j] : 0;
            const T* src = in + (size_t)idx * CIN + q * C::kLaneElems;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                Vec v = C::zero();
                if (live) v = *reinterpret_cast<const Vec*>(src + g * C::kChannels);
                a[blk][g] = v;
            }
        }
    };
    auto load_a = [&](int k, int cnt, Vec (&a)[kMaxBlk][G]) {
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk) load_a_block(k, cnt, blk, a);
    };
    // chunk g of W[k] -> operand registers (buffer path: k < 0 = nothing to fetch)
    auto load_b = [&](int k, int g, Vec (&b)[NB]) {
        if constexpr (kBuf) {
            const unsigned at = k >= 0 ? (unsigned)(((((k * G + g) * NBT + chalf * NB) * 64) + lane) * (int)sizeof(Vec))
                                       : kOutOfRange;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) b[nb] = buffer_load<Vec>(rs_w, at + nb * 64 * (unsigned)sizeof(Vec));
        } else {
            const Vec* wk = wp + (((size_t)k * G + g) * NBT + chalf * NB) * 64;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) b[nb] = wk[nb * 64];
        }
    };

    int k_cur = my_mask ? __ffs(my_mask) - 1 : -1;
    my_mask &= my_mask - 1;
    Vec a_cur[kMaxBlk][G], a_nxt[kMaxBlk][G], b[G][NB];
    int cnt_cur = 0, cnt_nxt = 0;
    if (k_cur >= 0) {
        cnt_cur = __builtin_amdgcn_readfirstlane(s_cnt[k_cur]);
        load_a(k_cur, cnt_cur, a_cur);
#pragma unroll
        for (int g = 0; g < G; ++g) load_b(k_cur, g, b[g]);
    }
    while (k_cur >= 0) {
        const int k_nxt = my_mask ? __ffs(my_mask) - 1 : -1;
        my_mask &= my_mask - 1;
        if constexpr (kBuf) {
            // (the next offset's rows are requested block by block between the chunks below)
            cnt_nxt = k_nxt >= 0 ? __builtin_amdgcn_readfirstlane(s_cnt[k_nxt]) : 0;  // wave-uniform: keep it scalar
        } else {
            // Everything requested during the previous offset is consumed by this one: wait for all of it here,
            // before this offset's own requests go out.  Left to itself the compiler waits chunk by chunk, and
            // because some requests sit under branches its count is inexact: the wait before the second chunk
            // then also covers the rows and weights requested a moment ago for the NEXT offset.
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            if (k_nxt >= 0) {
                cnt_nxt = __builtin_amdgcn_readfirstlane(s_cnt[k_nxt]);
                load_a(k_nxt, cnt_nxt, a_nxt);
            }
        }
        v4f acc[kMaxBlk][NB];
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) acc[blk][nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int blk = 0; blk < kMaxBlk; ++blk) {
                if (blk * 16 >= cnt_cur) continue;  // wave-uniform: this offset has fewer pairs
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) C::mma(b[g][nb], a_cur[blk][g], acc[blk][nb]);
            }
            // The next offset's chunk g replaces this one, without a branch: FP32 asks out of range after the
            // last offset, FP16 asks for the same chunk once more.
            if constexpr (kBuf) load_b(k_nxt, g, b[g]);
            else load_b(k_nxt >= 0 ? k_nxt : k_cur, g, b[g]);
            // FP32: the next offset's rows follow, one block behind each chunk, instead of all at the top of the
            // offset: the address unit sees the requests spread over the offset (frame 0.396 -> 0.390 ms)
            if constexpr (kBuf) {
#pragma unroll
                for (int blk = g; blk < kMaxBlk; blk += G) load_a_block(k_nxt >= 0 ? k_nxt : 0, cnt_nxt, blk, a_nxt);
            }
        }
        // block results -> partial tile.  D is the transposed block: lane (pair j = lane%16, q = lane/16)
        // holds output channels 16nb+4q .. +3 of pair j -- one 16-byte LDS read-modify-write per column
        // block.
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk) {
            if (blk * 16 >= cnt_cur) continue;
            const int j = blk * 16 + i;
            if (j < cnt_cur) {
                float* dst = part + (int)s_row[k_cur * kTileRows + j] * LDP + q * 4;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    float4 v = *reinterpret_cast<float4*>(dst + nb * 16);
                    v.x += acc[blk][nb][0];
                    v.y += acc[blk][nb][1];
                    v.z += acc[blk][nb][2];
                    v.w += acc[blk][nb][3];
                    *reinterpret_cast<float4*>(dst + nb * 16) = v;
                }
            }
        }
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk)
#pragma unroll
            for (int g = 0; g < G; ++g) a_cur[blk][g] = a_nxt[blk][g];
        k_cur = k_nxt;
        cnt_cur = cnt_nxt;
    }
    __syncthreads();

    // fixed-order sum of the four partials, epilogue, coalesced stores
    for (int v = tid; v < rows * kVecPerRow; v += kWaves * 64) {
        const int r = v / kVecPerRow;
        // the partial tiles of the KG waves that hold this column, in a fixed order
        const float* col = s_part + ((ec4 / CW) * kTileRows + r) * LDP + ec4 % CW;
        float4 acc4 = *reinterpret_cast<const float4*>(col);
#pragma unroll
        for (int w = 1; w < KG; ++w) {
            const float4 p4 = *reinterpret_cast<const float4*>(col + w * CS * kTileRows * LDP);
            acc4.x += p4.x;
            acc4.y += p4.y;
            acc4.z += p4.z;
            acc4.w += p4.w;
        }
        float o[4] = {acc4.x, acc4.y, acc4.z, acc4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float s = o[e];
            if (scale) s = s * s_epi[ec4 + e];
            if (shift) s = s + s_epi[COUT + ec4 + e];
            if (relu) s = s > 0.f ? s : 0.f;
            o[e] = s;
        }
        store4(out + (size_t)(row0 + r) * COUT + ec4, o);
        if (dt.dense) {  // the sparse2Dense scatter of this row, fused (uniform branch)
            const int4 cc = reinterpret_cast<const int4*>(dt.coors)[row0 + r];  // (b,z,y,x)
            if (cc.x != 0 || cc.y < 0 || cc.y >= dt.D || cc.z < 0 || cc.z >= dt.H || cc.w < 0 || cc.w >= dt.W) {
                if (dt.status && ec4 == 0) atomicOr(dt.status, SESSD_STATUS_BAD_COORD);
            } else {
                TO* d = static_cast<TO*>(dt.dense) + ((size_t)cc.y * dt.Hp + cc.z + dt.pad_top) * dt.Wp + cc.w + dt.pad_left;
                const size_t plane = (size_t)dt.D * dt.Hp * dt.Wp;  // channel stride
#pragma unroll
                for (int e = 0; e < 4; ++e) store1(d + (size_t)(ec4 + e) * plane, o[e]);
            }
        }
    }
    __syncthreads();  // the next piece reuses the lists and partial tiles
    }
}

int compute_units() {
    static int cu = 0;
    if (cu == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cu = v;
        else
            cu = 256;
    }
    return cu;
}

template <typename T, int CIN, int COUT, typename TO = T>
int launch(const GemmArgs& a, hipStream_t stream) {
    // the FP32 kernels address their operands with 32-bit byte offsets and use 2^31 as "out of range"
    if (sizeof(T) == 4 && ((size_t)a.max_voxels * CIN * sizeof(T) >= kOutOfRange ||
                           (size_t)a.K * CIN * COUT * sizeof(T) >= kOutOfRange))
        return SESSD_E_UNSUPPORTED;
    const int num_cu = compute_units();
    // enough workgroups for any cut of any n <= max_voxels rows: tile_plan() never makes more tiles for fewer
    // rows or a taller target (surplus workgroups return at once)
    const unsigned blocks = (unsigned)tile_plan(a.max_voxels, num_cu, kGemmMinTileRows).count;
    hipLaunchKernelGGL((conv_mfma<T, CIN, COUT, TO>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                       static_cast<const T*>(a.in_feat), static_cast<TO*>(a.out_feat), a.w_packed, a.nbr,
                       a.num_out, a.max_voxels, a.K, a.scale, a.shift, a.relu, a.write_pad_rows, num_cu, a.tiles,
                       a.dense);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

bool mfma_shape(int K, int cin, int cout, int dtype) {
    if (K > kMaxK) return false;
    if (cin == 4) return cout == 16 || cout == 32;  // FP32 operands whatever the pipeline's feature dtype
    const int shapes[][2] = {{16, 16}, {16, 32}, {32, 32}, {32, 64}, {64, 64}, {64, 128}, {128, 128}};
    for (auto& s : shapes)
        if (s[0] == cin && s[1] == cout) return true;
    return false;
}

// channels per K-chunk and elements per lane, as in Chunk<>
void chunk_shape(int dtype, int cin, int* channels, int* lane_elems) {
    if (cin == 4) {
        *channels = 4;
        *lane_elems = 1;
    } else if (dtype == SESSD_FLOAT) {
        *channels = 16;
        *lane_elems = 4;
    } else if (cin == 16) {
        *channels = 16;
        *lane_elems = 4;
    } else {
        *channels = 32;
        *lane_elems = 8;
    }
}

}  // namespace

int gemm_compute_units() { return compute_units(); }

int gemm_tile_rows(int cin, int cout, int dtype) {
    if (gemm_runs_wide(kMaxK, cin, cout, dtype, dtype)) return gemm_wide_tile_rows();
    return tile_rows(dtype == SESSD_HALF && cin != 4, cin, cout);
}

bool gemm_runs_on_mfma(int K, int cin, int cout, int in_type, int out_type) {
    if (!mfma_shape(K, cin, cout, out_type)) return false;
    return in_type == out_type || (cin == 4 && in_type == SESSD_FLOAT && out_type == SESSD_HALF);
}

size_t packed_weight_bytes(int K, int cin, int cout, int dtype) {
    if (!mfma_shape(K, cin, cout, dtype)) return 0;
    return (size_t)K * cin * cout * (dtype == SESSD_HALF && cin != 4 ? sizeof(__half) : sizeof(float));
}

// Operand order: Wp[k][g][nb][lane][e] = W[k][C*g + E*(lane/16) + e][16nb + lane%16] with C channels per
// K-chunk and E elements per lane (FP32: 16/4, FP16: 32/8, FP16 with Cin = 16: 16/4, Cin = 4: 4/1).  Cin = 4
// always takes FP32 operands (the voxel means are FP32); in an FP16 pipeline its weights are the
// half-rounded values, as in every other layer of that pipeline.
void pack_weights(const float* w, int K, int cin, int cout, int dtype, void* dst) {
    int C, E;
    chunk_shape(dtype, cin, &C, &E);
    const int G = cin / C, NB = cout / 16;
    for (int k = 0; k < K; ++k)
        for (int g = 0; g < G; ++g)
            for (int nb = 0; nb < NB; ++nb)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < E; ++e) {
                        const size_t o = ((((size_t)k * G + g) * NB + nb) * 64 + lane) * E + e;
                        const float v = w[((size_t)k * cin + C * g + E * (lane / 16) + e) * cout + 16 * nb + lane % 16];
                        if (dtype == SESSD_HALF && cin != 4) static_cast<__half*>(dst)[o] = __float2half_rn(v);
                        else if (dtype == SESSD_HALF) static_cast<float*>(dst)[o] = __half2float(__float2half_rn(v));
                        else static_cast<float*>(dst)[o] = v;
                    }
}

// -> SESSD_OK when an MFMA kernel was launched, SESSD_E_UNSUPPORTED when the shape/dtype is not covered
int launch_mfma(const GemmArgs& a, hipStream_t stream) {
    if (!a.w_packed || !mfma_shape(a.K, a.cin, a.cout, a.out_type)) return SESSD_E_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.in_feat) | reinterpret_cast<uintptr_t>(a.out_feat)) & 15)
        return SESSD_E_UNSUPPORTED;
    if (a.cin == 4 && a.in_type == SESSD_FLOAT && a.out_type == SESSD_HALF) {  // first layer of an FP16 pipeline
        if (a.cout == 16) return launch<float, 4, 16, __half>(a, stream);
        if (a.cout == 32) return launch<float, 4, 32, __half>(a, stream);
    }
    if (a.in_type != a.out_type) return SESSD_E_UNSUPPORTED;
#define SESSD_CASE(CI, CO)                                                        \
    if (a.cin == CI && a.cout == CO)                                              \
    return a.in_type == SESSD_HALF ? launch<__half, CI, CO>(a, stream) : launch<float, CI, CO>(a, stream)
    if (a.cin == 4 && a.cout == 16) return launch<float, 4, 16>(a, stream);  // (FP32 only: mfma_shape)
    if (a.cin == 4 && a.cout == 32) return launch<float, 4, 32>(a, stream);
    SESSD_CASE(16, 16);
    SESSD_CASE(16, 32);
    SESSD_CASE(32, 32);
    SESSD_CASE(32, 64);
    SESSD_CASE(64, 64);
    SESSD_CASE(64, 128);
    SESSD_CASE(128, 128);
#undef SESSD_CASE
    return SESSD_E_UNSUPPORTED;
}

}  // namespace sessd
