// conv_split.hip -- gather-GEMM for FP32 features on the BF16 matrix pipeline, with FP32 accuracy.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// gfx950's FP32 MFMA (16x16x4, 32 cycles) multiplies 64 FLOP per cycle and SIMD, its BF16 MFMA (16x16x32, 16 cycles)
// 1024.  Every FP32 value is the sum of three BF16 values, x = x0 + x1 + x2 (x0 = bf16(x), x1 = bf16(x - x0),
// x2 = bf16(x - x0 - x1); the subtractions are exact, what is left is below 2^-26 |x|), and a product of two BF16
// values is exact in FP32.  So
//     x * w = x0 w0 + (x0 w1 + x1 w0) + (x0 w2 + x1 w1 + x2 w0) + O(2^-26 |x w|)
// -- six BF16 MFMAs with FP32 accumulation do the work of sixteen FP32 MFMAs in 3/8 of their time, and the three
// products that are left out are smaller than the rounding of one FP32 product.  The leading products x0 w0 have
// an accumulator of their own and the five small ones share a second one, added in at the end: with all six in one
// accumulator the rounding of the large sum swallows the small terms and the result is 2-4x further from an FP64
// evaluation than a sequential FP32 sum is; with two it is as close as that sum (the parity tests measure both).
// Infinities in the features turn into NaN (inf - inf in the split); finite inputs of any magnitude are exact to
// the above, BF16 having FP32's exponent range.
//
// The split is done once per feature element, not once per use: the kernel reads its input rows in split form
// (row r = [part 0: Cin BF16][part 1][part 2], 6*Cin bytes) and can write its output rows in that form beside the
// FP32 rows, for the next layer.  split_rows converts an FP32 tensor for a layer whose producer does not.
//
// With the multiplications that cheap the kernel is built like the FP16 tall-tile kernel (conv_tall.hip), dense:
//   * a workgroup (4 wave64) owns 64 consecutive output rows (32 in launches with few rows); a wave owns 16 of
//     them and all columns (half of the columns in the 32-row tiles) and keeps their accumulators in registers
//     over all K offsets: no pair compaction, no partial tiles, no reduction.  A row without a neighbour at an
//     offset is a request that points out of range (zeros, no memory touched);
//   * the weights are split on the host into their three BF16 parts in MFMA operand order; W[k] (all three parts)
//     is copied once per workgroup and offset into one of two LDS buffers, requested DW offsets ahead into
//     registers and stored one offset before its use; one barrier per offset;
//   * every gathered row is requested once, D offsets ahead, straight into MFMA operand registers;
//   * all requests of the offset loop are unconditional and in a fixed order, so the compiler's waits cover exactly
//     the operands about to be used.
// Summation order per output element: offsets ascending, then K-chunks, then weight part 0, 1, 2 and inside each
// the feature parts 0..2: fixed, run-to-run identical.
#include <type_traits>

#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned int v4u32 __attribute__((__vector_size__(16)));

constexpr int kWaves = 4;
constexpr unsigned kOutOfRange = 0x80000000u;
constexpr int kRawBuffer = 0x00020000;

// see conv_tall.hip: a barrier that publishes this wave's LDS stores without draining its global requests
__device__ __forceinline__ void ring_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One of the three weight buffers in LDS (U units of 64 lanes x 16 bytes)
template <int U, int slot>
__device__ __forceinline__ float4* weight_slot() {
    __shared__ float4 s_w[U * 64];
    return s_w;
}

#ifdef SESSD_TRACE
__device__ unsigned long long g_trace[8 * 4 * 40];
__device__ unsigned long long g_blocks[2 * 4096];
#define TRACE(slot)                                                                                   \
    do {                                                                                              \
        if (KC == 27 && CIN == 64 && CS == SESSD_TRACE && (blockIdx.x & 31) == 0 && blockIdx.x < 256 && lane == 0)          \
            g_trace[((blockIdx.x >> 5) * 4 + wave) * 40 + (slot)] = __builtin_readcyclecounter();       \
    } while (0)
#else
#define TRACE(slot)
#endif

// K-chunks of 32 channels; 16 input channels fill half of one (the other lanes' operands are zero)
constexpr int chunks(int cin) { return cin <= 32 ? 1 : cin / 32; }

// The tile of one workgroup.  RB = 16-row blocks per wave, CS = waves that share a row block and split the columns,
// D = offsets the rows are requested ahead, DW = register sets for weights in flight.
template <int CIN, int COUT, int RB, int CS, int D, int DW, int KC>
__device__ __forceinline__ void split_tile(const void* __restrict__ in_split, float* __restrict__ out,
                                           void* __restrict__ out_split, const void* __restrict__ Wp,
                                           const int32_t* __restrict__ nbr, int n, int row0, int max_voxels,
                                           bool has_scale, bool has_shift, int relu, DenseTarget dt, int32_t* s_nbr,
                                           const float* s_epi) {
    constexpr int G = chunks(CIN);
    constexpr int NBT = COUT / 16;     // 16-column blocks of the layer
    constexpr int NBW = NBT / CS;      // ... of one wave
    constexpr int RG = kWaves / CS;    // row groups of the tile
    constexpr int U = G * 3 * NBT;     // 1 KB units of one offset's weights: [chunk][part][column block]
    constexpr int NBUF = D + 1;        // row register sets
    constexpr int TR = RG * RB * 16;
    constexpr int UW = (U + kWaves - 1) / kWaves;  // weight units a wave copies per offset
    constexpr int kRowBytes = split_row_bytes(CIN);
    static_assert(NBT % CS == 0 && kWaves % CS == 0, "column split");
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave / CS, cg = wave % CS;
    if (row0 >= n) return;
    TRACE(0);
#ifdef SESSD_TRACE
    if (KC == 27 && CIN == 64 && CS == SESSD_TRACE && (blockIdx.x & 31) == 0 && blockIdx.x < 256 && lane == 0)
        g_trace[((blockIdx.x >> 5) * 4 + wave) * 40 + 31] = __builtin_amdgcn_s_memrealtime();
#endif

    // the tile's neighbour lists (rows beyond n: none) -> LDS; all requests out before the first store
    {
        constexpr int kPer = (KC * TR + kWaves * 64 - 1) / (kWaves * 64);
        int32_t v[kPer];
#pragma unroll
        for (int it = 0; it < kPer; ++it) {
            const int e = tid + it * kWaves * 64;
            const int k = e / TR, r = e - k * TR;
            v[it] = e < KC * TR && row0 + r < n ? nbr[(size_t)k * max_voxels + row0 + r] : -1;
        }
#pragma unroll
        for (int it = 0; it < kPer; ++it) {
            const int e = tid + it * kWaves * 64;
            if (e < KC * TR) s_nbr[e] = v[it];
        }
    }
    TRACE(1);

    const int i = lane & 15;  // row inside a 16-row block
    const int q = lane >> 4;  // 8-channel group inside a K-chunk
    const __amdgpu_buffer_rsrc_t rs_in = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(in_split), 0, (int)((size_t)max_voxels * kRowBytes), kRawBuffer);
    const float4* wsrc = reinterpret_cast<const float4*>(Wp) + lane;
    const bool lane_has_channels = q * 8 < CIN;  // (CIN = 16: the upper half of the chunk is padding)

    constexpr int NG = G * 3;         // fragment groups of an offset: (chunk g, weight part t), NBW fragments each
    constexpr int PD = 2;             // groups a fragment is requested from LDS ahead of its MFMAs
    constexpr int R = PD + 1;         // fragment register sets
    static_assert(NG % R == 0, "the fragment ring must close over an offset");
    v4u32 a[NBUF][3][RB][G];  // feature parts of the offsets in flight, as MFMA operands
    v4f wreg[DW][UW];
    v4f b[R][NBW];
    v4f acc[2][RB][NBW];      // [0]: the leading products x0 w0, [1]: the five small ones
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int blk = 0; blk < RB; ++blk)
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) acc[c][blk][nb] = (v4f){0.f, 0.f, 0.f, 0.f};

    // period of the unrolled offset loop: register sets and the three LDS buffers get compile-time names
    constexpr int P1 = NBUF % 3 == 0 ? NBUF : 3 * NBUF;
    constexpr int P = P1 % DW == 0 ? P1 : P1 * DW;
    static_assert(P % NBUF == 0 && P % 3 == 0 && P % DW == 0, "period");
    auto unit_of = [&](int j) { return U % kWaves == 0 ? wave + j * kWaves : (wave + j * kWaves) % U; };
    // unit j of this wave's share of W[k] -> registers (beyond the last offset: the last one again, never used)
    auto load_w1 = [&](int k, int set, int j) {
        const int kw = k < KC ? k : KC - 1;
        wreg[set % DW][j] = *reinterpret_cast<const v4f*>(wsrc + ((size_t)kw * U + unit_of(j)) * 64);
    };
    // ... -> LDS buffer `slot` (one of three)
    auto store_w1 = [&](auto slot_c, int set, int j) {
        *reinterpret_cast<v4f*>(weight_slot<U, decltype(slot_c)::value % 3>() + unit_of(j) * 64 + lane) = wreg[set % DW][j];
    };
    // block blk of this wave's rows of offset k -> registers, in two steps: the rows' numbers from the neighbour
    // list in LDS, and (an offset's last group later, so that nothing waits for that read) the requests themselves
    // (no neighbour, or beyond the last offset: requests that fetch nothing)
    int row_idx[RB];
    auto fetch_row_numbers = [&](int k, int blk) {
        const int kr = k < KC ? k : KC - 1;
        const int idx = s_nbr[kr * TR + (rg * RB + blk) * 16 + i];
        row_idx[blk] = k < KC && lane_has_channels ? idx : -1;
    };
    auto load_rows1 = [&](int set, int blk) {
        const int idx = row_idx[blk];
        const unsigned at = idx >= 0 ? (unsigned)(idx * kRowBytes + q * 16) : kOutOfRange;
#pragma unroll
        for (int t = 0; t < 3; ++t)
#pragma unroll
            for (int g = 0; g < G; ++g)
                a[set % NBUF][t][blk][g] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, at + t * (2u * CIN) + g * 64u, 0, 0);
    };
    // fragment group grp of the offset whose weights are in LDS buffer `slot` -> fragment register set
    auto load_frags = [&](auto slot_c, int grp, int set) {
        const v4f* const s_w = reinterpret_cast<const v4f*>(weight_slot<U, decltype(slot_c)::value % 3>()) + cg * NBW * 64 + lane;
#pragma unroll
        for (int j = 0; j < NBW; ++j) b[set % R][j] = s_w[(grp * NBT + j) * 64];
    };
    // Offset k at position s of the period.  During it: its MFMAs, group by group (group (g, t) = the column blocks of
    // weight part t of chunk g, multiplied with the feature parts 0 .. 2-t), with the fragments requested from LDS two
    // groups ahead -- across the end of the offset as well, so the matrix cores never wait for the first fragments
    // of an offset; the rows of offset k+D requested; W[k+2] stored to the LDS buffer that W[k-1] has left and
    // W[k+2+DW] requested.  One barrier, before the first read of the next offset's weights: behind it everybody's
    // W[k+1] is in place (stored during offset k-1) and nobody reads W[k-1] any more.  Every MFMA is followed by at
    // most one of the other instructions (sched_group_barrier), which therefore issue while it executes.
    auto offset_step = [&](int k, auto s_c) {
        constexpr int s = decltype(s_c)::value;
        // The weight units go to groups ahead of the barrier, the row requests to the first group of a chunk; which
        // ones: where the group's MFMAs leave issue slots (12, 8, 4 MFMAs per chunk at 64 columns, 4 fragment
        // requests each): with two chunks units [0, UW/3) in group 1, the rest in group 3; with one chunk all in
        // group 0.
        constexpr int NGS = NG - PD;
        auto units_begin = [](int grp) { return NGS < 4 ? 0 : (grp <= 1 ? 0 : (grp <= 3 ? UW / 3 : UW)); };
        auto units_end = [](int grp) { return NGS < 4 ? (grp == 0 ? UW : 0) : (grp == 1 ? UW / 3 : (grp == 3 ? UW : 0)); };
#pragma unroll
        for (int grp = 0; grp < NG; ++grp) {
            const int g = grp / 3, t = grp % 3;
            int n_dsr = NBW, n_dsw = 0, n_vm = 0;
            if (grp == NG - PD) ring_barrier();
            // (the interleaving below is per group: across groups the scheduler would pull a fragment request down
            // to its first use)
            __builtin_amdgcn_sched_barrier(0);
            if (grp + PD < NG) load_frags(std::integral_constant<int, s>{}, grp + PD, s * NG + grp + PD);
            else load_frags(std::integral_constant<int, s + 1>{}, grp + PD - NG, s * NG + grp + PD);
            if (grp < NGS) {
#pragma unroll
                for (int j = units_begin(grp); j < units_end(grp); ++j) {
                    store_w1(std::integral_constant<int, s + 2>{}, s + 2, j);
                    load_w1(k + 2 + DW, s + 2 + DW, j);
                    ++n_dsw;
                    ++n_vm;
                }
            }
#pragma unroll
            for (int blk = 0; blk < RB; ++blk)
                if (grp == (3 * blk < NG ? 3 * blk : 0)) {
                    load_rows1(s + D, blk);
                    n_vm += 3 * G;
                }
            if (grp == NG - 1) {
#pragma unroll
                for (int blk = 0; blk < RB; ++blk) fetch_row_numbers(k + 1 + D, blk);
                n_dsr += RB;
            }
#pragma unroll
            for (int f = 0; f + t < 3; ++f)
#pragma unroll
                for (int j = 0; j < NBW; ++j)
#pragma unroll
                    for (int blk = 0; blk < RB; ++blk)
                        acc[f + t == 0 ? 0 : 1][blk][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            *reinterpret_cast<const v8bf*>(&b[(s * NG + grp) % R][j]),
                            *reinterpret_cast<const v8bf*>(&a[s % NBUF][f][blk][g]), acc[f + t == 0 ? 0 : 1][blk][j], 0, 0, 0);
            // issue order of the group: MFMA, one other instruction, MFMA, ...
            const int nm = (3 - t) * NBW * RB;
#pragma unroll
            for (int m = 0; m < nm; ++m) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (n_dsr > 0) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    --n_dsr;
                } else if (n_vm > 0) {
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    --n_vm;
                } else if (n_dsw > 0) {
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    --n_dsw;
                }
            }
        }
    };
    // prologue: W[0] and W[1] into their buffers, W[2 .. 1+DW] and the rows of offsets 0 .. D-1 requested
#pragma unroll
    for (int j = 0; j < UW; ++j) load_w1(0, 0, j);
#pragma unroll
    for (int j = 0; j < UW; ++j) store_w1(std::integral_constant<int, 0>{}, 0, j);
#pragma unroll
    for (int j = 0; j < UW; ++j) load_w1(1, 1, j);
#pragma unroll
    for (int j = 0; j < UW; ++j) store_w1(std::integral_constant<int, 1>{}, 1, j);
#pragma unroll
    for (int kk = 0; kk < DW; ++kk)
#pragma unroll
        for (int j = 0; j < UW; ++j) load_w1(2 + kk, 2 + kk, j);
    __syncthreads();  // the neighbour lists and W[0], W[1] are in LDS
#pragma unroll
    for (int kk = 0; kk < D; ++kk)
#pragma unroll
        for (int blk = 0; blk < RB; ++blk) {
            fetch_row_numbers(kk, blk);
            load_rows1(kk, blk);
        }
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) fetch_row_numbers(D, blk);
#pragma unroll
    for (int grp = 0; grp < PD; ++grp) load_frags(std::integral_constant<int, 0>{}, grp, grp);
    TRACE(2);

    auto steps = [&](auto self, int k0, auto s_c, auto last_c) -> void {
        constexpr int s = decltype(s_c)::value;
        if constexpr (s < decltype(last_c)::value) {
            TRACE(3 + k0 + s);
            offset_step(k0 + s, s_c);
            self(self, k0, std::integral_constant<int, s + 1>{}, last_c);
        }
    };
    int k0 = 0;
    for (; k0 + P <= KC; k0 += P) steps(steps, k0, std::integral_constant<int, 0>{}, std::integral_constant<int, P>{});
    steps(steps, k0, std::integral_constant<int, 0>{}, std::integral_constant<int, KC % P>{});

    TRACE(30);
#ifdef SESSD_TRACE
    if (KC == 27 && CIN == 64 && CS == SESSD_TRACE && (blockIdx.x & 31) == 0 && blockIdx.x < 256 && lane == 0)
        g_trace[((blockIdx.x >> 5) * 4 + wave) * 40 + 32] = __builtin_amdgcn_s_memrealtime();
#endif
    // epilogue: lane (i, q) holds output channels 16nb+4q .. +3 of row i of each of its blocks
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) {
        const int row = row0 + (rg * RB + blk) * 16 + i;
        if (row >= n) continue;
        bool to_dense = false;
        float* d = nullptr;
        size_t plane = 0;
        if (dt.dense) {  // the sparse2Dense scatter of this row, fused (uniform branch)
            const int4 cc = reinterpret_cast<const int4*>(dt.coors)[row];  // (b,z,y,x)
            if (cc.x != 0 || cc.y < 0 || cc.y >= dt.D || cc.z < 0 || cc.z >= dt.H || cc.w < 0 || cc.w >= dt.W) {
                if (dt.status && q == 0 && cg == 0) atomicOr(dt.status, SESSD_STATUS_BAD_COORD);
            } else {
                to_dense = true;
                d = static_cast<float*>(dt.dense) + ((size_t)cc.y * dt.Hp + cc.z + dt.pad_top) * dt.Wp + cc.w + dt.pad_left;
                plane = (size_t)dt.D * dt.Hp * dt.Wp;
            }
        }
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int c4 = (cg * NBW + nb) * 16 + q * 4;
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float s = acc[1][blk][nb][e] + acc[0][blk][nb][e];
                if (has_scale) s = s * s_epi[c4 + e];
                if (has_shift) s = s + s_epi[COUT + c4 + e];
                if (relu) s = s > 0.f ? s : 0.f;
                o[e] = s;
            }
            *reinterpret_cast<float4*>(out + (size_t)row * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
            if (out_split) store_split4(out_split, row, COUT, c4, o);
            if (to_dense) {
#pragma unroll
                for (int e = 0; e < 4; ++e) d[(size_t)(c4 + e) * plane] = o[e];
            }
        }
    }
}

template <int CIN, int COUT, int D, int DW, int KC>
__global__ void __launch_bounds__(kWaves * 64, 2)
conv_split(const void* __restrict__ in_split, float* __restrict__ out, void* __restrict__ out_split,
           const void* __restrict__ Wp, const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out,
           int max_voxels, const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad,
           int short_below, DenseTarget dt) {
    __shared__ int32_t s_nbr[KC * 64];
    __shared__ float s_epi[2 * COUT];
#ifdef SESSD_TRACE
    if (KC == 27 && CIN == 64 && threadIdx.x == 0 && blockIdx.x < 4096) g_blocks[2 * blockIdx.x] = __builtin_amdgcn_s_memrealtime();
#endif
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int tid = threadIdx.x;
    constexpr int kVecPerRow = COUT / 4;

    // rows >= n: epilogue(0), as the reference's zero fill followed by BN + ReLU (FP32 rows only: nothing reads
    // the split form of a row that is not active)
    if (write_pad) {
        const int chunks = (max_voxels - n + 63) / 64;
        for (int c = blockIdx.x; c < chunks; c += gridDim.x)
            for (int v = tid; v < 64 * kVecPerRow; v += kWaves * 64) {
                const int row = n + c * 64 + v / kVecPerRow, c4 = (v % kVecPerRow) * 4;
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
                *reinterpret_cast<float4*>(out + (size_t)row * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
            }
    }
    if (tid < COUT) {  // (published by the barrier behind the tile's prologue)
        s_epi[tid] = scale ? scale[tid] : 1.f;
        s_epi[COUT + tid] = shift ? shift[tid] : 0.f;
    }
    // Tile heights: 64 rows, a wave owning 16 rows and all columns; launches with fewer than `short_below` rows
    // (too few 64-row tiles for the compute units) run 32-row tiles, two waves sharing 16 rows and splitting the
    // columns.
    constexpr bool kCanSplitColumns = COUT >= 32;
    if (kCanSplitColumns && n < short_below)
        split_tile<CIN, COUT, 1, kCanSplitColumns ? 2 : 1, D, DW, KC>(in_split, out, out_split, Wp, nbr, n, blockIdx.x * 32, max_voxels, scale != nullptr, shift != nullptr, relu, dt, s_nbr, s_epi);
    else
        split_tile<CIN, COUT, 1, 1, D, DW, KC>(in_split, out, out_split, Wp, nbr, n, blockIdx.x * 64, max_voxels, scale != nullptr, shift != nullptr, relu, dt, s_nbr, s_epi);
#ifdef SESSD_TRACE
    if (KC == 27 && CIN == 64 && threadIdx.x == 0 && blockIdx.x < 4096) g_blocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime();
#endif
}

template <int CIN, int COUT, int D, int DW, int KC>
int launch(const GemmArgs& a, hipStream_t stream) {
    if ((size_t)a.max_voxels * split_row_bytes(CIN) >= kOutOfRange) return SESSD_E_UNSUPPORTED;
    const int num_cu = gemm_compute_units();
    const unsigned blocks = (unsigned)((a.max_voxels + 31) / 32);
    // below this many rows the 64-row tiles would leave compute units without one
    const int short_below = 40 * num_cu;
    hipLaunchKernelGGL((conv_split<CIN, COUT, D, DW, KC>), dim3(blocks), dim3(kWaves * 64), 0, stream, a.in_split,
                       static_cast<float*>(a.out_feat), a.out_split, a.w_split, a.nbr, a.num_out, a.max_voxels, a.scale,
                       a.shift, a.relu, a.write_pad_rows, short_below, a.dense);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

// FP32 rows [max_voxels][C] -> split rows, active rows only; a thread converts four consecutive channels
__global__ void __launch_bounds__(256)
split_rows_kernel(const float* __restrict__ in, void* __restrict__ out_split, const int32_t* __restrict__ num,
                  int max_voxels, int C) {
    int n = *num;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int vec_per_row = C / 4;
    const long long total = (long long)n * vec_per_row;
    for (long long v = (long long)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (long long)gridDim.x * blockDim.x) {
        const int row = (int)(v / vec_per_row), c4 = (int)(v % vec_per_row) * 4;
        const float4 x = *reinterpret_cast<const float4*>(in + (size_t)row * C + c4);
        const float o[4] = {x.x, x.y, x.z, x.w};
        store_split4(out_split, row, C, c4, o);
    }
}

#ifdef SESSD_TRACE
}  // namespace
}  // namespace sessd
extern "C" int sessd_debug_blocks(unsigned long long* out) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(sessd::g_blocks), sizeof(unsigned long long) * 2 * 4096);
}
extern "C" int sessd_debug_trace(unsigned long long* out) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(sessd::g_trace), sizeof(unsigned long long) * 8 * 4 * 40);
}
namespace sessd {
namespace {
#endif
// float -> BF16 bits, round to nearest even (finite inputs; NaN stays NaN)
uint16_t bf16_bits(float x) {
    uint32_t u;
    std::memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float bf16_value(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float x;
    std::memcpy(&x, &u, 4);
    return x;
}

}  // namespace

bool gemm_runs_split(int K, int cin, int cout, int in_type, int out_type) {
    if (in_type != SESSD_FLOAT || out_type != SESSD_FLOAT) return false;
    if (K != 27 && K != 3) return false;
    const int shapes[][2] = {{16, 16}, {16, 32}, {32, 32}, {32, 64}, {64, 64}};
    for (auto& s : shapes)
        if (s[0] == cin && s[1] == cout) return true;
    return false;
}

size_t split_weight_bytes(int K, int cin, int cout) {
    return (size_t)K * chunks(cin) * 3 * (cout / 16) * 64 * 16;
}

// Operand order: Ws[k][g][t][nb][lane][e] = part t of W[k][32g + 8*(lane/16) + e][16nb + lane%16] as BF16 bits,
// e = 0..7 (zero where the channel is beyond Cin)
void pack_weights_split(const float* w, int K, int cin, int cout, void* dst) {
    const int G = chunks(cin), NB = cout / 16;
    uint16_t* o = static_cast<uint16_t*>(dst);
    for (int k = 0; k < K; ++k)
        for (int g = 0; g < G; ++g)
            for (int t = 0; t < 3; ++t)
                for (int nb = 0; nb < NB; ++nb)
                    for (int lane = 0; lane < 64; ++lane)
                        for (int e = 0; e < 8; ++e) {
                            const int ch = 32 * g + 8 * (lane / 16) + e;
                            uint16_t bits = 0;
                            if (ch < cin) {
                                float r = w[((size_t)k * cin + ch) * cout + 16 * nb + lane % 16];
                                for (int p = 0; p <= t; ++p) {
                                    bits = bf16_bits(r);
                                    r -= bf16_value(bits);
                                }
                            }
                            *o++ = bits;
                        }
}

size_t split_feature_bytes(int max_voxels, int channels) { return (size_t)max_voxels * split_row_bytes(channels); }

int launch_split_rows(const float* in, void* out_split, const int32_t* num, int max_voxels, int channels,
                      hipStream_t stream) {
    if (!in || !out_split || !num || channels % 4) return fail(SESSD_E_INVALID, "split_rows: bad argument");
    const long long vecs = (long long)max_voxels * (channels / 4);
    const unsigned blocks = (unsigned)(vecs / 256 + 1 < 4096 ? vecs / 256 + 1 : 4096);
    hipLaunchKernelGGL(split_rows_kernel, dim3(blocks), dim3(256), 0, stream, in, out_split, num, max_voxels, channels);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

// FP32 layers whose shape the kernel covers, given their input rows in split form; SESSD_E_UNSUPPORTED otherwise
int launch_split(const GemmArgs& a, hipStream_t stream) {
    if (!a.w_split || !a.in_split || !gemm_runs_split(a.K, a.cin, a.cout, a.in_type, a.out_type)) return SESSD_E_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.in_feat) | reinterpret_cast<uintptr_t>(a.out_feat)) & 15) return SESSD_E_UNSUPPORTED;
    // <Cin, Cout, offsets the rows are requested ahead, weight register sets, K>
#define SESSD_SPLIT_CASE(CI, CO, D, DW)                                      \
    if (a.cin == CI && a.cout == CO)                                         \
    return a.K == 27 ? launch<CI, CO, D, DW, 27>(a, stream) : launch<CI, CO, D, DW, 3>(a, stream)
#ifndef SESSD_D64
#define SESSD_D64 2
#define SESSD_DW64 2
#endif
    SESSD_SPLIT_CASE(64, 64, SESSD_D64, SESSD_DW64);
    SESSD_SPLIT_CASE(32, 64, 3, 2);
    SESSD_SPLIT_CASE(32, 32, 3, 2);
    SESSD_SPLIT_CASE(16, 32, 3, 2);
    SESSD_SPLIT_CASE(16, 16, 3, 2);
#undef SESSD_SPLIT_CASE
    return SESSD_E_UNSUPPORTED;
}

}  // namespace sessd
