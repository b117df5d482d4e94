// conv_tall.hip -- gather-GEMM for FP16 features with many active rows: tall tiles, weights through LDS.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// The split-K kernel of conv_mfma.hip requests all of W once per 48..64-row tile; in FP16, where the matrix cores
// are far from busy, those requests (and, at 128 columns, every row gathered twice) are what the compute units'
// load path spends its time on.  Here a workgroup (4 wave64) owns 64 or 128 consecutive output rows:
//   * W[k] is copied once per workgroup and offset into LDS (two buffers; the host's MFMA operand order is also
//     the LDS order): every wave requests its share a few offsets ahead into registers and stores it one offset
//     before its use;
//   * a wave owns 16 or 32 of the rows and ALL columns, and keeps their accumulators in registers over all K
//     offsets: no compaction, no partial tiles.  A row without a neighbour at offset k contributes a zero operand
//     (a buffer load that points out of range: zeros, no memory touched), so the matrix cores multiply about twice
//     the useful pairs -- in FP16 they have the headroom;
//   * every gathered row is requested once, D offsets ahead, by the wave that uses it;
//   * all requests of the offset loop are unconditional and in a fixed order, so the compiler's waits cover exactly
//     the operands about to be used; one barrier per offset publishes the next offset's weights and frees the buffer
//     they overwrite.
// (Copying the weights with direct-to-LDS loads needs no registers, but a wait for "all but the N youngest
// requests" did not reliably cover such a copy when ordinary loads were in flight behind it -- stale weights in a
// few tiles per thousand launches -- and waiting for everything gives up the prefetch.)
// Summation order per output element: offsets ascending, channels inside the MFMA: fixed, run-to-run identical.
#include <type_traits>

#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned int v4u32 __attribute__((__vector_size__(16)));

constexpr int kWaves = 4;
constexpr int kGroupsAhead = 3;  // groups of weight fragments a wave has requested from LDS ahead of the one it multiplies
constexpr int kMaxK = kGemmMaxOffsets;
constexpr unsigned kOutOfRange = 0x80000000u;
constexpr int kRawBuffer = 0x00020000;

__device__ __forceinline__ void store4h(__half* dst, const float (&o)[4]) {
    union {
        __half2 h[2];
        uint2 u;
    } p;
    p.h[0] = __floats2half2_rn(o[0], o[1]);
    p.h[1] = __floats2half2_rn(o[2], o[3]);
    *reinterpret_cast<uint2*>(dst) = p.u;
}

// The barrier of the offset loop.  __syncthreads() would add workgroup-scope fences, for which the compiler drains
// every request in flight -- the rows and weights just requested for later offsets included.  What the loop needs
// published are this wave's LDS stores (waited for explicitly); the compiler must only keep its LDS accesses on
// their side of the barrier.
__device__ __forceinline__ void ring_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): vmcnt and expcnt fields at their maximum = no wait
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One of the two weight buffers in LDS
template <int U, int slot>
__device__ __forceinline__ float4* weight_slot() {
    __shared__ float4 s_w[U * 64];
    return s_w;
}

// The tile of one workgroup.  RB = 16-row blocks per wave, D = offsets the rows are requested ahead, DW = register
// sets for weights in flight.
template <int CIN, int COUT, int RB, int D, int DW, int KC>
__device__ __forceinline__ void tall_tile(const __half* __restrict__ in, __half* __restrict__ out,
                                          const void* __restrict__ Wp, const int32_t* __restrict__ nbr, int n,
                                          int row0, int max_voxels, bool has_scale, bool has_shift, int relu,
                                          DenseTarget dt, int32_t* s_nbr, const float* s_epi) {
    constexpr int G = CIN / 32;        // K-chunks (32 channels) of the inner dimension
    constexpr int NBT = COUT / 16;     // 16-column blocks
    constexpr int U = G * NBT;         // 1 KB units (64 lanes x 16 bytes) of one offset's weights
    constexpr int NBUF = D + 1;        // row register sets
    constexpr int TR = kWaves * RB * 16;
    constexpr int UW = (U + kWaves - 1) / kWaves;  // weight units a wave copies per offset
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (row0 >= n) return;

    // the tile's neighbour lists (rows beyond n: none) -> LDS
    for (int e = tid; e < KC * TR; e += kWaves * 64) {
        const int k = e / TR, r = e - k * TR;
        s_nbr[e] = row0 + r < n ? nbr[(size_t)k * max_voxels + row0 + r] : -1;
    }
    __syncthreads();

    const int i = lane & 15;  // row inside a 16-row block
    const int q = lane >> 4;  // 8-channel group inside a K-chunk
    const __amdgpu_buffer_rsrc_t rs_in = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<__half*>(in), 0, (int)((size_t)max_voxels * CIN * sizeof(__half)), kRawBuffer);
    const float4* wsrc = reinterpret_cast<const float4*>(Wp) + lane;

    float4 a[NBUF][RB][G];
    v4f wreg[DW][UW];  // (a native vector type: as an array of structs these registers ended up on the stack)
    v4f acc[RB][NBT];
#pragma unroll
    for (int blk = 0; blk < RB; ++blk)
#pragma unroll
        for (int nb = 0; nb < NBT; ++nb) acc[blk][nb] = (v4f){0.f, 0.f, 0.f, 0.f};

    // The offset loop runs in periods of P offsets (P = a common multiple of the row register sets, the two weight
    // buffers and the weight register sets), the period unrolled, so that every register set and buffer has a
    // compile-time name: s = position inside the period, k = k0 + s the offset.
    constexpr int P = NBUF % 2 == 0 ? NBUF : 2 * NBUF;
    static_assert(P % NBUF == 0 && P % 2 == 0 && P % DW == 0, "period");
    // unit j of this wave's share of W[k] -> registers (beyond the last offset: the last one again, never used)
    auto load_w1 = [&](int k, auto s_c, int j) {
        constexpr int set = decltype(s_c)::value % DW;
        const int kw = k < KC ? k : KC - 1;
        // (fewer units than waves: some are copied twice, same bytes to the same place)
        const int u = U % kWaves == 0 ? wave + j * kWaves : (wave + j * kWaves) % U;
        wreg[set][j] = *reinterpret_cast<const v4f*>(wsrc + ((size_t)kw * U + u) * 64);
    };
    // ... -> LDS (beyond the last offset: into the buffer nobody reads any more)
    auto store_w1 = [&](auto s_c, int j) {
        constexpr int s = decltype(s_c)::value;
        const int u = U % kWaves == 0 ? wave + j * kWaves : (wave + j * kWaves) % U;
        *reinterpret_cast<v4f*>(weight_slot<U, s % 2>() + u * 64 + lane) = wreg[s % DW][j];
    };
    // block blk of this wave's rows of offset k -> registers (beyond the last offset: requests that fetch nothing)
    auto load_rows1 = [&](int k, auto s_c, int blk) {
        constexpr int set = decltype(s_c)::value % NBUF;
        const int kr = k < KC ? k : KC - 1;
        int idx = s_nbr[kr * TR + (wave * RB + blk) * 16 + i];
        idx = k < KC ? idx : -1;
        const unsigned at = idx >= 0 ? (unsigned)((idx * CIN + q * 8) * (int)sizeof(__half)) : kOutOfRange;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            v4u32 v = __builtin_amdgcn_raw_buffer_load_b128(rs_in, at + g * 64u, 0, 0);
            a[set][blk][g] = *reinterpret_cast<float4*>(&v);
        }
    };
    // Offset k at position s of the period.  Its weight fragments (one per K-chunk and column block, 16 bytes per
    // lane) come from LDS in groups of BG, requested kGroupsAhead groups before they multiply.  The offset's other
    // work -- the rows of offset k+D requested, W[k+1] stored to its buffer, W[k+1+DW] requested -- is dealt over
    // the groups, so that those instructions issue while the matrix cores work on the group before (issued in one
    // piece ahead of the first MFMA they took as long as the MFMAs themselves).
    auto offset_step = [&](int k, auto s_c) {
        constexpr int s = decltype(s_c)::value;
        const v4f* const s_w = reinterpret_cast<const v4f*>(weight_slot<U, s % 2>()) + lane;
        constexpr int BG = U < 4 ? U : 4;
        constexpr int NG = U / BG;
        static_assert(U % BG == 0, "whole groups");
        constexpr int NI = RB + UW;                  // side items: RB row blocks, then UW weight units
        constexpr int IPG = (NI + NG - 1) / NG;      // ... per group
        constexpr int PD = NG >= 3 ? kGroupsAhead : 1;  // groups requested ahead
        v4f b[PD + 1][BG];
#pragma unroll
        for (int g0 = 0; g0 < PD; ++g0)
#pragma unroll
            for (int j = 0; j < BG; ++j) b[g0][j] = s_w[(g0 * BG + j) * 64];
#pragma unroll
        for (int grp = 0; grp < NG; ++grp) {
            if (grp + PD < NG) {
#pragma unroll
                for (int j = 0; j < BG; ++j) b[(grp + PD) % (PD + 1)][j] = s_w[((grp + PD) * BG + j) * 64];
            }
#pragma unroll
            for (int it = grp * IPG; it < (grp + 1) * IPG && it < NI; ++it) {
                if (it < RB) {
                    load_rows1(k + D, std::integral_constant<int, s + D>{}, it);
                } else {
                    store_w1(std::integral_constant<int, s + 1>{}, it - RB);
                    load_w1(k + 1 + DW, std::integral_constant<int, s + 1 + DW>{}, it - RB);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < BG; ++j) {
                const int f = grp * BG + j, g = f / NBT, nb = f % NBT;
#pragma unroll
                for (int blk = 0; blk < RB; ++blk)
                    acc[blk][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const v8h*>(&b[grp % (PD + 1)][j]),
                                                                         *reinterpret_cast<const v8h*>(&a[s % NBUF][blk][g]),
                                                                         acc[blk][nb], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // prologue: W[0] into its buffer, W[1 .. DW] and the rows of offsets 0 .. D-1 requested
#pragma unroll
    for (int j = 0; j < UW; ++j) load_w1(0, std::integral_constant<int, 0>{}, j);
#pragma unroll
    for (int j = 0; j < UW; ++j) store_w1(std::integral_constant<int, 0>{}, j);
    auto ahead = [&](auto self, auto k_c) -> void {
        constexpr int k = decltype(k_c)::value;
        if constexpr (k <= DW) {
#pragma unroll
            for (int j = 0; j < UW; ++j) load_w1(k, k_c, j);
            self(self, std::integral_constant<int, k + 1>{});
        }
    };
    ahead(ahead, std::integral_constant<int, 1>{});
    auto rows_ahead = [&](auto self, auto k_c) -> void {
        constexpr int k = decltype(k_c)::value;
        if constexpr (k < D) {
#pragma unroll
            for (int blk = 0; blk < RB; ++blk) load_rows1(k, k_c, blk);
            self(self, std::integral_constant<int, k + 1>{});
        }
    };
    rows_ahead(rows_ahead, std::integral_constant<int, 0>{});

    // positions s .. `last` - 1 of the period that starts at offset k0
    auto steps = [&](auto self, int k0, auto s_c, auto last_c) -> void {
        constexpr int s = decltype(s_c)::value;
        if constexpr (s < decltype(last_c)::value) {
            // behind this barrier W[k] is in its buffer (every wave stored its share during the previous offset)
            // and every wave is done with offset k-1, whose buffer W[k+1] now overwrites
            ring_barrier();
            offset_step(k0 + s, s_c);
            self(self, k0, std::integral_constant<int, s + 1>{}, last_c);
        }
    };
    int k0 = 0;
    for (; k0 + P <= KC; k0 += P) steps(steps, k0, std::integral_constant<int, 0>{}, std::integral_constant<int, P>{});
    steps(steps, k0, std::integral_constant<int, 0>{}, std::integral_constant<int, KC % P>{});

    // epilogue: lane (i, q) holds output channels 16nb+4q .. +3 of row i of each of its blocks
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) {
        const int row = row0 + (wave * RB + blk) * 16 + i;
        if (row >= n) continue;
        bool to_dense = false;
        __half* d = nullptr;
        size_t plane = 0;
        if (dt.dense) {  // the sparse2Dense scatter of this row, fused (uniform branch)
            const int4 cc = reinterpret_cast<const int4*>(dt.coors)[row];  // (b,z,y,x)
            if (cc.x != 0 || cc.y < 0 || cc.y >= dt.D || cc.z < 0 || cc.z >= dt.H || cc.w < 0 || cc.w >= dt.W) {
                if (dt.status && q == 0) atomicOr(dt.status, SESSD_STATUS_BAD_COORD);
            } else {
                to_dense = true;
                d = static_cast<__half*>(dt.dense) + ((size_t)cc.y * dt.Hp + cc.z + dt.pad_top) * dt.Wp + cc.w + dt.pad_left;
                plane = (size_t)dt.D * dt.Hp * dt.Wp;
            }
        }
#pragma unroll
        for (int nb = 0; nb < NBT; ++nb) {
            const int c4 = nb * 16 + q * 4;
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float s = acc[blk][nb][e];
                if (has_scale) s = s * s_epi[c4 + e];
                if (has_shift) s = s + s_epi[COUT + c4 + e];
                if (relu) s = s > 0.f ? s : 0.f;
                o[e] = s;
            }
            store4h(out + (size_t)row * COUT + c4, o);
            if (to_dense) {
#pragma unroll
                for (int e = 0; e < 4; ++e) d[(size_t)(c4 + e) * plane] = __float2half_rn(o[e]);
            }
        }
    }
}

// RB = 16-row blocks a wave owns in a tall tile (one in a short tile: the heights are chosen on the device from
// the row count), D = offsets the rows are requested ahead, DW = register sets for weights in flight
template <int CIN, int COUT, int RB, int D, int DW, int KC>
__global__ void __launch_bounds__(kWaves * 64, 2)
conv_tall(const __half* __restrict__ in, __half* __restrict__ out, const void* __restrict__ Wp,
          const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels,
          const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad,
          int slots, DenseTarget dt) {
    static_assert(CIN % 32 == 0 && COUT % 16 == 0, "whole MFMA chunks");
    __shared__ int32_t s_nbr[KC * kWaves * RB * 16];
    __shared__ float s_epi[2 * COUT];
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int tid = threadIdx.x;
    constexpr int kVecPerRow = COUT / 4;

    // rows >= n: epilogue(0), as the reference's zero fill followed by BN + ReLU
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
                store4h(out + (size_t)row * COUT + c4, o);
            }
    }
    if (tid < COUT) {  // (published by the barrier behind the list staging)
        s_epi[tid] = scale ? scale[tid] : 1.f;
        s_epi[COUT + tid] = shift ? shift[tid] : 0.f;
    }
    // Tile heights.  `slots` workgroups are resident at a time.  Up to 64 * slots rows every
    // tile is 64 rows (one block per wave); beyond that just enough tiles at the head of the grid take RB blocks
    // per wave for the launch to stay one round of resident workgroups -- a second, mostly empty round costs a
    // whole tile's time; beyond 64 * RB * slots rows every tile is tall.
    constexpr int kShort = kWaves * 16, kTall = kShort * RB;
    int n_tall = 0;
    if (RB > 1 && n > kShort * slots) {
        n_tall = (n - kShort * slots + (kTall - kShort) - 1) / (kTall - kShort);
        if (n_tall > slots) n_tall = (n + kTall - 1) / kTall;
    }
    const int b = blockIdx.x;
    if (b < n_tall)
        tall_tile<CIN, COUT, RB, D, DW, KC>(in, out, Wp, nbr, n, b * kTall, max_voxels, scale != nullptr, shift != nullptr, relu, dt, s_nbr, s_epi);
    else
        tall_tile<CIN, COUT, 1, D, DW, KC>(in, out, Wp, nbr, n, n_tall * kTall + (b - n_tall) * kShort, max_voxels, scale != nullptr, shift != nullptr, relu, dt, s_nbr, s_epi);
}

template <int CIN, int COUT, int RB, int D, int DW, int KC>
int launch(const GemmArgs& a, hipStream_t stream) {
    if ((size_t)a.max_voxels * CIN * sizeof(__half) >= kOutOfRange) return SESSD_E_UNSUPPORTED;
    const int num_cu = gemm_compute_units();
    const unsigned blocks = (unsigned)((a.max_voxels + 63) / 64);
    // workgroups of this instantiation a compute unit holds at a time (registers and LDS decide; asked once)
    static int per_cu = 0;
    if (per_cu == 0) {
        int v = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, conv_tall<CIN, COUT, RB, D, DW, KC>, kWaves * 64, 0) != hipSuccess || v < 1)
            v = 2;
        per_cu = v;
    }
    hipLaunchKernelGGL((conv_tall<CIN, COUT, RB, D, DW, KC>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                       static_cast<const __half*>(a.in_feat), static_cast<__half*>(a.out_feat), a.w_packed, a.nbr,
                       a.num_out, a.max_voxels, a.scale, a.shift, a.relu, a.write_pad_rows,
                       per_cu * num_cu, a.dense);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace

bool gemm_runs_tall(int K, int cin, int cout, int in_type, int out_type) {
    if (in_type != SESSD_HALF || out_type != SESSD_HALF) return false;
    if (K == 3) return cin == cout && (cin == 64 || cin == 128);  // the (3,1,1) layer that ends the backbone
    if (K != 27) return false;
    return (cin == 128 && cout == 128) || (cin == 64 && (cout == 128 || cout == 64)) || (cin == 32 && (cout == 64 || cout == 32));
}

// FP16 layers with 3x3x3 (or the reference's last 3x1x1) kernels whose inner dimension fills whole 32-channel chunks;
// SESSD_E_UNSUPPORTED otherwise
int launch_tall(const GemmArgs& a, hipStream_t stream) {
    if (!a.w_packed || !gemm_runs_tall(a.K, a.cin, a.cout, a.in_type, a.out_type)) return SESSD_E_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.in_feat) | reinterpret_cast<uintptr_t>(a.out_feat)) & 15) return SESSD_E_UNSUPPORTED;
    // <Cin, Cout, row blocks per wave in tall tiles, offsets the rows are requested ahead, weight register sets, K>
    if (a.K == 3) {
        if (a.cin == 128) return launch<128, 128, 2, 1, 1, 3>(a, stream);
        return launch<64, 64, 2, 2, 2, 3>(a, stream);
    }
    if (a.cin == 128 && a.cout == 128) return launch<128, 128, 2, 1, 1, 27>(a, stream);
    if (a.cin == 64 && a.cout == 128) return launch<64, 128, 2, 2, 1, 27>(a, stream);
    if (a.cin == 64 && a.cout == 64) return launch<64, 64, 2, 3, 2, 27>(a, stream);
    if (a.cin == 32 && a.cout == 64) return launch<32, 64, 2, 3, 2, 27>(a, stream);
    if (a.cin == 32 && a.cout == 32) return launch<32, 32, 2, 3, 2, 27>(a, stream);
    return SESSD_E_UNSUPPORTED;
}

}  // namespace sessd
