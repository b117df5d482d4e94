// conv_wide.hip -- FP32 gather-GEMM for the layers with 64 output columns (Cin 32 or 64): one tall tile per compute
// unit, sixteen waves.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// conv_mfma.hip gives a workgroup of four waves a tile of at most 48 rows; a wave there holds the rows of all
// 16-pair blocks of two offsets and the whole W[k] in registers (247 of them in the 64 -> 64 layer), so a SIMD
// holds two waves, and with ~17 000 rows a compute unit runs two 33-row tiles whose per-offset pair lists fill
// 69 % of the 16-row MFMA blocks they occupy.  This kernel turns both knobs the other way:
//   * one tile per compute unit, up to 96 rows: at 66 rows the pair lists fill 81 % of their blocks;
//   * sixteen waves per tile: four groups share the tile's offsets (split-K), the four waves of a group take
//     a quarter of the output columns each (more groups would need more partial tiles than LDS holds).  A wave
//     works on ONE 16-pair block at a time -- the block's rows, its columns of W[k] and the next block's rows are
//     all it holds -- so it stays far below 128 registers and a SIMD holds four waves: while one waits for rows
//     or adds a block into its partial tile, the matrix core runs the others' blocks.
// Pair lists, operand order (the packed weights are conv_mfma.hip's), partial tiles in LDS (one per group and
// column quarter, private to a wave, so the sum order is fixed), fixed-order reduction, fused scale/shift/ReLU and
// the optional dense scatter are as in conv_mfma.hip; results are bit-identical run to run.
#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int v4u32 __attribute__((__vector_size__(16)));

constexpr int kWaves = 16;          // wave64s per workgroup: four per SIMD
constexpr int kTileRows = 96;       // tile capacity (rows): what the partial tiles leave of the 160 KB of LDS
constexpr int kMaxBlk = kTileRows / 16;
constexpr int kMaxK = kGemmMaxOffsets;
constexpr unsigned kOutOfRange = 0x80000000u;  // beyond any buffer the kernel is given (launch() checks)
constexpr int kRawBuffer = 0x00020000;         // descriptor word 3: raw 32-bit data format, no swizzle

__device__ __forceinline__ float4 buffer_load16(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {
    v4u32 v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, 0);
    return *reinterpret_cast<float4*>(&v);
}

__device__ __forceinline__ void mma16(const float4& w, const float4& x, v4f& acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, x.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, x.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, x.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, x.w, acc, 0, 0, 0);
}

// DENSE: the epilogue also scatters the rows into a dense tensor (the layer in front of sparse2Dense).  A variant of
// its own because the scatter's addresses cost ten registers, and what this kernel leaves of the register file is
// what the coordinate kernels of the frame's other branch run in beside it.
template <int CIN, int COUT, bool DENSE>
__global__ void __launch_bounds__(kWaves * 64)
conv_wide(const float* __restrict__ in, float* __restrict__ out, const void* __restrict__ Wp,
          const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
          const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad, int num_cu,
          const int32_t* __restrict__ tiles, DenseTarget dt) {
    constexpr int G = CIN / 16;     // 16-channel chunks of the inner dimension
    constexpr int NBT = COUT / 16;  // 16-column blocks of the layer
    constexpr int kCS = 4;               // waves of a group (column quarters)
    constexpr int kKG = kWaves / kCS;    // groups the offsets are dealt to
    constexpr int NB = NBT / kCS;   // column blocks of one wave
    constexpr int CW = COUT / kCS;  // columns of one wave
    constexpr int LDP = CW + 4;     // padded row stride of a partial tile
    static_assert(kTileRows <= 128 && kTileRows % 16 == 0, "the lists are staged in two halves of 64 rows");
    constexpr int kVecPerRow = COUT / 4;
    constexpr int kThreads = kWaves * 64;
    static_assert(CIN % 16 == 0 && NBT % kCS == 0, "channel counts must fill whole MFMA chunks per wave");
    static_assert(kThreads % kVecPerRow == 0, "a thread must keep its columns from row to row");
    __shared__ int32_t s_in[kMaxK * kTileRows];   // compacted pair lists: input row ...
    __shared__ uint8_t s_row[kMaxK * kTileRows];  // ... and local output row of pair j of offset k
    __shared__ int32_t s_cnt[kMaxK + 5];          // pairs per offset
    __shared__ float s_epi[2 * COUT];
    __shared__ float s_part[kWaves * kTileRows * LDP];

    int n = *num_out;
    const int cut_count = tiles ? tiles[0] : 0;
    const int cut_begin = tiles ? tiles[4 + blockIdx.x] : 0;
    const int cut_end = tiles ? tiles[5 + blockIdx.x] : 0;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (tells the compiler that it is wave-uniform)
    const int kgrp = wave / kCS;   // offsets are dealt to this group ...
    const int chalf = wave % kCS;  // ... and this wave computes this part of their columns
    float epi_scale = 1.f, epi_shift = 0.f;
    if (tid < COUT) {
        if (scale) epi_scale = scale[tid];
        if (shift) epi_shift = shift[tid];
    }
    const int ec4 = (tid % kVecPerRow) * 4;  // this thread's epilogue columns, the same for every row it stores

    // rows >= n: the reference zero-fills them (then BN+ReLU): epilogue(0), spread over all workgroups
    if (write_pad) {
        const int chunks = (max_voxels - n + kTileRows - 1) / kTileRows;
        for (int c = blockIdx.x; c < chunks; c += gridDim.x)
            for (int v = tid; v < kTileRows * kVecPerRow; v += kThreads) {
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
                *reinterpret_cast<float4*>(out + (size_t)row * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
            }
    }
    // The grid is one workgroup per compute unit (a workgroup takes most of a unit's LDS, so workgroups with no
    // tile would queue behind the busy ones just to return); workgroup b walks tiles b, b + grid, ...: runs of rows
    // from the rulebook's equal-work cuts, or runs of equal length.
    const TilePlan plan = tile_plan(n, num_cu, kTileRows);
    const int tile_count = cut_count > 0 ? cut_count : (n > 0 ? plan.count : 0);
    const int i = lane & 15;  // pair inside a 16-pair block
    const int q = lane >> 4;  // channel group inside a 16-channel chunk
    const __amdgpu_buffer_rsrc_t rs_in = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(in), 0, (int)((size_t)max_voxels * CIN * sizeof(float)), kRawBuffer);
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(Wp), 0, (int)((size_t)K * CIN * COUT * sizeof(float)), kRawBuffer);

    for (int tile = blockIdx.x; tile < tile_count; tile += gridDim.x) {
    int run_begin, run_end;
    if (cut_count > 0) {
        run_begin = tile == (int)blockIdx.x ? cut_begin : tiles[4 + tile];
        run_end = tile == (int)blockIdx.x ? cut_end : tiles[5 + tile];
    } else {
        run_begin = tile * plan.height;
        run_end = run_begin + plan.height < n ? run_begin + plan.height : n;
    }
    // a run longer than the tile capacity (sparse stretches under equal-work cuts) is walked in pieces
    for (int row0 = run_begin; row0 < run_end; row0 += kTileRows) {
    const int rows = run_end - row0 < kTileRows ? run_end - row0 : kTileRows;

    // ---- stage + compact: a wave turns an offset's neighbour list (two halves of 64 rows) into a pair list ----
    constexpr int kListsPerWave = (kMaxK + kWaves - 1) / kWaves;
    int staged[kListsPerWave][2];
#pragma unroll
    for (int s = 0; s < kListsPerWave; ++s) {
        const int k = wave + s * kWaves;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r = h * 64 + lane;
            staged[s][h] = (k < K && r < rows) ? nbr[(size_t)k * max_voxels + row0 + r] : -1;
        }
    }
    if (row0 == run_begin && tid < COUT) {
        s_epi[tid] = epi_scale;
        s_epi[COUT + tid] = epi_shift;
    }
    // zero this wave's partial tile (while the lists are on their way)
    float* part = s_part + wave * kTileRows * LDP;
    for (int t = lane; t < rows * LDP / 4; t += 64) reinterpret_cast<float4*>(part)[t] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int s = 0; s < kListsPerWave; ++s) {
        const int k = wave + s * kWaves;
        if (k >= K) break;
        int base = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int v = staged[s][h];
            const uint64_t m = __ballot(v >= 0);
            if (v >= 0) {
                const int j = base + __popcll(m & ((1ull << lane) - 1ull));
                s_in[k * kTileRows + j] = v;
                s_row[k * kTileRows + j] = (uint8_t)(h * 64 + lane);
            }
            base += __popcll(m);
        }
        if (lane == 0) s_cnt[k] = base;
    }
    __syncthreads();

    // offsets of this wave's group: ranked by their number of 16-pair blocks (ballots: lane k holds offset k)
    // and dealt in that order back and forth over the groups (0 1 2 3 3 2 1 0 ...)
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
        const int r2 = rank % (2 * kKG);
        const int w = r2 < kKG ? r2 : 2 * kKG - 1 - r2;
        my_mask = (uint32_t)__ballot(b > 0 && w == kgrp);
    }

    // Rows are requested with four neighbouring lanes on the 64 contiguous bytes of one row (lane l: pair l / 4 of
    // the block, bytes 16 * (l % 4) ..): the cache looks up one line per group of four lanes.  In the MFMA's
    // operand order -- lane l: pair l % 16, bytes 16 * (l / 16) .. -- the four lanes of a group name four
    // different rows and the same request takes four lookups: 18 instead of 48 bytes per cycle and compute unit,
    // measured.  The operand order is restored by a lane permutation (fetch()) before the MFMAs.
    // Padding lanes ask out of range (such a request returns zeros and touches no memory).
    auto row_at = [&](int k, int cnt, int blk) -> unsigned {
        const int j = blk * 16 + (lane >> 2);
        const bool live = j < cnt;
        const int idx = s_in[k * kTileRows + (live ? j : 0)];
        return live ? (unsigned)((idx * CIN + (lane & 3) * 4) * (int)sizeof(float)) : kOutOfRange;
    };
    const int from_lane4 = (4 * i + q) * 4;  // ds_bpermute address: this lane's operand sits in lane 4 * i + q
    auto fetch = [&](const float4& v) -> float4 {
        float4 r;
        r.x = __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane4, __float_as_int(v.x)));
        r.y = __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane4, __float_as_int(v.y)));
        r.z = __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane4, __float_as_int(v.z)));
        r.w = __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane4, __float_as_int(v.w)));
        return r;
    };
    auto load_a = [&](unsigned at, float4 (&a)[G]) {
#pragma unroll
        for (int g = 0; g < G; ++g) a[g] = buffer_load16(rs_in, at + g * 16 * (unsigned)sizeof(float));
    };
    // chunk g of this wave's columns of W[k] -> operand registers (k < 0: nothing to fetch)
    auto load_b = [&](int k, int g, float4 (&b)[NB]) {
        const unsigned at = k >= 0 ? (unsigned)(((((k * G + g) * NBT + chalf * NB) * 64) + lane) * 16) : kOutOfRange;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) b[nb] = buffer_load16(rs_w, at + nb * 64 * 16u);
    };

    int k_cur = my_mask ? __ffs(my_mask) - 1 : -1;
    my_mask &= my_mask - 1;
    float4 a0[G], a1[G], b[G][NB];
    int cnt_cur = 0;
    if (k_cur >= 0) {
        cnt_cur = __builtin_amdgcn_readfirstlane(s_cnt[k_cur]);
#pragma unroll
        for (int g = 0; g < G; ++g) load_b(k_cur, g, b[g]);
        load_a(row_at(k_cur, cnt_cur, 0), a0);
    }
    int k_nxt = -1, cnt_nxt = 0, nblk = 0, blk = 0;
    auto begin_offset = [&]() {
        k_nxt = my_mask ? __ffs(my_mask) - 1 : -1;
        my_mask &= my_mask - 1;
        cnt_nxt = k_nxt >= 0 ? __builtin_amdgcn_readfirstlane(s_cnt[k_nxt]) : 0;  // wave-uniform
        nblk = (cnt_cur + 15) >> 4;
        blk = 0;
    };
    auto item = [&](float4 (&a_use)[G], float4 (&a_fill)[G]) {
        const bool last = blk + 1 == nblk;  // wave-uniform
        // the next block's rows: of this offset, or the first block of the next one (cnt_nxt = 0: none)
        load_a(last ? row_at(k_nxt >= 0 ? k_nxt : 0, cnt_nxt, 0) : row_at(k_cur, cnt_cur, blk + 1), a_fill);
        v4f acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float4 x = fetch(a_use[g]);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) mma16(b[g][nb], x, acc[nb]);
            // behind the offset's last block the next offset's chunk g replaces this one
            if (last) load_b(k_nxt, g, b[g]);
        }
        const int j = blk * 16 + i;
        if (j < cnt_cur) {
            float* dst = part + (int)s_row[k_cur * kTileRows + j] * LDP + q * 4;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                float4 v = *reinterpret_cast<float4*>(dst + nb * 16);
                v.x += acc[nb][0];
                v.y += acc[nb][1];
                v.z += acc[nb][2];
                v.w += acc[nb][3];
                *reinterpret_cast<float4*>(dst + nb * 16) = v;
            }
        }
        if (last) {
            k_cur = k_nxt;
            cnt_cur = cnt_nxt;
            if (k_cur >= 0) begin_offset();
        } else {
            ++blk;
        }
    };
    if (k_cur >= 0) begin_offset();
    while (k_cur >= 0) {
        item(a0, a1);
        if (k_cur < 0) break;
        item(a1, a0);
    }
    __syncthreads();

    // fixed-order sum of the groups' partial tiles, epilogue, coalesced stores
    for (int v = tid; v < rows * kVecPerRow; v += kThreads) {
        const int r = v / kVecPerRow;
        const float* col = s_part + ((ec4 / CW) * kTileRows + r) * LDP + ec4 % CW;
        float4 acc4 = *reinterpret_cast<const float4*>(col);
#pragma unroll
        for (int w = 1; w < kKG; ++w) {
            const float4 p4 = *reinterpret_cast<const float4*>(col + w * kCS * kTileRows * LDP);
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
        *reinterpret_cast<float4*>(out + (size_t)(row0 + r) * COUT + ec4) = make_float4(o[0], o[1], o[2], o[3]);
        if (DENSE && dt.dense) {  // the sparse2Dense scatter of this row, fused (uniform branch)
            const int4 cc = reinterpret_cast<const int4*>(dt.coors)[row0 + r];  // (b,z,y,x)
            if (cc.x != 0 || cc.y < 0 || cc.y >= dt.D || cc.z < 0 || cc.z >= dt.H || cc.w < 0 || cc.w >= dt.W) {
                if (dt.status && ec4 == 0) atomicOr(dt.status, SESSD_STATUS_BAD_COORD);
            } else {
                float* d = static_cast<float*>(dt.dense) + ((size_t)cc.y * dt.Hp + cc.z + dt.pad_top) * dt.Wp + cc.w + dt.pad_left;
                const size_t plane = (size_t)dt.D * dt.Hp * dt.Wp;  // channel stride
#pragma unroll
                for (int e = 0; e < 4; ++e) d[(size_t)(ec4 + e) * plane] = o[e];
            }
        }
    }
    __syncthreads();  // the next piece reuses the lists and partial tiles
    }
    }
}

template <int CIN, int COUT>
int launch(const GemmArgs& a, hipStream_t stream) {
    // operands are addressed with 32-bit byte offsets, 2^31 means "out of range"
    if ((size_t)a.max_voxels * CIN * sizeof(float) >= kOutOfRange || (size_t)a.K * CIN * COUT * sizeof(float) >= kOutOfRange)
        return SESSD_E_UNSUPPORTED;
    const int num_cu = gemm_compute_units();
    const unsigned blocks = (unsigned)num_cu;
    if (a.dense.dense)
        hipLaunchKernelGGL((conv_wide<CIN, COUT, true>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                           static_cast<const float*>(a.in_feat), static_cast<float*>(a.out_feat), a.w_packed, a.nbr,
                           a.num_out, a.max_voxels, a.K, a.scale, a.shift, a.relu, a.write_pad_rows, num_cu, a.tiles,
                           a.dense);
    else
        hipLaunchKernelGGL((conv_wide<CIN, COUT, false>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                           static_cast<const float*>(a.in_feat), static_cast<float*>(a.out_feat), a.w_packed, a.nbr,
                           a.num_out, a.max_voxels, a.K, a.scale, a.shift, a.relu, a.write_pad_rows, num_cu, a.tiles,
                           a.dense);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace

bool gemm_runs_wide(int K, int cin, int cout, int in_type, int out_type) {
    if (in_type != SESSD_FLOAT || out_type != SESSD_FLOAT || K > kMaxK) return false;
    return cout == 64 && (cin == 64 || cin == 32);
}

int gemm_wide_tile_rows() { return kTileRows; }

int launch_wide(const GemmArgs& a, hipStream_t stream) {
    if (!a.w_packed || !gemm_runs_wide(a.K, a.cin, a.cout, a.in_type, a.out_type)) return SESSD_E_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.in_feat) | reinterpret_cast<uintptr_t>(a.out_feat)) & 15) return SESSD_E_UNSUPPORTED;
    if (a.cin == 64 && a.cout == 64) return launch<64, 64>(a, stream);
    if (a.cin == 32 && a.cout == 64) return launch<32, 64>(a, stream);
    return SESSD_E_UNSUPPORTED;
}

}  // namespace sessd
