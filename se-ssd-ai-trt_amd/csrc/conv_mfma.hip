// conv_mfma.hip -- gather-GEMM on the matrix cores (gfx950 MFMA), FP32 features.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// One workgroup (4 wave64) owns a tile of output rows and all Cout columns.  The tile height is chosen
// per launch from the device-side row count so that every CU gets the same number of tiles
// (tile_height()).
//   * The tile's neighbour lists nbr[k][row0 .. row0+TM) are staged in LDS and compacted per offset
//     with wave64 ballot + popcount: pair list k = the (input row, local output row) pairs of the rows
//     that really have a neighbour at offset k.  Only those rows enter an MFMA block, so the matrix
//     cores do not multiply the zero rows a dense [TM x K*Cin] gather matrix would be half full of.
//   * Non-empty offsets are dealt round-robin to the four waves (split-K over offsets): tiles x 4 waves
//     is what fills 256 CUs with a ~17k-row problem.
//   * A wave gathers 16 pairs per MFMA block straight into A-operand registers: lane (i = lane%16,
//     q = lane/16) loads 16 bytes = channels 16g+4q .. 16g+4q+3 of pair i's input row, i.e. every row is
//     read as 64-byte segments.  The weights were reordered on the host so that the B operand of the same
//     four MFMA steps is one 16-byte load per lane; one pass over W[k] serves all blocks of the offset.
//     Next offset's rows and next chunk's weights are in flight while the current MFMAs issue.
//   * v_mfma_f32_16x16x4_f32 accumulates a block in FP32 registers (weights as the A operand, gathered
//     rows as B, so a lane ends up with four consecutive output channels of one pair); the block is then
//     added into the wave's private partial tile in LDS at the pairs' output rows with 16-byte
//     read-modify-writes (only this wave touches its partial and LDS keeps a wave's operations in order,
//     so the sum order is fixed; LDS float atomics measured several times slower).
//   * The four partial tiles are summed in a fixed order, scale/shift/ReLU is applied and each output
//     row is written once, coalesced.  No global atomics; results are bit-identical run to run.
#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

#ifndef SESSD_MFMA_WAVES
#define SESSD_MFMA_WAVES 4
#endif
#ifndef SESSD_MFMA_TM
#define SESSD_MFMA_TM 48
#endif
#ifndef SESSD_MFMA_TARGET
#define SESSD_MFMA_TARGET 40
#endif
constexpr int kWaves = SESSD_MFMA_WAVES;
constexpr int kTileRows = SESSD_MFMA_TM;      // capacity: most output rows a workgroup can own (<= 64)
constexpr int kTargetRows = SESSD_MFMA_TARGET;  // tile height aimed for when choosing tiles per CU
constexpr int kMaxBlk = (kTileRows + 15) / 16;  // MFMA row blocks an offset can need
constexpr int kMaxK = 27;

// Tile height for `n` active rows on `num_cu` compute units: the rows are split into num_cu * r tiles
// of equal height, r = the smallest tiles-per-CU count that keeps the height at or below the target.
// Every CU then gets the same number of tiles (a fixed 32-row tiling leaves e.g. 529 tiles for 256 CUs:
// some CUs run three tiles, most two, and the kernel lasts as long as the three).
static_assert(kTargetRows <= kTileRows && kTileRows <= 64, "tile height must fit the capacity and one wave");
__host__ __device__ inline int tile_height(int n, int num_cu) {
    if (n <= 0) return kTileRows;
    const int r = (n + num_cu * kTargetRows - 1) / (num_cu * kTargetRows);
    int h = (n + num_cu * r - 1) / (num_cu * r);
    return h > kTileRows ? kTileRows : (h < 1 ? 1 : h);
}

template <int CIN, int COUT>
__global__ void __launch_bounds__(kWaves * 64)
conv_mfma_f32(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ Wp,
              const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
              const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad,
              int num_cu) {
    constexpr int G = CIN / 16;    // 16-channel chunks of the inner dimension
    constexpr int NB = COUT / 16;  // 16-column blocks
    constexpr int LDP = COUT + 4;  // padded row stride of the partial tiles in LDS
    __shared__ int32_t s_in[kMaxK * kTileRows];   // compacted pair lists: input row ...
    __shared__ uint8_t s_row[kMaxK * kTileRows];  // ... and local output row of pair j of offset k
    __shared__ int32_t s_cnt[kMaxK + 5];          // pairs per offset
    __shared__ float s_part[kWaves * kTileRows * LDP];

    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int kVecPerRow = COUT / 4;

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
                *reinterpret_cast<float4*>(out + (size_t)row * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
            }
    }
    const int R = tile_height(n, num_cu);  // rows of this launch's tiles
    const int row0 = blockIdx.x * R;
    if (row0 >= n) return;
    const int rows = n - row0 < R ? n - row0 : R;

    // ---- stage + compact: a wave turns one offset's neighbour list into a pair list per step ----
    for (int k = wave; k < K; k += kWaves) {
        const int v = lane < rows ? nbr[(size_t)k * max_voxels + row0 + lane] : -1;
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

    const int i = lane & 15;  // pair inside a 16-pair block
    const int q = lane >> 4;  // 4-channel group inside a 16-channel chunk

    // offsets this wave handles: the non-empty ones, dealt round-robin (all wave-uniform)
    uint32_t my_mask = 0;
    {
        int live = 0;
        for (int k = 0; k < K; ++k)
            if (s_cnt[k] > 0) {
                if ((live % kWaves) == wave) my_mask |= 1u << k;
                ++live;
            }
    }

    const float4* wp4 = reinterpret_cast<const float4*>(Wp) + lane;
    // gathered rows of all blocks of offset k -> A-operand registers (zeros for the padding pairs)
    auto load_a = [&](int k, int cnt, float4 (&a)[kMaxBlk][G]) {
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk) {
            const int j = blk * 16 + i;
            const bool live = j < cnt;
            const int idx = live ? s_in[k * kTileRows + j] : 0;
            const float4* src = reinterpret_cast<const float4*>(in + (size_t)idx * CIN + q * 4);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#ifdef SESSD_EXP_NO_LOADS
                v.x = (float)idx;
#else
                if (live) v = src[g * 4];
#endif
                a[blk][g] = v;
            }
        }
    };
    auto load_b = [&](int k, int g, float4 (&b)[NB]) {
        const float4* wk = wp4 + ((size_t)k * G + g) * NB * 64;
#pragma unroll
#ifdef SESSD_EXP_NO_LOADS
        for (int nb = 0; nb < NB; ++nb) b[nb] = make_float4((float)(k + g), 1.f, 2.f, (float)nb);
#else
        for (int nb = 0; nb < NB; ++nb) b[nb] = wk[nb * 64];
#endif
    };

    int k_cur = my_mask ? __ffs(my_mask) - 1 : -1;
    my_mask &= my_mask - 1;
    // Pipeline: the gathered rows of the NEXT offset are loaded at the top of the current one; the
    // weight registers of chunk g are refilled with the next offset's chunk g as soon as the MFMAs that
    // read them have issued, so every weight load has a whole offset of MFMA work to hide behind
    // without a second register set.
    float4 a_cur[kMaxBlk][G], a_nxt[kMaxBlk][G], b[G][NB];
    int cnt_cur = 0, cnt_nxt = 0;
    if (k_cur >= 0) {
        cnt_cur = s_cnt[k_cur];
        load_a(k_cur, cnt_cur, a_cur);
#pragma unroll
        for (int g = 0; g < G; ++g) load_b(k_cur, g, b[g]);
    }
    while (k_cur >= 0) {
        const int k_nxt = my_mask ? __ffs(my_mask) - 1 : -1;
        my_mask &= my_mask - 1;
        if (k_nxt >= 0) {
            cnt_nxt = s_cnt[k_nxt];
            load_a(k_nxt, cnt_nxt, a_nxt);
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
                const float av[4] = {a_cur[blk][g].x, a_cur[blk][g].y, a_cur[blk][g].z, a_cur[blk][g].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const float bv[4] = {b[g][nb].x, b[g][nb].y, b[g][nb].z, b[g][nb].w};
                        acc[blk][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv[e], av[e], acc[blk][nb], 0, 0, 0);
                    }
            }
            if (k_nxt >= 0) load_b(k_nxt, g, b[g]);
        }
        // block results -> partial tile.  The weights are the MFMA's A operand and the gathered rows its
        // B operand, so D is the transposed block: lane (pair j = lane%16, q = lane/16) holds output
        // channels 16nb+4q .. +3 of pair j -- one 16-byte LDS read-modify-write per column block.
#pragma unroll
        for (int blk = 0; blk < kMaxBlk; ++blk) {
            if (blk * 16 >= cnt_cur) continue;
            const int j = blk * 16 + i;
            if (j < cnt_cur) {
                float* dst = part + (int)s_row[k_cur * kTileRows + j] * LDP + q * 4;
#ifndef SESSD_EXP_NO_ACCUM
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    float4 v = *reinterpret_cast<float4*>(dst + nb * 16);
                    v.x += acc[blk][nb][0];
                    v.y += acc[blk][nb][1];
                    v.z += acc[blk][nb][2];
                    v.w += acc[blk][nb][3];
                    *reinterpret_cast<float4*>(dst + nb * 16) = v;
                }
#else
                float t = 0.f;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) t += acc[blk][nb][0] + acc[blk][nb][1] + acc[blk][nb][2] + acc[blk][nb][3];
                if (t == 123.f) dst[0] = 1.f;
#endif
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

    // fixed-order sum of the four partials, epilogue, coalesced 16-byte stores
    for (int v = tid; v < rows * kVecPerRow; v += kWaves * 64) {
        const int r = v / kVecPerRow, c4 = (v % kVecPerRow) * 4;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float s = s_part[(0 * kTileRows + r) * LDP + c4 + e];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) s += s_part[(w * kTileRows + r) * LDP + c4 + e];
            if (scale) s = s * scale[c4 + e];
            if (shift) s = s + shift[c4 + e];
            if (relu) s = s > 0.f ? s : 0.f;
            o[e] = s;
        }
        *reinterpret_cast<float4*>(out + (size_t)(row0 + r) * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
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

template <int CIN, int COUT>
int launch_f32(const GemmArgs& a, hipStream_t stream) {
    const int num_cu = compute_units();
    // tile_height() never cuts n <= max_voxels rows into more than num_cu * r_max tiles
    const int r_max = ceil_div(a.max_voxels, (int64_t)num_cu * kTargetRows);
    const unsigned blocks = (unsigned)(num_cu * (r_max < 1 ? 1 : r_max));
    hipLaunchKernelGGL((conv_mfma_f32<CIN, COUT>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                       static_cast<const float*>(a.in_feat), static_cast<float*>(a.out_feat),
                       static_cast<const float*>(a.w_packed), a.nbr, a.num_out, a.max_voxels, a.K, a.scale,
                       a.shift, a.relu, a.write_pad_rows, num_cu);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

bool mfma_f32_shape(int K, int cin, int cout) {
    if (K > 27) return false;
    const int shapes[][2] = {{16, 16}, {16, 32}, {32, 32}, {32, 64}, {64, 64}, {64, 128}, {128, 128}};
    for (auto& s : shapes)
        if (s[0] == cin && s[1] == cout) return true;
    return false;
}

}  // namespace

size_t packed_weight_bytes(int K, int cin, int cout, int dtype) {
    if (dtype == SESSD_FLOAT && mfma_f32_shape(K, cin, cout)) return (size_t)K * cin * cout * sizeof(float);
    return 0;
}

// FP32 operand order: Wp[k][g][nb][lane][e] = W[k][16g + 4(lane/16) + e][16nb + lane%16]
void pack_weights(const float* w, int K, int cin, int cout, int dtype, void* dst) {
    if (dtype != SESSD_FLOAT) return;
    float* p = static_cast<float*>(dst);
    const int G = cin / 16, NB = cout / 16;
    for (int k = 0; k < K; ++k)
        for (int g = 0; g < G; ++g)
            for (int nb = 0; nb < NB; ++nb)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < 4; ++e)
                        p[((((size_t)k * G + g) * NB + nb) * 64 + lane) * 4 + e] =
                            w[((size_t)k * cin + 16 * g + 4 * (lane / 16) + e) * cout + 16 * nb + lane % 16];
}

// -> SESSD_OK when an MFMA kernel was launched, SESSD_E_UNSUPPORTED when the shape/dtype is not covered
int launch_mfma(const GemmArgs& a, hipStream_t stream) {
    if (a.in_type != SESSD_FLOAT || a.out_type != SESSD_FLOAT || !a.w_packed || !mfma_f32_shape(a.K, a.cin, a.cout))
        return SESSD_E_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.in_feat) | reinterpret_cast<uintptr_t>(a.out_feat)) & 15)
        return SESSD_E_UNSUPPORTED;
#define SESSD_CASE(CI, CO) \
    if (a.cin == CI && a.cout == CO) return launch_f32<CI, CO>(a, stream)
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
