// conv_mfma.hip -- gather-GEMM on the matrix cores (gfx950 MFMA), FP32 features.
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )
//
// One workgroup (4 wave64) owns a tile of 16 output rows (one MFMA row block) and all Cout columns.
//   * The tile's neighbour lists nbr[k][row0..row0+15] for all K offsets are staged in LDS once.
//   * Offsets for which the tile has no neighbour at all are skipped (wave64 ballot over the staged
//     list); the remaining ones are dealt round-robin to the four waves (split-K over offsets), so a
//     small frame still fills the chip: tiles x 4 waves.
//   * A wave gathers the input rows of an offset straight into MFMA A-operand registers: lane
//     (i = lane%16, q = lane/16) loads 16 bytes = channels 16g+4q .. 16g+4q+3 of row i, i.e. every
//     row is read as 64-byte segments.  The weights were reordered on the host so that the B operand
//     of the same four MFMA steps is one 16-byte load per lane as well.
//   * v_mfma_f32_16x16x4_f32 accumulates in FP32.  The tile height trades weight re-reads (one pass
//     over W[k] per tile and offset) against load balance: at ~17k active rows a 16-row tile gives
//     ~1000 workgroups for 256 CUs and measured fastest.
//   * The four partial tiles are summed through LDS in a fixed order (deterministic), the
//     scale/shift/ReLU epilogue is applied and each output row is written once, coalesced.
#include "kernels.h"

namespace sessd {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

#ifndef SESSD_MFMA_WAVES
#define SESSD_MFMA_WAVES 4
#endif
#ifndef SESSD_MFMA_RB
#define SESSD_MFMA_RB 1
#endif
constexpr int kWaves = SESSD_MFMA_WAVES;
constexpr int kRB = SESSD_MFMA_RB;   // 16-row MFMA blocks per wave
constexpr int kTileRows = kRB * 16;

template <int CIN, int COUT>
__global__ void __launch_bounds__(kWaves * 64)
conv_mfma_f32(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ Wp,
              const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
              const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad) {
    constexpr int G = CIN / 16;    // 16-channel chunks of the inner dimension
    constexpr int NB = COUT / 16;  // 16-column blocks
    constexpr int LDP = COUT + 4;  // padded row stride of the partial tiles in LDS
    __shared__ int32_t s_nbr[27 * kTileRows];
    __shared__ float s_part[kWaves * kTileRows * LDP];

    const int row0 = blockIdx.x * kTileRows;
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    if (row0 >= n && !write_pad) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    for (int t = tid; t < K * kTileRows; t += kWaves * 64) {
        const int k = t / kTileRows, r = t % kTileRows;
        const int row = row0 + r;
        s_nbr[t] = row < n ? nbr[(size_t)k * max_voxels + row] : -1;
    }
    __syncthreads();

    v4f acc[kRB][NB];
#pragma unroll
    for (int rb = 0; rb < kRB; ++rb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[rb][nb] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int i = lane & 15;  // row inside a 16-row block
    const int q = lane >> 4;  // 4-channel group inside a 16-channel chunk

    // offsets this wave handles: the non-empty ones of the tile, dealt round-robin to the four waves;
    // bit k of rb_mask[rb] = "16-row block rb has a neighbour at offset k" (all wave-uniform)
    uint32_t my_mask = 0, rb_mask[kRB];
#pragma unroll
    for (int rb = 0; rb < kRB; ++rb) rb_mask[rb] = 0;
    {
        int live = 0;
        for (int k = 0; k < K; ++k) {
            bool any = false;
#pragma unroll
            for (int rb = 0; rb < kRB; ++rb) {
                const bool any_rb = __ballot(s_nbr[k * kTileRows + rb * 16 + i] >= 0) != 0ull;
                if (any_rb) rb_mask[rb] |= 1u << k;
                any = any || any_rb;
            }
            if (any) {
                if ((live % kWaves) == wave) my_mask |= 1u << k;
                ++live;
            }
        }
    }

    // Software pipeline: the gathered rows of the NEXT offset and the weights of the NEXT 16-channel
    // chunk are in flight while the MFMAs of the current chunk issue.
    const float4* wp4 = reinterpret_cast<const float4*>(Wp) + lane;
    auto load_a = [&](int k, float4 (&a)[kRB][G]) {
#pragma unroll
        for (int rb = 0; rb < kRB; ++rb) {
            const int idx = s_nbr[k * kTileRows + rb * 16 + i];
            const float4* src = reinterpret_cast<const float4*>(in + (size_t)(idx < 0 ? 0 : idx) * CIN + q * 4);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx >= 0) v = src[g * 4];
                a[rb][g] = v;
            }
        }
    };
    auto load_b = [&](int k, int g, float4 (&b)[NB]) {
        const float4* wk = wp4 + ((size_t)k * G + g) * NB * 64;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) b[nb] = wk[nb * 64];
    };

    int k_cur = my_mask ? __ffs(my_mask) - 1 : -1;
    my_mask &= my_mask - 1;
    float4 a_cur[kRB][G], a_nxt[kRB][G], b_cur[NB], b_nxt[NB];
    if (k_cur >= 0) {
        load_a(k_cur, a_cur);
        load_b(k_cur, 0, b_cur);
    }
    while (k_cur >= 0) {
        const int k_nxt = my_mask ? __ffs(my_mask) - 1 : -1;
        my_mask &= my_mask - 1;
        if (k_nxt >= 0) load_a(k_nxt, a_nxt);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (g + 1 < G) load_b(k_cur, g + 1, b_nxt);
            else if (k_nxt >= 0) load_b(k_nxt, 0, b_nxt);
#pragma unroll
            for (int rb = 0; rb < kRB; ++rb) {
                if (!((rb_mask[rb] >> k_cur) & 1u)) continue;  // wave-uniform: block has no neighbour here
                const float av[4] = {a_cur[rb][g].x, a_cur[rb][g].y, a_cur[rb][g].z, a_cur[rb][g].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const float bv[4] = {b_cur[nb].x, b_cur[nb].y, b_cur[nb].z, b_cur[nb].w};
                        acc[rb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[e], bv[e], acc[rb][nb], 0, 0, 0);
                    }
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) b_cur[nb] = b_nxt[nb];
        }
#pragma unroll
        for (int rb = 0; rb < kRB; ++rb)
#pragma unroll
            for (int g = 0; g < G; ++g) a_cur[rb][g] = a_nxt[rb][g];
        k_cur = k_nxt;
    }

    // partial tile of this wave -> LDS.  D layout of the 16x16 MFMA: lane holds column lane%16 of rows
    // 4*(lane/16) .. +3.
    float* part = s_part + wave * kTileRows * LDP;
#pragma unroll
    for (int rb = 0; rb < kRB; ++rb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                part[(rb * 16 + q * 4 + r) * LDP + nb * 16 + i] = acc[rb][nb][r];
    __syncthreads();

    // fixed-order sum of the four partials, epilogue, coalesced 16-byte stores
    constexpr int kVecPerRow = COUT / 4;
    for (int v = tid; v < kTileRows * kVecPerRow; v += kWaves * 64) {
        const int r = v / kVecPerRow, c4 = (v % kVecPerRow) * 4;
        const int row = row0 + r;
        if (row >= max_voxels || (row >= n && !write_pad)) continue;
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
        *reinterpret_cast<float4*>(out + (size_t)row * COUT + c4) = make_float4(o[0], o[1], o[2], o[3]);
    }
}

template <int CIN, int COUT>
int launch_f32(const GemmArgs& a, hipStream_t stream) {
    const unsigned blocks = (unsigned)ceil_div(a.max_voxels, kTileRows);
    hipLaunchKernelGGL((conv_mfma_f32<CIN, COUT>), dim3(blocks), dim3(kWaves * 64), 0, stream,
                       static_cast<const float*>(a.in_feat), static_cast<float*>(a.out_feat),
                       static_cast<const float*>(a.w_packed), a.nbr, a.num_out, a.max_voxels, a.K, a.scale,
                       a.shift, a.relu, a.write_pad_rows);
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
