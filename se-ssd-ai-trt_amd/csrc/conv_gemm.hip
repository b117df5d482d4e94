// conv_gemm.hip -- the gather-GEMM stage of SubmConv3d / SparseConv3d and the rulebook export.
//
// Replaces sparseGatherConvScatter (submConv3dlayer.cu:479-518 == sparseConv3dlayer.cu:557-589),
// which the reference launches once per kernel offset with one thread per rulebook pair, a scalar
// Cin x Cout mat-vec per thread and Cout float atomicAdds per pair.
//
// Here the rulebook is a gather table nbr[k][o] (for a fixed output row o and offset k there is
// at most one input row), so the layer is output-stationary:
//
//     out[o][:] = epilogue( sum_k  in[nbr[k][o]][:] @ W[k] )          k ascending
//
// Every output row is written exactly once, without atomics, and the result is deterministic.
#include "kernels.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }

__device__ __forceinline__ float apply_epilogue(float acc, int c, const float* scale, const float* shift, int relu) {
    if (scale) acc = acc * scale[c];
    if (shift) acc = acc + shift[c];
    if (relu) acc = acc > 0.f ? acc : 0.f;
    return acc;
}

// Shape-agnostic VALU path: one thread per output element.  The threads of one row read the same
// input values (broadcast) and consecutive weight columns (coalesced).  Used for channel counts the
// MFMA kernels do not cover and as their cross-check.
template <typename Tin, typename Tw, typename Tout>
__global__ void __launch_bounds__(kBlock)
conv_valu_generic(const Tin* __restrict__ in, Tout* __restrict__ out, const Tw* __restrict__ W,
                  const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels,
                  int K, int cin, int cout, const float* __restrict__ scale,
                  const float* __restrict__ shift, int relu, int write_pad) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int row = (int)(e / cout);
    const int c = (int)(e - (int64_t)row * cout);
    if (row >= max_voxels) return;
    int n = *num_out;
    n = n > max_voxels ? max_voxels : n;
    if (row >= n) {
        if (write_pad) out[e] = from_f32<Tout>(apply_epilogue(0.f, c, scale, shift, relu));
        return;
    }
    float acc = 0.f;
    for (int k = 0; k < K; ++k) {
        const int idx = nbr[(size_t)k * max_voxels + row];
        if (idx < 0) continue;
        const Tin* x = in + (size_t)idx * cin;
        const Tw* w = W + (size_t)k * cin * cout + c;
        float s = 0.f;
        for (int j = 0; j < cin; ++j) s = fmaf(to_f32(x[j]), to_f32(w[(size_t)j * cout]), s);
        acc += s;
    }
    out[e] = from_f32<Tout>(apply_epilogue(acc, c, scale, shift, relu));
}

// First layer of the backbone (voxel means, Cin = 4): the inner dimension is too thin for MFMA tiles
// (4 per offset).  One thread owns four output channels of one row; the whole weight tensor
// (K*4*Cout floats, < 14 KB) sits in LDS, a gathered input row is one 16-byte load shared by the
// row's threads.
template <typename Tw, typename Tout, int COUT>
__global__ void __launch_bounds__(kBlock)
conv_valu_cin4(const float* __restrict__ in, Tout* __restrict__ out, const Tw* __restrict__ W,
               const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
               const float* __restrict__ scale, const float* __restrict__ shift, int relu, int write_pad) {
    constexpr int TPR = COUT / 4;         // threads per row
    constexpr int ROWS = kBlock / TPR;    // rows per block
    __shared__ float4 s_w[27 * 4 * TPR];  // [k][j][c4]
    for (int t = threadIdx.x; t < K * 4 * TPR; t += kBlock)
        s_w[t] = make_float4(to_f32(W[4 * t]), to_f32(W[4 * t + 1]), to_f32(W[4 * t + 2]), to_f32(W[4 * t + 3]));
    __syncthreads();
    const int row = blockIdx.x * ROWS + threadIdx.x / TPR;
    const int c4 = threadIdx.x % TPR;
    if (row >= max_voxels) return;
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    if (row >= n && !write_pad) return;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < n) {
        for (int k = 0; k < K; ++k) {
            const int idx = nbr[(size_t)k * max_voxels + row];
            if (idx < 0) continue;
            const float4 x = reinterpret_cast<const float4*>(in)[idx];
            const float4* w = s_w + k * 4 * TPR + c4;
            float4 s;
            s.x = x.x * w[0].x; s.y = x.x * w[0].y; s.z = x.x * w[0].z; s.w = x.x * w[0].w;
            s.x = fmaf(x.y, w[TPR].x, s.x); s.y = fmaf(x.y, w[TPR].y, s.y); s.z = fmaf(x.y, w[TPR].z, s.z); s.w = fmaf(x.y, w[TPR].w, s.w);
            s.x = fmaf(x.z, w[2 * TPR].x, s.x); s.y = fmaf(x.z, w[2 * TPR].y, s.y); s.z = fmaf(x.z, w[2 * TPR].z, s.z); s.w = fmaf(x.z, w[2 * TPR].w, s.w);
            s.x = fmaf(x.w, w[3 * TPR].x, s.x); s.y = fmaf(x.w, w[3 * TPR].y, s.y); s.z = fmaf(x.w, w[3 * TPR].z, s.z); s.w = fmaf(x.w, w[3 * TPR].w, s.w);
            acc.x += s.x; acc.y += s.y; acc.z += s.z; acc.w += s.w;
        }
    }
    const int c = c4 * 4;
    float o[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = apply_epilogue(o[e], c + e, scale, shift, relu);
    Tout* dst = out + (size_t)row * COUT + c;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[e] = from_f32<Tout>(o[e]);
}

template <typename Tw, typename Tout, int COUT>
int launch_cin4(const GemmArgs& a, const Tw* w, hipStream_t stream) {
    constexpr int ROWS = kBlock / (COUT / 4);
    hipLaunchKernelGGL((conv_valu_cin4<Tw, Tout, COUT>), dim3(ceil_div(a.max_voxels, ROWS)), dim3(kBlock), 0, stream,
                       static_cast<const float*>(a.in_feat), static_cast<Tout*>(a.out_feat), w, a.nbr,
                       a.num_out, a.max_voxels, a.K, a.scale, a.shift, a.relu, a.write_pad_rows);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

template <typename Tin, typename Tw, typename Tout>
int launch_generic(const GemmArgs& a, const Tw* w, hipStream_t stream) {
    const int64_t elems = (int64_t)a.max_voxels * a.cout;
    const unsigned blocks = (unsigned)((elems + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((conv_valu_generic<Tin, Tw, Tout>), dim3(blocks), dim3(kBlock), 0, stream,
                       static_cast<const Tin*>(a.in_feat), static_cast<Tout*>(a.out_feat), w, a.nbr,
                       a.num_out, a.max_voxels, a.K, a.cin, a.cout, a.scale, a.shift, a.relu,
                       a.write_pad_rows);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

// ------------------------------------------------------------------------------------------
// rulebook export: wave64 ballot + prefix-scan compaction of nbr[k][:] into per-offset pair lists
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
export_masks(const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels,
             int words_per_k, uint64_t* __restrict__ masks) {
    const int row = blockIdx.x * kBlock + threadIdx.x;
    const int k = blockIdx.y;
    int n = *num_out;
    n = n > max_voxels ? max_voxels : n;
    const bool valid = row < n && nbr[(size_t)k * max_voxels + row] >= 0;
    const uint64_t m = __ballot(valid);
    if ((threadIdx.x & 63) == 0 && (row >> 6) < words_per_k) masks[(size_t)k * words_per_k + (row >> 6)] = m;
}

// one block per offset: exclusive scan of the popcounts of that offset's mask words
__global__ void __launch_bounds__(kBlock)
export_scan(const uint64_t* __restrict__ masks, int words_per_k, uint32_t* __restrict__ word_prefix,
            uint32_t* __restrict__ indice_num) {
    __shared__ uint32_t part[kBlock];
    const int k = blockIdx.x;
    const uint64_t* m = masks + (size_t)k * words_per_k;
    uint32_t* pre = word_prefix + (size_t)k * words_per_k;
    const int chunk = (words_per_k + kBlock - 1) / kBlock;
    const int lo = threadIdx.x * chunk;
    const int hi = lo + chunk < words_per_k ? lo + chunk : words_per_k;
    uint32_t s = 0;
    for (int w = lo; w < hi; ++w) s += __popcll(m[w]);
    part[threadIdx.x] = s;
    __syncthreads();
    for (int off = 1; off < kBlock; off <<= 1) {  // inclusive Hillis-Steele scan of the partials
        uint32_t v = threadIdx.x >= off ? part[threadIdx.x - off] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    uint32_t run = threadIdx.x ? part[threadIdx.x - 1] : 0;
    for (int w = lo; w < hi; ++w) {
        pre[w] = run;
        run += __popcll(m[w]);
    }
    if (threadIdx.x == kBlock - 1) indice_num[k] = part[kBlock - 1];
}

__global__ void __launch_bounds__(kBlock)
export_pairs(const int32_t* __restrict__ nbr, int max_voxels, int words_per_k,
             const uint64_t* __restrict__ masks, const uint32_t* __restrict__ word_prefix,
             int32_t* __restrict__ indice_pairs) {
    const int row = blockIdx.x * kBlock + threadIdx.x;
    const int k = blockIdx.y;
    if (row >= max_voxels) return;
    const uint64_t m = masks[(size_t)k * words_per_k + (row >> 6)];
    if (!((m >> (row & 63)) & 1ull)) return;
    const uint32_t pos = word_prefix[(size_t)k * words_per_k + (row >> 6)] + __popcll(m & ((1ull << (row & 63)) - 1ull));
    int32_t* base = indice_pairs + (size_t)k * 2 * max_voxels;
    base[pos] = nbr[(size_t)k * max_voxels + row];  // [k][0][pos] input row
    base[max_voxels + pos] = row;                   // [k][1][pos] output row
}

}  // namespace

int launch_mfma(const GemmArgs& a, hipStream_t stream);  // conv_mfma.hip

int launch_tall(const GemmArgs& a, hipStream_t stream);  // conv_tall.hip
int launch_wide(const GemmArgs& a, hipStream_t stream);  // conv_wide.hip

int launch_gather_gemm(const GemmArgs& a, hipStream_t stream) {
    if (!a.force_valu) {  // FP16 3x3x3 layers from 32 channels up: the tall-tile kernel
        const int rc = launch_tall(a, stream);
        if (rc != SESSD_E_UNSUPPORTED) return rc;
    }
    if (!a.force_valu) {  // FP32, 64 output columns: one tall tile per compute unit
        const int rc = launch_wide(a, stream);
        if (rc != SESSD_E_UNSUPPORTED) return rc;
    }
    if (!a.force_valu) {
        const int rc = launch_mfma(a, stream);
        if (rc != SESSD_E_UNSUPPORTED) return rc;  // launched (or failed for good)
    }
    if (a.dense.dense) return fail(SESSD_E_UNSUPPORTED, "gather-GEMM: the fused dense scatter needs the MFMA kernel");
    if (!a.force_valu && a.cin == 4 && a.K <= 27 && a.in_type == SESSD_FLOAT &&
        !(reinterpret_cast<uintptr_t>(a.in_feat) & 15)) {
        // FP16 output = the FP16 configuration: half-rounded weights, as in every other layer
        if (a.cout == 16 && a.out_type == SESSD_FLOAT) return launch_cin4<float, float, 16>(a, a.w_f32, stream);
        if (a.cout == 32 && a.out_type == SESSD_FLOAT) return launch_cin4<float, float, 32>(a, a.w_f32, stream);
        if (a.cout == 16 && a.out_type == SESSD_HALF) return launch_cin4<__half, __half, 16>(a, a.w_f16, stream);
        if (a.cout == 32 && a.out_type == SESSD_HALF) return launch_cin4<__half, __half, 32>(a, a.w_f16, stream);
    }
    if (a.in_type == SESSD_FLOAT && a.out_type == SESSD_FLOAT)
        return launch_generic<float, float, float>(a, a.w_f32, stream);
    if (a.in_type == SESSD_FLOAT && a.out_type == SESSD_HALF)
        return launch_generic<float, __half, __half>(a, a.w_f16, stream);
    if (a.in_type == SESSD_HALF && a.out_type == SESSD_HALF)
        return launch_generic<__half, __half, __half>(a, a.w_f16, stream);
    if (a.in_type == SESSD_HALF && a.out_type == SESSD_FLOAT)
        return launch_generic<__half, __half, float>(a, a.w_f16, stream);
    return fail(SESSD_E_UNSUPPORTED, "gather-GEMM: unsupported feature dtypes %d -> %d", a.in_type, a.out_type);
}

static int words_per_offset(int max_voxels) { return (max_voxels + 63) / 64; }

size_t export_scratch_bytes(int K, int max_voxels) {
    const size_t w = (size_t)K * words_per_offset(max_voxels);
    return align_up(w * sizeof(uint64_t)) + align_up(w * sizeof(uint32_t));
}

int launch_count_pairs(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels, void* scratch,
                       uint32_t* indice_num, hipStream_t stream) {
    if (!nbr || !num_out || !scratch || !indice_num) return fail(SESSD_E_INVALID, "count_pairs: null argument");
    const int wpk = words_per_offset(max_voxels);
    uint64_t* masks = static_cast<uint64_t*>(scratch);
    uint32_t* prefix = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(scratch) +
                                                   align_up((size_t)K * wpk * sizeof(uint64_t)));
    hipLaunchKernelGGL(export_masks, dim3(ceil_div(max_voxels, kBlock), K), dim3(kBlock), 0, stream, nbr, num_out,
                       max_voxels, wpk, masks);
    hipLaunchKernelGGL(export_scan, dim3(K), dim3(kBlock), 0, stream, masks, wpk, prefix, indice_num);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

int launch_export_rulebook(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels,
                           void* scratch, int32_t* indice_pairs, uint32_t* indice_num,
                           hipStream_t stream) {
    if (!nbr || !num_out || !scratch || !indice_pairs || !indice_num)
        return fail(SESSD_E_INVALID, "export_rulebook: null argument");
    const int wpk = words_per_offset(max_voxels);
    uint64_t* masks = static_cast<uint64_t*>(scratch);
    uint32_t* prefix = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(scratch) +
                                                   align_up((size_t)K * wpk * sizeof(uint64_t)));
    FillArgs f;
    f.add(indice_pairs, (uint64_t)K * 2 * max_voxels, kEmpty);  // -1, as submConv3dlayer.cu:583
    SESSD_TRY(launch_fill(f, stream));
    const dim3 grid(ceil_div(max_voxels, kBlock), K);
    hipLaunchKernelGGL(export_masks, grid, dim3(kBlock), 0, stream, nbr, num_out, max_voxels, wpk, masks);
    hipLaunchKernelGGL(export_scan, dim3(K), dim3(kBlock), 0, stream, masks, wpk, prefix, indice_num);
    hipLaunchKernelGGL(export_pairs, grid, dim3(kBlock), 0, stream, nbr, max_voxels, wpk, masks, prefix,
                       indice_pairs);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
