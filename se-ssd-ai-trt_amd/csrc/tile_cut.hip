// tile_cut.hip -- cuts the active output rows of a rulebook into tiles of equal WORK for the MFMA
// gather-GEMM.
//
// The GEMM kernel gives every workgroup a run of consecutive output rows.  With runs of equal length the
// busiest compute unit of the headline frame issues 37 % more MFMA blocks than the average one (pairs per
// row vary between 1 and 27 with the local density of the scene), and the launch lasts as long as the
// busiest unit.  Here every row gets the weight  pairs(row) + row_weight  and the rows are cut where the
// running sum crosses multiples of W = ceil(total / T), T = the tile count the equal-length rule would
// use (tile_plan() with the target height the caller names).  The per-row constant is the caller's: what a row
// costs its GEMM kernel beside its pairs (20 pairs' worth on the split-K kernel, 4 on the one-tile-per-unit kernel,
// whose tile time measured 732 cycles per 16-pair block + 22 per row); it also keeps sparse runs from growing far
// beyond the kernel's tile capacity.  Runs that still do are walked in capacity-sized pieces by the kernel, so any
// cut is correct.
//
// Two launches over the rows:
//   tile_weights  row weight -> w[row], per-block sums -> bsum[block]
//   tile_cuts     every block re-derives its offset and the total from bsum (a few hundred values),
//                 scans its rows, and the first row of every tile writes start[tile]; the last active row
//                 writes the end marker and the tile count.
// Region layout (int32): [0] tile count (0 = no cuts: the kernel falls back to equal lengths), [1] W,
// [2] total weight, [3] unused, [4 ..] start[0 .. count], then w[max_voxels], bsum[blocks].
#include "kernels.h"

namespace sessd {

namespace {

constexpr int kBlock = 256;

__host__ __device__ inline int max_tiles(int max_voxels) { return max_voxels / kGemmMinTileRows + 1024 + 1; }

// 256 rows per block, four threads per row (each sums every fourth offset): 1024 threads
constexpr int kSplit = 4;
__global__ void __launch_bounds__(kBlock * kSplit)
tile_weights(const int32_t* __restrict__ nbr, const int32_t* __restrict__ num_out, int max_voxels, int K,
             int row_weight, int32_t* __restrict__ w, int32_t* __restrict__ bsum) {
    __shared__ int32_t s_cnt[kSplit][kBlock];
    __shared__ int32_t s_part[kBlock / 64];
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    const int r = threadIdx.x % kBlock, kg = threadIdx.x / kBlock;
    const int row = blockIdx.x * kBlock + r;
    int c = 0;
    if (row < n) {
        constexpr int kPer = (kGemmMaxOffsets + kSplit - 1) / kSplit;
        int32_t e[kPer];  // all loads of the thread are requested before the first is used
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int k = kg + j * kSplit;
            e[j] = k < K ? nbr[(size_t)k * max_voxels + row] : -1;
        }
#pragma unroll
        for (int j = 0; j < kPer; ++j) c += e[j] >= 0 ? 1 : 0;
    }
    s_cnt[kg][r] = c;
    __syncthreads();
    int v = 0;
    if (kg == 0 && row < n) {
        v = row_weight;
#pragma unroll
        for (int g = 0; g < kSplit; ++g) v += s_cnt[g][r];
    }
    if (kg == 0 && row < max_voxels) w[row] = v;
    int s = v;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) s += __shfl_xor(s, d, 64);
    if (kg == 0 && (r & 63) == 0) s_part[r >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) bsum[blockIdx.x] = s_part[0] + s_part[1] + s_part[2] + s_part[3];
}

__global__ void __launch_bounds__(kBlock)
tile_cuts(const int32_t* __restrict__ num_out, int max_voxels, int num_cu, int target, int row_weight, const int32_t* __restrict__ w,
          const int32_t* __restrict__ bsum, int32_t* __restrict__ hdr) {
    __shared__ int32_t s_before[kBlock / 64], s_total[kBlock / 64], s_wave[kBlock / 64];
    int n = *num_out;
    n = n < 0 ? 0 : (n > max_voxels ? max_voxels : n);
    if (n == 0) return;  // the count stays 0
    const int nb = (n + kBlock - 1) / kBlock;  // blocks that hold active rows
    if ((int)blockIdx.x >= nb) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // weight before this block and in total
    int before = 0, total = 0;
    for (int b = threadIdx.x; b < nb; b += kBlock) {
        const int v = bsum[b];
        total += v;
        if (b < (int)blockIdx.x) before += v;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        before += __shfl_xor(before, d, 64);
        total += __shfl_xor(total, d, 64);
    }
    if (lane == 0) {
        s_before[wave] = before;
        s_total[wave] = total;
    }
    // inclusive scan of the block's row weights
    const int row = blockIdx.x * kBlock + threadIdx.x;
    const int mine = row < n ? w[row] : 0;
    int inc = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(inc, d, 64);
        if (lane >= d) inc += o;
    }
    if (lane == 63) s_wave[wave] = inc;
    __syncthreads();
    before = s_before[0] + s_before[1] + s_before[2] + s_before[3];
    total = s_total[0] + s_total[1] + s_total[2] + s_total[3];
    for (int v = 0; v < wave; ++v) before += s_wave[v];
    const int excl = before + inc - mine;  // weight of all rows before this one
    const int tiles = tile_plan(n, num_cu, target).count;
    // W is kept above the heaviest possible row: a row then advances the tile id by at most one, so every id
    // up to the last gets its start written (with few rows -- fewer than tiles -- total / tiles would fall
    // below a row's weight, ids would skip, and the skipped entries of the table would be read unwritten)
    int W = (total + tiles - 1) / tiles;
    W = W > kGemmMaxOffsets + row_weight ? W : kGemmMaxOffsets + row_weight + 1;
    if (row < n) {
        const int id = excl / W;
        const int prev = row == 0 ? -1 : (excl - w[row - 1]) / W;
        int32_t* start = hdr + 4;
        if (id != prev) start[id] = row;  // ids grow by at most one per row (W exceeds every row weight)
        if (row == n - 1) {
            start[id + 1] = n;
            hdr[1] = W;
            hdr[2] = total;
            hdr[0] = id + 1;
        }
    }
}

}  // namespace

size_t tile_cut_bytes(int max_voxels) {
    const size_t ints = 4 + (size_t)max_tiles(max_voxels) + 1 + (size_t)max_voxels + (size_t)ceil_div(max_voxels, kBlock);
    return align_up(ints * sizeof(int32_t));
}

int launch_tile_cuts(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels, int target_rows, int row_weight,
                     void* region, hipStream_t stream) {
    if (target_rows < kGemmMinTileRows) return fail(SESSD_E_INVALID, "tile cuts: target of %d rows is below %d", target_rows, kGemmMinTileRows);
    int32_t* hdr = static_cast<int32_t*>(region);
    int32_t* w = hdr + 4 + max_tiles(max_voxels) + 1;
    int32_t* bsum = w + max_voxels;
    const int blocks = ceil_div(max_voxels, kBlock);
    hipLaunchKernelGGL(tile_weights, dim3(blocks), dim3(kBlock * kSplit), 0, stream, nbr, num_out, max_voxels, K, row_weight, w, bsum);
    hipLaunchKernelGGL(tile_cuts, dim3(blocks), dim3(kBlock), 0, stream, num_out, max_voxels, gemm_compute_units(), target_rows, row_weight, w,
                       bsum, hdr);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
