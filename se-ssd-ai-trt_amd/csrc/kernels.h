// kernels.h -- launchers of the gather-GEMM kernels (conv_gemm.hip) used by both conv plugins.
#pragma once

#include "common.h"

namespace sessd {

struct GemmArgs {
    const void* in_feat;     // [max_voxels][cin]   FP32 or FP16
    void* out_feat;          // [max_voxels][cout]  FP32 or FP16
    const void* in_split = nullptr;  // the input rows in split form (split_row_bytes(cin) per row), or null
    void* out_split = nullptr;       // where to also write the output rows in split form, or null
    const int32_t* nbr;      // [K][max_voxels] input row feeding (offset k, output row), -1 = none
    const int32_t* num_out;  // device scalar: active output rows
    int max_voxels;
    int K, cin, cout;
    int in_type, out_type;   // SESSD_FLOAT / SESSD_HALF
    const float* w_f32;      // [K][cin][cout]
    const __half* w_f16;     // same layout, rounded to half (used when in_type is HALF)
    const void* w_packed;    // MFMA operand order, or null
    const void* w_split;     // three BF16 parts in MFMA operand order (conv_split.hip), or null
    const float* scale;      // [cout] or null
    const float* shift;      // [cout] or null
    int relu;
    int write_pad_rows;      // rows >= *num_out get epilogue(0) (the reference zero-fills them)
    int force_valu;          // skip the MFMA kernels (cross-check)
    int fp32_mfma;           // FP32 layers on the FP32 matrix instructions, not on the split-BF16 kernel
    const int32_t* tiles;    // tile cuts of this rulebook (launch_tile_cuts) or null: tiles of equal length
    DenseTarget dense;       // dense.dense != null: also scatter the rows there (MFMA kernel only)
};

// Tiling of the MFMA gather-GEMM: n active rows on num_cu compute units are cut into num_cu * r tiles,
// r = the smallest tiles-per-CU count that keeps the mean tile at or below the target height, so that every
// CU gets the same number of tiles (a fixed 32-row tiling leaves e.g. 529 tiles for 256 CUs: some CUs run
// three tiles, most two, and the kernel lasts as long as the three).
// The target is the tile capacity of the kernel the rulebook's owner runs (gemm_tile_rows()): the tallest
// tiles the quantisation to whole tiles per CU allows.  Any cut is correct for any kernel: runs longer than
// a kernel's capacity are walked in pieces.
constexpr int kGemmMinTileRows = 48;  // smallest capacity of any kernel: bounds the tile count
constexpr int kGemmMaxOffsets = 27;  // kernel volumes the rulebook holds (3 x 3 x 3)
struct TilePlan {
    int count;   // tiles
    int height;  // rows per tile when all tiles have the same length
};
__host__ __device__ inline TilePlan tile_plan(int n, int num_cu, int target) {
    TilePlan p;
    if (n <= 0) {
        p.count = num_cu;
        p.height = 1;
        return p;
    }
    const int r = (n + num_cu * target - 1) / (num_cu * target);
    p.count = num_cu * r;
    p.height = (n + p.count - 1) / p.count;
    return p;
}
// tile capacity (rows) of the MFMA kernel that serves this layer shape
int gemm_tile_rows(int cin, int cout, int dtype);
int gemm_compute_units();

// equal-work tile cuts for the MFMA kernel, written into `region` (tile_cut_bytes() bytes of the layer's
// workspace; its first word must be zero before the launch and stays zero when there are no active rows);
// target_rows >= kGemmMinTileRows is the tile height aimed at
size_t tile_cut_bytes(int max_voxels);
int launch_tile_cuts(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels, int target_rows,
                     void* region, hipStream_t stream);

// picks the kernel for the layer shape; returns SESSD_E_UNSUPPORTED for dtype pairs not covered, and when a
// dense target is set but the layer does not run on the MFMA kernel (see gemm_runs_on_mfma)
int launch_gather_gemm(const GemmArgs& a, hipStream_t stream);
bool gemm_runs_on_mfma(int K, int cin, int cout, int in_type, int out_type);
// whether the layer runs on the tall-tile FP16 kernel (conv_tall.hip), which cuts its own tiles: a rulebook whose
// owner does needs no equal-work cuts
bool gemm_runs_tall(int K, int cin, int cout, int in_type, int out_type);

// whether the layer runs on the split-BF16 kernel (conv_split.hip: FP32 features, fixed-height tiles, no cuts)
bool gemm_runs_split(int K, int cin, int cout, int in_type, int out_type);
size_t split_weight_bytes(int K, int cin, int cout);
void pack_weights_split(const float* w, int K, int cin, int cout, void* dst);

// Split form of an FP32 feature tensor (conv_split.hip): row r = [part 0: C BF16][part 1][part 2], the three BF16
// values a channel's FP32 value is the sum of.  Written by the epilogues of the kernels that can (the split-BF16
// kernel, the FP32 MFMA kernel) when GemmArgs::out_split is set, or from FP32 rows by launch_split_rows.
__host__ __device__ constexpr int split_row_bytes(int channels) { return 6 * channels; }
size_t split_feature_bytes(int max_voxels, int channels);
// whether the kernel launch_gather_gemm picks for these arguments honours GemmArgs::out_split
bool gemm_writes_split(const GemmArgs& a);
int launch_split_rows(const float* in, void* out_split, const int32_t* num, int max_voxels, int channels,
                      hipStream_t stream);
#ifdef __HIPCC__
// two floats -> two BF16 (round to nearest even) in one register: v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef float v2f_t __attribute__((ext_vector_type(2)));
    typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
    const v2f_t v = {lo, hi};
    const v2bf_t r = __builtin_convertvector(v, v2bf_t);
    return *reinterpret_cast<const uint32_t*>(&r);
}
// channels c4 .. c4+3 of row `row` (C channels per row) -> their three BF16 parts in the split tensor
__device__ __forceinline__ void store_split4(void* split, int row, int C, int c4, const float (&x)[4]) {
    uint8_t* dst = static_cast<uint8_t*>(split) + (size_t)row * split_row_bytes(C) + 2 * c4;
    uint32_t p[3][2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float a = x[2 * e], b = x[2 * e + 1];
        p[0][e] = pack_bf16(a, b);
        const float ra = a - __uint_as_float(p[0][e] << 16), rb = b - __uint_as_float(p[0][e] & 0xffff0000u);
        p[1][e] = pack_bf16(ra, rb);
        const float sa = ra - __uint_as_float(p[1][e] << 16), sb = rb - __uint_as_float(p[1][e] & 0xffff0000u);
        p[2][e] = pack_bf16(sa, sb);
    }
#pragma unroll
    for (int t = 0; t < 3; ++t) *reinterpret_cast<uint2*>(dst + t * 2 * C) = make_uint2(p[t][0], p[t][1]);
}
#endif

// size in bytes of the packed weight copy for this shape/dtype (0 = shape runs on the VALU path)
size_t packed_weight_bytes(int K, int cin, int cout, int dtype);
// host-side packing into MFMA operand order; dst has packed_weight_bytes() bytes
void pack_weights(const float* w, int K, int cin, int cout, int dtype, void* dst);

// rulebook export (reference layout indice_pairs[K][2][max_voxels], indice_num[K])
size_t export_scratch_bytes(int K, int max_voxels);
int launch_export_rulebook(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels,
                           void* scratch, int32_t* indice_pairs, uint32_t* indice_num,
                           hipStream_t stream);

// indice_num[k] only (pairs per offset), same scratch as the export
int launch_count_pairs(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels, void* scratch,
                       uint32_t* indice_num, hipStream_t stream);

}  // namespace sessd
