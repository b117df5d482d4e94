// kernels.h -- launchers of the gather-GEMM kernels (conv_gemm.hip) used by both conv plugins.
#pragma once

#include "common.h"

namespace sessd {

struct GemmArgs {
    const void* in_feat;     // [max_voxels][cin]   FP32 or FP16
    void* out_feat;          // [max_voxels][cout]  FP32 or FP16
    const int32_t* nbr;      // [K][max_voxels] input row feeding (offset k, output row), -1 = none
    const int32_t* num_out;  // device scalar: active output rows
    int max_voxels;
    int K, cin, cout;
    int in_type, out_type;   // SESSD_FLOAT / SESSD_HALF
    const float* w_f32;      // [K][cin][cout]
    const __half* w_f16;     // same layout, rounded to half (used when in_type is HALF)
    const void* w_packed;    // MFMA operand order, or null
    const float* scale;      // [cout] or null
    const float* shift;      // [cout] or null
    int relu;
    int write_pad_rows;      // rows >= *num_out get epilogue(0) (the reference zero-fills them)
    int force_valu;          // skip the MFMA kernels (cross-check)
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
int launch_tile_cuts(const int32_t* nbr, const int32_t* num_out, int K, int max_voxels, int target_rows, int row_weight,
                     void* region, hipStream_t stream);

// picks the kernel for the layer shape; returns SESSD_E_UNSUPPORTED for dtype pairs not covered, and when a
// dense target is set but the layer does not run on the MFMA kernel (see gemm_runs_on_mfma)
int launch_gather_gemm(const GemmArgs& a, hipStream_t stream);
bool gemm_runs_on_mfma(int K, int cin, int cout, int in_type, int out_type);
// whether the layer runs on the tall-tile FP16 kernel (conv_tall.hip), which cuts its own tiles: a rulebook whose
// owner does needs no equal-work cuts
bool gemm_runs_tall(int K, int cin, int cout, int in_type, int out_type);
// whether the layer runs on the FP32 kernel with one tall tile per compute unit (conv_wide.hip), and that kernel's
// tile capacity
bool gemm_runs_wide(int K, int cin, int cout, int in_type, int out_type);
int gemm_wide_tile_rows();

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
