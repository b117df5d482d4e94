// sessd_oracle.cpp -- scalar CPU restatement of the SE-SSD-AI-TRT 3-D front-end plugins.
//
// TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP library: it is built
// into oracle/_build/libsessd_oracle.so and may be loaded only by tests/, by
// __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  Nothing in the product
// (the package, the C-ABI library) links, loads or calls it.
//
// Every function restates one piece of the reference, cited as file:line relative to the
// reference checkout.  Where the reference's GPU code is order-dependent on atomics, the
// sequential meaning is used: points / voxels are processed in index order.
//
// Build: g++ -O2 -fno-fast-math -ffp-contract=off (IEEE FP32 division and no FMA contraction are
// required for bit-exact voxel coordinates and a reproducible summation order).
//
// What pins each function (tests/test_oracle_*.py):
//   oracle_np_round / oracle_grid_size  closed form 1408x1600x40 + half-even cases
//   oracle_voxelize                     KITTI frame 000000 known answers held in the reference's
//                                       comments (16825 voxels; point 0 -> (38,800,366)),
//                                       an independent numpy-float32 recomputation, brute-force
//                                       grouping, FP32 boundary cases
//   oracle_valid_out_pos                brute force over (out cell, offset) on small grids
//   oracle_subm_rulebook                centre-offset identity, (i,o,k)<->(o,i,26-k) symmetry,
//                                       brute force
//   oracle_sparse_rulebook              brute-force out set, out-grid formula, KITTI counts
//   oracle_gather_gemm_scatter          dense equivalence with torch.nn.functional.conv3d,
//                                       neighbour-count special case, linearity
//   oracle_scale_shift_relu / fold_bn   closed form (the reference has no test at this boundary:
//                                       TensorRT IScaleLayer semantics are the textbook ones)
//   oracle_sparse2dense                 closed-form index + inverse gather
//   oracle_zero_pad2d                   equality with torch.nn.functional.pad (constant 0)
//   oracle_frame                        composition of the above (checked against calling them
//                                       one by one)

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../include/sessd3d.h"

namespace {

// Dense index grid as the reference keeps in its workspace (submConv3dlayer.cu:253,582:
// int grid over the whole volume, memset to -1).  Kept between calls and reset sparsely so a
// call costs O(active sites) instead of O(volume); the observable content during a call is the
// reference's.
struct DenseGrid {
    std::vector<int32_t> cells;
    std::vector<size_t> touched;
    int32_t* acquire(size_t volume) {
        if (cells.size() < volume) cells.assign(volume, -1);
        touched.clear();
        return cells.data();
    }
    void set(size_t idx, int32_t v) {
        if (cells[idx] == -1) touched.push_back(idx);
        cells[idx] = v;
    }
    void release() {
        for (size_t i : touched) cells[i] = -1;
        touched.clear();
    }
};
thread_local DenseGrid g_grid;
int g_threads = 1;  // see oracle_set_threads

// Round an FP32 value to the nearest IEEE binary16 value (ties to even, subnormals kept,
// overflow to infinity) and return it as FP32.
float round_to_half(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return f;  // inf / nan
    float r;
    if (a >= 0x477ff000u) {  // >= 65520 rounds to infinity
        a = 0x7f800000u;
    } else if (a < 0x38800000u) {  // below the smallest normal half: quantum 2^-24
        float mag;
        std::memcpy(&mag, &a, 4);
        mag = (mag + 0.5f) - 0.5f;  // 0.5f has ulp 2^-24 for sums in [0.5,1): rounds ties-to-even
        std::memcpy(&a, &mag, 4);
    } else {
        const uint32_t lsb = (a >> 13) & 1u;
        a = (a + 0x0fffu + lsb) & ~0x1fffu;
    }
    a |= sign;
    std::memcpy(&r, &a, 4);
    return r;
}

}  // namespace

extern "C" {

// voxelGenerator.cu:61-68 -- round half to even, as np.round.
int oracle_np_round(float x) {
    int x2 = int(x * 2.0f);
    if (x != int(x) && x2 == x * 2.0f) {
        return int(x / 2.0f + 0.5f) * 2;
    }
    return int(x + 0.5f);
}

// voxelGenerator.cu:228-235 -- grid dims (x,y,z) from range (xmin,ymin,zmin,xmax,ymax,zmax).
void oracle_grid_size(const float* range, const float* vsize, int32_t* grid_xyz) {
    grid_xyz[0] = oracle_np_round((range[3] - range[0]) / vsize[0]);
    grid_xyz[1] = oracle_np_round((range[4] - range[1]) / vsize[1]);
    grid_xyz[2] = oracle_np_round((range[5] - range[2]) / vsize[2]);
}

// voxelGenerator.cu:348-451 (generateVoxels_kernel) + :255-321 (generateAverage_kernel), with
// points taken in index order.  Returns a SESSD_STATUS_* mask.
//   points      f32[n_points][point_features]   (x,y,z,i first)
//   voxels      f32[max_voxels][4]              mean of the kept points, rows >= voxel_num are 0
//   coors       i32[max_voxels][4]              (0,z,y,x)
//   num_points  i32[max_voxels] or NULL         kept points per voxel (<= max_pts)
int oracle_voxelize(const float* points, int32_t n_points, int32_t point_features,
                    const float* range, const float* vsize, int32_t max_pts, int32_t max_voxels,
                    float* voxels, int32_t* coors, int32_t* voxel_num, int32_t* num_points) {
    int32_t g[3];
    oracle_grid_size(range, vsize, g);
    const int gx = g[0], gy = g[1], gz = g[2];
    const float min_x = range[0], min_y = range[1], min_z = range[2];
    const float max_x = range[3], max_y = range[4], max_z = range[5];
    int status = 0;

    std::memset(voxels, 0, sizeof(float) * 4 * (size_t)max_voxels);  // :524
    std::memset(coors, 0, sizeof(int32_t) * 4 * (size_t)max_voxels); // :525
    // slot table voxel_[vid][slot][4] and per-cell arrival count (:506-517)
    std::vector<float> slots((size_t)max_voxels * max_pts * 4, 0.0f);
    std::vector<int32_t> kept((size_t)max_voxels, 0);
    int32_t* grid = g_grid.acquire((size_t)gx * gy * gz);
    int32_t nvox = 0;

    for (int32_t p = 0; p < n_points; ++p) {
        const float* pt = points + (size_t)p * point_features;
        const float x = pt[0], y = pt[1], z = pt[2], w = pt[3];
        if (!(x >= min_x && x < max_x && y >= min_y && y < max_y && z >= min_z && z < max_z))
            continue;  // :363-367
        int ix = (int)floorf((x - min_x) / vsize[0]);  // :369-371
        int iy = (int)floorf((y - min_y) / vsize[1]);
        int iz = (int)floorf((z - min_z) / vsize[2]);
        if (ix < 0 || ix >= gx || iy < 0 || iy >= gy || iz < 0 || iz >= gz) continue;  // :375
        size_t cell = (size_t)iz * ((size_t)gy * gx) + (size_t)iy * gx + ix;      // :378
        int32_t vid = grid[cell];
        if (vid == -1) {  // first point of the cell: allocate a voxel id (:387-407)
            if (nvox >= max_voxels) {
                // the reference has no capacity check and overflows; here the cell is dropped
                g_grid.set(cell, -2);
                status |= SESSD_STATUS_VOXEL_OVERFLOW;
                continue;
            }
            vid = nvox++;
            g_grid.set(cell, vid);
            coors[vid * 4 + 0] = 0;
            coors[vid * 4 + 1] = iz;
            coors[vid * 4 + 2] = iy;
            coors[vid * 4 + 3] = ix;
        } else if (vid == -2) {
            continue;
        }
        int32_t slot = kept[vid];
        if (slot >= max_pts) continue;  // :383
        float* dst = &slots[((size_t)vid * max_pts + slot) * 4];  // :426-430
        dst[0] = x; dst[1] = y; dst[2] = z; dst[3] = w;
        kept[vid] = slot + 1;  // :433-437
    }
    g_grid.release();

    // generateAverage_kernel :274-296 -- all max_pts slots are summed left to right (unfilled
    // slots hold 0) and divided by the kept count.
    for (int32_t v = 0; v < nvox; ++v) {
        for (int c = 0; c < 4; ++c) {
            float s = slots[((size_t)v * max_pts + 0) * 4 + c];
            for (int32_t k = 1; k < max_pts; ++k) s = s + slots[((size_t)v * max_pts + k) * 4 + c];
            voxels[v * 4 + c] = s / (float)kept[v];
        }
        if (num_points) num_points[v] = kept[v];
    }
    *voxel_num = nvox;
    return status;
}

// submConv3dlayer.cu:271-358 == sparseConv3dlayer.cu:310-386 (getValidOutPosKernel).
//   c[3], ksize[3], stride[3], padding[3], out_shape[3] all (z,y,x); out[27][4] = (oz,oy,ox,offset)
// Returns the number of valid rows, in the reference's enumeration order.
int oracle_valid_out_pos(const int32_t* c, const int32_t* ksize, const int32_t* stride,
                         const int32_t* padding, int32_t dilation, const int32_t* out_shape,
                         int32_t* out) {
    const int NDim = 3;
    int lowers[3], uppers[3], counter[3] = {0, 0, 0}, counter_size[3];
    int num_points = 1, point_counter = 0;
    for (int i = 0; i < NDim; i++) {
        lowers[i] = (c[i] - (ksize[i] - 1) * dilation - 1 + stride[i] + padding[i]) / stride[i];
        uppers[i] = (c[i] + padding[i]) / stride[i];
    }
    for (int i = 0; i < NDim; i++) {
        counter_size[i] = ((uppers[i] - lowers[i]) / dilation + 1);
        num_points *= counter_size[i];
    }
    for (int i = 0; i < num_points; i++) {
        int valid = 1, m = 1, offset = 0;
        int32_t* row = out + point_counter * 4;
        for (int j = NDim - 1; j >= 0; j--) {
            int val = uppers[j] - counter[j] * dilation;
            row[j] = val;
            if (val < 0 || (val > out_shape[j] - 1)) valid = 0;
            offset += m * (c[j] - val * stride[j] + padding[j]) / dilation;
            m *= ksize[j];
        }
        row[NDim] = offset;
        if (valid) point_counter += 1;
        counter[NDim - 1] += 1;
        for (int k = NDim - 1; k >= 0; k--) {
            if (counter[k] == counter_size[k] && k > 0) {
                counter[k - 1] += 1;
                counter[k] = 0;
            }
        }
    }
    return point_counter;
}

// submConv3dlayer.cu:441-459 (prepareSubMGridKernel) + :376-424 (getSubMIndicePairsKernel).
//   coors i32[n][4] (b,z,y,x); out_shape (x,y,z) as the plugin field
//   indice_pairs i32[K][2][max_voxels] filled with -1 first (:583); indice_num u32[K]
int oracle_subm_rulebook(const int32_t* coors, int32_t n, const int32_t* out_shape_xyz,
                         int32_t ksize, int32_t stride, int32_t padding, int32_t dilation,
                         int32_t max_voxels, int32_t* indice_pairs, uint32_t* indice_num) {
    const int K = ksize * ksize * ksize;
    const int X = out_shape_xyz[0], Y = out_shape_xyz[1], Z = out_shape_xyz[2];
    const int32_t ks[3] = {ksize, ksize, ksize}, st[3] = {stride, stride, stride};
    const int32_t pd[3] = {padding, padding, padding}, os[3] = {Z, Y, X};
    int status = 0;
    for (size_t i = 0; i < (size_t)K * 2 * max_voxels; ++i) indice_pairs[i] = -1;
    for (int k = 0; k < K; ++k) indice_num[k] = 0;
    int32_t* grid = g_grid.acquire((size_t)X * Y * Z);
    std::vector<char> in_grid((size_t)n, 0);
    for (int32_t v = 0; v < n; ++v) {  // :452-457
        const int32_t z = coors[v * 4 + 1], y = coors[v * 4 + 2], x = coors[v * 4 + 3];
        if (z < 0 || z >= Z || y < 0 || y >= Y || x < 0 || x >= X) {
            status |= SESSD_STATUS_BAD_COORD;  // the reference would write out of bounds
            continue;
        }
        in_grid[v] = 1;
        g_grid.set((size_t)z * Y * X + (size_t)y * X + x, v);
    }
    int32_t vp[27 * 4];
    for (int32_t v = 0; v < n; ++v) {  // :393-422
        if (!in_grid[v]) continue;
        const int32_t c[3] = {coors[v * 4 + 1], coors[v * 4 + 2], coors[v * 4 + 3]};
        int cnt = oracle_valid_out_pos(c, ks, st, pd, dilation, os, vp);
        for (int i = 0; i < cnt; ++i) {
            size_t index = (size_t)vp[i * 4 + 0] * Y * X + (size_t)vp[i * 4 + 1] * X + vp[i * 4 + 2];
            int offset = vp[i * 4 + 3];
            if (grid[index] > -1) {
                uint32_t old_num = indice_num[offset]++;
                indice_pairs[(size_t)offset * 2 * max_voxels + 1 * (size_t)max_voxels + old_num] = grid[index];
                indice_pairs[(size_t)offset * 2 * max_voxels + 0 * (size_t)max_voxels + old_num] = v;
            }
        }
    }
    g_grid.release();
    return status;
}

// sparseConv3dlayer.cu:475-541 (fillGridKernel1/2) + :405-454 (getSparseIndicePairsKernel);
// output numbering = the author's host restatement sparseConv3dlayer.cu:738-757 (input voxels in
// order, first-seen out cell gets the next index).
//   ksize/stride/padding (z,y,x); out_shape (x,y,z)
//   out_coors i32[max_voxels][4] zeroed first (:668); out_num i32[1]
int oracle_sparse_rulebook(const int32_t* coors, int32_t n, const int32_t* out_shape_xyz,
                           const int32_t* ksize, const int32_t* stride, const int32_t* padding,
                           int32_t dilation, int32_t max_voxels, int32_t* indice_pairs,
                           uint32_t* indice_num, int32_t* out_coors, int32_t* out_num) {
    const int K = ksize[0] * ksize[1] * ksize[2];
    const int X = out_shape_xyz[0], Y = out_shape_xyz[1], Z = out_shape_xyz[2];
    const int32_t os[3] = {Z, Y, X};
    int status = 0;
    for (size_t i = 0; i < (size_t)K * 2 * max_voxels; ++i) indice_pairs[i] = -1;
    for (int k = 0; k < K; ++k) indice_num[k] = 0;
    std::memset(out_coors, 0, sizeof(int32_t) * 4 * (size_t)max_voxels);
    int32_t* grid = g_grid.acquire((size_t)X * Y * Z);
    int32_t m = 0;
    int32_t vp[27 * 4];
    for (int32_t v = 0; v < n; ++v) {
        const int32_t c[3] = {coors[v * 4 + 1], coors[v * 4 + 2], coors[v * 4 + 3]};
        // A negative coordinate: with C's truncating division getValidOutPos then yields kernel offsets outside
        // [0, K) (e.g. c = -2, k = 3, s = 2, p = 1: o = 0, c - o*s + p = -1) and the reference indexes its rulebook
        // with them.  Defined here: the row contributes nothing and the status word says so.
        if (c[0] < 0 || c[1] < 0 || c[2] < 0) {
            status |= SESSD_STATUS_BAD_COORD;
            continue;
        }
        int cnt = oracle_valid_out_pos(c, ksize, stride, padding, dilation, os, vp);
        for (int i = 0; i < cnt; ++i) {
            size_t index = (size_t)vp[i * 4 + 0] * Y * X + (size_t)vp[i * 4 + 1] * X + vp[i * 4 + 2];
            if (grid[index] == -1) {
                if (m < max_voxels) {
                    g_grid.set(index, m);
                    out_coors[m * 4 + 0] = 0;
                    out_coors[m * 4 + 1] = vp[i * 4 + 0];
                    out_coors[m * 4 + 2] = vp[i * 4 + 1];
                    out_coors[m * 4 + 3] = vp[i * 4 + 2];
                    ++m;
                } else {
                    // the reference overflows its buffers here; the site is dropped instead
                    g_grid.set(index, -2);
                    status |= SESSD_STATUS_VOXEL_OVERFLOW;
                }
            }
        }
    }
    for (int32_t v = 0; v < n; ++v) {
        const int32_t c[3] = {coors[v * 4 + 1], coors[v * 4 + 2], coors[v * 4 + 3]};
        if (c[0] < 0 || c[1] < 0 || c[2] < 0) continue;
        int cnt = oracle_valid_out_pos(c, ksize, stride, padding, dilation, os, vp);
        for (int i = 0; i < cnt; ++i) {
            size_t index = (size_t)vp[i * 4 + 0] * Y * X + (size_t)vp[i * 4 + 1] * X + vp[i * 4 + 2];
            int offset = vp[i * 4 + 3];
            if (grid[index] < 0) continue;  // dropped site
            uint32_t old_num = indice_num[offset]++;
            indice_pairs[(size_t)offset * 2 * max_voxels + 1 * (size_t)max_voxels + old_num] = grid[index];
            indice_pairs[(size_t)offset * 2 * max_voxels + 0 * (size_t)max_voxels + old_num] = v;
        }
    }
    g_grid.release();
    *out_num = m;
    return status;
}

// submConv3dlayer.cu:479-518 == sparseConv3dlayer.cu:557-589 (sparseGatherConvScatter), launched
// for k = 0..K-1 in order (:632-638).  out is zeroed over all max_voxels rows first (:594).
// Per pair: s[c] = sum_j in[i][j]*W[k][j][c] with j ascending from 0.0f, then out[o][c] += s[c].
// (The j loop is hoisted outside the c loop; each s[c] still accumulates in the same order.)
//
// Threads (oracle_set_threads, default 1): the pairs of ONE offset are split over threads.  Inside an
// offset every output row occurs at most once (in = out*stride - pad + k is injective for fixed k), so
// threads never share an output row and every out[o][c] still receives its terms in offset order: the
// result is bit-identical for any thread count.  Used only to time a multi-core CPU baseline.
void oracle_gather_gemm_scatter(const float* in_feat, const float* weights,
                                const int32_t* indice_pairs, const uint32_t* indice_num, int32_t K,
                                int32_t max_voxels, int32_t cin, int32_t cout, float* out_feat) {
    if (cout > 512) std::abort();  // the per-pair accumulator below is a fixed array
    std::memset(out_feat, 0, sizeof(float) * (size_t)max_voxels * cout);
    for (int k = 0; k < K; ++k) {
        const float* W = weights + (size_t)k * cin * cout;
        const int32_t* in_idx = indice_pairs + (size_t)k * 2 * max_voxels;
        const int32_t* out_idx = in_idx + max_voxels;
        const int64_t pairs = indice_num[k];
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && pairs > 256)
        for (int64_t a = 0; a < pairs; ++a) {
            const float* x = in_feat + (size_t)in_idx[a] * cin;
            float* y = out_feat + (size_t)out_idx[a] * cout;
            float s[512];
            for (int c = 0; c < cout; ++c) s[c] = 0.0f;
            for (int j = 0; j < cin; ++j) {
                const float xj = x[j];
                const float* w = W + (size_t)j * cout;
                for (int c = 0; c < cout; ++c) s[c] = s[c] + xj * w[c];
            }
            for (int c = 0; c < cout; ++c) y[c] = y[c] + s[c];
        }
    }
}

// Threads oracle_gather_gemm_scatter may use (>= 1); everything else stays sequential.
void oracle_set_threads(int32_t n) { g_threads = n < 1 ? 1 : n; }

// Test helper: nearest binary16 value of every element (ties to even), as FP32.
void oracle_round_to_half(float* x, int64_t n) {
    for (int64_t i = 0; i < n; ++i) x[i] = round_to_half(x[i]);
}

// se-ssd-ai-trt.cpp:816-824 -- BatchNorm folding on the host.  The file includes <cmath> and is
// `using namespace std` (:24,29), so `sqrt(var[i] + eps)` on a float argument is the float overload
// and both expressions are evaluated in FP32, left to right: gamma / sqrtf(var + eps) and
// beta - (mean * gamma) / sqrtf(var + eps).  `eps` arrives as a float parameter (:808).
void oracle_fold_bn(const float* gamma, const float* beta, const float* mean, const float* var,
                    float eps, int32_t c, float* scale, float* shift) {
    for (int i = 0; i < c; ++i) {
        scale[i] = gamma[i] / sqrtf(var[i] + eps);
        shift[i] = beta[i] - mean[i] * gamma[i] / sqrtf(var[i] + eps);
    }
}

// se-ssd-ai-trt.cpp:843-855 -- IScaleLayer(kCHANNEL, shift, scale, power=1) then kRELU, applied to
// `rows` rows (the reference applies it to all max_voxels rows).  scale/shift may be NULL.
void oracle_scale_shift_relu(float* x, int32_t rows, int32_t c, const float* scale,
                             const float* shift, int32_t relu) {
    for (int32_t r = 0; r < rows; ++r) {
        for (int i = 0; i < c; ++i) {
            float v = x[(size_t)r * c + i];
            if (scale) v = v * scale[i];
            if (shift) v = v + shift[i];
            if (relu) v = v > 0.0f ? v : 0.0f;
            x[(size_t)r * c + i] = v;
        }
    }
}

// sparse2Dense.cu:182-207 + :240-242 -- dense[(c*D+z)][y][x] = feat[v][c], everything else 0.
//   size (x,y,z) = (W,H,D)
void oracle_sparse2dense(const float* feat, const int32_t* coors, int32_t n, int32_t channels,
                         const int32_t* size_xyz, float* dense) {
    const int W = size_xyz[0], H = size_xyz[1], D = size_xyz[2];
    std::memset(dense, 0, sizeof(float) * (size_t)W * H * D * channels);
    for (int32_t v = 0; v < n; ++v) {
        const int32_t b = coors[v * 4 + 0], z = coors[v * 4 + 1], y = coors[v * 4 + 2],
                      x = coors[v * 4 + 3];
        for (int i = 0; i < channels; ++i) {
            dense[(size_t)b * channels * W * H * D + ((size_t)(i * D) + z) * W * H + (size_t)y * W + x] =
                feat[(size_t)v * channels + i];
        }
    }
}

// zeroPad2d.cu:183-244 -- out[c][y + top][x + left] = in[c][y][x] over a zero-filled
// [channels][height + top + bottom][width + left + right] tensor (the memset of :230, then one
// thread per (y,x) looping over the channels, :188-200).
void oracle_zero_pad2d(const float* in, int32_t channels, int32_t height, int32_t width, int32_t top,
                       int32_t bottom, int32_t left, int32_t right, float* out) {
    const int output_height = height + top + bottom, output_width = width + left + right;
    std::memset(out, 0, sizeof(float) * (size_t)channels * output_height * output_width);
    for (int idx = 0; idx < height * width; ++idx) {
        const int height_index = idx / width, width_index = idx % width;
        const int oh = height_index + top, ow = width_index + left;
        for (int i = 0; i < channels; ++i)
            out[(size_t)i * output_height * output_width + (size_t)oh * output_width + ow] =
                in[(size_t)i * height * width + (size_t)height_index * width + width_index];
    }
}

// Whole frame, the reference's graph order (se-ssd-ai-trt.cpp:1138-1252): voxelGenerator, then per
// layer {rulebook, gather-GEMM-scatter, scale/shift/ReLU}, then sparse2Dense.
//   counts_out i32[n_layers+1]: voxel_num after the voxelizer and after every layer
//   pairs_out  i64[n_layers]  : rulebook pairs per layer (or NULL)
//   round_half != 0: every layer's output features are rounded to IEEE half after the epilogue
//   (the FP16 configs store features in half; accumulation and epilogue stay FP32)
// Returns the OR of the status masks.
int oracle_frame(const float* points, int32_t n_points, int32_t point_features,
                 const sessd_voxelgen_desc* vg, int32_t n_layers, const sessd_layer_spec* layers,
                 const float* const* weights, const float* const* scale, const float* const* shift,
                 int32_t relu, int32_t round_half, const sessd_sparse2dense_desc* dd, float* dense,
                 int32_t* counts_out, int64_t* pairs_out, float* last_feat, int32_t* last_coors) {
    const int32_t mv = vg->max_voxels;
    int status = 0;
    std::vector<float> feat((size_t)mv * 4);
    std::vector<int32_t> coors((size_t)mv * 4);
    int32_t n = 0;
    status |= oracle_voxelize(points, n_points, point_features, vg->point_cloud_range,
                              vg->voxel_size, vg->max_num_points_per_voxel, mv, feat.data(),
                              coors.data(), &n, nullptr);
    if (counts_out) counts_out[0] = n;
    std::vector<int32_t> pairs;
    std::vector<uint32_t> num(27);
    std::vector<float> out;
    std::vector<int32_t> ocoors((size_t)mv * 4);
    for (int l = 0; l < n_layers; ++l) {
        const sessd_layer_spec& L = layers[l];
        const int K = L.ksize[0] * L.ksize[1] * L.ksize[2];
        pairs.resize((size_t)K * 2 * mv);
        out.resize((size_t)mv * L.out_channel);
        if (L.type == SESSD_LAYER_SUBM) {
            status |= oracle_subm_rulebook(coors.data(), n, L.out_shape, L.ksize[0], L.stride[0],
                                           L.padding[0], 1, mv, pairs.data(), num.data());
        } else {
            int32_t m = 0;
            status |= oracle_sparse_rulebook(coors.data(), n, L.out_shape, L.ksize, L.stride,
                                             L.padding, 1, mv, pairs.data(), num.data(),
                                             ocoors.data(), &m);
            coors = ocoors;
            n = m;
        }
        if (pairs_out) {
            int64_t p = 0;
            for (int k = 0; k < K; ++k) p += num[k];
            pairs_out[l] = p;
        }
        oracle_gather_gemm_scatter(feat.data(), weights[l], pairs.data(), num.data(), K, mv,
                                   L.in_channel, L.out_channel, out.data());
        oracle_scale_shift_relu(out.data(), n, L.out_channel, scale ? scale[l] : nullptr,
                                shift ? shift[l] : nullptr, relu);
        if (round_half)
            for (size_t i = 0; i < (size_t)n * L.out_channel; ++i) out[i] = round_to_half(out[i]);
        feat.swap(out);
        if (counts_out) counts_out[l + 1] = n;
    }
    const int32_t c_last = n_layers ? layers[n_layers - 1].out_channel : 4;
    if (last_feat) std::memcpy(last_feat, feat.data(), sizeof(float) * (size_t)n * c_last);
    if (last_coors) std::memcpy(last_coors, coors.data(), sizeof(int32_t) * 4 * (size_t)n);
    if (dense) oracle_sparse2dense(feat.data(), coors.data(), n, dd->feature_map_channel,
                                   dd->feature_map_size, dense);
    return status;
}

}  // extern "C"
