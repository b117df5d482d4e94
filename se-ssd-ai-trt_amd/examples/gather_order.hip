// gather_order.hip -- measures what the order of a wave's 16-byte row requests costs on gfx950.
//
// A gather-GEMM wave asks for 16 rows of 256 bytes (64 FP32 channels) in four requests of 16 bytes per lane.  The
// MFMA wants the data in operand order -- lane l holds pair l % 16, bytes 16 * (l / 16) of each 64-byte chunk --
// but a request issued in that order has four neighbouring lanes on four different rows.  The other order puts
// four neighbouring lanes on the 64 contiguous bytes of one row (lane l: pair l / 4, bytes 16 * (l % 4)); the data
// then needs a lane permutation before the MFMA.  This program times both orders over rows drawn like the
// neighbours of a tile (48 consecutive candidates per block of 16) at 4, 8 and 16 waves per compute unit and prints
// the bytes per cycle and compute unit each reaches.  conv_wide.hip requests in the second order because of it.
//
//   hipcc --offload-arch=gfx950 -O3 gather_order.hip -o gather_order && ./gather_order
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(expr)                                                                              \
    do {                                                                                         \
        hipError_t e_ = (expr);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            return 1;                                                                            \
        }                                                                                        \
    } while (0)

typedef unsigned int v4u32 __attribute__((__vector_size__(16)));

constexpr int kRowBytes = 256;

template <int ORDER>
__global__ void __launch_bounds__(256) gather(const float* in, unsigned in_bytes, const int* rows, int n_blocks, float* out, int iters) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(in), 0, (int)in_bytes, 0x00020000);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    int blk = (blockIdx.x * 4 + wave) % n_blocks;
    for (int it = 0; it < iters; ++it) {
        const int pair = ORDER == 0 ? (lane & 15) : (lane >> 2);   // operand order : contiguous order
        const int part = ORDER == 0 ? (lane >> 4) : (lane & 3);
        const unsigned at = (unsigned)(rows[blk * 16 + pair] * kRowBytes + part * 16);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4u32 v = __builtin_amdgcn_raw_buffer_load_b128(rs, at + g * 64, 0, 0);
            const float4 f = *reinterpret_cast<const float4*>(&v);
            acc.x += f.x;
            acc.y += f.y;
            acc.z += f.z;
            acc.w += f.w;
        }
        blk = (blk + 97) % n_blocks;
    }
    if (acc.x == 12345.f) out[0] = acc.y + acc.z + acc.w;  // (keeps the loads alive; the input is all zeros)
}

int main() {
    const int n_rows = 16914, n_blocks = 4096, iters = 200, num_cu = 256;
    float *in = nullptr, *out = nullptr;
    int* rows = nullptr;
    CHECK(hipMalloc(reinterpret_cast<void**>(&in), (size_t)n_rows * kRowBytes));
    CHECK(hipMemset(in, 0, (size_t)n_rows * kRowBytes));
    CHECK(hipMalloc(reinterpret_cast<void**>(&out), 64));
    std::vector<int> h((size_t)n_blocks * 16);
    std::srand(1);
    for (int b = 0; b < n_blocks; ++b) {
        const int base = std::rand() % (n_rows - 64);
        for (int i = 0; i < 16; ++i) h[(size_t)b * 16 + i] = base + std::rand() % 48;   // always inside the buffer
    }
    CHECK(hipMalloc(reinterpret_cast<void**>(&rows), h.size() * sizeof(int)));
    CHECK(hipMemcpy(rows, h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int blocks : {256, 512, 1024}) {
        for (int order = 0; order < 2; ++order) {
            float best = 1e9f;
            for (int rep = 0; rep < 5; ++rep) {
                CHECK(hipEventRecord(e0));
                if (order == 0)
                    hipLaunchKernelGGL(gather<0>, dim3(blocks), dim3(256), 0, 0, in, (unsigned)(n_rows * kRowBytes), rows, n_blocks, out, iters);
                else
                    hipLaunchKernelGGL(gather<1>, dim3(blocks), dim3(256), 0, 0, in, (unsigned)(n_rows * kRowBytes), rows, n_blocks, out, iters);
                CHECK(hipGetLastError());
                CHECK(hipEventRecord(e1));
                CHECK(hipEventSynchronize(e1));
                float ms = 0.f;
                CHECK(hipEventElapsedTime(&ms, e0, e1));
                if (ms < best) best = ms;
            }
            const double bytes = (double)blocks * 4 * iters * 4 * 1024;
            std::printf("%2d waves per compute unit, %s order: %.3f ms, %.2f TB/s, %.1f bytes per cycle and compute unit (2.1 GHz)\n",
                        blocks * 4 / num_cu, order == 0 ? "operand   " : "contiguous", best, bytes / best / 1e9,
                        bytes / (best * 1e-3) / num_cu / 2.1e9);
        }
    }
    return 0;
}
