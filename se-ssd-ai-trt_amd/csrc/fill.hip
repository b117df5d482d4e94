// fill.hip -- multi-region fill kernel and the library's error bookkeeping.
#include <cstdarg>

#include "common.h"

namespace sessd {

namespace {
thread_local std::string g_last_error;
}

void set_last_error(const std::string& msg) { g_last_error = msg; }

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

const char* last_error_cstr() { return g_last_error.c_str(); }

// One launch clears up to FillArgs::kMaxRegions regions.  The grid is flat: region i owns the blocks
// [first_block[i], first_block[i+1]), as many as its size asks for (a small region gets one block, not the grid of
// the largest one), and its blocks stride over it with 16-byte stores (pure write stream, HBM-bound).
struct FillPlan {
    FillArgs a;
    uint32_t first_block[FillArgs::kMaxRegions + 1];
};

__global__ void __launch_bounds__(256) fill_kernel(FillPlan p) {
    int i = 0;
    while (i + 1 < p.a.n && blockIdx.x >= p.first_block[i + 1]) ++i;  // (uniform: scalar loads of the arguments)
    const FillRegion r = p.a.r[i];
    const uint32_t blocks = p.first_block[i + 1] - p.first_block[i];
    const uint32_t local = blockIdx.x - p.first_block[i];
    const uint64_t vec = r.words / 4;
    uint4* p4 = reinterpret_cast<uint4*>(r.ptr);
    const uint4 v4 = make_uint4(r.value, r.value, r.value, r.value);
    const uint64_t stride = (uint64_t)blocks * blockDim.x;
    for (uint64_t j = (uint64_t)local * blockDim.x + threadIdx.x; j < vec; j += stride) p4[j] = v4;
    if (local == 0 && threadIdx.x < (r.words & 3)) r.ptr[vec * 4 + threadIdx.x] = r.value;
}

int launch_fill(const FillArgs& a, hipStream_t stream) {
    if (a.n == 0) return SESSD_OK;
    FillPlan p;
    p.a = a;
    uint32_t total = 0;
    for (int i = 0; i < a.n; ++i) {
        if (reinterpret_cast<uintptr_t>(a.r[i].ptr) & 15)
            return fail(SESSD_E_INVALID, "fill: region %d is not 16-byte aligned", i);
        // 4 stores of 16 B per thread is enough to saturate HBM; at most 8 blocks per CU for one region
        uint64_t blocks = (a.r[i].words / 4 + 256 * 4 - 1) / (256 * 4);
        if (blocks > 2048) blocks = 2048;
        if (blocks < 1) blocks = 1;
        p.first_block[i] = total;
        total += (uint32_t)blocks;
    }
    for (int i = a.n; i <= FillArgs::kMaxRegions; ++i) p.first_block[i] = total;
    hipLaunchKernelGGL(fill_kernel, dim3(total), dim3(256), 0, stream, p);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
