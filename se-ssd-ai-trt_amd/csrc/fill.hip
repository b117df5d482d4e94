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

// One launch clears up to FillArgs::kMaxRegions regions: blockIdx.y picks the region, blockIdx.x strides over it with
// 16-byte stores (pure write stream, HBM-bound).
__global__ void __launch_bounds__(256) fill_kernel(FillArgs a) {
    const FillRegion r = a.r[blockIdx.y];
    const uint64_t vec = r.words / 4;
    uint4* p4 = reinterpret_cast<uint4*>(r.ptr);
    const uint4 v4 = make_uint4(r.value, r.value, r.value, r.value);
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < vec; i += stride) p4[i] = v4;
    if (blockIdx.x == 0 && threadIdx.x < (r.words & 3)) r.ptr[vec * 4 + threadIdx.x] = r.value;
}

int launch_fill(const FillArgs& a, hipStream_t stream) {
    if (a.n == 0) return SESSD_OK;
    uint64_t max_vec = 1;
    for (int i = 0; i < a.n; ++i) {
        if (reinterpret_cast<uintptr_t>(a.r[i].ptr) & 15)
            return fail(SESSD_E_INVALID, "fill: region %d is not 16-byte aligned", i);
        if (a.r[i].words / 4 > max_vec) max_vec = a.r[i].words / 4;
    }
    // 4 stores of 16 B per thread is enough to saturate HBM; cap the grid at 8 blocks per CU
    uint64_t blocks = (max_vec + 256 * 4 - 1) / (256 * 4);
    if (blocks > 2048) blocks = 2048;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks, a.n), dim3(256), 0, stream, a);
    SESSD_HIP_TRY(hipGetLastError());
    return SESSD_OK;
}

}  // namespace sessd
