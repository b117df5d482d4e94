// frame_io.hip -- host side only: reading one LiDAR frame file into a points buffer.
//
// Replaces loadData (se-ssd-ai-trt.cpp:1515-1559) and the size arithmetic of its caller (:1849-1850):
// a KITTI velodyne `.bin` is a headerless array of float32 (x, y, z, intensity); the number of points is
// bytes / 4 / sizeof(float), integer division, so trailing bytes that do not fill a point are ignored.
// A file larger than the buffer is an error code here (the reference prints and exits).
#include <cerrno>
#include <cstdio>
#include <cstring>

#include "common.h"

using namespace sessd;

extern "C" int sessd_load_frame(const char* path, float* points, int32_t max_points, int32_t point_features,
                                int32_t* points_size) {
    if (!path || !points || !points_size || max_points < 0 || point_features <= 0)
        return fail(SESSD_E_INVALID, "load_frame: bad argument");
    FILE* f = std::fopen(path, "rb");
    if (!f) return fail(SESSD_E_INVALID, "load_frame: cannot open '%s': %s", path, std::strerror(errno));
    if (std::fseek(f, 0, SEEK_END) != 0) {
        std::fclose(f);
        return fail(SESSD_E_INVALID, "load_frame: cannot seek in '%s'", path);
    }
    const long len = std::ftell(f);
    std::rewind(f);
    const size_t point_bytes = sizeof(float) * (size_t)point_features;
    if (len < 0 || (size_t)len > (size_t)max_points * point_bytes) {
        std::fclose(f);
        return fail(SESSD_E_INVALID, "load_frame: '%s' holds %ld bytes, the points buffer %zu", path, len,
                    (size_t)max_points * point_bytes);
    }
    const size_t n = (size_t)len / point_bytes;
    const size_t got = std::fread(points, point_bytes, n, f);
    std::fclose(f);
    if (got != n) return fail(SESSD_E_INVALID, "load_frame: short read on '%s'", path);
    // rows past the last point are never read by the voxelizer (it gates on points_size); zero them so the
    // buffer is fully defined, as the reference's zero-initialised staging buffer intends
    std::memset(points + n * (size_t)point_features, 0, ((size_t)max_points - n) * point_bytes);
    *points_size = (int32_t)n;
    return SESSD_OK;
}
