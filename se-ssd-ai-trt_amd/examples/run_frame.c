/* run_frame.c -- a C host of libsessd3d: one LiDAR frame through the 3-D front end.
 *
 *     run_frame <frame.bin> <model.wts> [dense_out.bin] [repeats]
 *
 * The counterpart, for the 3-D front end, of what the reference's main() does per frame
 * (se-ssd-ai-trt.cpp:1824-1868: loadData, copy to the device, enqueue, copy back): the frame is read
 * with sessd_load_frame (KITTI velodyne layout, float32 x,y,z,intensity), the weights with
 * sessd_wts_load (the text format of tools/gen_wts.py), the backbone is the reference's 14 layers
 * (sessd_reference_backbone), and the frame runs `repeats` times through sessd_pipeline_enqueue on a
 * stream of the caller.  Prints the voxel count, the status word, the time per frame and a checksum of
 * the dense tensor; writes the tensor (float32 [128][200][176]) when a path is given.
 *
 * Plain C99 against include/sessd3d.h and the HIP runtime API; se-ssd-ai-trt_amd/build.py builds it
 * into se-ssd-ai-trt_amd/lib/run_frame. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "sessd3d.h"

#define MAX_POINTS 80000 /* params.h:30 */

static void die_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return;
    fprintf(stderr, "run_frame: %s: %s\n", what, hipGetErrorString(e));
    exit(2);
}

static void die_sessd(int rc, const char* what) {
    if (rc == SESSD_OK) return;
    fprintf(stderr, "run_frame: %s: error %d: %s\n", what, rc, sessd_last_error());
    exit(3);
}

int main(int argc, char** argv) {
    if (argc < 3) {
        fprintf(stderr, "usage: run_frame <frame.bin> <model.wts> [dense_out.bin] [repeats]\n");
        return 1;
    }
    const char* dense_path = argc > 3 && argv[3][0] ? argv[3] : NULL;
    const int repeats = argc > 4 ? atoi(argv[4]) : 1;

    /* host side: the frame and the weights */
    float* points = (float*)malloc((size_t)MAX_POINTS * 4 * sizeof(float));
    int32_t n_points = 0;
    die_sessd(sessd_load_frame(argv[1], points, MAX_POINTS, 4, &n_points), "sessd_load_frame");
    sessd_wts* wts = NULL;
    die_sessd(sessd_wts_load(argv[2], &wts), "sessd_wts_load");

    /* the reference's network (params.h), folded BatchNorm + ReLU behind every layer */
    sessd_layer_spec layers[14];
    sessd_pipeline_desc pd;
    memset(&pd, 0, sizeof pd);
    if (sessd_reference_backbone(layers, 14, &pd.voxelgen, &pd.dense) != 14) return 4;
    pd.max_points = MAX_POINTS;
    pd.point_features = 4;
    pd.n_layers = 14;
    pd.layers = layers;
    pd.feature_dtype = SESSD_FLOAT;
    pd.share_rulebooks = 1;
    pd.flags = SESSD_FLAG_SKIP_PAD_ROWS;
    pd.use_graph = 1;
    pd.overlap_streams = 1;
    sessd_pipeline* pipe = NULL;
    die_sessd(sessd_pipeline_create_from_wts(&pd, wts, NULL, NULL, 1e-5f, &pipe), "sessd_pipeline_create_from_wts");
    sessd_wts_destroy(wts);

    /* device side: the caller owns the points, the count, the dense tensor and the stream */
    const size_t dense_elems = (size_t)pd.dense.feature_map_channel * pd.dense.feature_map_size[2] *
                               pd.dense.feature_map_size[1] * pd.dense.feature_map_size[0];
    void *d_points = NULL, *d_size = NULL, *d_dense = NULL;
    hipStream_t stream;
    hipEvent_t t0, t1;
    die_hip(hipMalloc(&d_points, (size_t)MAX_POINTS * 4 * sizeof(float)), "hipMalloc");
    die_hip(hipMalloc(&d_size, sizeof(int32_t)), "hipMalloc");
    die_hip(hipMalloc(&d_dense, dense_elems * sizeof(float)), "hipMalloc");
    die_hip(hipStreamCreate(&stream), "hipStreamCreate");
    die_hip(hipEventCreate(&t0), "hipEventCreate");
    die_hip(hipEventCreate(&t1), "hipEventCreate");
    die_hip(hipMemcpyAsync(d_points, points, (size_t)MAX_POINTS * 4 * sizeof(float), hipMemcpyHostToDevice, stream), "copy");
    die_hip(hipMemcpyAsync(d_size, &n_points, sizeof n_points, hipMemcpyHostToDevice, stream), "copy");

    die_sessd(sessd_pipeline_enqueue(pipe, d_points, d_size, d_dense, stream), "sessd_pipeline_enqueue");
    die_hip(hipEventRecord(t0, stream), "hipEventRecord");
    for (int r = 1; r < repeats; ++r)
        die_sessd(sessd_pipeline_enqueue(pipe, d_points, d_size, d_dense, stream), "sessd_pipeline_enqueue");
    die_hip(hipEventRecord(t1, stream), "hipEventRecord");
    die_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    float ms = 0.f;
    if (repeats > 1) die_hip(hipEventElapsedTime(&ms, t0, t1), "hipEventElapsedTime");

    int32_t status = 0, n_voxels = 0;
    void* d_voxel_num = NULL;
    die_sessd(sessd_pipeline_status(pipe, stream, &status), "sessd_pipeline_status");
    die_sessd(sessd_pipeline_layer_io(pipe, -1, NULL, NULL, &d_voxel_num, NULL, NULL), "sessd_pipeline_layer_io");
    die_hip(hipMemcpy(&n_voxels, d_voxel_num, sizeof n_voxels, hipMemcpyDeviceToHost), "copy");

    float* dense = (float*)malloc(dense_elems * sizeof(float));
    die_hip(hipMemcpy(dense, d_dense, dense_elems * sizeof(float), hipMemcpyDeviceToHost), "copy");
    double sum = 0.0;
    size_t nonzero = 0;
    for (size_t i = 0; i < dense_elems; ++i) {
        sum += dense[i];
        nonzero += dense[i] != 0.f;
    }
    printf("points %d voxels %d status %d dense_sum %.6f dense_nonzero %zu", n_points, n_voxels, status, sum, nonzero);
    if (repeats > 1) printf(" ms_per_frame %.4f", ms / (repeats - 1));
    printf("\n");
    if (dense_path) {
        FILE* f = fopen(dense_path, "wb");
        if (!f || fwrite(dense, sizeof(float), dense_elems, f) != dense_elems) {
            fprintf(stderr, "run_frame: cannot write %s\n", dense_path);
            return 5;
        }
        fclose(f);
    }

    sessd_pipeline_destroy(pipe);
    hipEventDestroy(t0);
    hipEventDestroy(t1);
    hipStreamDestroy(stream);
    hipFree(d_points);
    hipFree(d_size);
    hipFree(d_dense);
    free(points);
    free(dense);
    return 0;
}
