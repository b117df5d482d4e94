/*
 * sessd3d.h -- C-ABI of the MI355X (gfx950) implementation of the SE-SSD 3-D front end:
 * voxelGenerator, SubmConv3dLayer, SparseConv3dLayer and sparse2Dense.
 *
 * One set of entry points per layer type.  Each set mirrors the life cycle TensorRT drives on
 * the reference's IPluginV2DynamicExt plugins:
 *
 *     create(fields, weights) | deserialize(bytes)          ctor / PluginCreator
 *     configure(inDescs, outDescs)                          configurePlugin
 *     workspace_size(inDescs, outDescs)                     getWorkspaceSize
 *     enqueue(inDesc, outDesc, inputs, outputs, ws, stream) enqueue
 *     serialization_size / serialize                        getSerializationSize / serialize
 *     destroy                                               terminate + destroy
 *
 * Tensor contract (same as the reference): every tensor is linear, batch dimension 1, device
 * memory owned by the caller; `voxel_num` / `points_size` are int32 scalars in DEVICE memory and
 * are only read inside kernels.  enqueue only enqueues work on `stream` (a hipStream_t); it never
 * synchronises, allocates or frees.  Outputs and workspace are (re)initialised inside every
 * enqueue.  Return value 0 = success, anything else is a SESSD_E_* code (the reference aborts).
 *
 * All plain C: no HIP, torch or C++ types appear in any signature.
 */
#ifndef SESSD3D_H_
#define SESSD3D_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------ */
/* common types                                                                               */
/* ------------------------------------------------------------------------------------------ */

typedef void* sessd_stream_t; /* a hipStream_t; NULL = the default stream */
/* For sessd_pipeline_submit only: "the inputs are ready now, order this frame after no stream" (the caller has
 * synchronised, or the inputs have long been resident).  Without it the frame waits for a marker on the
 * caller's stream, and where that stream shares a hardware queue with one of the pipeline's own, the marker
 * sits behind that queue's kernels. */
#define SESSD_STREAM_NONE ((sessd_stream_t)(intptr_t)-1)

/* Values follow nvinfer1::DataType so descriptors can be copied field by field. */
enum { SESSD_FLOAT = 0, SESSD_HALF = 1, SESSD_INT32 = 3 };

/* Mirrors nvinfer1::PluginTensorDesc {Dims dims; DataType type; TensorFormat format; float scale;}
 * (format is always 0 = kLINEAR here). */
typedef struct sessd_tensor_desc {
    int32_t nbDims;
    int32_t d[8];
    int32_t type;
    int32_t format;
    float scale;
} sessd_tensor_desc;

enum {
    SESSD_OK = 0,
    SESSD_E_INVALID = 1,     /* bad argument / descriptor mismatch */
    SESSD_E_UNSUPPORTED = 2, /* dtype or shape the kernels do not cover */
    SESSD_E_HIP = 3,         /* a HIP runtime call failed; see sessd_last_error() */
    SESSD_E_NOMEM = 4
};

/* Bits of the device-side status word (kept in the last 256-byte block of a layer's workspace and
 * cleared by every enqueue), read back by *_status(). */
enum {
    SESSD_STATUS_VOXEL_OVERFLOW = 1, /* more active sites than max_voxels; the excess was dropped  */
    SESSD_STATUS_HASH_FULL = 2,      /* hash table could not place a key (cannot happen when sized
                                        by workspace_size; reported instead of spinning)          */
    SESSD_STATUS_BAD_COORD = 4       /* an input coordinate was outside the layer's grid          */
};

/* Behaviour flags set with *_set_flags(); 0 = behave exactly like the reference plugin. */
enum {
    /* Do not write feature rows >= voxel_num.  The reference zero-fills every output up to
     * max_voxels rows; consumers gate on voxel_num, so a fused pipeline can skip that traffic. */
    SESSD_FLAG_SKIP_PAD_ROWS = 1,
    /* Run the gather-GEMM on the shape-agnostic VALU kernel even where an MFMA kernel exists
     * (cross-check of the matrix-core path). */
    SESSD_FLAG_FORCE_VALU = 2
};

const char* sessd_last_error(void); /* thread-local text of the last failure */
/* Copy `bytes` from device memory to host memory on `stream` and wait for it: lets a host that has
 * no HIP binding of its own read back tensors the library owns (see sessd_pipeline_layer_io). */
int sessd_copy_to_host(void* dst_host, const void* src_device, size_t bytes, sessd_stream_t stream);
const char* sessd_version(void);

/* ------------------------------------------------------------------------------------------ */
/* VoxelGeneratorPlugin   (reference: voxelGenerator.h:15-77, voxelGenerator.cu:105-616)       */
/* ------------------------------------------------------------------------------------------ */
/* inputs : 0 points f32[1,max_points,point_features]   1 points_size i32[1]
 * outputs: 0 voxels f32[1,max_voxels,4] (mean x,y,z,i) 1 coors i32[1,max_voxels,4] (b,z,y,x)
 *          2 voxel_num i32[1]
 * Voxel ids follow first appearance in point order, the first max_num_points_per_voxel points of
 * a cell (by point index) are averaged, new cells beyond max_voxels are dropped. */

typedef struct sessd_voxelgen sessd_voxelgen;

/* Field names = the PluginFields the reference creator accepts (voxelGenerator.cu:624-628). */
typedef struct sessd_voxelgen_desc {
    int32_t max_num_points_per_voxel;
    int32_t max_voxels;
    float point_cloud_range[6]; /* xmin,ymin,zmin,xmax,ymax,zmax */
    int32_t voxel_feature_num;
    float voxel_size[3]; /* x,y,z */
} sessd_voxelgen_desc;

/* replaces VoxelGeneratorPluginCreator::createPlugin (voxelGenerator.cu:649-701) */
int sessd_voxelgen_create(const sessd_voxelgen_desc* desc, sessd_voxelgen** out);
/* replaces VoxelGeneratorPlugin(const void*, size_t) (voxelGenerator.cu:131-150) */
int sessd_voxelgen_deserialize(const void* bytes, size_t n, sessd_voxelgen** out);
/* replaces getSerializationSize / serialize (voxelGenerator.cu:576-600): 7 int32 + 9 float */
size_t sessd_voxelgen_serialization_size(const sessd_voxelgen* h);
int sessd_voxelgen_serialize(const sessd_voxelgen* h, void* buf);
/* replaces configurePlugin (voxelGenerator.cu:228-235): point feature count + grid dims */
int sessd_voxelgen_configure(sessd_voxelgen* h, const sessd_tensor_desc* in, int nIn,
                             const sessd_tensor_desc* out, int nOut);
/* grid dims derived by configure, (x,y,z); for tests and for sizing downstream layers */
int sessd_voxelgen_grid_size(const sessd_voxelgen* h, int32_t grid_xyz[3]);
/* replaces getWorkspaceSize (voxelGenerator.cu:237-252) */
size_t sessd_voxelgen_workspace_size(const sessd_voxelgen* h, const sessd_tensor_desc* in, int nIn,
                                     const sessd_tensor_desc* out, int nOut);
/* replaces enqueue (voxelGenerator.cu:480-542) */
int sessd_voxelgen_enqueue(sessd_voxelgen* h, const sessd_tensor_desc* inDesc,
                           const sessd_tensor_desc* outDesc, const void* const* inputs,
                           void* const* outputs, void* workspace, sessd_stream_t stream);
/* No counterpart in the reference.  For callers that cannot allocate device memory or hand over a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * sessd_voxelgen_enqueue without the workspace argument.  The scratch memory is a static device array
 * inside the library, 8 MiB on every GPU the library runs on, held until the process ends; that is
 * enough for the reference's shape (80000-row points tensor, 5 points per voxel: 7.7 MB) and a request
 * that needs more is rejected with SESSD_E_INVALID before anything is launched.  The call allocates and
 * frees nothing; its first use on a device looks the array's address up (make that call outside a
 * stream capture).  All calls on one GPU share the array: it is cleared by each call, and two calls that
 * overlap in time on one GPU (different streams, different handles) race.  Outputs are bit-identical
 * to sessd_voxelgen_enqueue's. */
int sessd_voxelgen_enqueue_static(sessd_voxelgen* h, const sessd_tensor_desc* inDesc,
                                  const sessd_tensor_desc* outDesc, const void* const* inputs,
                                  void* const* outputs, sessd_stream_t stream);
/* workspace NULL = the static scratch of sessd_voxelgen_enqueue_static on the current device */
int sessd_voxelgen_status(const sessd_voxelgen* h, const void* workspace, sessd_stream_t stream,
                          int32_t* status);
int sessd_voxelgen_set_flags(sessd_voxelgen* h, int32_t flags);
/* replaces terminate + destroy (voxelGenerator.cu:572-605) */
void sessd_voxelgen_destroy(sessd_voxelgen* h);

/* ------------------------------------------------------------------------------------------ */
/* SubmConv3dLayerPlugin  (reference: submConv3dlayer.h:19-92, submConv3dlayer.cu:126-730)     */
/* ------------------------------------------------------------------------------------------ */
/* inputs : 0 feat [1,max_voxels,Cin] f32|f16   1 coors i32[1,max_voxels,4]   2 voxel_num i32[1]
 * outputs: 0 feat [1,max_voxels,Cout] f32|f16
 * out[o] = sum_k W[k]^T in[nbr(o,k)], weights FP32 [K][Cin][Cout] (K = ksize^3, offset index
 * kz*9+ky*3+kx), no bias; optional fused y = max(0, x*scale[c]+shift[c]) epilogue. */

typedef struct sessd_submconv3d sessd_submconv3d;

/* Field names = submConv3dlayer.cu:737-748; 3-vectors are (x,y,z) as at every call site. */
typedef struct sessd_submconv3d_desc {
    int32_t in_channel;
    int32_t out_channel;
    int32_t max_voxels;
    int32_t feature_num;
    int32_t out_shape[3];     /* x,y,z */
    int32_t spatial_shape[3]; /* x,y,z (carried, unused -- as in the reference) */
    int32_t ksize;
    int32_t stride;
    int32_t padding;
    int32_t dilation;
    int32_t out_padding;
} sessd_submconv3d_desc;

/* replaces SubmConv3dLayerPluginCreator::createPlugin (submConv3dlayer.cu:770-850) and the
 * weight-uploading ctor (submConv3dlayer.cu:126-152).  `weights`: host FP32 [K][Cin][Cout]. */
int sessd_submconv3d_create(const sessd_submconv3d_desc* desc, const float* weights,
                            sessd_submconv3d** out);
/* replaces SubmConv3dLayerPlugin(const void*, size_t) (submConv3dlayer.cu:154-186) + clone() */
int sessd_submconv3d_deserialize(const void* bytes, size_t n, sessd_submconv3d** out);
/* replaces getSerializationSize / serialize (submConv3dlayer.cu:684-714): 16 int32 + weights */
size_t sessd_submconv3d_serialization_size(const sessd_submconv3d* h);
int sessd_submconv3d_serialize(const sessd_submconv3d* h, void* buf);
/* replaces configurePlugin (submConv3dlayer.cu:242-245); records the feature dtypes */
int sessd_submconv3d_configure(sessd_submconv3d* h, const sessd_tensor_desc* in, int nIn,
                               const sessd_tensor_desc* out, int nOut);
/* replaces getWorkspaceSize (submConv3dlayer.cu:247-267) */
size_t sessd_submconv3d_workspace_size(const sessd_submconv3d* h, const sessd_tensor_desc* in,
                                       int nIn, const sessd_tensor_desc* out, int nOut);
/* replaces enqueue (submConv3dlayer.cu:539-641) */
int sessd_submconv3d_enqueue(sessd_submconv3d* h, const sessd_tensor_desc* inDesc,
                             const sessd_tensor_desc* outDesc, const void* const* inputs,
                             void* const* outputs, void* workspace, sessd_stream_t stream);
/* No counterpart in the reference (it rebuilds the rulebook in every layer although consecutive
 * SubM layers share one coors tensor, se-ssd-ai-trt.cpp:1147-1239): run the layer on the rulebook
 * a previous sessd_submconv3d_enqueue left in `rulebook_workspace` (same coors, same max_voxels,
 * same out_shape).  Only the gather-GEMM kernel is launched. */
int sessd_submconv3d_enqueue_shared(sessd_submconv3d* h, const sessd_tensor_desc* inDesc,
                                    const sessd_tensor_desc* outDesc, const void* const* inputs,
                                    void* const* outputs, const void* rulebook_workspace,
                                    sessd_stream_t stream);
/* Materialise the rulebook of the last enqueue on `workspace` in the reference's layout
 * (submConv3dlayer.cu:254-255, 413-419): indice_pairs i32[K][2][max_voxels] ([k][0]=input row,
 * [k][1]=output row, unused entries -1), indice_num u32[K].  Within one offset the pairs are in
 * ascending output-row order (the reference's order is atomics-dependent).  Device pointers. */
int sessd_submconv3d_export_rulebook(const sessd_submconv3d* h, const void* workspace,
                                     int32_t* indice_pairs, uint32_t* indice_num,
                                     sessd_stream_t stream);
/* Fused BatchNorm1d+ReLU epilogue replacing the IScaleLayer + kRELU pair the reference inserts
 * after every conv (se-ssd-ai-trt.cpp:808-856).  scale/shift: host FP32 [Cout]; NULL = none. */
int sessd_submconv3d_set_epilogue(sessd_submconv3d* h, const float* scale, const float* shift,
                                  int relu);
int sessd_submconv3d_set_flags(sessd_submconv3d* h, int32_t flags);
int sessd_submconv3d_status(const sessd_submconv3d* h, const void* workspace,
                            sessd_stream_t stream, int32_t* status);
/* replaces terminate + destroy (submConv3dlayer.cu:671-682, 716-719) */
void sessd_submconv3d_destroy(sessd_submconv3d* h);

/* ------------------------------------------------------------------------------------------ */
/* SparseConv3dLayerPlugin (reference: sparseConv3dlayer.h:19-97, sparseConv3dlayer.cu:137-915) */
/* ------------------------------------------------------------------------------------------ */
/* inputs : as SubmConv3d.
 * outputs: 0 feat [1,max_voxels,Cout]   1 coors i32[1,max_voxels,4]   2 voxel_num i32[1]
 * Output sites are numbered in first-seen order over (input row ascending, candidate order of
 * getValidOutPos), i.e. the order of the author's host restatement sparseConv3dlayer.cu:738-757;
 * sites beyond max_voxels are dropped and SESSD_STATUS_VOXEL_OVERFLOW is raised. */

typedef struct sessd_sparseconv3d sessd_sparseconv3d;

/* Field names = sparseConv3dlayer.cu:923-934; shapes (x,y,z), ksize/stride/padding (z,y,x). */
typedef struct sessd_sparseconv3d_desc {
    int32_t in_channel;
    int32_t out_channel;
    int32_t max_voxels;
    int32_t feature_num;
    int32_t out_shape[3];     /* x,y,z */
    int32_t spatial_shape[3]; /* x,y,z */
    int32_t ksize[3];         /* z,y,x */
    int32_t stride[3];        /* z,y,x */
    int32_t padding[3];       /* z,y,x */
    int32_t dilation;
    int32_t out_padding;
} sessd_sparseconv3d_desc;

/* replaces SparseConv3dLayerPluginCreator::createPlugin (sparseConv3dlayer.cu:956-1079) + ctor
 * (sparseConv3dlayer.cu:137-163) */
int sessd_sparseconv3d_create(const sessd_sparseconv3d_desc* desc, const float* weights,
                              sessd_sparseconv3d** out);
/* replaces SparseConv3dLayerPlugin(const void*, size_t) (sparseConv3dlayer.cu:165-202) */
int sessd_sparseconv3d_deserialize(const void* bytes, size_t n, sessd_sparseconv3d** out);
/* replaces getSerializationSize / serialize (sparseConv3dlayer.cu:863-899): 22 int32 + weights */
size_t sessd_sparseconv3d_serialization_size(const sessd_sparseconv3d* h);
int sessd_sparseconv3d_serialize(const sessd_sparseconv3d* h, void* buf);
/* replaces configurePlugin (sparseConv3dlayer.cu:281-284) */
int sessd_sparseconv3d_configure(sessd_sparseconv3d* h, const sessd_tensor_desc* in, int nIn,
                                 const sessd_tensor_desc* out, int nOut);
/* replaces getWorkspaceSize (sparseConv3dlayer.cu:286-306) */
size_t sessd_sparseconv3d_workspace_size(const sessd_sparseconv3d* h, const sessd_tensor_desc* in,
                                         int nIn, const sessd_tensor_desc* out, int nOut);
/* replaces enqueue (sparseConv3dlayer.cu:606-813) */
int sessd_sparseconv3d_enqueue(sessd_sparseconv3d* h, const sessd_tensor_desc* inDesc,
                               const sessd_tensor_desc* outDesc, const void* const* inputs,
                               void* const* outputs, void* workspace, sessd_stream_t stream);
/* As sessd_submconv3d_export_rulebook; K = ksize[0]*ksize[1]*ksize[2]
 * (layout sparseConv3dlayer.cu:627-628, 444-451). */
int sessd_sparseconv3d_export_rulebook(const sessd_sparseconv3d* h, const void* workspace,
                                       int32_t* indice_pairs, uint32_t* indice_num,
                                       sessd_stream_t stream);
int sessd_sparseconv3d_set_epilogue(sessd_sparseconv3d* h, const float* scale, const float* shift,
                                    int relu);
int sessd_sparseconv3d_set_flags(sessd_sparseconv3d* h, int32_t flags);
int sessd_sparseconv3d_status(const sessd_sparseconv3d* h, const void* workspace,
                              sessd_stream_t stream, int32_t* status);
/* replaces terminate + destroy (sparseConv3dlayer.cu:845-861, 901-904) */
void sessd_sparseconv3d_destroy(sessd_sparseconv3d* h);

/* ------------------------------------------------------------------------------------------ */
/* Sparse2DensePlugin     (reference: sparse2Dense.h:15-60, sparse2Dense.cu:105-300)           */
/* ------------------------------------------------------------------------------------------ */
/* inputs : 0 feat [1,max_voxels,C] f32|f16   1 coors i32[1,max_voxels,4]   2 voxel_num i32[1]
 * outputs: 0 dense [1, C*D, H, W], dense[(c*D+z)][y][x] = feat[v][c]; every other cell 0. */

typedef struct sessd_sparse2dense sessd_sparse2dense;

/* Field names = sparse2Dense.cu:321-322. */
typedef struct sessd_sparse2dense_desc {
    int32_t feature_map_size[3]; /* x,y,z  (W,H,D) */
    int32_t feature_map_channel;
} sessd_sparse2dense_desc;

/* replaces Sparse2DensePluginCreator::createPlugin (sparse2Dense.cu:343-373) */
int sessd_sparse2dense_create(const sessd_sparse2dense_desc* desc, sessd_sparse2dense** out);
/* replaces Sparse2DensePlugin(const void*, size_t) (sparse2Dense.cu:111-118) */
int sessd_sparse2dense_deserialize(const void* bytes, size_t n, sessd_sparse2dense** out);
/* replaces getSerializationSize / serialize (sparse2Dense.cu:283-295): 4 int32 */
size_t sessd_sparse2dense_serialization_size(const sessd_sparse2dense* h);
int sessd_sparse2dense_serialize(const sessd_sparse2dense* h, void* buf);
/* replaces configurePlugin (sparse2Dense.cu:170-173) */
int sessd_sparse2dense_configure(sessd_sparse2dense* h, const sessd_tensor_desc* in, int nIn,
                                 const sessd_tensor_desc* out, int nOut);
/* replaces getWorkspaceSize (sparse2Dense.cu:175-179: the reference needs none); here the status word, one word per
 * 256 rows and a cell -> row map of D*H*W ints (282 KB for 2 x 200 x 176) */
size_t sessd_sparse2dense_workspace_size(const sessd_sparse2dense* h, const sessd_tensor_desc* in,
                                         int nIn, const sessd_tensor_desc* out, int nOut);
/* replaces enqueue (sparse2Dense.cu:224-249).  The workspace is required (SESSD_E_INVALID when NULL); its contents
 * need not be cleared or kept between calls.  Every element of the output is written, zeros included. */
int sessd_sparse2dense_enqueue(sessd_sparse2dense* h, const sessd_tensor_desc* inDesc,
                               const sessd_tensor_desc* outDesc, const void* const* inputs,
                               void* const* outputs, void* workspace, sessd_stream_t stream);
/* Folds the reference's ZeroPad2dPlugin (zeroPad2d.cu:183-244; creator field zero_padding_2d_size =
 * top, bottom, left, right, zeroPad2d.cu:311, se-ssd-ai-trt.cpp:615-619), which the reference runs
 * right after sparse2Dense (se-ssd-ai-trt.cpp:1253), into this plugin: the output becomes
 * [1, C*D, H + top + bottom, W + left + right] with a zero border and the unpadded tensor is never
 * written.  Call before configure.  All zeros (the default) = the reference's Sparse2DensePlugin. */
int sessd_sparse2dense_set_padding(sessd_sparse2dense* h, int32_t top, int32_t bottom, int32_t left,
                                   int32_t right);
/* replaces destroy (sparse2Dense.cu:297-300) */
void sessd_sparse2dense_destroy(sessd_sparse2dense* h);

/* ------------------------------------------------------------------------------------------ */
/* Creators by name and clone()  (reference: the four XxxPluginCreator classes and               */
/* IPluginV2DynamicExt::clone, e.g. submConv3dlayer.cu:732-878, 188-196)                         */
/* ------------------------------------------------------------------------------------------ */
/* Values follow nvinfer1::PluginFieldType. */
enum {
    SESSD_FIELD_FLOAT16 = 0, SESSD_FIELD_FLOAT32 = 1, SESSD_FIELD_FLOAT64 = 2, SESSD_FIELD_INT8 = 3,
    SESSD_FIELD_INT16 = 4, SESSD_FIELD_INT32 = 5, SESSD_FIELD_CHAR = 6, SESSD_FIELD_DIMS = 7,
    SESSD_FIELD_UNKNOWN = 8
};
/* Mirrors nvinfer1::PluginField {name, data, type, length} and PluginFieldCollection {nbFields, fields}. */
typedef struct sessd_plugin_field {
    const char* name;
    const void* data;
    int32_t type;   /* SESSD_FIELD_* */
    int32_t length; /* elements behind `data` */
} sessd_plugin_field;
typedef struct sessd_plugin_field_collection {
    int32_t nbFields;
    const sessd_plugin_field* fields;
} sessd_plugin_field_collection;
/* replaces XxxPluginCreator::getFieldNames (voxelGenerator.cu:618-647, submConv3dlayer.cu:732-768,
 * sparseConv3dlayer.cu:918-954, sparse2Dense.cu:316-341): the fields createPlugin reads, `data` NULL,
 * `length` = the number of elements it reads (0 for weights: the layer shape decides).  plugin_name is the
 * reference's PLUGIN_NAME: "VoxelGeneratorPlugin", "SubmConv3dLayerPlugin", "SparseConv3dLayerPlugin",
 * "Sparse2DensePlugin".  NULL for any other name. */
const sessd_plugin_field_collection* sessd_plugin_field_names(const char* plugin_name);
/* replaces XxxPluginCreator::createPlugin(name, fc) (voxelGenerator.cu:649-701, submConv3dlayer.cu:770-878,
 * sparseConv3dlayer.cu:956-1079, sparse2Dense.cu:343-373): fields are picked by name, in any order, unknown
 * names are ignored; a missing field or a field of the wrong type is an error (the reference builds the
 * plugin from zeros).  Array fields may carry length 1, as the reference's own creators declare them.
 * *handle is a sessd_voxelgen* / sessd_submconv3d* / sessd_sparseconv3d* / sessd_sparse2dense*. */
int sessd_plugin_create(const char* plugin_name, const sessd_plugin_field_collection* fc, void** handle);
/* replace clone() (voxelGenerator.cu:152-159, submConv3dlayer.cu:188-196, sparseConv3dlayer.cu:204-210,
 * sparse2Dense.cu:120-125): an independent plugin with its own device copy of the weights, plus what this
 * library adds to a plugin (epilogue, flags, configured tensor types, dense border). */
int sessd_voxelgen_clone(const sessd_voxelgen* h, sessd_voxelgen** out);
int sessd_submconv3d_clone(const sessd_submconv3d* h, sessd_submconv3d** out);
int sessd_sparseconv3d_clone(const sessd_sparseconv3d* h, sessd_sparseconv3d** out);
int sessd_sparse2dense_clone(const sessd_sparse2dense* h, sessd_sparse2dense** out);

/* ------------------------------------------------------------------------------------------ */
/* Frame pipeline: voxelGenerator -> SpMiddleFHD conv stack (+BN+ReLU) -> sparse2Dense          */
/* (reference wiring: se-ssd-ai-trt.cpp:1138-1252; layer shapes: params.h:19-197)               */
/* ------------------------------------------------------------------------------------------ */
/* The pipeline owns its plugins, intermediate tensors and workspaces (allocated at create);
 * enqueue allocates nothing.  It is what TensorRT's executor does for the reference: call each
 * plugin's enqueue in graph order on one stream. */

typedef struct sessd_pipeline sessd_pipeline;

enum { SESSD_LAYER_SUBM = 0, SESSD_LAYER_SPARSE = 1 };

typedef struct sessd_layer_spec {
    int32_t type; /* SESSD_LAYER_* */
    int32_t in_channel, out_channel;
    int32_t ksize[3], stride[3], padding[3]; /* z,y,x (SubM: 3,1,1 on every axis) */
    int32_t out_shape[3];                    /* x,y,z */
} sessd_layer_spec;

typedef struct sessd_pipeline_desc {
    sessd_voxelgen_desc voxelgen;
    int32_t max_points;       /* rows of the points tensor */
    int32_t point_features;   /* columns of the points tensor (4) */
    int32_t n_layers;
    const sessd_layer_spec* layers;
    const float* const* weights; /* per layer: host FP32 [K][Cin][Cout] */
    const float* const* scale;   /* per layer: host FP32 [Cout] folded BN scale, or NULL */
    const float* const* shift;   /* per layer: host FP32 [Cout] folded BN shift, or NULL */
    int32_t relu;                /* ReLU after every layer */
    int32_t feature_dtype;       /* SESSD_FLOAT or SESSD_HALF: dtype of conv features */
    sessd_sparse2dense_desc dense;
    int32_t share_rulebooks;     /* consecutive SubM layers on one coors tensor build it once */
    int32_t flags;               /* SESSD_FLAG_* applied to every layer */
    int32_t use_graph;           /* replay the enqueue sequence from a captured hipGraph */
    int32_t layer_max_voxels;    /* rows of the conv layers' tensors; 0 = voxelgen.max_voxels.  May exceed the
                                    voxelizer's cap: strided layers can produce more sites than they get */
    int32_t overlap_streams;     /* run the coordinate chain (voxelizer + rulebook builds) on a second
                                    stream owned by the pipeline, overlapping the GEMMs of earlier layers */
    int32_t dense_padding[4];    /* top, bottom, left, right: zero border around the dense tensor
                                    (sessd_sparse2dense_set_padding); the reference network uses 1,1,1,1
                                    (params.h:200-203).  The caller's dense buffer has the padded size */
    int32_t frames_in_flight;    /* 0 or 1: one frame at a time.  R = 2..8: throughput mode, needs
                                    overlap_streams.  The pipeline keeps R replicas of its tensors, workspaces and
                                    graph, each with a stream of its own, and gives successive frames to
                                    successive replicas, so that frame t + 1 starts while frame t still runs:
                                    sessd_pipeline_submit / sessd_pipeline_join */
} sessd_pipeline_desc;

/* Fills `layers[14]` with the reference backbone (params.h:39-192) and `dense`/`voxelgen` with
 * params.h:19-36, 194-197; returns the number of layers written (14). */
int sessd_reference_backbone(sessd_layer_spec* layers, int max_layers,
                             sessd_voxelgen_desc* voxelgen, sessd_sparse2dense_desc* dense);

int sessd_pipeline_create(const sessd_pipeline_desc* desc, sessd_pipeline** out);

/* ------------------------------------------------------------------------------------------ */
/* `.wts` weight files and BatchNorm folding (host side; no GPU call)                          */
/* ------------------------------------------------------------------------------------------ */
/* replaces loadWeights (se-ssd-ai-trt.cpp:276-314; writer: tools/gen_wts.py:86-99): text, the blob
 * count, then per blob `name count` and `count` tokens of big-endian hex float bits.  Malformed input
 * is an error code where the reference asserts. */
typedef struct sessd_wts sessd_wts;
int sessd_wts_load(const char* path, sessd_wts** out);
int sessd_wts_parse(const char* text, size_t length, sessd_wts** out);
int sessd_wts_count(const sessd_wts* w);
/* blob names in file order; the pointer lives as long as the handle */
int sessd_wts_name(const sessd_wts* w, int index, const char** name);
/* replaces weightMap[name] (e.g. se-ssd-ai-trt.cpp:1148); an unknown name is an error, not an empty blob */
int sessd_wts_find(const sessd_wts* w, const char* name, const float** values, int64_t* count);
void sessd_wts_destroy(sessd_wts* w);
/* replaces the folding in add_batchNorm1d_relu (se-ssd-ai-trt.cpp:808-824), FP32 arithmetic:
 * scale = gamma / sqrtf(var + eps), shift = beta - mean * gamma / sqrtf(var + eps) */
int sessd_fold_batchnorm(const float* gamma, const float* beta, const float* mean, const float* var,
                         int32_t n, float eps, float* scale, float* shift);
/* replaces loadData + the point count of its caller (se-ssd-ai-trt.cpp:1515-1559, 1849-1850): reads a
 * headerless float32 [n][point_features] file (KITTI velodyne `.bin`: x,y,z,intensity) into the host
 * buffer points[max_points][point_features], zero-fills the rest, and returns n = bytes / (4 *
 * point_features).  A file that does not fit is an error (the reference exits). */
int sessd_load_frame(const char* path, float* points, int32_t max_points, int32_t point_features,
                     int32_t* points_size);
/* replaces the weightMap lookups of the reference's network builder (se-ssd-ai-trt.cpp:1147-1249):
 * layer l takes `<prefix><conv_index[l]>.weight` and the BatchNorm blobs `<prefix><conv_index[l]+1>.
 * {weight,bias,running_mean,running_var}`, folded with `eps` (the reference passes 1e-5) + ReLU.
 * prefix NULL = "backbone.middle_conv."; conv_index NULL = 0,3,6,...,39 (needs n_layers == 14).
 * desc->weights/scale/shift/relu are ignored. */
int sessd_pipeline_create_from_wts(const sessd_pipeline_desc* desc, const sessd_wts* wts,
                                   const char* prefix, const int32_t* conv_index, float eps,
                                   sessd_pipeline** out);
/* points f32[max_points,point_features], points_size i32[1], dense [C*D,H,W]: device pointers */
int sessd_pipeline_enqueue(sessd_pipeline* h, const void* points, const void* points_size,
                           void* dense, sessd_stream_t stream);
/* The two halves of sessd_pipeline_enqueue, for hosts that keep several frames in flight (frames_in_flight
 * >= 2): submit starts the frame once the work already on `stream` is done (the inputs are ready) and
 * returns a ticket; it does not make `stream` wait for the frame.  join makes `stream` wait until the dense
 * tensor of that ticket's frame is complete.  Submit frame t + 1 before joining frame t and the two overlap;
 * enqueue = submit + join.  points, points_size and dense of a frame must stay untouched until its join has
 * been waited for.  More than frames_in_flight submitted frames without a join in between are safe (a
 * replica is not reused before its previous frame has finished), they just do not overlap any further.  The
 * per-layer queries below (layer_io, status, layer_stats, num_launches) then refer to the frame submitted
 * last.  With frames_in_flight < 2: submit = enqueue, join does nothing. */
int sessd_pipeline_submit(sessd_pipeline* h, const void* points, const void* points_size, void* dense,
                          sessd_stream_t stream, int64_t* ticket);
/* (join with stream = SESSD_STREAM_NONE blocks the calling thread, as sessd_pipeline_wait does.  With frames in
 * flight, sessd_pipeline_status / _layer_stats first make `stream` wait for the last submitted frame; a caller
 * that reads tensors of sessd_pipeline_layer_io itself has to join that frame first; sessd_pipeline_enqueue_timed
 * is refused.) */
int sessd_pipeline_join(sessd_pipeline* h, int64_t ticket, sessd_stream_t stream);
/* join for a host loop: blocks the calling thread (not a stream) until the frame of `ticket` is complete.  A
 * stream-side join puts a wait into the caller's stream, and where that stream shares a hardware queue with
 * one of the pipeline's own, everything behind the wait in that queue stands still until the frame is done;
 * a throughput loop that submits frame t + 1, then waits for frame t + 1 - frames_in_flight here, has no such
 * coupling.  Only with frames_in_flight >= 2. */
int sessd_pipeline_wait(sessd_pipeline* h, int64_t ticket);
/* Device pointers to the tensors a layer produced in the last enqueue (layer = -1: voxelizer).
 * feat: [max_voxels, C]; coors: i32[max_voxels,4]; voxel_num: i32[1]; workspace of that layer. */
int sessd_pipeline_layer_io(sessd_pipeline* h, int layer, void** feat, void** coors,
                            void** voxel_num, void** workspace, int32_t* channels);
/* Profiling variant of enqueue: records HIP events on `stream` around the voxelizer, around each
 * layer's rulebook build and gather-GEMM launch and around sparse2dense, synchronises, and returns
 * the 2*n_layers+2 segment durations in milliseconds, in that order.  When max_segments leaves room
 * for one more value, segment_ms[2*n_layers+2] receives the time between two events recorded back to
 * back (what the timer itself adds to every segment).  Never uses the graph. */
int sessd_pipeline_enqueue_timed(sessd_pipeline* h, const void* points, const void* points_size,
                                 void* dense, sessd_stream_t stream, float* segment_ms,
                                 int max_segments, int* n_segments);
/* Active output rows and rulebook pairs of a layer in the last enqueue (layer = -1: voxelizer,
 * pairs = 0).  Launches small counting kernels and synchronises; for reporting, not the hot path. */
int sessd_pipeline_layer_stats(sessd_pipeline* h, int layer, sessd_stream_t stream, int64_t* n_out,
                               int64_t* pairs);
/* OR of every layer's status word (synchronises the stream) */
int sessd_pipeline_status(sessd_pipeline* h, sessd_stream_t stream, int32_t* status);
size_t sessd_pipeline_device_bytes(const sessd_pipeline* h);
int sessd_pipeline_num_launches(const sessd_pipeline* h);
void sessd_pipeline_destroy(sessd_pipeline* h);

#ifdef __cplusplus
}
#endif
#endif /* SESSD3D_H_ */
