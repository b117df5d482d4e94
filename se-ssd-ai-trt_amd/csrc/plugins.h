// plugins.h -- host classes behind the C-ABI.  One class per reference plugin, with the methods
// TensorRT drives on IPluginV2DynamicExt (configurePlugin, getWorkspaceSize, enqueue,
// getSerializationSize, serialize) under the same names; include/sessd3d.h forwards to them.
#pragma once

#include <vector>

#include "common.h"

namespace sessd {

struct Epilogue {
    float* scale_dev = nullptr;  // [Cout] or null
    float* shift_dev = nullptr;  // [Cout] or null
    int relu = 0;
    std::vector<float> scale_host, shift_host;
};

// ---------------------------------------------------------------------------------------------
// reference: voxelGenerator.h:15-77 / voxelGenerator.cu
// ---------------------------------------------------------------------------------------------
class VoxelGeneratorPlugin {
  public:
    static int create(const sessd_voxelgen_desc& d, VoxelGeneratorPlugin** out);
    static int deserialize(const void* data, size_t length, VoxelGeneratorPlugin** out);

    int configurePlugin(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                        int nbOutputs);
    size_t getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs,
                            const sessd_tensor_desc* outputs, int nbOutputs) const;
    // `mirror`: the neighbour table of the SubM layer that will run its symmetric lookup on these voxels;
    // `also_clear`: regions cleared in the same launch as the voxelizer's own tables
    int enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                const void* const* inputs, void* const* outputs, void* workspace,
                hipStream_t stream, const MirrorInit* mirror = nullptr, const FillArgs* also_clear = nullptr);
    // enqueue() on the library's own static scratch array instead of a caller's workspace: allocates nothing;
    // rejects points tensors whose layout does not fit the array.  Calls that overlap on one GPU race.
    int enqueueStatic(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                      const void* const* inputs, void* const* outputs, hipStream_t stream);
    size_t getSerializationSize() const;
    void serialize(void* buffer) const;
    size_t statusOffset(int max_points) const;
    // After an enqueue the workspace's hash maps linear cell (z*Y + y)*X + x -> voxel row (kEmpty for cells
    // dropped at the cap): a SubM layer on the same x/y grid can use it as its cell table
    // (SubmConv3dLayerPlugin::enqueueBuild) instead of inserting every voxel into its own.
    HashTable cellTable(void* workspace, int max_points) const;

    // serialized fields, in the reference's order (voxelGenerator.cu:584-599)
    int voxelNum_ = 0;      // max_voxels
    int pointNum_ = 0;      // max points per voxel
    int featureNum_ = 4;    // voxel feature count
    float min_x_range_ = 0, max_x_range_ = 0, min_y_range_ = 0, max_y_range_ = 0, min_z_range_ = 0,
          max_z_range_ = 0;
    float voxel_x_size_ = 0, voxel_y_size_ = 0, voxel_z_size_ = 0;
    int pointFeatureNum_ = 4;
    int grid_x_size_ = 0, grid_y_size_ = 0, grid_z_size_ = 0;

    int flags_ = 0;
    int lastMaxPoints_ = 0;  // rows of the points tensor seen by the last configure/enqueue

  private:
    struct Layout;
    Layout carve(void* workspace, int max_points) const;
    void deriveGrid();
};

// ---------------------------------------------------------------------------------------------
// Shared by both conv plugins: device weights (+ epilogue), dtype bookkeeping, GEMM dispatch
// ---------------------------------------------------------------------------------------------
bool gemm_runs_tall(int K, int cin, int cout, int in_type, int out_type);  // kernels.h
// Cin * Cout (of the layer that builds it) from which a rulebook gets equal-work tile cuts.  At 32 x 32 the GEMM
// measured the same with and without them, and the two launches lengthen the coordinate branch: frame 0.387 -> 0.377 ms.
constexpr int kTileCutMinWork = 32 * 64;
class ConvPluginBase {
  public:
    virtual ~ConvPluginBase();
    int setEpilogue(const float* scale, const float* shift, int relu);
    int uploadWeights(const float* w, size_t count);
    int configureTypes(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                       int nbOutputs);
    // whether this layer's gather-GEMM runs on the MFMA kernel (the one that can take a DenseTarget)
    bool gemmOnMatrixCores() const;
    // after in_type_ / out_type_ were set by hand (clone): the operand-ordered weight copy for those types
    int preparePackedForTypes() { return preparePacked(); }

    int in_channel_ = 0, out_channel_ = 0, max_voxels_ = 0, feature_num_ = 0;
    int out_shape_x_ = 0, out_shape_y_ = 0, out_shape_z_ = 0;
    int spatial_shape_x_ = 0, spatial_shape_y_ = 0, spatial_shape_z_ = 0;
    int dilation_ = 1, out_padding_ = 0;
    int weights_size_ = 0;
    int kernel_volume_ = 0;
    std::vector<float> weights_data_;  // host copy, FP32 [K][Cin][Cout]
    float* weights_dev_ = nullptr;     // FP32 [K][Cin][Cout]
    __half* weights_half_dev_ = nullptr;  // FP16 copy of the same layout
    void* weights_packed_dev_ = nullptr;  // MFMA B-operand order (see conv_gemm.hip)
    int packed_dtype_ = -1;
    Epilogue epi_;
    int in_type_ = SESSD_FLOAT, out_type_ = SESSD_FLOAT;
    int flags_ = 0;
    // when set, recorded on the stream right before / after the gather-GEMM launch (profiling)
    hipEvent_t ev_gemm_begin_ = nullptr, ev_gemm_end_ = nullptr;

  protected:
    // gather-GEMM over the neighbour table nbr[K][max_voxels] (device), rows < *num_out
    // `dense`: also scatter the output rows into the dense tensor of a sparse2Dense step (MFMA kernel only)
    int runGemm(const void* in_feat, void* out_feat, const int32_t* nbr, const int32_t* tiles,
                const int32_t* num_out, hipStream_t stream, const DenseTarget* dense = nullptr);
    // whether a rulebook built by this layer gets equal-work tile cuts: worth two small launches when the
    // GEMM runs on the matrix cores and is not tiny
    bool wantTileCuts() const {
        return weights_packed_dev_ != nullptr && !(flags_ & SESSD_FLAG_FORCE_VALU) &&
               in_channel_ * out_channel_ >= kTileCutMinWork &&
               !gemm_runs_tall(kernel_volume_, in_channel_, out_channel_, in_type_, out_type_);
    }
    // tile height those cuts aim at: the capacity of this layer's own GEMM kernel
    int tileRows() const;
    // weight of a row beside its pairs in those cuts
    int tileRowWeight() const;
    int exportRulebook(const int32_t* nbr, const int32_t* num_out, void* scratch,
                       int32_t* indice_pairs, uint32_t* indice_num, hipStream_t stream) const;
    int freeDevice();
    int preparePacked();
};

// ---------------------------------------------------------------------------------------------
// reference: submConv3dlayer.h:19-92 / submConv3dlayer.cu
// ---------------------------------------------------------------------------------------------
class SubmConv3dLayerPlugin : public ConvPluginBase {
  public:
    static int create(const sessd_submconv3d_desc& d, const float* weights,
                      SubmConv3dLayerPlugin** out);
    static int deserialize(const void* data, size_t length, SubmConv3dLayerPlugin** out);

    int configurePlugin(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                        int nbOutputs);
    size_t getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs,
                            const sessd_tensor_desc* outputs, int nbOutputs) const;
    int enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                const void* const* inputs, void* const* outputs, void* workspace,
                hipStream_t stream);
    int enqueueShared(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                      const void* const* inputs, void* const* outputs,
                      const void* rulebook_workspace, hipStream_t stream);
    // enqueue = enqueueBuild (coordinates -> rulebook) + enqueueGemm (features)
    // `cells`: a cell -> row table over this layer's grid that some earlier kernel already built (the
    // voxelizer's, or that of the strided layer that produced `coors`); the insert pass is skipped then
    // `mirrored`: the producer of `coors` has initialised this layer's mirrored neighbour entries (mirrorInit()):
    // the lookup then probes 13 offsets per row instead of 27 and writes both directions of every hit
    int enqueueBuild(const int32_t* coors, const int32_t* voxel_num, void* workspace, hipStream_t stream,
                     bool prefilled = false, const HashTable* cells = nullptr, bool mirrored = false);
    // what the producer of this layer's coors tensor needs for that (nbr == nullptr: this layer cannot use it)
    MirrorInit mirrorInit(void* workspace) const;
    void collectFill(void* workspace, FillArgs& f, bool own_table = true) const;
    int enqueueGemm(const void* in_feat, void* out_feat, const int32_t* voxel_num,
                    const void* rulebook_workspace, hipStream_t stream, const DenseTarget* dense = nullptr);
    int exportRulebook(const void* workspace, int32_t* indice_pairs, uint32_t* indice_num,
                       hipStream_t stream) const;
    int countPairs(const void* workspace, uint32_t* indice_num, hipStream_t stream) const;
    size_t getSerializationSize() const;
    void serialize(void* buffer) const;
    size_t statusOffset() const;

    int ksize_ = 3, stride_ = 1, padding_ = 1;

  private:
    struct Layout;
    Layout carve(void* workspace) const;
    int validate() const;
};

// ---------------------------------------------------------------------------------------------
// reference: sparseConv3dlayer.h:19-97 / sparseConv3dlayer.cu
// ---------------------------------------------------------------------------------------------
class SparseConv3dLayerPlugin : public ConvPluginBase {
  public:
    static int create(const sessd_sparseconv3d_desc& d, const float* weights,
                      SparseConv3dLayerPlugin** out);
    static int deserialize(const void* data, size_t length, SparseConv3dLayerPlugin** out);

    int configurePlugin(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                        int nbOutputs);
    size_t getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs,
                            const sessd_tensor_desc* outputs, int nbOutputs) const;
    int enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                const void* const* inputs, void* const* outputs, void* workspace,
                hipStream_t stream);
    int exportRulebook(const void* workspace, int32_t* indice_pairs, uint32_t* indice_num,
                       hipStream_t stream) const;
    int countPairs(const void* workspace, uint32_t* indice_num, hipStream_t stream) const;
    int enqueueBuild(const int32_t* coors, const int32_t* voxel_num, int32_t* out_coors, int32_t* out_num,
                     void* workspace, hipStream_t stream, bool prefilled = false, const MirrorInit* mirror = nullptr);
    // after enqueueBuild the workspace's hash maps output cell -> output row (see VoxelGeneratorPlugin::cellTable)
    HashTable cellTable(void* workspace) const;
    void collectFill(void* workspace, int32_t* out_coors, FillArgs& f) const;
    int enqueueGemm(const void* in_feat, void* out_feat, const int32_t* out_num, const void* workspace,
                    hipStream_t stream, const DenseTarget* dense = nullptr);
    size_t getSerializationSize() const;
    void serialize(void* buffer) const;
    size_t statusOffset() const;

    int ksize0_ = 3, ksize1_ = 3, ksize2_ = 3;        // z,y,x
    int stride0_ = 1, stride1_ = 1, stride2_ = 1;
    int padding0_ = 0, padding1_ = 0, padding2_ = 0;

  private:
    struct Layout;
    Layout carve(void* workspace) const;
    int validate() const;
    int maxCandidates() const;  // enumeration slots per input voxel
};

// ---------------------------------------------------------------------------------------------
// reference: sparse2Dense.h:15-60 / sparse2Dense.cu
// ---------------------------------------------------------------------------------------------
class Sparse2DensePlugin {
  public:
    static int create(const sessd_sparse2dense_desc& d, Sparse2DensePlugin** out);
    static int deserialize(const void* data, size_t length, Sparse2DensePlugin** out);
    int configurePlugin(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                        int nbOutputs);
    size_t getWorkspaceSize(const sessd_tensor_desc* inputs, int nbInputs,
                            const sessd_tensor_desc* outputs, int nbOutputs) const;
    int enqueue(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                const void* const* inputs, void* const* outputs, void* workspace,
                hipStream_t stream);
    void collectFill(void* dense, void* workspace, FillArgs& f) const;
    // the scatter of enqueue() as an epilogue of the gather-GEMM that produces `coors`' feature rows
    DenseTarget denseTarget(void* dense, const int32_t* coors, void* workspace) const;
    size_t getSerializationSize() const;
    void serialize(void* buffer) const;

    int setPadding(int top, int bottom, int left, int right);
    int outHeight() const { return feature_map_size_y_ + zero_padding_2d_top_ + zero_padding_2d_bottom_; }
    int outWidth() const { return feature_map_size_x_ + zero_padding_2d_left_ + zero_padding_2d_right_; }
    bool padded() const {
        return (zero_padding_2d_top_ | zero_padding_2d_bottom_ | zero_padding_2d_left_ | zero_padding_2d_right_) != 0;
    }

    int feature_map_size_x_ = 0, feature_map_size_y_ = 0, feature_map_size_z_ = 0;
    int feature_map_channel_ = 0;
    // border written around every channel plane: the reference's ZeroPad2dPlugin (zeroPad2d.cu:183-244),
    // which follows sparse2Dense in its network (se-ssd-ai-trt.cpp:1253), folded into this scatter
    int zero_padding_2d_top_ = 0, zero_padding_2d_bottom_ = 0, zero_padding_2d_left_ = 0, zero_padding_2d_right_ = 0;
    int in_type_ = SESSD_FLOAT, out_type_ = SESSD_FLOAT;
};

// little-endian field (de)serialisation in declaration order, as the reference's
// writeToBuffer / readFromBuffer (voxelGenerator.cu:44-58)
template <typename T>
inline void writeToBuffer(char*& buffer, const T& val) {
    std::memcpy(buffer, &val, sizeof(T));
    buffer += sizeof(T);
}
template <typename T>
inline T readFromBuffer(const char*& buffer) {
    T val;
    std::memcpy(&val, buffer, sizeof(T));
    buffer += sizeof(T);
    return val;
}

int read_status_word(const void* workspace, size_t offset, hipStream_t stream, int32_t* status);
// device address of the voxelizer's static scratch array on the current device (voxel_generator.hip)
int voxelgen_static_scratch(void** out);

// helpers shared by the two conv plugins (conv_base.hip)
int conv_check_io(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                  const void* const* inputs, void* const* outputs, int in_type, int out_type, int max_voxels,
                  int cin, int cout, const char* who);
int read_epilogue_trailer(const char* d, size_t remaining, ConvPluginBase* p);
size_t conv_epilogue_trailer_size(const Epilogue& e);
void conv_write_epilogue_trailer(char*& d, const Epilogue& e);

}  // namespace sessd
