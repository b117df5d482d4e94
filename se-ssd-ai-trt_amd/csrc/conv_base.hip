// conv_base.hip -- what SubmConv3dLayerPlugin and SparseConv3dLayerPlugin share: the device copies
// of the weights, the fused scale/shift/ReLU epilogue, dtype bookkeeping and the GEMM dispatch.
#include "kernels.h"
#include "plugins.h"

namespace sessd {

ConvPluginBase::~ConvPluginBase() { freeDevice(); }

int ConvPluginBase::freeDevice() {
    // the reference frees in terminate() and again in the destructor (submConv3dlayer.cu:671-682);
    // here every pointer is released once and cleared
    void** ptrs[] = {reinterpret_cast<void**>(&weights_dev_), reinterpret_cast<void**>(&weights_half_dev_),
                     &weights_packed_dev_, reinterpret_cast<void**>(&epi_.scale_dev),
                     reinterpret_cast<void**>(&epi_.shift_dev)};
    for (void** p : ptrs) {
        if (*p) (void)hipFree(*p);
        *p = nullptr;
    }
    return SESSD_OK;
}

// Uploads FP32 [K][Cin][Cout] weights (the ctor of the reference does the same with a synchronous
// cudaMemcpy, submConv3dlayer.cu:147-150) plus a half-rounded copy for the FP16 feature path.
int ConvPluginBase::uploadWeights(const float* w, size_t count) {
    if (!w) return fail(SESSD_E_INVALID, "conv: weights pointer is null");
    weights_data_.assign(w, w + count);
    weights_size_ = (int)count;
    SESSD_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&weights_dev_), count * sizeof(float)));
    SESSD_HIP_TRY(hipMemcpy(weights_dev_, w, count * sizeof(float), hipMemcpyHostToDevice));
    std::vector<__half> h(count);
    for (size_t i = 0; i < count; ++i) h[i] = __float2half_rn(w[i]);
    SESSD_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&weights_half_dev_), count * sizeof(__half)));
    SESSD_HIP_TRY(hipMemcpy(weights_half_dev_, h.data(), count * sizeof(__half), hipMemcpyHostToDevice));
    packed_dtype_ = -1;
    return preparePacked();
}

int ConvPluginBase::setEpilogue(const float* scale, const float* shift, int relu) {
    for (float** p : {&epi_.scale_dev, &epi_.shift_dev}) {
        if (*p) (void)hipFree(*p);
        *p = nullptr;
    }
    epi_.scale_host.clear();
    epi_.shift_host.clear();
    epi_.relu = relu ? 1 : 0;
    const size_t bytes = (size_t)out_channel_ * sizeof(float);
    if (scale) {
        epi_.scale_host.assign(scale, scale + out_channel_);
        SESSD_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&epi_.scale_dev), bytes));
        SESSD_HIP_TRY(hipMemcpy(epi_.scale_dev, scale, bytes, hipMemcpyHostToDevice));
    }
    if (shift) {
        epi_.shift_host.assign(shift, shift + out_channel_);
        SESSD_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&epi_.shift_dev), bytes));
        SESSD_HIP_TRY(hipMemcpy(epi_.shift_dev, shift, bytes, hipMemcpyHostToDevice));
    }
    return SESSD_OK;
}

// The reference accepts only kFLOAT features (submConv3dlayer.cu:218-240); FP16 features with FP32
// accumulation are accepted here as well.
int ConvPluginBase::configureTypes(const sessd_tensor_desc* in, int nbInputs, const sessd_tensor_desc* out,
                                   int nbOutputs) {
    if (!in || !out || nbInputs < 3 || nbOutputs < 1)
        return fail(SESSD_E_INVALID, "conv.configure: expected 3 inputs and >= 1 output");
    for (const sessd_tensor_desc* d : {&in[0], &out[0]})
        if (d->type != SESSD_FLOAT && d->type != SESSD_HALF)
            return fail(SESSD_E_UNSUPPORTED, "conv.configure: features must be FP32 or FP16");
    if (in[0].nbDims != 3 || in[0].d[0] != 1 || in[0].d[2] != in_channel_)
        return fail(SESSD_E_INVALID, "conv.configure: input features must be [1,max_voxels,%d]", in_channel_);
    if (in[0].d[1] != max_voxels_ || out[0].d[1] != max_voxels_ || out[0].d[2] != out_channel_)
        return fail(SESSD_E_INVALID, "conv.configure: tensors must have max_voxels=%d rows, %d output channels",
                    max_voxels_, out_channel_);
    in_type_ = in[0].type;
    out_type_ = out[0].type;
    return preparePacked();
}

// Operand-ordered weights for the MFMA kernels, packed for the compute dtype the configured feature
// dtypes imply.  Runs at create/configure time so that enqueue never allocates.
int ConvPluginBase::preparePacked() {
    const int compute_type = in_type_ == SESSD_HALF || out_type_ == SESSD_HALF ? SESSD_HALF : SESSD_FLOAT;
    if (packed_dtype_ == compute_type) return SESSD_OK;
    if (weights_packed_dev_) (void)hipFree(weights_packed_dev_);
    weights_packed_dev_ = nullptr;
    const size_t bytes = packed_weight_bytes(kernel_volume_, in_channel_, out_channel_, compute_type);
    if (bytes) {
        std::vector<uint8_t> host(bytes);
        pack_weights(weights_data_.data(), kernel_volume_, in_channel_, out_channel_, compute_type, host.data());
        SESSD_HIP_TRY(hipMalloc(&weights_packed_dev_, bytes));
        SESSD_HIP_TRY(hipMemcpy(weights_packed_dev_, host.data(), bytes, hipMemcpyHostToDevice));
    }
    packed_dtype_ = compute_type;
    return SESSD_OK;
}

bool ConvPluginBase::gemmOnMatrixCores() const {
    return weights_packed_dev_ != nullptr && !(flags_ & SESSD_FLAG_FORCE_VALU) &&
           gemm_runs_on_mfma(kernel_volume_, in_channel_, out_channel_, in_type_, out_type_);
}

int ConvPluginBase::tileRows() const { return gemm_tile_rows(in_channel_, out_channel_, out_type_); }
int ConvPluginBase::tileRowWeight() const {
    return gemm_runs_wide(kernel_volume_, in_channel_, out_channel_, in_type_, out_type_) ? 4 : 20;
}

int ConvPluginBase::runGemm(const void* in_feat, void* out_feat, const int32_t* nbr, const int32_t* tiles,
                            const int32_t* num_out, hipStream_t stream, const DenseTarget* dense) {
    GemmArgs a;
    if (dense) a.dense = *dense;
    a.in_feat = in_feat;
    a.out_feat = out_feat;
    a.nbr = nbr;
    a.num_out = num_out;
    a.max_voxels = max_voxels_;
    a.K = kernel_volume_;
    a.cin = in_channel_;
    a.cout = out_channel_;
    a.in_type = in_type_;
    a.out_type = out_type_;
    a.w_f32 = weights_dev_;
    a.w_f16 = weights_half_dev_;
    a.w_packed = weights_packed_dev_;
    a.scale = epi_.scale_dev;
    a.shift = epi_.shift_dev;
    a.relu = epi_.relu;
    a.write_pad_rows = (flags_ & SESSD_FLAG_SKIP_PAD_ROWS) ? 0 : 1;
    a.force_valu = (flags_ & SESSD_FLAG_FORCE_VALU) ? 1 : 0;
    a.tiles = tiles;
    if (ev_gemm_begin_) SESSD_HIP_TRY(hipEventRecord(ev_gemm_begin_, stream));
    SESSD_TRY(launch_gather_gemm(a, stream));
    if (ev_gemm_end_) SESSD_HIP_TRY(hipEventRecord(ev_gemm_end_, stream));
    return SESSD_OK;
}

int ConvPluginBase::exportRulebook(const int32_t* nbr, const int32_t* num_out, void* scratch,
                                   int32_t* indice_pairs, uint32_t* indice_num, hipStream_t stream) const {
    return launch_export_rulebook(nbr, num_out, kernel_volume_, max_voxels_, scratch, indice_pairs,
                                  indice_num, stream);
}

// Serialised conv plugins carry the reference's fields (submConv3dlayer.cu:684-714,
// sparseConv3dlayer.cu:863-899).  A fused epilogue (not part of the reference plugin) is appended as a
// trailer: int magic, int relu, int has_scale, int has_shift, floats.
static constexpr int kEpilogueMagic = 0x49504553;  // "SEPI"

static size_t epilogue_trailer_size(const Epilogue& e) {
    if (e.scale_host.empty() && e.shift_host.empty() && !e.relu) return 0;
    return 4 * sizeof(int) + (e.scale_host.size() + e.shift_host.size()) * sizeof(float);
}
static void write_epilogue_trailer(char*& d, const Epilogue& e) {
    if (!epilogue_trailer_size(e)) return;
    writeToBuffer<int>(d, kEpilogueMagic);
    writeToBuffer<int>(d, e.relu);
    writeToBuffer<int>(d, e.scale_host.empty() ? 0 : 1);
    writeToBuffer<int>(d, e.shift_host.empty() ? 0 : 1);
    for (float v : e.scale_host) writeToBuffer<float>(d, v);
    for (float v : e.shift_host) writeToBuffer<float>(d, v);
}
int read_epilogue_trailer(const char* d, size_t remaining, ConvPluginBase* p) {
    if (remaining == 0) return SESSD_OK;
    if (remaining < 4 * sizeof(int)) return fail(SESSD_E_INVALID, "conv: truncated epilogue trailer");
    if (readFromBuffer<int>(d) != kEpilogueMagic) return fail(SESSD_E_INVALID, "conv: unknown trailer");
    const int relu = readFromBuffer<int>(d);
    const int has_scale = readFromBuffer<int>(d), has_shift = readFromBuffer<int>(d);
    const size_t need = (size_t)(has_scale + has_shift) * p->out_channel_ * sizeof(float);
    if (remaining - 4 * sizeof(int) < need) return fail(SESSD_E_INVALID, "conv: truncated epilogue trailer");
    std::vector<float> sc, sh;
    if (has_scale) for (int i = 0; i < p->out_channel_; ++i) sc.push_back(readFromBuffer<float>(d));
    if (has_shift) for (int i = 0; i < p->out_channel_; ++i) sh.push_back(readFromBuffer<float>(d));
    return p->setEpilogue(has_scale ? sc.data() : nullptr, has_shift ? sh.data() : nullptr, relu);
}
size_t conv_epilogue_trailer_size(const Epilogue& e) { return epilogue_trailer_size(e); }
void conv_write_epilogue_trailer(char*& d, const Epilogue& e) { write_epilogue_trailer(d, e); }


static int check_conv_io_impl(const sessd_tensor_desc* inputDesc, const sessd_tensor_desc* outputDesc,
                         const void* const* inputs, void* const* outputs, int in_type, int out_type,
                         int max_voxels, int cin, int cout, const char* who) {
    if (!inputDesc || !outputDesc || !inputs || !outputs) return fail(SESSD_E_INVALID, "%s: null argument", who);
    if (!inputs[0] || !inputs[1] || !inputs[2] || !outputs[0]) return fail(SESSD_E_INVALID, "%s: null tensor pointer", who);
    if (inputDesc[0].d[0] != 1) return fail(SESSD_E_UNSUPPORTED, "%s: batch size must be 1", who);
    if (inputDesc[0].type != in_type || outputDesc[0].type != out_type)
        return fail(SESSD_E_INVALID, "%s: tensor dtypes differ from the configured ones", who);
    if (inputDesc[0].d[1] != max_voxels || inputDesc[0].d[2] != cin || outputDesc[0].d[1] != max_voxels ||
        outputDesc[0].d[2] != cout)
        return fail(SESSD_E_INVALID, "%s: tensor shapes do not match the layer", who);
    if ((reinterpret_cast<uintptr_t>(inputs[0]) | reinterpret_cast<uintptr_t>(inputs[1]) |
         reinterpret_cast<uintptr_t>(outputs[0])) & 15)
        return fail(SESSD_E_INVALID, "%s: tensors must be 16-byte aligned", who);
    return SESSD_OK;
}
int conv_check_io(const sessd_tensor_desc* a, const sessd_tensor_desc* b, const void* const* c, void* const* d,
                  int e, int f, int g, int h, int i, const char* who) {
    return check_conv_io_impl(a, b, c, d, e, f, g, h, i, who);
}


}  // namespace sessd
