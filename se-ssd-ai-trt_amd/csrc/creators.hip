// creators.hip -- the by-name half of the plugin surface: what TensorRT reaches through IPluginCreator
// (getFieldNames / createPlugin(name, PluginFieldCollection*)) and IPluginV2::clone(), as C entry points.
//
// The reference has one creator class per plugin; each walks the field collection, picks the fields it knows by
// name and calls the plugin's constructor (voxelGenerator.cu:618-701, submConv3dlayer.cu:732-878,
// sparseConv3dlayer.cu:918-1079, sparse2Dense.cu:316-373).  Here one function does that for the four plugins of
// the 3-D front end, keyed by the reference's plugin names.  Where the reference constructs a plugin from zeros
// when a field is missing, this returns an error that names the field.
#include <cstring>

#include "plugins.h"

namespace sessd {
namespace {

struct FieldSpec {
    const char* name;
    int32_t type;    // SESSD_FIELD_*
    int32_t length;  // elements the creator reads from `data`
};

const FieldSpec kVoxelGenFields[] = {  // voxelGenerator.cu:624-628
    {"max_num_points_per_voxel", SESSD_FIELD_INT32, 1}, {"max_voxels", SESSD_FIELD_INT32, 1},
    {"point_cloud_range", SESSD_FIELD_FLOAT32, 6},      {"voxel_feature_num", SESSD_FIELD_INT32, 1},
    {"voxel_size", SESSD_FIELD_FLOAT32, 3}};
const FieldSpec kSubmFields[] = {  // submConv3dlayer.cu:737-748 (scalar ksize/stride/padding: :834-848)
    {"in_channel", SESSD_FIELD_INT32, 1}, {"out_channel", SESSD_FIELD_INT32, 1}, {"max_voxels", SESSD_FIELD_INT32, 1},
    {"feature_num", SESSD_FIELD_INT32, 1}, {"out_shape", SESSD_FIELD_INT32, 3}, {"spatial_shape", SESSD_FIELD_INT32, 3},
    {"ksize", SESSD_FIELD_INT32, 1},      {"stride", SESSD_FIELD_INT32, 1},     {"padding", SESSD_FIELD_INT32, 1},
    {"dilation", SESSD_FIELD_INT32, 1},   {"out_padding", SESSD_FIELD_INT32, 1}, {"weights", SESSD_FIELD_FLOAT32, 0}};
const FieldSpec kSparseFields[] = {  // sparseConv3dlayer.cu:923-934 (3-vectors in z,y,x order: :1028-1048)
    {"in_channel", SESSD_FIELD_INT32, 1}, {"out_channel", SESSD_FIELD_INT32, 1}, {"max_voxels", SESSD_FIELD_INT32, 1},
    {"feature_num", SESSD_FIELD_INT32, 1}, {"out_shape", SESSD_FIELD_INT32, 3}, {"spatial_shape", SESSD_FIELD_INT32, 3},
    {"ksize", SESSD_FIELD_INT32, 3},      {"stride", SESSD_FIELD_INT32, 3},     {"padding", SESSD_FIELD_INT32, 3},
    {"dilation", SESSD_FIELD_INT32, 1},   {"out_padding", SESSD_FIELD_INT32, 1}, {"weights", SESSD_FIELD_FLOAT32, 0}};
const FieldSpec kDenseFields[] = {  // sparse2Dense.cu:321-322
    {"feature_map_size", SESSD_FIELD_INT32, 3}, {"feature_map_channel", SESSD_FIELD_INT32, 1}};

struct Registry {
    const char* plugin_name;
    const FieldSpec* specs;
    int n;
    sessd_plugin_field fields[12];
    sessd_plugin_field_collection fc;
};

template <int N>
Registry make_registry(const char* name, const FieldSpec (&specs)[N]) {
    Registry r;
    r.plugin_name = name;
    r.specs = specs;
    r.n = N;
    for (int i = 0; i < N; ++i) r.fields[i] = sessd_plugin_field{specs[i].name, nullptr, specs[i].type, specs[i].length};
    r.fc.nbFields = N;
    r.fc.fields = nullptr;  // set by registry(): the array lives in the static object
    return r;
}

Registry* registry(const char* plugin_name) {
    static Registry all[4] = {make_registry("VoxelGeneratorPlugin", kVoxelGenFields),
                              make_registry("SubmConv3dLayerPlugin", kSubmFields),
                              make_registry("SparseConv3dLayerPlugin", kSparseFields),
                              make_registry("Sparse2DensePlugin", kDenseFields)};
    if (!plugin_name) return nullptr;
    for (Registry& r : all)
        if (!std::strcmp(r.plugin_name, plugin_name)) {
            r.fc.fields = r.fields;
            return &r;
        }
    return nullptr;
}

// the field `name` of the collection, checked against what the creator reads: type and a length that covers it
// (a length of 1 on an array field is accepted: the reference's creators declare every field with length 1 and
// read 3 or 6 elements all the same)
int find_field(const sessd_plugin_field_collection* fc, const Registry& r, const char* name, const void** data,
               int32_t* length) {
    const FieldSpec* spec = nullptr;
    for (int i = 0; i < r.n; ++i)
        if (!std::strcmp(r.specs[i].name, name)) spec = &r.specs[i];
    for (int i = 0; i < fc->nbFields; ++i) {
        const sessd_plugin_field& f = fc->fields[i];
        if (!f.name || std::strcmp(f.name, name)) continue;
        if (!f.data) return fail(SESSD_E_INVALID, "%s: field '%s' has no data", r.plugin_name, name);
        if (spec && f.type != spec->type)
            return fail(SESSD_E_INVALID, "%s: field '%s' has type %d, the creator reads type %d", r.plugin_name, name, f.type,
                        spec->type);
        if (spec && spec->length > 1 && f.length != 1 && f.length < spec->length)
            return fail(SESSD_E_INVALID, "%s: field '%s' declares %d elements, the creator reads %d", r.plugin_name, name,
                        f.length, spec->length);
        *data = f.data;
        if (length) *length = f.length;
        return SESSD_OK;
    }
    return fail(SESSD_E_INVALID, "%s: field '%s' is missing", r.plugin_name, name);
}

int get_ints(const sessd_plugin_field_collection* fc, const Registry& r, const char* name, int32_t* dst, int count) {
    const void* p = nullptr;
    SESSD_TRY(find_field(fc, r, name, &p, nullptr));
    std::memcpy(dst, p, sizeof(int32_t) * (size_t)count);
    return SESSD_OK;
}

int get_floats(const sessd_plugin_field_collection* fc, const Registry& r, const char* name, float* dst, int count) {
    const void* p = nullptr;
    SESSD_TRY(find_field(fc, r, name, &p, nullptr));
    std::memcpy(dst, p, sizeof(float) * (size_t)count);
    return SESSD_OK;
}

// the `weights` field: FP32 [K][Cin][Cout]; a length other than 0 or 1 (the reference declares 1) must be the element count
int get_weights(const sessd_plugin_field_collection* fc, const Registry& r, int64_t expect, const float** w) {
    const void* p = nullptr;
    int32_t length = 0;
    SESSD_TRY(find_field(fc, r, "weights", &p, &length));
    if (length > 1 && length != expect)
        return fail(SESSD_E_INVALID, "%s: field 'weights' holds %d values, the layer shape needs %lld", r.plugin_name, length,
                    (long long)expect);
    *w = static_cast<const float*>(p);
    return SESSD_OK;
}

}  // namespace
}  // namespace sessd

using namespace sessd;

template <typename P>
static int clone_conv(const P* src, P** out) {
    std::vector<char> blob(src->getSerializationSize());
    src->serialize(blob.data());
    P* p = nullptr;
    SESSD_TRY(P::deserialize(blob.data(), blob.size(), &p));
    p->flags_ = src->flags_;
    p->in_type_ = src->in_type_;
    p->out_type_ = src->out_type_;
    const int rc = p->preparePackedForTypes();
    if (rc != SESSD_OK) {
        delete p;
        return rc;
    }
    *out = p;
    return SESSD_OK;
}

extern "C" {

const sessd_plugin_field_collection* sessd_plugin_field_names(const char* plugin_name) {
    Registry* r = registry(plugin_name);
    if (!r) {
        fail(SESSD_E_INVALID, "no plugin named '%s'", plugin_name ? plugin_name : "(null)");
        return nullptr;
    }
    return &r->fc;
}

static int plugin_create_unguarded(const char* plugin_name, const sessd_plugin_field_collection* fc, void** handle) {
    if (!plugin_name || !fc || !handle || (fc->nbFields > 0 && !fc->fields) || fc->nbFields < 0)
        return fail(SESSD_E_INVALID, "plugin_create: null argument");
    const Registry* rp = registry(plugin_name);
    if (!rp) return fail(SESSD_E_INVALID, "plugin_create: no plugin named '%s'", plugin_name);
    const Registry& r = *rp;
    if (r.specs == kVoxelGenFields) {
        sessd_voxelgen_desc d;
        std::memset(&d, 0, sizeof(d));
        SESSD_TRY(get_ints(fc, r, "max_num_points_per_voxel", &d.max_num_points_per_voxel, 1));
        SESSD_TRY(get_ints(fc, r, "max_voxels", &d.max_voxels, 1));
        SESSD_TRY(get_floats(fc, r, "point_cloud_range", d.point_cloud_range, 6));
        SESSD_TRY(get_ints(fc, r, "voxel_feature_num", &d.voxel_feature_num, 1));
        SESSD_TRY(get_floats(fc, r, "voxel_size", d.voxel_size, 3));
        return sessd_voxelgen_create(&d, reinterpret_cast<sessd_voxelgen**>(handle));
    }
    if (r.specs == kDenseFields) {
        sessd_sparse2dense_desc d;
        std::memset(&d, 0, sizeof(d));
        SESSD_TRY(get_ints(fc, r, "feature_map_size", d.feature_map_size, 3));
        SESSD_TRY(get_ints(fc, r, "feature_map_channel", &d.feature_map_channel, 1));
        return sessd_sparse2dense_create(&d, reinterpret_cast<sessd_sparse2dense**>(handle));
    }
    if (r.specs == kSubmFields) {
        sessd_submconv3d_desc d;
        std::memset(&d, 0, sizeof(d));
        SESSD_TRY(get_ints(fc, r, "in_channel", &d.in_channel, 1));
        SESSD_TRY(get_ints(fc, r, "out_channel", &d.out_channel, 1));
        SESSD_TRY(get_ints(fc, r, "max_voxels", &d.max_voxels, 1));
        SESSD_TRY(get_ints(fc, r, "feature_num", &d.feature_num, 1));
        SESSD_TRY(get_ints(fc, r, "out_shape", d.out_shape, 3));
        SESSD_TRY(get_ints(fc, r, "spatial_shape", d.spatial_shape, 3));
        SESSD_TRY(get_ints(fc, r, "ksize", &d.ksize, 1));
        SESSD_TRY(get_ints(fc, r, "stride", &d.stride, 1));
        SESSD_TRY(get_ints(fc, r, "padding", &d.padding, 1));
        SESSD_TRY(get_ints(fc, r, "dilation", &d.dilation, 1));
        SESSD_TRY(get_ints(fc, r, "out_padding", &d.out_padding, 1));
        if (d.in_channel <= 0 || d.out_channel <= 0 || d.ksize <= 0 || d.ksize > 3)
            return fail(SESSD_E_INVALID, "%s: in_channel, out_channel and ksize (1..3) must be positive", r.plugin_name);
        const float* w = nullptr;
        SESSD_TRY(get_weights(fc, r, (int64_t)d.in_channel * d.out_channel * d.ksize * d.ksize * d.ksize, &w));  // :866
        return sessd_submconv3d_create(&d, w, reinterpret_cast<sessd_submconv3d**>(handle));
    }
    sessd_sparseconv3d_desc d;
    std::memset(&d, 0, sizeof(d));
    SESSD_TRY(get_ints(fc, r, "in_channel", &d.in_channel, 1));
    SESSD_TRY(get_ints(fc, r, "out_channel", &d.out_channel, 1));
    SESSD_TRY(get_ints(fc, r, "max_voxels", &d.max_voxels, 1));
    SESSD_TRY(get_ints(fc, r, "feature_num", &d.feature_num, 1));
    SESSD_TRY(get_ints(fc, r, "out_shape", d.out_shape, 3));
    SESSD_TRY(get_ints(fc, r, "spatial_shape", d.spatial_shape, 3));
    SESSD_TRY(get_ints(fc, r, "ksize", d.ksize, 3));
    SESSD_TRY(get_ints(fc, r, "stride", d.stride, 3));
    SESSD_TRY(get_ints(fc, r, "padding", d.padding, 3));
    SESSD_TRY(get_ints(fc, r, "dilation", &d.dilation, 1));
    SESSD_TRY(get_ints(fc, r, "out_padding", &d.out_padding, 1));
    for (int a = 0; a < 3; ++a)
        if (d.ksize[a] <= 0 || d.ksize[a] > 3)
            return fail(SESSD_E_INVALID, "%s: ksize must be 1..3 on every axis", r.plugin_name);
    if (d.in_channel <= 0 || d.out_channel <= 0) return fail(SESSD_E_INVALID, "%s: channels must be positive", r.plugin_name);
    const float* w = nullptr;
    SESSD_TRY(get_weights(fc, r, (int64_t)d.in_channel * d.out_channel * d.ksize[0] * d.ksize[1] * d.ksize[2], &w));  // :1065
    return sessd_sparseconv3d_create(&d, w, reinterpret_cast<sessd_sparseconv3d**>(handle));
}

int sessd_plugin_create(const char* plugin_name, const sessd_plugin_field_collection* fc, void** handle) {
    return guarded(__func__, [&]() -> int { return plugin_create_unguarded(plugin_name, fc, handle); });
}

// clone(): the reference builds a new plugin from the members of the old one, device weights included
// (submConv3dlayer.cu:188-196); here the copy also carries what this library adds to a plugin (epilogue, flags,
// the configured tensor types, the dense border).  The serialised form is the member list, so a clone is a
// deserialisation of it plus the members that are not serialised.
int sessd_voxelgen_clone(const sessd_voxelgen* h, sessd_voxelgen** out) {
    if (!h || !out) return fail(SESSD_E_INVALID, "voxelgen_clone: null argument");
    return guarded(__func__, [&]() -> int {
        const auto* src = reinterpret_cast<const VoxelGeneratorPlugin*>(h);
        std::vector<char> blob(src->getSerializationSize());
        src->serialize(blob.data());
        VoxelGeneratorPlugin* p = nullptr;
        SESSD_TRY(VoxelGeneratorPlugin::deserialize(blob.data(), blob.size(), &p));
        p->flags_ = src->flags_;
        p->lastMaxPoints_ = src->lastMaxPoints_;
        *out = reinterpret_cast<sessd_voxelgen*>(p);
        return SESSD_OK;
    });
}

int sessd_submconv3d_clone(const sessd_submconv3d* h, sessd_submconv3d** out) {
    if (!h || !out) return fail(SESSD_E_INVALID, "submconv3d_clone: null argument");
    return guarded(__func__, [&]() -> int {
        return clone_conv(reinterpret_cast<const SubmConv3dLayerPlugin*>(h), reinterpret_cast<SubmConv3dLayerPlugin**>(out));
    });
}

int sessd_sparseconv3d_clone(const sessd_sparseconv3d* h, sessd_sparseconv3d** out) {
    if (!h || !out) return fail(SESSD_E_INVALID, "sparseconv3d_clone: null argument");
    return guarded(__func__, [&]() -> int {
        return clone_conv(reinterpret_cast<const SparseConv3dLayerPlugin*>(h), reinterpret_cast<SparseConv3dLayerPlugin**>(out));
    });
}

int sessd_sparse2dense_clone(const sessd_sparse2dense* h, sessd_sparse2dense** out) {
    if (!h || !out) return fail(SESSD_E_INVALID, "sparse2dense_clone: null argument");
    return guarded(__func__, [&]() -> int {
        const auto* src = reinterpret_cast<const Sparse2DensePlugin*>(h);
        std::vector<char> blob(src->getSerializationSize());
        src->serialize(blob.data());
        Sparse2DensePlugin* p = nullptr;
        SESSD_TRY(Sparse2DensePlugin::deserialize(blob.data(), blob.size(), &p));
        p->in_type_ = src->in_type_;
        p->out_type_ = src->out_type_;
        *out = reinterpret_cast<sessd_sparse2dense*>(p);
        return SESSD_OK;
    });
}

}  // extern "C"
