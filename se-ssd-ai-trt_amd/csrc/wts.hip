// wts.hip -- host side only: the reference's `.wts` weight file, BatchNorm folding, and a pipeline
// built from such a file.
//
// File format (writer: tools/gen_wts.py:86-99, reader: se-ssd-ai-trt.cpp:276-314): text; the first token
// is the number of blobs, then per blob `name count` followed by `count` tokens of 8 hex digits, each the
// IEEE-754 bits of one float, most significant byte first (struct.pack('>f', v).hex()).  The reference
// reader parses every token with `>> std::hex` into a uint32_t and reinterprets it as float, and asserts
// on a missing file or a non-positive count; here every malformed input is an error code.
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <new>
#include <memory>
#include <string>
#include <vector>

#include "common.h"

struct sessd_wts {
    std::vector<std::string> names;  // file order
    std::map<std::string, std::vector<float>> blobs;
};

namespace sessd {
namespace {

struct Tokens {
    const char* p;
    const char* end;
    // next whitespace-delimited token -> [b, e); false at the end of the file
    bool next(const char** b, const char** e) {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t' || *p == '\f' || *p == '\v')) ++p;
        if (p >= end) return false;
        *b = p;
        while (p < end && !(*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t' || *p == '\f' || *p == '\v')) ++p;
        *e = p;
        return true;
    }
};

bool parse_decimal(const char* b, const char* e, int64_t* out) {
    if (b == e) return false;
    bool neg = false;
    if (*b == '-' || *b == '+') {
        neg = *b == '-';
        ++b;
        if (b == e) return false;
    }
    int64_t v = 0;
    for (; b < e; ++b) {
        if (*b < '0' || *b > '9') return false;
        v = v * 10 + (*b - '0');
        if (v > (int64_t)1 << 40) return false;
    }
    *out = neg ? -v : v;
    return true;
}

// 1..8 hex digits (an optional 0x prefix is accepted as `>> std::hex` does) -> the 32-bit pattern
bool parse_hex32(const char* b, const char* e, uint32_t* out) {
    if (e - b > 2 && b[0] == '0' && (b[1] == 'x' || b[1] == 'X')) b += 2;
    if (b == e || e - b > 8) return false;
    uint32_t v = 0;
    for (; b < e; ++b) {
        const char c = *b;
        uint32_t d;
        if (c >= '0' && c <= '9') d = c - '0';
        else if (c >= 'a' && c <= 'f') d = 10 + c - 'a';
        else if (c >= 'A' && c <= 'F') d = 10 + c - 'A';
        else return false;
        v = (v << 4) | d;
    }
    *out = v;
    return true;
}

// middle_conv indices of the reference's 14 conv layers (se-ssd-ai-trt.cpp:1147-1249); BatchNorm of conv i
// is middle_conv.(i+1)
const int32_t kReferenceConvIndex[14] = {0, 3, 6, 9, 12, 15, 18, 21, 24, 27, 30, 33, 36, 39};

}  // namespace
}  // namespace sessd

using namespace sessd;

extern "C" {

int sessd_wts_parse(const char* text, size_t length, sessd_wts** out) {
    if (!text || !out) return fail(SESSD_E_INVALID, "wts_parse: null argument");
    Tokens t{text, text + length};
    const char *b, *e;
    int64_t count = 0;
    if (!t.next(&b, &e) || !parse_decimal(b, e, &count) || count <= 0)
        return fail(SESSD_E_INVALID, "wts: the file must start with a positive blob count");
    std::unique_ptr<sessd_wts> w(new sessd_wts());
    for (int64_t i = 0; i < count; ++i) {
        if (!t.next(&b, &e)) return fail(SESSD_E_INVALID, "wts: %lld blobs announced, %lld found", (long long)count, (long long)i);
        std::string name(b, e);
        int64_t size = 0;
        if (!t.next(&b, &e) || !parse_decimal(b, e, &size) || size < 0)
            return fail(SESSD_E_INVALID, "wts: blob '%s' has no valid element count", name.c_str());
        // every element is a token of at least one character behind a separator: a count the rest of the text cannot
        // hold is refused before anything of that size is allocated
        if (size > (int64_t)(t.end - t.p + 1) / 2)
            return fail(SESSD_E_INVALID, "wts: blob '%s' announces %lld elements, the file ends before that", name.c_str(),
                        (long long)size);
        std::vector<float> v;
        try {
            v.resize((size_t)size);
        } catch (const std::bad_alloc&) {
            return fail(SESSD_E_NOMEM, "wts: blob '%s': no memory for %lld elements", name.c_str(), (long long)size);
        }
        for (int64_t x = 0; x < size; ++x) {
            uint32_t bits;
            if (!t.next(&b, &e) || !parse_hex32(b, e, &bits))
                return fail(SESSD_E_INVALID, "wts: blob '%s': element %lld of %lld is missing or not 32-bit hex",
                            name.c_str(), (long long)x, (long long)size);
            std::memcpy(&v[(size_t)x], &bits, 4);
        }
        if (!w->blobs.count(name)) w->names.push_back(name);
        w->blobs[name] = std::move(v);  // a repeated name replaces the earlier blob, as map assignment does (:308)
    }
    *out = w.release();
    return SESSD_OK;
}

int sessd_wts_load(const char* path, sessd_wts** out) {
    if (!path || !out) return fail(SESSD_E_INVALID, "wts_load: null argument");
    FILE* f = std::fopen(path, "rb");
    if (!f) return fail(SESSD_E_INVALID, "wts_load: cannot open '%s': %s", path, std::strerror(errno));
    std::string text;
    char buf[1 << 16];
    size_t n;
    while ((n = std::fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, n);
    const bool bad = std::ferror(f) != 0;
    std::fclose(f);
    if (bad) return fail(SESSD_E_INVALID, "wts_load: read error on '%s'", path);
    return sessd_wts_parse(text.data(), text.size(), out);
}

int sessd_wts_count(const sessd_wts* w) { return w ? (int)w->names.size() : 0; }

int sessd_wts_name(const sessd_wts* w, int index, const char** name) {
    if (!w || !name || index < 0 || index >= (int)w->names.size()) return fail(SESSD_E_INVALID, "wts_name: bad argument");
    *name = w->names[(size_t)index].c_str();
    return SESSD_OK;
}

int sessd_wts_find(const sessd_wts* w, const char* name, const float** values, int64_t* count) {
    if (!w || !name || !values || !count) return fail(SESSD_E_INVALID, "wts_find: null argument");
    auto it = w->blobs.find(name);
    if (it == w->blobs.end()) return fail(SESSD_E_INVALID, "wts: no blob named '%s'", name);
    *values = it->second.data();
    *count = (int64_t)it->second.size();
    return SESSD_OK;
}

void sessd_wts_destroy(sessd_wts* w) { delete w; }

// se-ssd-ai-trt.cpp:808-824.  All FP32: the reference's translation unit is `using namespace std` with
// <cmath>, so sqrt on a float is the float overload.
int sessd_fold_batchnorm(const float* gamma, const float* beta, const float* mean, const float* var, int32_t n,
                         float eps, float* scale, float* shift) {
    if (!gamma || !beta || !mean || !var || !scale || !shift || n < 0)
        return fail(SESSD_E_INVALID, "fold_batchnorm: bad argument");
    for (int i = 0; i < n; ++i) {
        scale[i] = gamma[i] / sqrtf(var[i] + eps);
        shift[i] = beta[i] - mean[i] * gamma[i] / sqrtf(var[i] + eps);
    }
    return SESSD_OK;
}

int sessd_pipeline_create_from_wts(const sessd_pipeline_desc* desc, const sessd_wts* wts, const char* prefix,
                                   const int32_t* conv_index, float eps, sessd_pipeline** out) {
    if (!desc || !wts || !out) return fail(SESSD_E_INVALID, "pipeline_create_from_wts: null argument");
    const int L = desc->n_layers;
    if (L <= 0 || !desc->layers) return fail(SESSD_E_INVALID, "pipeline_create_from_wts: the desc has no layers");
    if (!conv_index) {
        if (L != 14)
            return fail(SESSD_E_INVALID, "pipeline_create_from_wts: conv_index may be NULL only for the reference's 14 layers");
        conv_index = kReferenceConvIndex;
    }
    const std::string pre = prefix ? prefix : "backbone.middle_conv.";
    std::vector<const float*> w((size_t)L), sc((size_t)L), sh((size_t)L);
    std::vector<std::vector<float>> scale((size_t)L), shift((size_t)L);
    for (int l = 0; l < L; ++l) {
        const sessd_layer_spec& s = desc->layers[l];
        const int64_t kvol = (int64_t)s.ksize[0] * s.ksize[1] * s.ksize[2];
        const std::string conv = pre + std::to_string(conv_index[l]) + ".weight";
        const std::string bn = pre + std::to_string(conv_index[l] + 1);
        int64_t n = 0;
        SESSD_TRY(sessd_wts_find(wts, conv.c_str(), &w[(size_t)l], &n));
        if (n != kvol * s.in_channel * s.out_channel)
            return fail(SESSD_E_INVALID, "wts: '%s' has %lld elements, layer %d needs %lld x %d x %d", conv.c_str(),
                        (long long)n, l, (long long)kvol, s.in_channel, s.out_channel);
        const float* p[4];
        const char* key[4] = {".weight", ".bias", ".running_mean", ".running_var"};
        for (int j = 0; j < 4; ++j) {
            SESSD_TRY(sessd_wts_find(wts, (bn + key[j]).c_str(), &p[j], &n));
            if (n != s.out_channel)
                return fail(SESSD_E_INVALID, "wts: '%s%s' has %lld elements, layer %d has %d output channels", bn.c_str(),
                            key[j], (long long)n, l, s.out_channel);
        }
        scale[(size_t)l].resize((size_t)s.out_channel);
        shift[(size_t)l].resize((size_t)s.out_channel);
        SESSD_TRY(sessd_fold_batchnorm(p[0], p[1], p[2], p[3], s.out_channel, eps, scale[(size_t)l].data(),
                                       shift[(size_t)l].data()));
        sc[(size_t)l] = scale[(size_t)l].data();
        sh[(size_t)l] = shift[(size_t)l].data();
    }
    sessd_pipeline_desc d = *desc;
    d.weights = w.data();
    d.scale = sc.data();
    d.shift = sh.data();
    d.relu = 1;
    return sessd_pipeline_create(&d, out);
}

}  // extern "C"
