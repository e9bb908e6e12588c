// GGUF v2/v3 parser (crates/slai/src/gguf.rs:504-765) and its C-ABI accessors.
#include "host_gguf.h"
#include "common.h"
#include "quant_formats.h"

#include <cerrno>
#include <cstdio>
#include <cstring>
#include <iterator>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace slai {
namespace {

struct Reader {
    const uint8_t *b; size_t len; size_t off = 0; bool bad = false;
    template <class T> T pod() {              // gguf.rs:720-725 read_pod
        T v{};
        if (bad || off + sizeof(T) > len) { bad = true; return v; }
        memcpy(&v, b + off, sizeof(T)); off += sizeof(T);
        return v;
    }
    std::string str() {                       // gguf.rs:714-718 read_string
        uint64_t n = pod<uint64_t>();
        if (bad || n > len - off) { bad = true; return {}; }
        std::string s((const char *)b + off, (size_t)n); off += (size_t)n;
        return s;
    }
};

size_t scalar_size(uint32_t t) {
    switch (t) { case 0: case 1: case 7: return 1; case 2: case 3: return 2; case 4: case 5: case 6: return 4;
                 case 10: case 11: case 12: return 8; default: return 0; }
}

// gguf.rs:463-500 read_array: skip over the payload, remembering nothing but its extent
bool skip_array(Reader &r, uint32_t et, uint64_t n, std::string &err) {
    if (et > 12) { err = "metadata value of type " + std::to_string(et) + " is not part of the supported gguf version"; return false; }
    if (et == 8) { for (uint64_t i = 0; i < n && !r.bad; ++i) r.str(); return true; }
    if (et == 9) {
        for (uint64_t i = 0; i < n && !r.bad; ++i) {
            uint32_t t = r.pod<uint32_t>(); uint64_t l = r.pod<uint64_t>();
            if (!skip_array(r, t, l, err)) return false;
        }
        return true;
    }
    size_t sz = scalar_size(et);
    if (n > (r.len - r.off) / (sz ? sz : 1)) { r.bad = true; return true; }
    r.off += sz * (size_t)n;
    return true;
}

}  // namespace

int Gguf::parse(const uint8_t *data, size_t n, std::string &err) {
    bytes = data; len = n;
    Reader r{data, n};
    uint32_t magic = r.pod<uint32_t>();
    if (r.bad) { err = "truncated file"; return SLAI_E_PARSE; }
    if (magic != 0x46554747u && magic != 0x47475546u) {   // gguf.rs:21-22,529-531
        char buf[128];
        snprintf(buf, sizeof buf, "the input file isn't a ggml binary file. Got a magic number of %#x instead of 0x46554747 or 0x47475546.", magic);
        err = buf; return SLAI_E_PARSE;
    }
    version = r.pod<uint32_t>();
    uint64_t tensor_count = r.pod<uint64_t>(), metadata_count = r.pod<uint64_t>();
    if (r.bad || tensor_count > n || metadata_count > n) { err = "truncated file"; return SLAI_E_PARSE; }
    for (uint64_t i = 0; i < metadata_count; ++i) {      // gguf.rs:544-557
        std::string key = r.str();
        GgufMetaValue v;
        v.type = r.pod<uint32_t>();
        if (r.bad) { err = "truncated file"; return SLAI_E_PARSE; }
        if (v.type > 12) { err = "metadata value of type " + std::to_string(v.type) + " is not part of the supported gguf version"; return SLAI_E_PARSE; }
        switch (v.type) {
        case 0: v.u = r.pod<uint8_t>(); break;
        case 1: v.i = r.pod<int8_t>(); break;
        case 2: v.u = r.pod<uint16_t>(); break;
        case 3: v.i = r.pod<int16_t>(); break;
        case 4: v.u = r.pod<uint32_t>(); break;
        case 5: v.i = r.pod<int32_t>(); break;
        case 6: v.f = r.pod<float>(); break;
        case 7: v.u = r.pod<uint8_t>() != 0; break;       // gguf.rs:451
        case 8: v.s = r.str(); break;
        case 9:
            v.arr_type = r.pod<uint32_t>(); v.arr_len = r.pod<uint64_t>(); v.arr_offset = r.off;
            if (!skip_array(r, v.arr_type, v.arr_len, err)) return SLAI_E_PARSE;
            break;
        case 10: v.u = r.pod<uint64_t>(); break;
        case 11: v.i = r.pod<int64_t>(); break;
        case 12: v.f = r.pod<double>(); break;
        }
        if (r.bad) { err = "truncated file"; return SLAI_E_PARSE; }
        metadata[key] = v;                                // HashMap::insert: the last duplicate wins
    }
    // gguf.rs:508-516: only a U32 `general.alignment` overrides the default 32
    auto al = metadata.find("general.alignment");
    alignment = (al != metadata.end() && al->second.type == 4 && al->second.u) ? (uint32_t)al->second.u : 32;
    tensors.reserve((size_t)tensor_count);
    for (uint64_t i = 0; i < tensor_count; ++i) {        // gguf.rs:559-593
        GgufTensorInfo t;
        t.name = r.str();
        t.ndims = r.pod<uint32_t>();
        if (r.bad) { err = "truncated file"; return SLAI_E_PARSE; }
        if (t.ndims > 4) { err = "Tensors of dimensions larger than 4 are not supported yet."; return SLAI_E_PARSE; }
        for (uint32_t d = 0; d < t.ndims; ++d) t.dims[d] = r.pod<uint64_t>();
        std::swap(t.dims[0], t.dims[1]);                  // gguf.rs:579-581
        t.type = r.pod<uint32_t>();
        t.offset = r.pod<uint64_t>();
        if (r.bad) { err = "truncated file"; return SLAI_E_PARSE; }
        if (t.type > 29) { err = "tensor of type " + std::to_string(t.type) + " is not part of the supported gguf version"; return SLAI_E_PARSE; }
        tensors.push_back(t);
    }
    data_start = r.off + (alignment - (r.off % alignment)) % alignment;   // gguf.rs:596,763-765
    for (size_t i = 0; i < tensors.size(); ++i) {
        GgufTensorInfo &t = tensors[i];
        t.offset += data_start;
        // element counts per block as in gguf.rs:604-673; Q4_1/Q5_0/Q5_1/Q8_K are located but have no device kernels
        uint64_t be = 0, bb = 0;
        switch (t.type) {
        case 0: be = 1; bb = 4; break;   case 1: be = 1; bb = 2; break;
        case 2: be = 32; bb = 18; break; case 3: be = 32; bb = 20; break;
        case 6: be = 32; bb = 22; break; case 7: be = 32; bb = 24; break;
        case 8: be = 32; bb = 34; break; case 12: be = 256; bb = 144; break;
        case 13: be = 256; bb = 176; break; case 14: be = 256; bb = 210; break;
        case 15: be = 256; bb = 292; break;
        default: break;
        }
        if (be) {
            uint64_t count = t.dims[0] * t.dims[1] * t.dims[2] * t.dims[3];
            t.nbytes = count / be * bb;
            if (t.offset > n || t.nbytes > n - t.offset) { err = "tensor '" + t.name + "' extends past the end of the file"; return SLAI_E_PARSE; }
        }
        tensor_index[t.name] = i;
    }
    return SLAI_OK;
}

const GgufTensorInfo *Gguf::find(const std::string &name) const {
    auto it = tensor_index.find(name);
    return it == tensor_index.end() ? nullptr : &tensors[it->second];
}
const GgufMetaValue *Gguf::meta(const std::string &key) const {
    auto it = metadata.find(key);
    return it == metadata.end() ? nullptr : &it->second;
}

}  // namespace slai

using namespace slai;

SLAI_EXPORT int slai_gguf_parse(const void *bytes, size_t len, slai_gguf **out, char *err, size_t err_len) {
    if (!bytes || !out) return SLAI_E_ARG;
    *out = nullptr;
    slai_gguf *g = new slai_gguf();
    std::string e;
    int rc = g->g.parse((const uint8_t *)bytes, len, e);
    if (rc) {
        if (err && err_len) { snprintf(err, err_len, "%s", e.c_str()); }
        delete g;
        return rc;
    }
    *out = g;
    return SLAI_OK;
}
// slai-chat/src/cli.rs:43-57: the model file is mapped, not read; tensor data is then uploaded straight from the
// mapping.  The mapping lives as long as the handle.
SLAI_EXPORT int slai_gguf_open_file(const char *path, slai_gguf **out, char *err, size_t err_len) {
    if (!path || !out) return SLAI_E_ARG;
    *out = nullptr;
    auto fail = [&](const std::string &m, int rc) { if (err && err_len) snprintf(err, err_len, "%s", m.c_str()); return rc; };
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail(std::string("unable to open '") + path + "': " + strerror(errno), SLAI_E_IO);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) { close(fd); return fail(std::string("'") + path + "' is empty or cannot be examined", SLAI_E_PARSE); }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return fail(std::string("unable to map '") + path + "': " + strerror(errno), SLAI_E_IO);
    slai_gguf *g = new slai_gguf();
    g->map = map; g->map_len = (size_t)st.st_size;
    std::string e;
    const int rc = g->g.parse((const uint8_t *)map, g->map_len, e);
    if (rc) { slai_gguf_free(g); return fail(e, rc); }
    *out = g;
    return SLAI_OK;
}
SLAI_EXPORT void slai_gguf_free(slai_gguf *g) {
    if (!g) return;
    if (g->map) munmap(g->map, g->map_len);
    delete g;
}
SLAI_EXPORT uint32_t slai_gguf_version(const slai_gguf *g) { return g ? g->g.version : 0; }
SLAI_EXPORT uint64_t slai_gguf_tensor_count(const slai_gguf *g) { return g ? g->g.tensors.size() : 0; }
SLAI_EXPORT uint64_t slai_gguf_metadata_count(const slai_gguf *g) { return g ? g->g.metadata.size() : 0; }
SLAI_EXPORT uint64_t slai_gguf_data_start(const slai_gguf *g) { return g ? g->g.data_start : 0; }

SLAI_EXPORT int slai_gguf_tensor_info(const slai_gguf *g, uint64_t i, const char **name, uint64_t dims[4], uint32_t *ggml_type,
                                      uint64_t *offset) {
    if (!g || i >= g->g.tensors.size()) return SLAI_E_ARG;
    const GgufTensorInfo &t = g->g.tensors[(size_t)i];
    if (name) *name = t.name.c_str();
    if (dims) for (int d = 0; d < 4; ++d) dims[d] = t.dims[d];
    if (ggml_type) *ggml_type = t.type;
    if (offset) *offset = t.offset;
    return SLAI_OK;
}
SLAI_EXPORT int slai_gguf_find_tensor(const slai_gguf *g, const char *name, uint64_t *index) {
    if (!g || !name) return SLAI_E_ARG;
    auto it = g->g.tensor_index.find(name);
    if (it == g->g.tensor_index.end()) return SLAI_E_MISSING;
    if (index) *index = it->second;
    return SLAI_OK;
}
// gguf.rs:284-290 `unwrap_u32`: only a U32 value qualifies
SLAI_EXPORT int slai_gguf_meta_u32(const slai_gguf *g, const char *key, uint32_t *out) {
    if (!g || !key || !out) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 4) return SLAI_E_TYPE;
    *out = (uint32_t)v->u;
    return SLAI_OK;
}
// gguf.rs:300-306 `as_f32`
SLAI_EXPORT int slai_gguf_meta_f32(const slai_gguf *g, const char *key, float *out) {
    if (!g || !key || !out) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 6) return SLAI_E_TYPE;
    *out = (float)v->f;
    return SLAI_OK;
}
// gguf.rs:308-314 `as_string`
SLAI_EXPORT int slai_gguf_meta_str(const slai_gguf *g, const char *key, const char **out) {
    if (!g || !key || !out) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 8) return SLAI_E_TYPE;
    *out = v->s.c_str();
    return SLAI_OK;
}
// gguf.rs:292-298 `unwrap_array_len`
SLAI_EXPORT int slai_gguf_meta_array_len(const slai_gguf *g, const char *key, uint64_t *out) {
    if (!g || !key || !out) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 9) return SLAI_E_TYPE;
    *out = v->arr_len;
    return SLAI_OK;
}

// gguf.rs:686-695 `metadata_debug_strings`: entry i (keys in sorted order; the reference's map has no order) as
// "key = value" for scalars and strings, "key = array[len]" for arrays
SLAI_EXPORT int slai_gguf_meta_describe(const slai_gguf *g, uint64_t i, char *out, size_t out_len) {
    if (!g || !out || !out_len || i >= g->g.metadata.size()) return SLAI_E_ARG;
    auto it = g->g.metadata.begin();
    std::advance(it, (size_t)i);
    const GgufMetaValue &v = it->second;
    static const char *const names[] = {"U8", "I8", "U16", "I16", "U32", "I32", "F32", "Bool", "String", "Array", "U64", "I64", "F64"};
    std::string val;
    switch (v.type) {
    case 0: case 2: case 4: case 10: val = std::string(names[v.type]) + "(" + std::to_string(v.u) + ")"; break;
    case 1: case 3: case 5: case 11: val = std::string(names[v.type]) + "(" + std::to_string(v.i) + ")"; break;
    case 6: case 12: { char b[64]; snprintf(b, sizeof b, "%s(%g)", names[v.type], v.f); val = b; break; }
    case 7: val = v.u ? "Bool(true)" : "Bool(false)"; break;
    case 8: val = "String(\"" + v.s + "\")"; break;
    default: val = "array[" + std::to_string(v.arr_len) + "]"; break;
    }
    snprintf(out, out_len, "%s = %s", it->first.c_str(), val.c_str());
    return SLAI_OK;
}

// gguf.rs:316-322 `as_string_array`: pointers into the file bytes (not NUL-terminated) and lengths of the first
// `capacity` elements; returns the element count through `count`
SLAI_EXPORT int slai_gguf_meta_array_str(const slai_gguf *g, const char *key, const char **ptrs, uint64_t *lens, uint64_t capacity,
                                         uint64_t *count) {
    if (!g || !key) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 9 || v->arr_type != 8) return SLAI_E_TYPE;
    if (count) *count = v->arr_len;
    size_t off = (size_t)v->arr_offset;
    for (uint64_t i = 0; i < v->arr_len && i < capacity; ++i) {     // extents were validated by the parse
        uint64_t n;
        memcpy(&n, g->g.bytes + off, 8); off += 8;
        if (ptrs) ptrs[i] = (const char *)g->g.bytes + off;
        if (lens) lens[i] = n;
        off += (size_t)n;
    }
    return SLAI_OK;
}
// gguf.rs:324-330 `as_f32_array`
SLAI_EXPORT int slai_gguf_meta_array_f32(const slai_gguf *g, const char *key, float *out, uint64_t capacity, uint64_t *count) {
    if (!g || !key) return SLAI_E_ARG;
    const GgufMetaValue *v = g->g.meta(key);
    if (!v) return SLAI_E_MISSING;
    if (v->type != 9 || v->arr_type != 6) return SLAI_E_TYPE;
    if (count) *count = v->arr_len;
    const uint64_t n = v->arr_len < capacity ? v->arr_len : capacity;
    if (out && n) memcpy(out, g->g.bytes + v->arr_offset, (size_t)n * sizeof(float));
    return SLAI_OK;
}

// gguf.rs:357-366 `GgufTensor::to_gpu_matrix` -> gguf.rs:133-194: packed upload, row-major,
// without the reference's even-block-count / ncols%{64,512} conditions and f32 fallbacks.
SLAI_EXPORT int slai_gguf_tensor_to_qmat(slai_ctx *ctx, const slai_gguf *g, const char *name, slai_qmat **out) {
    return slai_gguf_tensor_to_qmat_layout(ctx, g, name, SLAI_LAYOUT_AUTO, out);
}
SLAI_EXPORT int slai_gguf_tensor_to_qmat_layout(slai_ctx *ctx, const slai_gguf *g, const char *name, int layout, slai_qmat **out) {
    if (!ctx || !g || !name || !out) return SLAI_E_ARG;
    const GgufTensorInfo *t = g->g.find(name);
    if (!t) return set_error(ctx, SLAI_E_MISSING, std::string("missing tensor '") + name + "'");
    if (t->dims[2] != 1 || t->dims[3] != 1) return set_error(ctx, SLAI_E_SHAPE, std::string("tensor '") + name + "' is not a matrix");  // gguf.rs:362-363
    if (!block_elems((int)t->type)) return set_error(ctx, SLAI_E_TYPE, std::string("tensor '") + name + "' has ggml type " + std::to_string(t->type) + " which has no device kernel");
    return slai_qmat_create_layout(ctx, t->type, (uint32_t)t->dims[0], (uint32_t)t->dims[1], g->g.bytes + t->offset, layout, out);
}
