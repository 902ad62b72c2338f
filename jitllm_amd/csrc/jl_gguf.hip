// GGUF reader: header, metadata, tensor infos, and upload of a tensor's blocks straight from the
// mapped file (host code only; no kernels).
//
// Follows the reference's parser, J/format/GGUF.java (J = src/main/java/org/beehive/jitllm):
//   :40-115   loadGGUFMetadata -- header, tensor infos, padding to the alignment, data offset
//   :297-322  readTensorInfo   -- name, n_dimensions, dimensions (ne order), type, relative offset
//   :365-392  readHeader       -- magic "GGUF", version 2 or 3, counts, key/value pairs
//   :394-474  value types and arrays (nested arrays included)
//   :511-518  getAlignment     -- general.alignment, default 32
//   :236-247  a tensor that runs past the end of the file is refused, the file never grown
// and J/format/GGMLType.java:5-54 for type ids and block geometry.  Where the reference maps each
// tensor with a 16-byte TornadoVM array header in front (:214-268), this reader hands the bare
// blocks to jl_weight_upload, which is what the device wants.
#include "jl_internal.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <map>
#include <new>
#include <string>
#include <vector>

namespace {

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF", little-endian
constexpr int kDefaultAlignment = 32;
constexpr int kMaxAlignment = 1 << 20;

// gguf_metadata_value_type
enum ValueType { U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64, VALUE_TYPES };

struct TypeGeometry {
    int bytes, elems;  // bytes per block, elements per block; bytes 0 = no layout known here
};

// J/format/GGMLType.java:5-54, by ggml type id.  Types the reference marks unreadable
// (Integer.MAX_VALUE) have no geometry here either.
TypeGeometry geometry(int type) {
    switch (type) {
        case 0: return {4, 1};       // F32
        case 1: return {2, 1};       // F16
        case 2: return {18, 32};     // Q4_0
        case 3: return {20, 32};     // Q4_1
        case 6: return {22, 32};     // Q5_0
        case 8: return {34, 32};     // Q8_0
        case 9: return {40, 32};     // Q8_1 (32 quants + two floats, as the reference sizes it)
        case 12: return {144, 256};  // Q4_K
        case 13: return {176, 256};  // Q5_K
        case 14: return {210, 256};  // Q6_K
        case 23: return {136, 256};  // IQ4_XS
        case 24: return {1, 1};      // I8
        case 25: return {2, 1};      // I16
        case 26: return {4, 1};      // I32
        case 27: return {8, 1};      // I64
        case 28: return {8, 1};      // F64
        case 30: return {2, 1};      // BF16
        case 31: case 32: case 33: return {18, 32};  // Q4_0_4_4 / _4_8 / _8_8
        default: return {0, 0};
    }
}

struct Value {
    int type = -1;          // ValueType; ARRAY: `elem_type` and `count` describe it, elements are skipped
    int64_t i = 0;          // integers and bool
    double f = 0.0;         // F32 / F64
    std::string s;          // STRING
    int elem_type = -1;
    int64_t count = 0;
};

struct TensorInfo {
    std::string name;
    int n_dims = 0;
    int64_t dims[4] = {1, 1, 1, 1};
    int type = -1;
    int64_t offset = 0;  // relative to the tensor-data section
    int64_t bytes = -1;  // -1: a type without geometry
};

}  // namespace

struct jl_gguf {
    int fd = -1;
    const uint8_t *base = nullptr;
    int64_t size = 0;
    int version = 0;
    int alignment = kDefaultAlignment;
    int64_t data_offset = 0;
    std::map<std::string, Value> metadata;
    std::vector<TensorInfo> tensors;
    std::map<std::string, int64_t> by_name;
};

namespace {

// Bounds-checked little-endian cursor over the mapped file.
struct Cursor {
    const uint8_t *base;
    int64_t size, pos = 0;
    bool ok = true;

    bool need(int64_t n) {
        if (!ok || n < 0 || pos + n > size) ok = false;
        return ok;
    }
    template <typename T> T get() {
        T v{};
        if (need((int64_t)sizeof(T))) {
            memcpy(&v, base + pos, sizeof(T));
            pos += sizeof(T);
        }
        return v;
    }
    std::string str() {
        const uint64_t len = get<uint64_t>();
        std::string s;
        if (len > (uint64_t)size || !need((int64_t)len)) {
            ok = false;
            return s;
        }
        s.assign((const char *)base + pos, (size_t)len);
        pos += (int64_t)len;
        return s;
    }
};

int scalar_bytes(int t) {
    switch (t) {
        case U8: case I8: case BOOL: return 1;
        case U16: case I16: return 2;
        case U32: case I32: case F32: return 4;
        case U64: case I64: case F64: return 8;
        default: return 0;
    }
}

// Skips the elements of an array whose element type and count have been read (GGUF.java:394-446).
bool skip_array(Cursor &c, int elem_type, uint64_t count, int depth) {
    if (depth > 8) return false;
    if (const int w = scalar_bytes(elem_type)) {
        if (count > (uint64_t)c.size) return false;
        if (!c.need((int64_t)count * w)) return false;
        c.pos += (int64_t)count * w;
        return true;
    }
    if (elem_type == STRING) {
        for (uint64_t i = 0; i < count && c.ok; i++) {
            const uint64_t len = c.get<uint64_t>();
            if (len > (uint64_t)c.size || !c.need((int64_t)len)) return false;
            c.pos += (int64_t)len;
        }
        return c.ok;
    }
    if (elem_type == ARRAY) {
        for (uint64_t i = 0; i < count && c.ok; i++) {
            const int inner = (int)c.get<uint32_t>();
            const uint64_t n = c.get<uint64_t>();
            if (!c.ok || inner < 0 || inner >= VALUE_TYPES || !skip_array(c, inner, n, depth + 1)) return false;
        }
        return c.ok;
    }
    return false;
}

bool read_value(Cursor &c, Value &v) {
    v.type = (int)c.get<uint32_t>();
    switch (v.type) {
        case U8: v.i = c.get<uint8_t>(); break;
        case I8: v.i = c.get<int8_t>(); break;
        case U16: v.i = c.get<uint16_t>(); break;
        case I16: v.i = c.get<int16_t>(); break;
        case U32: v.i = c.get<uint32_t>(); break;
        case I32: v.i = c.get<int32_t>(); break;
        case U64: v.i = (int64_t)c.get<uint64_t>(); break;
        case I64: v.i = c.get<int64_t>(); break;
        case BOOL: v.i = c.get<uint8_t>() != 0; break;
        case F32: v.f = c.get<float>(); break;
        case F64: v.f = c.get<double>(); break;
        case STRING: v.s = c.str(); break;
        case ARRAY: {
            v.elem_type = (int)c.get<uint32_t>();
            v.count = (int64_t)c.get<uint64_t>();
            if (!c.ok || v.elem_type < 0 || v.elem_type >= VALUE_TYPES) return false;
            return skip_array(c, v.elem_type, (uint64_t)v.count, 0);
        }
        default: return false;
    }
    return c.ok;
}

void close_file(jl_gguf *g) {
    if (g->base) munmap((void *)g->base, (size_t)g->size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

}  // namespace

extern "C" {

// Fills `g` from the file; the caller closes it when this fails or throws.
static int parse_file(const char *path, jl_gguf *g) {
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    if (g->fd < 0) {
        return jl_fail(JL_ERR_INVALID, "Model file not found: %s", path);
    }
    struct stat st;
    if (fstat(g->fd, &st) != 0 || st.st_size < 24) {
        return jl_fail(JL_ERR_INVALID, "%s is too short to be a GGUF file", path);
    }
    g->size = (int64_t)st.st_size;
    void *m = mmap(nullptr, (size_t)g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) {
        return jl_fail(JL_ERR_INVALID, "mapping %s failed", path);
    }
    g->base = (const uint8_t *)m;

    Cursor c{g->base, g->size};
    const uint32_t magic = c.get<uint32_t>();
    if (magic != kMagic) {
        return jl_fail(JL_ERR_INVALID, "unsupported header.magic %u", magic);
    }
    g->version = (int)c.get<uint32_t>();
    if (g->version != 2 && g->version != 3) {
        const int v = g->version;
        return jl_fail(JL_ERR_INVALID, "unsupported header.version %d", v);
    }
    const uint64_t tensor_count = c.get<uint64_t>();
    const uint64_t kv_count = c.get<uint64_t>();
    if (!c.ok || tensor_count > (uint64_t)g->size || kv_count > (uint64_t)g->size) {
        return jl_fail(JL_ERR_INVALID, "GGUF header of %s holds impossible counts", path);
    }
    for (uint64_t i = 0; i < kv_count; i++) {
        std::string key = c.str();
        Value v;
        if (!c.ok || !read_value(c, v)) {
            const long long at = (long long)c.pos;
                return jl_fail(JL_ERR_INVALID, "GGUF metadata ends early or is malformed at byte %lld", at);
        }
        g->metadata[key] = v;
    }
    auto al = g->metadata.find("general.alignment");
    if (al != g->metadata.end() && al->second.type != STRING && al->second.type != ARRAY && al->second.i > 0) {
        // range-checked as 64 bits before it is narrowed: 2^32 must not become 0
        const int64_t a = al->second.i;
        if (a > kMaxAlignment || (a & (a - 1))) {
                return jl_fail(JL_ERR_INVALID, "general.alignment %lld is not a power of two of at most %d",
                           (long long)a, kMaxAlignment);
        }
        g->alignment = (int)a;
    }
    // a tensor info takes at least 24 bytes (name length, dimension count, type, offset)
    if (tensor_count > (uint64_t)(g->size - c.pos) / 24) {
        return jl_fail(JL_ERR_INVALID, "GGUF header of %s holds impossible counts", path);
    }
    g->tensors.reserve((size_t)tensor_count);
    for (uint64_t i = 0; i < tensor_count; i++) {
        TensorInfo t;
        t.name = c.str();
        t.n_dims = (int)c.get<uint32_t>();
        if (!c.ok || t.n_dims < 0 || t.n_dims > 4) {
                return jl_fail(JL_ERR_INVALID, "GGUF tensor info %llu is malformed", (unsigned long long)i);
        }
        for (int k = 0; k < t.n_dims; k++) t.dims[k] = (int64_t)c.get<uint64_t>();
        t.type = (int)c.get<uint32_t>();
        t.offset = (int64_t)c.get<uint64_t>();
        if (!c.ok) {
                return jl_fail(JL_ERR_INVALID, "GGUF tensor infos end early at byte %lld", (long long)c.pos);
        }
        const TypeGeometry geo = geometry(t.type);
        if (geo.bytes) {
            // element count without overflow: a product past 2^62 leaves the tensor without a size,
            // and every later use refuses it
            uint64_t n = 1;
            bool fits = true;
            for (int k = 0; k < t.n_dims; k++) {
                const uint64_t dim = (uint64_t)t.dims[k];
                if (dim != 0 && n > (UINT64_C(1) << 62) / dim) fits = false;
                else n *= dim;
            }
            if (fits && n / geo.elems <= (UINT64_C(1) << 62) / geo.bytes) t.bytes = (int64_t)(n / geo.elems * geo.bytes);
        }
        g->by_name[t.name] = (int64_t)g->tensors.size();
        g->tensors.push_back(t);
    }
    // padding to the nearest multiple of the alignment, then the tensor data
    g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    return JL_OK;
}

int jl_gguf_open(const char *path, jl_gguf **out) {
    JL_REQUIRE(path && out, "jl_gguf_open: null argument");
    *out = nullptr;
    jl_gguf *g = new (std::nothrow) jl_gguf();
    JL_REQUIRE(g != nullptr, "jl_gguf_open: host allocation failed");
    int st;
    // strings, maps and the tensor table allocate: nothing may leave an extern "C" function by throwing
    try {
        st = parse_file(path, g);
    } catch (const std::bad_alloc &) {
        st = jl_fail(JL_ERR_OOM, "jl_gguf_open: out of host memory while reading %s", path);
    } catch (...) {
        st = jl_fail(JL_ERR_INVALID, "jl_gguf_open: reading %s failed", path);
    }
    if (st != JL_OK) {
        close_file(g);
        return st;
    }
    *out = g;
    return JL_OK;
}

int jl_gguf_close(jl_gguf *g) {
    if (g) close_file(g);
    return JL_OK;
}

int jl_gguf_version(const jl_gguf *g) { return g ? g->version : 0; }
int jl_gguf_alignment(const jl_gguf *g) { return g ? g->alignment : 0; }
int64_t jl_gguf_data_offset(const jl_gguf *g) { return g ? g->data_offset : -1; }
int64_t jl_gguf_tensor_count(const jl_gguf *g) { return g ? (int64_t)g->tensors.size() : -1; }
int64_t jl_gguf_metadata_count(const jl_gguf *g) { return g ? (int64_t)g->metadata.size() : -1; }

int64_t jl_gguf_find(const jl_gguf *g, const char *name) {
    if (!g || !name) return -1;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? -1 : it->second;
}

int jl_gguf_tensor_info(const jl_gguf *g, int64_t index, const char **name, int *ggml_type, int *n_dims,
                        int64_t dims[4], int64_t *file_offset, int64_t *bytes) {
    JL_REQUIRE(g != nullptr, "jl_gguf_tensor_info: file is null");
    JL_REQUIRE(index >= 0 && index < (int64_t)g->tensors.size(), "jl_gguf_tensor_info: tensor %lld of %zu",
               (long long)index, g->tensors.size());
    const TensorInfo &t = g->tensors[(size_t)index];
    if (name) *name = t.name.c_str();
    if (ggml_type) *ggml_type = t.type;
    if (n_dims) *n_dims = t.n_dims;
    if (dims)
        for (int k = 0; k < 4; k++) dims[k] = t.dims[k];
    if (file_offset) *file_offset = (t.offset < 0 || t.offset > INT64_MAX - g->data_offset) ? -1 : g->data_offset + t.offset;
    if (bytes) *bytes = t.bytes;
    return JL_OK;
}

int jl_gguf_metadata_int(const jl_gguf *g, const char *key, int64_t *value) {
    JL_REQUIRE(g && key && value, "jl_gguf_metadata_int: null argument");
    auto it = g->metadata.find(key);
    JL_REQUIRE(it != g->metadata.end(), "no metadata key %s", key);
    const int t = it->second.type;
    JL_REQUIRE(t != STRING && t != ARRAY && t != F32 && t != F64, "metadata key %s is not an integer", key);
    *value = it->second.i;
    return JL_OK;
}

int jl_gguf_metadata_float(const jl_gguf *g, const char *key, double *value) {
    JL_REQUIRE(g && key && value, "jl_gguf_metadata_float: null argument");
    auto it = g->metadata.find(key);
    JL_REQUIRE(it != g->metadata.end(), "no metadata key %s", key);
    JL_REQUIRE(it->second.type == F32 || it->second.type == F64, "metadata key %s is not a float", key);
    *value = it->second.f;
    return JL_OK;
}

int jl_gguf_metadata_string(const jl_gguf *g, const char *key, const char **value, int64_t *length) {
    JL_REQUIRE(g && key && value, "jl_gguf_metadata_string: null argument");
    auto it = g->metadata.find(key);
    JL_REQUIRE(it != g->metadata.end(), "no metadata key %s", key);
    JL_REQUIRE(it->second.type == STRING, "metadata key %s is not a string", key);
    *value = it->second.s.c_str();
    if (length) *length = (int64_t)it->second.s.size();
    return JL_OK;
}

int jl_gguf_metadata_array(const jl_gguf *g, const char *key, int *element_type, int64_t *count) {
    JL_REQUIRE(g && key, "jl_gguf_metadata_array: null argument");
    auto it = g->metadata.find(key);
    JL_REQUIRE(it != g->metadata.end(), "no metadata key %s", key);
    JL_REQUIRE(it->second.type == ARRAY, "metadata key %s is not an array", key);
    if (element_type) *element_type = it->second.elem_type;
    if (count) *count = it->second.count;
    return JL_OK;
}

int jl_gguf_upload(jl_context *ctx, const jl_gguf *g, const char *name, jl_weight **out) {
    JL_REQUIRE(g && name && out, "jl_gguf_upload: null argument");
    *out = nullptr;
    const int64_t i = jl_gguf_find(g, name);
    JL_REQUIRE(i >= 0, "no tensor %s in the file", name);
    const TensorInfo &t = g->tensors[(size_t)i];
    if (jl_block_elems(t.type) == 0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "tensor %s is ggml type %d, which has no projection kernel here",
                       name, t.type);
    }
    JL_REQUIRE(t.n_dims == 2, "tensor %s has %d dimensions, a projection weight has 2", name, t.n_dims);
    // compared as unsigned quantities against what is left of the file: a sum of offsets near
    // 2^63 would wrap and pass
    const uint64_t room = g->data_offset <= g->size ? (uint64_t)(g->size - g->data_offset) : 0;
    if (t.offset < 0 || t.bytes < 0 || (uint64_t)t.offset > room || (uint64_t)t.bytes > room - (uint64_t)t.offset) {
        return jl_fail(JL_ERR_INVALID, "tensor %s (%s, %lld bytes) runs past the end of the file", name,
                       jl_type_name(t.type), (long long)t.bytes);
    }
    // (the file's own faults are reported before a missing context is)
    JL_REQUIRE(ctx != nullptr, "jl_gguf_upload: null context");
    // GGUF dimensions are in ne order: dims[0] is the row length (the sum below is in range: checked above)
    const int64_t begin = g->data_offset + t.offset;
    return jl_weight_upload(ctx, t.type, g->base + begin, t.dims[1], t.dims[0], out);
}

}  // extern "C"
