// GGUF container reader (host code only): GgufMetadata::read, fusor-ml/gguf/src/lib.rs:559-613, the value
// conversions of :544-556, the suffix lookup of :301-311, tensor byte sizes of :262-286 and the VarBuilder
// tensor fetch of fusor-ml/fusor/src/varbuilder.rs:79-127.  The file is mapped read-only; metadata strings
// and tensor payloads are handed out as pointers into the mapping.
#include "fh_internal.h"

#include <cerrno>
#include <cstring>
#include <fcntl.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

namespace {

// GgufMetadataValueType, gguf/src/lib.rs:349-379
enum : uint32_t { VT_U8 = 0, VT_I8, VT_U16, VT_I16, VT_U32, VT_I32, VT_F32, VT_BOOL, VT_STRING, VT_ARRAY, VT_U64, VT_I64, VT_F64 };

struct Value {
    uint32_t type = 0;
    const uint8_t *p = nullptr; // scalars: the value; strings: first byte; arrays: first element
    uint64_t len = 0;           // strings: bytes without trailing NULs; arrays: element count
    uint32_t elem_type = 0;     // arrays
    std::vector<uint64_t> elem_off; // arrays of strings or arrays: offset of each element from p
};

struct TensorInfo {
    std::string name;
    uint32_t type = 0;
    int32_t rank = 0;
    int64_t shape[FH_GGUF_MAX_RANK] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint64_t offset = 0;
};

} // namespace

struct fh_gguf {
    const uint8_t *base = nullptr;
    size_t size = 0;
    bool mapped = false;
    uint32_t version = 0;
    uint64_t alignment = 32, data_offset = 0;
    std::vector<std::string> keys; // in file order; a repeated key keeps its first position and its last value
    std::vector<Value> values;
    std::unordered_map<std::string, size_t> key_index;
    std::vector<TensorInfo> tensors;
    std::unordered_map<std::string, size_t> tensor_index;
};

namespace {

struct Cursor {
    const uint8_t *base;
    size_t size, pos = 0;
    uint32_t version;
    bool need(uint64_t n) const { return n <= size && pos <= size - n; }
    template <typename T> bool get(T *out) {
        if (!need(sizeof(T))) return false;
        memcpy(out, base + pos, sizeof(T));
        pos += sizeof(T);
        return true;
    }
    // read_array_length, gguf/src/lib.rs:201-209: u32 in version 1, u64 afterwards
    bool length(uint64_t *out) {
        if (version == 1) {
            uint32_t v;
            if (!get(&v)) return false;
            *out = v;
            return true;
        }
        return get(out);
    }
};

#define GG_TRUNC() FH_FAIL(FH_ERR_IO, "GGUF data ends inside the header (offset %zu of %zu)", c.pos, c.size)

int scalar_size(uint32_t t) {
    switch (t) {
    case VT_U8: case VT_I8: case VT_BOOL: return 1;
    case VT_U16: case VT_I16: return 2;
    case VT_U32: case VT_I32: case VT_F32: return 4;
    case VT_U64: case VT_I64: case VT_F64: return 8;
    default: return 0;
    }
}

// read_string, gguf/src/lib.rs:321-335: length-prefixed, trailing NUL bytes dropped.
fh_status read_string(Cursor &c, const uint8_t **p, uint64_t *len) {
    uint64_t n;
    if (!c.length(&n)) GG_TRUNC();
    if (!c.need(n)) GG_TRUNC();
    *p = c.base + c.pos;
    c.pos += n;
    while (n && (*p)[n - 1] == 0) n--;
    *len = n;
    return FH_OK;
}

// GgufValue::read, gguf/src/lib.rs:430-465
fh_status read_value(Cursor &c, uint32_t type, Value *v, int depth) {
    v->type = type;
    if (type > VT_F64) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", type);
    if (int sz = scalar_size(type)) {
        if (!c.need(sz)) GG_TRUNC();
        v->p = c.base + c.pos;
        c.pos += sz;
        if (type == VT_BOOL && *v->p > 1) FH_FAIL(FH_ERR_INVALID, "invalid bool value");
        return FH_OK;
    }
    if (type == VT_STRING) return read_string(c, &v->p, &v->len);
    // array: element type, count, elements
    FH_REQUIRE(depth < 8, "arrays nested deeper than 8 levels");
    uint32_t et;
    if (!c.get(&et)) GG_TRUNC();
    if (et > VT_F64) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", et);
    uint64_t n;
    if (!c.length(&n)) GG_TRUNC();
    v->elem_type = et;
    v->len = n;
    v->p = c.base + c.pos;
    if (int sz = scalar_size(et)) {
        if (n > (c.size - c.pos) / sz) GG_TRUNC();
        if (et == VT_BOOL)
            for (uint64_t i = 0; i < n; i++)
                if (v->p[i] > 1) FH_FAIL(FH_ERR_INVALID, "invalid bool value");
        c.pos += n * sz;
        return FH_OK;
    }
    if (n > c.size - c.pos) GG_TRUNC(); // every element takes at least one byte
    v->elem_off.resize(n);
    for (uint64_t i = 0; i < n; i++) {
        v->elem_off[i] = (uint64_t)(c.base + c.pos - v->p);
        Value e;
        FH_TRY(read_value(c, et, &e, depth + 1));
    }
    return FH_OK;
}

// block_size / block_allocation_size, gguf/src/lib.rs:98-121 (elements and bytes per block; 0 bytes where the
// reference has no block layout either)
bool type_known(uint32_t t) { return t <= 3 || (t >= 6 && t <= 15); }
int64_t type_block_elems(uint32_t t) { return t <= 1 ? 1 : (t <= 9 ? 32 : 256); }
int64_t type_block_bytes(uint32_t t) {
    switch (t) {
    case 0: return 4;
    case 1: return 2;
    case 2: return 18;
    case 6: return 22;
    case 8: return 34;
    case 12: return 144;
    case 13: return 176;
    case 14: return 210;
    default: return 0;
    }
}

fh_status parse(fh_gguf *g) {
    Cursor c{g->base, g->size, 0, 0};
    uint8_t magic[4];
    if (!c.need(4)) GG_TRUNC();
    memcpy(magic, c.base, 4);
    c.pos = 4;
    // check_magic, gguf/src/lib.rs:16-31: "GGUF" or the same bytes reversed
    if (memcmp(magic, "GGUF", 4) && memcmp(magic, "FUGG", 4)) FH_FAIL(FH_ERR_INVALID, "invalid magic bytes");
    if (!c.get(&g->version)) GG_TRUNC();
    if (g->version < 1 || g->version > 3) FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported GGUF version %u", g->version);
    c.version = g->version;
    uint64_t n_tensors, n_kv;
    if (!c.length(&n_tensors) || !c.length(&n_kv)) GG_TRUNC();
    if (n_kv > c.size || n_tensors > c.size) GG_TRUNC();
    for (uint64_t i = 0; i < n_kv; i++) {
        const uint8_t *kp;
        uint64_t kl;
        FH_TRY(read_string(c, &kp, &kl));
        uint32_t vt;
        if (!c.get(&vt)) GG_TRUNC();
        Value v;
        FH_TRY(read_value(c, vt, &v, 0));
        std::string key((const char *)kp, kl);
        auto it = g->key_index.find(key);
        if (it != g->key_index.end()) g->values[it->second] = std::move(v); // map insert: the last one wins
        else {
            g->key_index.emplace(key, g->keys.size());
            g->keys.push_back(std::move(key));
            g->values.push_back(std::move(v));
        }
    }
    for (uint64_t i = 0; i < n_tensors; i++) {
        const uint8_t *np;
        uint64_t nl;
        FH_TRY(read_string(c, &np, &nl));
        TensorInfo t;
        t.name.assign((const char *)np, nl);
        uint32_t rank;
        if (!c.get(&rank)) GG_TRUNC();
        FH_REQUIRE(rank <= FH_GGUF_MAX_RANK, "tensor '%s' has %u dimensions (at most %d here)", t.name.c_str(), rank,
                   FH_GGUF_MAX_RANK);
        t.rank = (int32_t)rank;
        for (uint32_t d = 0; d < rank; d++) { // stored innermost first; the reference reverses (:583) and keeps u32
            uint64_t v;
            if (!c.length(&v)) GG_TRUNC();
            t.shape[rank - 1 - d] = (int64_t)(uint32_t)v;
        }
        if (!c.get(&t.type)) GG_TRUNC();
        if (!type_known(t.type)) FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported dtype %u", t.type);
        if (!c.get(&t.offset)) GG_TRUNC();
        auto it = g->tensor_index.find(t.name);
        if (it != g->tensor_index.end()) g->tensors[it->second] = t;
        else {
            g->tensor_index.emplace(t.name, g->tensors.size());
            g->tensors.push_back(std::move(t));
        }
    }
    // general.alignment, gguf/src/lib.rs:597-606: unsigned or non-negative signed values of at most 32 bits
    g->alignment = 32;
    auto it = g->key_index.find("general.alignment");
    if (it != g->key_index.end()) {
        const Value &v = g->values[it->second];
        int64_t a = -1;
        switch (v.type) {
        case VT_U8: a = *v.p; break;
        case VT_U16: { uint16_t x; memcpy(&x, v.p, 2); a = x; break; }
        case VT_U32: { uint32_t x; memcpy(&x, v.p, 4); a = x; break; }
        case VT_I8: a = (int8_t)*v.p; break;
        case VT_I16: { int16_t x; memcpy(&x, v.p, 2); a = x; break; }
        case VT_I32: { int32_t x; memcpy(&x, v.p, 4); a = x; break; }
        default: break;
        }
        if (a >= 0) g->alignment = (uint64_t)a;
    }
    FH_REQUIRE(g->alignment > 0, "general.alignment is 0");
    g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    return FH_OK;
}

// GgufMetadata::get_value, gguf/src/lib.rs:301-311: a key that starts with '.' matches the shortest stored key
// that ends with it (of several of that length: the first in the file).
const Value *find_value(const fh_gguf *g, const char *key, size_t *index) {
    size_t best = (size_t)-1;
    if (key[0] == '.') {
        const size_t kl = strlen(key);
        for (size_t i = 0; i < g->keys.size(); i++) {
            const std::string &s = g->keys[i];
            if (s.size() >= kl && !s.compare(s.size() - kl, kl, key) &&
                (best == (size_t)-1 || s.size() < g->keys[best].size()))
                best = i;
        }
    } else {
        auto it = g->key_index.find(key);
        if (it != g->key_index.end()) best = it->second;
    }
    if (best == (size_t)-1) return nullptr;
    if (index) *index = best;
    return &g->values[best];
}

#define GG_FIND(v, g, key)                                                                                         \
    FH_REQUIRE((g) && (key), "NULL argument");                                                                     \
    const Value *v = find_value((g), (key), nullptr);                                                              \
    if (!v) FH_FAIL(FH_ERR_NOT_FOUND, "Key '%s' not found in GGUF metadata", (key))

// scalar at p as the widest type of its class; class 0 unsigned, 1 signed, 2 float, 3 bool, -1 none
int load_scalar(uint32_t type, const uint8_t *p, uint64_t *u, int64_t *i, double *f) {
    switch (type) {
    case VT_U8: *u = *p; return 0;
    case VT_U16: { uint16_t x; memcpy(&x, p, 2); *u = x; return 0; }
    case VT_U32: { uint32_t x; memcpy(&x, p, 4); *u = x; return 0; }
    case VT_U64: memcpy(u, p, 8); return 0;
    case VT_I8: *i = (int8_t)*p; return 1;
    case VT_I16: { int16_t x; memcpy(&x, p, 2); *i = x; return 1; }
    case VT_I32: { int32_t x; memcpy(&x, p, 4); *i = x; return 1; }
    case VT_I64: memcpy(i, p, 8); return 1;
    case VT_F32: { float x; memcpy(&x, p, 4); *f = x; return 2; }
    case VT_F64: memcpy(f, p, 8); return 2;
    case VT_BOOL: *u = *p; return 3;
    default: return -1;
    }
}

// to_u64 / to_i64 (`as` casts between the integer types, gguf/src/lib.rs:544-551)
fh_status scalar_int(uint32_t type, const uint8_t *p, int64_t *out) {
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    int cls = load_scalar(type, p, &u, &i, &f);
    if (cls == 0) *out = (int64_t)u;
    else if (cls == 1) *out = i;
    else FH_FAIL(FH_ERR_INVALID, "invalid value type %u", type);
    return FH_OK;
}

// to_f32 / to_f64: float types only (gguf/src/lib.rs:552-553)
fh_status scalar_float(uint32_t type, const uint8_t *p, double *out) {
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    if (load_scalar(type, p, &u, &i, &f) != 2) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", type);
    *out = f;
    return FH_OK;
}

} // namespace

extern "C" fh_status fh_gguf_open_memory(const void *bytes, size_t len, fh_gguf **out) {
    FH_REQUIRE(bytes && out, "NULL argument");
    *out = nullptr;
    fh_gguf *g = new fh_gguf();
    g->base = (const uint8_t *)bytes;
    g->size = len;
    fh_status st = parse(g);
    if (st != FH_OK) {
        delete g;
        return st;
    }
    *out = g;
    return FH_OK;
}

extern "C" fh_status fh_gguf_open(const char *path, fh_gguf **out) {
    FH_REQUIRE(path && out, "NULL argument");
    *out = nullptr;
    int fd = open(path, O_RDONLY);
    if (fd < 0) FH_FAIL(FH_ERR_IO, "io error: open '%s': %s", path, strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size <= 0) {
        int e = errno;
        close(fd);
        FH_FAIL(FH_ERR_IO, "io error: '%s' is empty or cannot be examined (%s)", path, strerror(e));
    }
    void *p = mmap(nullptr, (size_t)sb.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    int e = errno;
    close(fd);
    if (p == MAP_FAILED) FH_FAIL(FH_ERR_IO, "io error: mmap '%s': %s", path, strerror(e));
    fh_status st = fh_gguf_open_memory(p, (size_t)sb.st_size, out);
    if (st != FH_OK) {
        munmap(p, (size_t)sb.st_size);
        return st;
    }
    (*out)->mapped = true;
    return FH_OK;
}

extern "C" fh_status fh_gguf_close(fh_gguf *g) {
    if (!g) return FH_OK;
    if (g->mapped) munmap((void *)g->base, g->size);
    delete g;
    return FH_OK;
}

extern "C" fh_status fh_gguf_info(const fh_gguf *g, uint32_t *version, uint64_t *tensor_count, uint64_t *metadata_count,
                                  uint64_t *alignment, uint64_t *tensor_data_offset) {
    FH_REQUIRE(g, "NULL argument");
    if (version) *version = g->version;
    if (tensor_count) *tensor_count = g->tensors.size();
    if (metadata_count) *metadata_count = g->keys.size();
    if (alignment) *alignment = g->alignment;
    if (tensor_data_offset) *tensor_data_offset = g->data_offset;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_key(const fh_gguf *g, uint64_t index, const char **key, uint32_t *value_type) {
    FH_REQUIRE(g, "NULL argument");
    FH_REQUIRE(index < g->keys.size(), "metadata index %llu out of range (%zu entries)", (unsigned long long)index,
               g->keys.size());
    if (key) *key = g->keys[index].c_str();
    if (value_type) *value_type = g->values[index].type;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_find(const fh_gguf *g, const char *key, const char **full_key, uint32_t *value_type) {
    FH_REQUIRE(g && key, "NULL argument");
    size_t idx = 0;
    const Value *v = find_value(g, key, &idx);
    if (!v) FH_FAIL(FH_ERR_NOT_FOUND, "Key '%s' not found in GGUF metadata", key);
    if (full_key) *full_key = g->keys[idx].c_str();
    if (value_type) *value_type = v->type;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_int(const fh_gguf *g, const char *key, int64_t *out) {
    GG_FIND(v, g, key);
    FH_REQUIRE(out, "NULL argument");
    return scalar_int(v->type, v->p, out);
}

extern "C" fh_status fh_gguf_meta_float(const fh_gguf *g, const char *key, double *out) {
    GG_FIND(v, g, key);
    FH_REQUIRE(out, "NULL argument");
    return scalar_float(v->type, v->p, out);
}

extern "C" fh_status fh_gguf_meta_bool(const fh_gguf *g, const char *key, int32_t *out) {
    GG_FIND(v, g, key);
    FH_REQUIRE(out, "NULL argument");
    if (v->type != VT_BOOL) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->type);
    *out = *v->p;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_string(const fh_gguf *g, const char *key, const char **bytes, uint64_t *len) {
    GG_FIND(v, g, key);
    FH_REQUIRE(bytes && len, "NULL argument");
    if (v->type != VT_STRING) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->type);
    *bytes = (const char *)v->p;
    *len = v->len;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_array(const fh_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count,
                                        const void **packed) {
    GG_FIND(v, g, key);
    if (v->type != VT_ARRAY) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->type);
    if (elem_type) *elem_type = v->elem_type;
    if (count) *count = v->len;
    if (packed) *packed = scalar_size(v->elem_type) ? v->p : nullptr;
    return FH_OK;
}

static fh_status array_elem(const fh_gguf *g, const char *key, uint64_t index, const Value **arr) {
    GG_FIND(v, g, key);
    if (v->type != VT_ARRAY) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->type);
    FH_REQUIRE(index < v->len, "array index %llu out of range (%llu elements)", (unsigned long long)index,
               (unsigned long long)v->len);
    *arr = v;
    return FH_OK;
}

extern "C" fh_status fh_gguf_meta_array_int(const fh_gguf *g, const char *key, uint64_t index, int64_t *out) {
    const Value *v = nullptr;
    FH_TRY(array_elem(g, key, index, &v));
    FH_REQUIRE(out, "NULL argument");
    int sz = scalar_size(v->elem_type);
    if (!sz) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->elem_type);
    return scalar_int(v->elem_type, v->p + index * sz, out);
}

extern "C" fh_status fh_gguf_meta_array_float(const fh_gguf *g, const char *key, uint64_t index, double *out) {
    const Value *v = nullptr;
    FH_TRY(array_elem(g, key, index, &v));
    FH_REQUIRE(out, "NULL argument");
    int sz = scalar_size(v->elem_type);
    if (!sz) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->elem_type);
    return scalar_float(v->elem_type, v->p + index * sz, out);
}

extern "C" fh_status fh_gguf_meta_array_string(const fh_gguf *g, const char *key, uint64_t index, const char **bytes,
                                               uint64_t *len) {
    const Value *v = nullptr;
    FH_TRY(array_elem(g, key, index, &v));
    FH_REQUIRE(bytes && len, "NULL argument");
    if (v->elem_type != VT_STRING) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", v->elem_type);
    Cursor c{v->p, (size_t)(g->base + g->size - v->p), (size_t)v->elem_off[index], g->version};
    const uint8_t *p;
    FH_TRY(read_string(c, &p, len));
    *bytes = (const char *)p;
    return FH_OK;
}

extern "C" fh_status fh_gguf_tensor_info(const fh_gguf *g, uint64_t index, fh_gguf_tensor *out) {
    FH_REQUIRE(g && out, "NULL argument");
    FH_REQUIRE(index < g->tensors.size(), "tensor index %llu out of range (%zu tensors)", (unsigned long long)index,
               g->tensors.size());
    const TensorInfo &t = g->tensors[index];
    out->name = t.name.c_str();
    out->ggml_type = t.type;
    out->rank = t.rank;
    for (int i = 0; i < FH_GGUF_MAX_RANK; i++) out->shape[i] = t.shape[i];
    out->offset = t.offset;
    return FH_OK;
}

extern "C" fh_status fh_gguf_tensor_find(const fh_gguf *g, const char *name, uint64_t *index) {
    FH_REQUIRE(g && name && index, "NULL argument");
    auto it = g->tensor_index.find(name);
    if (it == g->tensor_index.end()) FH_FAIL(FH_ERR_NOT_FOUND, "Key '%s' not found in GGUF metadata", name);
    *index = it->second;
    return FH_OK;
}

// GgufTensorMetadata::byte_size + read_tensor_bytes, gguf/src/lib.rs:262-286
extern "C" fh_status fh_gguf_tensor_data(const fh_gguf *g, uint64_t index, const void **bytes, size_t *len) {
    FH_REQUIRE(g && bytes && len, "NULL argument");
    FH_REQUIRE(index < g->tensors.size(), "tensor index %llu out of range (%zu tensors)", (unsigned long long)index,
               g->tensors.size());
    const TensorInfo &t = g->tensors[index];
    // the reference multiplies the dimensions in u32 (wrapping in release builds)
    uint32_t elems32 = 1;
    for (int i = 0; i < t.rank; i++) elems32 *= (uint32_t)t.shape[i];
    const int64_t elems = elems32, be = type_block_elems(t.type), bb = type_block_bytes(t.type);
    if (!bb) FH_FAIL(FH_ERR_UNSUPPORTED, "no block layout for dtype %u (tensor '%s')", t.type, t.name.c_str());
    if (elems % be)
        FH_FAIL(FH_ERR_INVALID, "tensor size (%lld) is not a multiple of the block size (%lld)", (long long)elems,
                (long long)be);
    const uint64_t need = (uint64_t)(elems / be) * (uint64_t)bb;
    const uint64_t start = g->data_offset + t.offset;
    if (start > g->size || need > g->size - start)
        FH_FAIL(FH_ERR_IO, "io error: tensor '%s' needs bytes [%llu, %llu) of a %zu-byte file", t.name.c_str(),
                (unsigned long long)start, (unsigned long long)(start + need), g->size);
    *bytes = g->base + start;
    *len = (size_t)need;
    return FH_OK;
}

// VarBuilder::get, fusor-ml/fusor/src/varbuilder.rs:79-127: the named tensor as a device weight matrix
// (rank 2, [n, k]; a rank-1 tensor is one row).
extern "C" fh_status fh_qmatrix_from_gguf_tensor(fh_device *dev, const fh_gguf *g, const char *name, fh_qmatrix **out) {
    FH_REQUIRE(dev && g && name && out, "NULL argument");
    *out = nullptr;
    uint64_t idx;
    FH_TRY(fh_gguf_tensor_find(g, name, &idx));
    const TensorInfo &t = g->tensors[idx];
    FH_REQUIRE(t.rank == 1 || t.rank == 2, "tensor '%s' has rank %d; a weight matrix has rank 1 or 2", name, t.rank);
    const void *bytes;
    size_t len;
    FH_TRY(fh_gguf_tensor_data(g, idx, &bytes, &len));
    const int64_t n = t.rank == 2 ? t.shape[0] : 1, k = t.shape[t.rank - 1];
    return fh_qmatrix_from_gguf_bytes(dev, t.type, n, k, bytes, len, out);
}

// ---------------------------------------------------------------------------------------------- decoder
static fh_status meta_int_or(const fh_gguf *g, const char *key, int64_t fallback, bool required, int64_t *out) {
    const Value *v = find_value(g, key, nullptr);
    if (!v) {
        if (required) FH_FAIL(FH_ERR_NOT_FOUND, "Key '%s' not found in GGUF metadata", key);
        *out = fallback;
        return FH_OK;
    }
    return scalar_int(v->type, v->p, out);
}

static const TensorInfo *tensor_named(const fh_gguf *g, const std::string &name) {
    auto it = g->tensor_index.find(name);
    return it == g->tensor_index.end() ? nullptr : &g->tensors[it->second];
}

// Parameter extraction of models/kalosm-llama/src/raw/mod.rs:377-416.  vocab and the feed-forward width are
// the row counts of token_embd.weight and blk.0.ffn_gate.weight (the reference takes them from the tensors too).
extern "C" fh_status fh_llama_config_from_gguf(const fh_gguf *g, fh_llama_config *cfg) {
    FH_REQUIRE(g && cfg, "NULL argument");
    memset(cfg, 0, sizeof(*cfg));
    const Value *arch = find_value(g, "general.architecture", nullptr);
    if (!arch) FH_FAIL(FH_ERR_NOT_FOUND, "Key 'general.architecture' not found in GGUF metadata");
    if (arch->type != VT_STRING) FH_FAIL(FH_ERR_INVALID, "invalid value type %u", arch->type);
    std::string a((const char *)arch->p, arch->len);
    if (a != "llama")
        FH_FAIL(FH_ERR_UNSUPPORTED, "architecture '%s': this decoder covers 'llama' (interleaved RoPE, separate q/k/v, "
                                    "gate/up/down feed-forward)", a.c_str());
    int64_t heads, kv_heads, blocks, d_model, ctx, key_len;
    FH_TRY(meta_int_or(g, ".attention.head_count", 0, true, &heads));
    FH_TRY(meta_int_or(g, ".attention.head_count_kv", 0, true, &kv_heads));
    FH_TRY(meta_int_or(g, ".block_count", 0, true, &blocks));
    FH_TRY(meta_int_or(g, ".embedding_length", 0, true, &d_model));
    FH_TRY(meta_int_or(g, ".context_length", 0, true, &ctx));
    FH_REQUIRE(heads > 0 && kv_heads > 0 && blocks > 0 && d_model > 0 && ctx > 0, "non-positive model dimensions");
    FH_TRY(meta_int_or(g, ".attention.key_length", d_model / heads, false, &key_len));
    const Value *eps = find_value(g, ".attention.layer_norm_rms_epsilon", nullptr);
    if (!eps) FH_FAIL(FH_ERR_NOT_FOUND, "Key '.attention.layer_norm_rms_epsilon' not found in GGUF metadata");
    double e = 0, theta = 1000000.0; // DEFAULT_ROPE_FREQUENCY, raw/mod.rs:104
    FH_TRY(scalar_float(eps->type, eps->p, &e));
    if (const Value *fb = find_value(g, ".rope.freq_base", nullptr)) {
        double t;
        if (scalar_float(fb->type, fb->p, &t) == FH_OK) theta = t; // a value of another type falls back (:385-388)
    }
    if (find_value(g, ".attention.sliding_window", nullptr))
        FH_FAIL(FH_ERR_UNSUPPORTED, "sliding-window attention is outside this decoder");
    const TensorInfo *embd = tensor_named(g, "token_embd.weight"), *gate = tensor_named(g, "blk.0.ffn_gate.weight");
    if (!embd) FH_FAIL(FH_ERR_NOT_FOUND, "Key 'token_embd.weight' not found in GGUF metadata");
    if (!gate) FH_FAIL(FH_ERR_NOT_FOUND, "Key 'blk.0.ffn_gate.weight' not found in GGUF metadata");
    FH_REQUIRE(embd->rank == 2 && gate->rank == 2, "token_embd.weight / blk.0.ffn_gate.weight are not matrices");
    cfg->n_layers = (int32_t)blocks;
    cfg->d_model = (int32_t)d_model;
    cfg->n_heads = (int32_t)heads;
    cfg->n_kv_heads = (int32_t)kv_heads;
    cfg->head_dim = (int32_t)key_len;
    cfg->ffn = (int32_t)gate->shape[0];
    cfg->vocab = (int32_t)embd->shape[0];
    cfg->ctx = (int32_t)ctx;
    cfg->eps = (float)e;
    cfg->theta = (float)theta;
    cfg->kv_dtype = FH_F32;
    cfg->fuse_qkv = cfg->fuse_gate_up = cfg->use_graph = 1;
    return FH_OK;
}

static float f16_bits_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023, u;
    if (e == 0) {
        if (!m) u = s;
        else {
            int sh = 0;
            while (!(m & 1024)) { m <<= 1; sh++; }
            u = s | ((uint32_t)(113 - sh) << 23) | ((m & 1023) << 13);
        }
    } else if (e == 31) u = s | 0x7F800000u | (m << 13);
    else u = s | ((e + 112) << 23) | (m << 13);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// Tensor loading of models/kalosm-llama/src/raw/mod.rs:418-604 for the variant this decoder covers.  Tensors of
// variants it does not cover (fused attn_qkv, biases, q/k norms, post norms) are refused rather than ignored.
extern "C" fh_status fh_llama_load_gguf(fh_llama *m, const fh_gguf *g) {
    FH_REQUIRE(m && g, "NULL argument");
    static const char *const refused[] = {"attn_qkv.weight", "attn_q.bias", "attn_k.bias", "attn_v.bias",
                                          "attn_q_norm.weight", "attn_k_norm.weight", "post_attention_norm.weight",
                                          "post_ffw_norm.weight"};
    std::vector<float> tmp;
    for (size_t i = 0; i < g->tensors.size(); i++) {
        const TensorInfo &t = g->tensors[i];
        const std::string &name = t.name;
        const bool global = name == "token_embd.weight" || name == "output.weight" || name == "output_norm.weight" ||
                            name == "rope_freqs.weight";
        if (!global && name.compare(0, 4, "blk.")) continue; // tokenizer or vision tensors: not the decoder's
        for (const char *r : refused)
            if (name.size() > strlen(r) && !name.compare(name.size() - strlen(r), strlen(r), r))
                FH_FAIL(FH_ERR_UNSUPPORTED, "tensor '%s': this attention / norm variant is outside this decoder",
                        name.c_str());
        const void *bytes;
        size_t len;
        FH_TRY(fh_gguf_tensor_data(g, i, &bytes, &len));
        FH_REQUIRE(t.rank == 1 || t.rank == 2, "tensor '%s' has rank %d", name.c_str(), t.rank);
        int64_t n = t.rank == 2 ? t.shape[0] : t.shape[0], k = t.rank == 2 ? t.shape[1] : 0;
        uint32_t type = t.type;
        if (type == 1 && (t.rank == 1 || n == 1 || k == 1)) { // f16 vector (norm weights, rope_freqs): widen on the host
            const size_t cnt = len / 2;
            tmp.resize(cnt);
            for (size_t j = 0; j < cnt; j++) {
                uint16_t h;
                memcpy(&h, (const uint8_t *)bytes + 2 * j, 2);
                tmp[j] = f16_bits_to_f32(h);
            }
            bytes = tmp.data();
            len = cnt * 4;
            type = 0;
        }
        FH_TRY(fh_llama_load_tensor(m, name.c_str(), type, n, k, bytes, len));
    }
    return FH_OK;
}
