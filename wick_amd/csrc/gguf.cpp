// GGUF v3 container reader behind include/wick_gguf.h (host only).
// Follows the parse order, limits and error cases of GgufFile::from_backing
// (wick/src/gguf.rs:404-545): header, key/value metadata, tensor infos, data section
// aligned to general.alignment (default 32), every tensor range checked against the file.
#include "../../include/wick_gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF" little-endian, wick/src/gguf.rs:18
constexpr uint64_t kMaxString = 1000000;  // wick/src/gguf.rs:219
constexpr uint64_t kMaxArray = 10000000;  // wick/src/gguf.rs:243

// {elements per block, bytes per block} of the ggml types the reference can size
// (ggml_type_to_dtype, wick/src/gguf.rs:250-270; DType::block_size / block_bytes).
bool type_layout(int t, uint64_t& block, uint64_t& bytes) {
    switch (t) {
        case 0: block = 1, bytes = 4; return true;      // F32
        case 1: block = 1, bytes = 2; return true;      // F16
        case 30: block = 1, bytes = 2; return true;     // BF16
        case 26: block = 1, bytes = 4; return true;     // I32
        case 2: block = 32, bytes = 18; return true;    // Q4_0
        case 8: block = 32, bytes = 34; return true;    // Q8_0
        case 12: block = 256, bytes = 144; return true; // Q4_K
        case 14: block = 256, bytes = 210; return true; // Q6_K
        default: return false;
    }
}

int scalar_size(int t) {
    switch (t) {
        case WICK_GGUF_T_U8: case WICK_GGUF_T_I8: case WICK_GGUF_T_BOOL: return 1;
        case WICK_GGUF_T_U16: case WICK_GGUF_T_I16: return 2;
        case WICK_GGUF_T_U32: case WICK_GGUF_T_I32: case WICK_GGUF_T_F32: return 4;
        case WICK_GGUF_T_U64: case WICK_GGUF_T_I64: case WICK_GGUF_T_F64: return 8;
        default: return 0;
    }
}

struct Value {
    int type = 0;
    size_t pos = 0;          // scalars: offset of the value; strings: offset of the bytes; arrays: offset of element 0
    uint64_t len = 0;        // strings: byte length; arrays: element count
    int elem_type = 0;       // arrays
    std::vector<std::pair<size_t, uint64_t>> strings;  // string arrays: {offset, length} per element
};

struct TensorRec {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[8] = {};
    int type = 0;
    uint64_t abs_offset = 0;
    uint64_t size_bytes = 0;  // 0: ggml type not sizeable here
};

}  // namespace

struct wick_gguf {
    const uint8_t* data = nullptr;
    size_t size = 0;
    bool mapped = false;
    std::vector<uint8_t> owned;
    std::vector<std::string> keys;
    std::unordered_map<std::string, Value> metadata;
    std::vector<TensorRec> tensors;
    std::unordered_map<std::string, size_t> tensor_index;
    size_t data_offset = 0;
    uint32_t alignment = 32;

    ~wick_gguf() {
        if (mapped && data) munmap(const_cast<uint8_t*>(data), size);
    }
};

namespace {

// Well-formed UTF-8 (no overlongs, no surrogates, <= U+10FFFF), what String::from_utf8 accepts.
bool valid_utf8(const uint8_t* p, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = p[i];
        if (c < 0x80) {
            i++;
            continue;
        }
        int extra;
        uint32_t cp;
        if ((c & 0xE0) == 0xC0) extra = 1, cp = c & 0x1Fu;
        else if ((c & 0xF0) == 0xE0) extra = 2, cp = c & 0x0Fu;
        else if ((c & 0xF8) == 0xF0) extra = 3, cp = c & 0x07u;
        else return false;
        if (n - i <= (size_t)extra) return false;
        for (int j = 1; j <= extra; j++) {
            if ((p[i + j] & 0xC0) != 0x80) return false;
            cp = (cp << 6) | (p[i + j] & 0x3Fu);
        }
        static const uint32_t kMin[4] = {0, 0x80, 0x800, 0x10000};
        if (cp < kMin[extra] || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
        i += extra + 1;
    }
    return true;
}

// Bounds-checked little-endian cursor over the file image.
struct Cursor {
    const uint8_t* p;
    size_t size, pos = 0;
    bool ok = true;
    const char* what = "";

    bool need(size_t n, const char* w) {
        if (!ok) return false;
        if (n > size - pos) {
            ok = false, what = w;
            return false;
        }
        return true;
    }
    template <typename T>
    T get(const char* w) {
        T v{};
        if (need(sizeof(T), w)) {
            memcpy(&v, p + pos, sizeof(T));
            pos += sizeof(T);
        }
        return v;
    }
    // u64 length + bytes; returns the offset of the bytes
    bool string(size_t& at, uint64_t& len) {
        len = get<uint64_t>("read string length");
        if (!ok) return false;
        if (len >= kMaxString) {
            ok = false, what = "string too long";
            return false;
        }
        if (!need((size_t)len, "read string")) return false;
        if (!valid_utf8(p + pos, (size_t)len)) {  // wick/src/gguf.rs:223
            ok = false, what = "invalid UTF-8 in string";
            return false;
        }
        at = pos;
        pos += (size_t)len;
        return true;
    }
};

// Reads one value of `type` into v (arrays recurse; nested arrays are walked but not indexed).
bool read_value(Cursor& c, int type, Value& v, int depth) {
    v.type = type;
    const int ss = scalar_size(type);
    if (ss) {
        if (!c.need(ss, "read value")) return false;
        v.pos = c.pos;
        c.pos += ss;
        return true;
    }
    if (type == WICK_GGUF_T_STRING) return c.string(v.pos, v.len);
    if (type == WICK_GGUF_T_ARRAY) {
        if (depth > 4) {
            c.ok = false, c.what = "arrays nested too deeply";
            return false;
        }
        v.elem_type = (int)c.get<uint32_t>("read array type");
        v.len = c.get<uint64_t>("read array count");
        if (!c.ok) return false;
        if (v.len >= kMaxArray) {
            c.ok = false, c.what = "array too long";
            return false;
        }
        v.pos = c.pos;
        const int es = scalar_size(v.elem_type);
        if (es) {
            if (!c.need((size_t)v.len * es, "read array")) return false;
            c.pos += (size_t)v.len * es;
            return true;
        }
        if (v.elem_type == WICK_GGUF_T_STRING) v.strings.reserve((size_t)v.len);
        for (uint64_t i = 0; i < v.len; i++) {
            Value e;
            if (!read_value(c, v.elem_type, e, depth + 1)) return false;
            if (v.elem_type == WICK_GGUF_T_STRING) v.strings.emplace_back(e.pos, e.len);
        }
        return true;
    }
    c.ok = false, c.what = "unknown GGUF value type";
    return false;
}

int parse(wick_gguf& g) {
    if (g.size < 24) return fail(WICK_GGUF_ERR_FORMAT, "GGUF buffer too small (%zu bytes; need at least 24 for the header)", g.size);
    Cursor c{g.data, g.size};
    const uint32_t magic = c.get<uint32_t>("read magic");
    if (magic != kMagic) return fail(WICK_GGUF_ERR_FORMAT, "not a GGUF file (magic: 0x%08X, expected 0x%08X)", magic, kMagic);
    const uint32_t version = c.get<uint32_t>("read version");
    if (version != 3) return fail(WICK_GGUF_ERR_FORMAT, "unsupported GGUF version %u (expected 3)", version);
    const uint64_t tensor_count = c.get<uint64_t>("read tensor count");
    const uint64_t kv_count = c.get<uint64_t>("read kv count");
    // every key/value and tensor info takes at least 13 / 24 bytes: counts beyond the file are malformed
    if (kv_count > g.size / 13 || tensor_count > g.size / 24)
        return fail(WICK_GGUF_ERR_FORMAT, "GGUF counts exceed the file (tensors=%llu, kv=%llu, file=%zu bytes)",
                    (unsigned long long)tensor_count, (unsigned long long)kv_count, g.size);

    for (uint64_t i = 0; i < kv_count; i++) {
        size_t at;
        uint64_t len;
        if (!c.string(at, len)) break;
        std::string key(reinterpret_cast<const char*>(g.data + at), (size_t)len);
        const int type = (int)c.get<uint32_t>("read value type");
        Value v;
        if (!c.ok || !read_value(c, type, v, 0)) break;
        if (g.metadata.find(key) == g.metadata.end()) g.keys.push_back(key);
        g.metadata[key] = std::move(v);  // a repeated key keeps the last value, like HashMap::insert
    }
    if (!c.ok) return fail(WICK_GGUF_ERR_FORMAT, "GGUF metadata: %s (offset %zu of %zu)", c.what, c.pos, g.size);

    struct Raw {
        std::string name;
        uint32_t n_dims;
        uint64_t dims[8];
        uint32_t type;
        uint64_t offset;
    };
    std::vector<Raw> raws;
    raws.reserve((size_t)tensor_count);
    for (uint64_t i = 0; i < tensor_count; i++) {
        size_t at;
        uint64_t len;
        if (!c.string(at, len)) break;
        Raw r{};
        r.name.assign(reinterpret_cast<const char*>(g.data + at), (size_t)len);
        r.n_dims = c.get<uint32_t>("read n_dims");
        if (!c.ok) break;
        if (r.n_dims > 8) return fail(WICK_GGUF_ERR_FORMAT, "tensor %s has too many dimensions: %u", r.name.c_str(), r.n_dims);
        for (uint32_t d = 0; d < r.n_dims; d++) r.dims[d] = c.get<uint64_t>("read dim");
        r.type = c.get<uint32_t>("read tensor type");
        r.offset = c.get<uint64_t>("read tensor offset");
        if (!c.ok) break;
        raws.push_back(std::move(r));
    }
    if (!c.ok) return fail(WICK_GGUF_ERR_FORMAT, "GGUF tensor infos: %s (offset %zu of %zu)", c.what, c.pos, g.size);

    // general.alignment counts only when stored as u32 (wick/src/gguf.rs:487-490)
    uint64_t alignment = 32;
    auto it = g.metadata.find("general.alignment");
    if (it != g.metadata.end() && it->second.type == WICK_GGUF_T_U32) {
        uint32_t a;
        memcpy(&a, g.data + it->second.pos, 4);
        alignment = a;
    }
    if (alignment == 0 || alignment > 1024 * 1024) return fail(WICK_GGUF_ERR_FORMAT, "invalid GGUF alignment: %llu", (unsigned long long)alignment);
    g.alignment = (uint32_t)alignment;
    const uint64_t header_end = c.pos;
    const uint64_t data_offset = (header_end + alignment - 1) / alignment * alignment;
    g.data_offset = (size_t)data_offset;

    for (Raw& r : raws) {
        TensorRec t;
        t.name = r.name, t.n_dims = r.n_dims, t.type = (int)r.type;
        memcpy(t.dims, r.dims, sizeof t.dims);
        uint64_t numel = 1;
        bool overflow = false;
        for (uint32_t d = 0; d < r.n_dims; d++) overflow |= __builtin_mul_overflow(numel, r.dims[d], &numel);
        uint64_t block, bytes;
        if (type_layout(t.type, block, bytes)) {  // other types stay listed with size 0, wick/src/gguf.rs:516-520
            if (overflow) return fail(WICK_GGUF_ERR_FORMAT, "tensor %s: tensor numel overflow", t.name.c_str());
            if (wick_gguf_tensor_data_size(t.type, numel, &t.size_bytes) != 0) {
                const std::string why = g_error;
                return fail(WICK_GGUF_ERR_FORMAT, "tensor %s: %s", t.name.c_str(), why.c_str());
            }
        }
        if (__builtin_add_overflow(data_offset, r.offset, &t.abs_offset))
            return fail(WICK_GGUF_ERR_FORMAT, "tensor %s offset overflow (data_offset=%llu, offset=%llu)", t.name.c_str(),
                        (unsigned long long)data_offset, (unsigned long long)r.offset);
        if (t.size_bytes > 0) {
            uint64_t end;
            if (__builtin_add_overflow(t.abs_offset, t.size_bytes, &end))
                return fail(WICK_GGUF_ERR_FORMAT, "tensor %s end offset overflow", t.name.c_str());
            if (end > g.size)
                return fail(WICK_GGUF_ERR_FORMAT, "tensor %s extends beyond file (offset=%llu, size=%llu, file_size=%zu)", t.name.c_str(),
                            (unsigned long long)t.abs_offset, (unsigned long long)t.size_bytes, g.size);
        }
        auto found = g.tensor_index.find(t.name);
        if (found != g.tensor_index.end()) {
            g.tensors[found->second] = std::move(t);  // a repeated name keeps the last info
        } else {
            g.tensor_index[t.name] = g.tensors.size();
            g.tensors.push_back(std::move(t));
        }
    }
    return WICK_GGUF_OK;
}

// Looks a key up; type < 0 accepts any stored type.
int find_value(const wick_gguf* g, const char* key, int type, const Value** out) {
    if (!g || !key) return fail(WICK_GGUF_ERR_INVALID_ARG, "null handle or key");
    auto it = g->metadata.find(key);
    if (it == g->metadata.end()) return fail(WICK_GGUF_ERR_NOT_FOUND, "metadata key %s not found", key);
    if (type >= 0 && it->second.type != type) return fail(WICK_GGUF_ERR_NOT_FOUND, "metadata key %s has another type", key);
    *out = &it->second;
    return WICK_GGUF_OK;
}

int find_tensor(const wick_gguf* g, const char* name, bool need_data, const TensorRec** out) {
    if (!g || !name) return fail(WICK_GGUF_ERR_INVALID_ARG, "null handle or tensor name");
    auto it = g->tensor_index.find(name);
    if (it == g->tensor_index.end()) return fail(WICK_GGUF_ERR_NOT_FOUND, "tensor not found: %s", name);
    const TensorRec* t = &g->tensors[it->second];
    if (need_data && t->size_bytes == 0)  // tensor_range, wick/src/gguf.rs:612-617
        return fail(WICK_GGUF_ERR_UNSUPPORTED, "tensor %s has unsupported GGML type %d (%s)", name, t->type, wick_gguf_type_name(t->type));
    *out = t;
    return WICK_GGUF_OK;
}

}  // namespace

extern "C" {

const char* wick_gguf_last_error(void) { return g_error.c_str(); }

int wick_gguf_open(const char* path, wick_gguf** out) {
    if (!path || !out) return fail(WICK_GGUF_ERR_INVALID_ARG, "open: null path or out pointer");
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail(WICK_GGUF_ERR_IO, "opening %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) {
        const int e = errno;
        ::close(fd);
        return fail(WICK_GGUF_ERR_IO, "stat %s: %s", path, strerror(e));
    }
    if (st.st_size < 24) {
        ::close(fd);
        return fail(WICK_GGUF_ERR_FORMAT, "GGUF buffer too small (%lld bytes; need at least 24 for the header)", (long long)st.st_size);
    }
    void* p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    const int e = errno;
    ::close(fd);
    if (p == MAP_FAILED) return fail(WICK_GGUF_ERR_IO, "mmap %s: %s", path, strerror(e));
    wick_gguf* g = new wick_gguf;
    g->data = static_cast<const uint8_t*>(p), g->size = (size_t)st.st_size, g->mapped = true;
    const int rc = parse(*g);
    if (rc != 0) {
        delete g;
        return rc;
    }
    *out = g;
    return WICK_GGUF_OK;
}

int wick_gguf_from_bytes(const void* bytes, size_t nbytes, wick_gguf** out) {
    if (!out || (!bytes && nbytes)) return fail(WICK_GGUF_ERR_INVALID_ARG, "from_bytes: null bytes or out pointer");
    *out = nullptr;
    wick_gguf* g = new wick_gguf;
    g->owned.assign(static_cast<const uint8_t*>(bytes), static_cast<const uint8_t*>(bytes) + nbytes);
    g->data = g->owned.data(), g->size = nbytes;
    const int rc = parse(*g);
    if (rc != 0) {
        delete g;
        return rc;
    }
    *out = g;
    return WICK_GGUF_OK;
}

void wick_gguf_close(wick_gguf* g) { delete g; }

const void* wick_gguf_data(const wick_gguf* g, size_t* nbytes) {
    if (!g) return nullptr;
    if (nbytes) *nbytes = g->size;
    return g->data;
}
size_t wick_gguf_data_offset(const wick_gguf* g) { return g ? g->data_offset : 0; }
uint32_t wick_gguf_alignment(const wick_gguf* g) { return g ? g->alignment : 0; }

uint64_t wick_gguf_metadata_count(const wick_gguf* g) { return g ? g->keys.size() : 0; }

int wick_gguf_metadata_key(const wick_gguf* g, uint64_t index, const char** key, size_t* len) {
    if (!g || !key) return fail(WICK_GGUF_ERR_INVALID_ARG, "metadata_key: null argument");
    if (index >= g->keys.size()) return fail(WICK_GGUF_ERR_INVALID_ARG, "metadata_key: index %llu out of range", (unsigned long long)index);
    *key = g->keys[(size_t)index].c_str();
    if (len) *len = g->keys[(size_t)index].size();
    return WICK_GGUF_OK;
}

int wick_gguf_value_type(const wick_gguf* g, const char* key, int* type, int* elem_type, uint64_t* count) {
    const Value* v = nullptr;
    if (int rc = find_value(g, key, -1, &v)) return rc;
    if (type) *type = v->type;
    if (elem_type) *elem_type = v->type == WICK_GGUF_T_ARRAY ? v->elem_type : 0;
    if (count) *count = v->type == WICK_GGUF_T_ARRAY ? v->len : 0;
    return WICK_GGUF_OK;
}

#define WICK_GGUF_FIND(var, type_id)                                                   \
    if (!out) return fail(WICK_GGUF_ERR_INVALID_ARG, "null out pointer");              \
    const Value* var = nullptr;                                                        \
    if (int rc = find_value(g, key, type_id, &var)) return rc;

int wick_gguf_get_u32(const wick_gguf* g, const char* key, uint32_t* out) {
    WICK_GGUF_FIND(v, WICK_GGUF_T_U32)
    memcpy(out, g->data + v->pos, 4);
    return WICK_GGUF_OK;
}

int wick_gguf_get_f32(const wick_gguf* g, const char* key, float* out) {
    WICK_GGUF_FIND(v, WICK_GGUF_T_F32)
    memcpy(out, g->data + v->pos, 4);
    return WICK_GGUF_OK;
}

int wick_gguf_get_bool(const wick_gguf* g, const char* key, int* out) {
    WICK_GGUF_FIND(v, WICK_GGUF_T_BOOL)
    *out = g->data[v->pos] != 0;
    return WICK_GGUF_OK;
}

int wick_gguf_get_int(const wick_gguf* g, const char* key, int64_t* out) {
    WICK_GGUF_FIND(v, -1)
    const uint8_t* p = g->data + v->pos;
    switch (v->type) {
        case WICK_GGUF_T_U8: case WICK_GGUF_T_BOOL: *out = *p; break;
        case WICK_GGUF_T_I8: *out = (int8_t)*p; break;
        case WICK_GGUF_T_U16: { uint16_t x; memcpy(&x, p, 2); *out = x; break; }
        case WICK_GGUF_T_I16: { int16_t x; memcpy(&x, p, 2); *out = x; break; }
        case WICK_GGUF_T_U32: { uint32_t x; memcpy(&x, p, 4); *out = x; break; }
        case WICK_GGUF_T_I32: { int32_t x; memcpy(&x, p, 4); *out = x; break; }
        case WICK_GGUF_T_U64: case WICK_GGUF_T_I64: memcpy(out, p, 8); break;
        default: return fail(WICK_GGUF_ERR_NOT_FOUND, "metadata key %s has another type", key);
    }
    return WICK_GGUF_OK;
}

#undef WICK_GGUF_FIND

int wick_gguf_get_str(const wick_gguf* g, const char* key, const char** s, size_t* len) {
    if (!s || !len) return fail(WICK_GGUF_ERR_INVALID_ARG, "get_str: null out pointer");
    const Value* v = nullptr;
    if (int rc = find_value(g, key, WICK_GGUF_T_STRING, &v)) return rc;
    *s = reinterpret_cast<const char*>(g->data + v->pos), *len = (size_t)v->len;
    return WICK_GGUF_OK;
}

int wick_gguf_get_array(const wick_gguf* g, const char* key, int elem_type, const void** data, uint64_t* count) {
    if (!data || !count) return fail(WICK_GGUF_ERR_INVALID_ARG, "get_array: null out pointer");
    const Value* v = nullptr;
    if (int rc = find_value(g, key, WICK_GGUF_T_ARRAY, &v)) return rc;
    if (v->elem_type != elem_type || scalar_size(elem_type) == 0)
        return fail(WICK_GGUF_ERR_NOT_FOUND, "metadata key %s is not an array of scalar type %d", key, elem_type);
    *data = g->data + v->pos, *count = v->len;
    return WICK_GGUF_OK;
}

int wick_gguf_get_array_str(const wick_gguf* g, const char* key, uint64_t index, const char** s, size_t* len) {
    if (!s || !len) return fail(WICK_GGUF_ERR_INVALID_ARG, "get_array_str: null out pointer");
    const Value* v = nullptr;
    if (int rc = find_value(g, key, WICK_GGUF_T_ARRAY, &v)) return rc;
    if (v->elem_type != WICK_GGUF_T_STRING) return fail(WICK_GGUF_ERR_NOT_FOUND, "metadata key %s is not a string array", key);
    if (index >= v->strings.size()) return fail(WICK_GGUF_ERR_INVALID_ARG, "get_array_str: index %llu out of range", (unsigned long long)index);
    *s = reinterpret_cast<const char*>(g->data + v->strings[(size_t)index].first), *len = (size_t)v->strings[(size_t)index].second;
    return WICK_GGUF_OK;
}

uint64_t wick_gguf_tensor_count(const wick_gguf* g) { return g ? g->tensors.size() : 0; }

int wick_gguf_tensor_name(const wick_gguf* g, uint64_t index, const char** name, size_t* len) {
    if (!g || !name) return fail(WICK_GGUF_ERR_INVALID_ARG, "tensor_name: null argument");
    if (index >= g->tensors.size()) return fail(WICK_GGUF_ERR_INVALID_ARG, "tensor_name: index %llu out of range", (unsigned long long)index);
    *name = g->tensors[(size_t)index].name.c_str();
    if (len) *len = g->tensors[(size_t)index].name.size();
    return WICK_GGUF_OK;
}

int wick_gguf_tensor_info(const wick_gguf* g, const char* name, int* ggml_type, uint32_t* n_dims, uint64_t* dims, uint64_t* abs_offset,
                          uint64_t* size_bytes) {
    const TensorRec* t = nullptr;
    if (int rc = find_tensor(g, name, false, &t)) return rc;
    if (ggml_type) *ggml_type = t->type;
    if (n_dims) *n_dims = t->n_dims;
    if (dims) memcpy(dims, t->dims, sizeof t->dims);
    if (abs_offset) *abs_offset = t->abs_offset;
    if (size_bytes) *size_bytes = t->size_bytes;
    return WICK_GGUF_OK;
}

int wick_gguf_tensor_data(const wick_gguf* g, const char* name, const void** data, size_t* nbytes) {
    if (!data || !nbytes) return fail(WICK_GGUF_ERR_INVALID_ARG, "tensor_data: null out pointer");
    const TensorRec* t = nullptr;
    if (int rc = find_tensor(g, name, true, &t)) return rc;
    *data = g->data + t->abs_offset, *nbytes = (size_t)t->size_bytes;
    return WICK_GGUF_OK;
}

int wick_gguf_tensor_meta(const wick_gguf* g, const char* name, uint64_t* abs_offset, uint64_t* rows, uint64_t* cols, int* ggml_type) {
    const TensorRec* t = nullptr;
    if (int rc = find_tensor(g, name, true, &t)) return rc;
    if (t->n_dims != 1 && t->n_dims != 2) return fail(WICK_GGUF_ERR_FORMAT, "tensor_meta: unexpected rank for %s: %u", name, t->n_dims);
    if (abs_offset) *abs_offset = t->abs_offset;
    if (rows) *rows = t->n_dims == 2 ? t->dims[1] : 1;
    if (cols) *cols = t->dims[0];
    if (ggml_type) *ggml_type = t->type;
    return WICK_GGUF_OK;
}

int wick_gguf_tensor_data_size(int ggml_type, uint64_t numel, uint64_t* nbytes) {
    if (!nbytes) return fail(WICK_GGUF_ERR_INVALID_ARG, "tensor_data_size: null out pointer");
    uint64_t block, bytes;
    if (!type_layout(ggml_type, block, bytes))
        return fail(WICK_GGUF_ERR_UNSUPPORTED, "ggml type %d (%s) has no known block size", ggml_type, wick_gguf_type_name(ggml_type));
    if (numel % block != 0)
        return fail(WICK_GGUF_ERR_FORMAT, "tensor element count %llu is not divisible by block size %llu", (unsigned long long)numel,
                    (unsigned long long)block);
    if (__builtin_mul_overflow(numel / block, bytes, nbytes)) return fail(WICK_GGUF_ERR_FORMAT, "tensor size overflow");
    return WICK_GGUF_OK;
}

const char* wick_gguf_type_name(int t) {
    switch (t) {
        case 0: return "F32";
        case 1: return "F16";
        case 30: return "BF16";
        case 2: return "Q4_0";
        case 3: return "Q4_1";
        case 6: return "Q5_0";
        case 7: return "Q5_1";
        case 8: return "Q8_0";
        case 9: return "Q8_1";
        case 10: return "Q2_K";
        case 11: return "Q3_K";
        case 12: return "Q4_K";
        case 13: return "Q5_K";
        case 14: return "Q6_K";
        case 15: return "Q8_K";
        case 26: return "I32";
        default: return "???";
    }
}

}  // extern "C"
