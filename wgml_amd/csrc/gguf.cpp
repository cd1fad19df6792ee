// GGUF container reader (host only).  Mirrors Gguf::from_bytes of the reference
// (gguf.rs:450-607): header, metadata key/values, tensor infos, tensor data
// located at `offset + align(end of infos, general.alignment or 32)`.  The file
// is memory-mapped; tensor data and POD arrays are handed out as pointers into
// the mapping, nothing is copied.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include <exception>
#include <new>

#include "common.h"

using namespace wgml;

namespace {

constexpr uint32_t kMagicLE = 0x46554747u;  // "GGUF"

// metadata value types (gguf.rs:330-361)
enum : uint32_t { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64 };

size_t scalar_size(uint32_t t) {
    switch (t) {
    case T_U8: case T_I8: case T_BOOL: return 1;
    case T_U16: case T_I16: return 2;
    case T_U32: case T_I32: case T_F32: return 4;
    case T_U64: case T_I64: case T_F64: return 8;
    default: return 0;
    }
}

struct Meta {
    std::string key;
    uint32_t type = 0;
    uint32_t array_type = 0;   // element type if type == T_ARRAY
    uint64_t array_len = 0;
    const uint8_t *data = nullptr;  // scalar: its bytes; string: its bytes; POD array: first element
    uint64_t str_len = 0;           // string: byte length
    std::vector<std::pair<const uint8_t *, uint64_t>> strings;  // string array elements
};

struct Tensor {
    std::string name;
    uint32_t ndims = 0;
    uint64_t dims[4] = {1, 1, 1, 1};
    uint32_t type = 0;
    uint64_t offset = 0;  // from the start of the file
    uint64_t nbytes = 0;  // 0 if the type is not one whose block size is known here
};

// bytes of `n` elements of a GGUF tensor type, 0 if unknown / not a whole number of blocks
uint64_t tensor_bytes(uint32_t type, uint64_t n) {
    uint64_t block = 0, bytes = 0;
    switch (type) {
    case 0: block = 1; bytes = 4; break;      // F32
    case 1: block = 1; bytes = 2; break;      // F16
    case 2: block = 32; bytes = 18; break;    // Q4_0
    case 3: block = 32; bytes = 20; break;    // Q4_1
    case 6: block = 32; bytes = 22; break;    // Q5_0
    case 7: block = 32; bytes = 24; break;    // Q5_1
    case 8: block = 32; bytes = 34; break;    // Q8_0
    case 9: block = 32; bytes = 36; break;    // Q8_1
    case 10: block = 256; bytes = 84; break;  // Q2_K
    case 11: block = 256; bytes = 110; break; // Q3_K
    case 12: block = 256; bytes = 144; break; // Q4_K
    case 13: block = 256; bytes = 176; break; // Q5_K
    case 14: block = 256; bytes = 210; break; // Q6_K
    case 15: block = 256; bytes = 292; break; // Q8_K
    case 24: block = 1; bytes = 1; break;     // I8
    case 25: block = 1; bytes = 2; break;     // I16
    case 26: block = 1; bytes = 4; break;     // I32
    case 27: block = 1; bytes = 8; break;     // I64
    case 28: block = 1; bytes = 8; break;     // F64
    default: return 0;
    }
    if (n % block) return 0;
    return n / block * bytes;
}

}  // namespace

struct wgml_gguf {
    const uint8_t *bytes = nullptr;
    uint64_t size = 0;
    void *map = nullptr;  // non-null if the bytes are our own mapping
    uint32_t version = 0;
    uint32_t alignment = 32;
    std::vector<Meta> meta;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, int> meta_index, tensor_index;
};

namespace {

struct Cursor {
    const uint8_t *b;
    uint64_t n, off = 0;
    bool ok = true;
    bool need(uint64_t k) {
        if (!ok || k > n - off) {
            ok = false;
            return false;
        }
        return true;
    }
    template <class T>
    T pod() {
        T v{};
        if (need(sizeof(T))) {
            std::memcpy(&v, b + off, sizeof(T));
            off += sizeof(T);
        }
        return v;
    }
    // length-prefixed string (gguf.rs:657-661)
    bool str(const uint8_t **p, uint64_t *len) {
        *len = pod<uint64_t>();
        if (!need(*len)) return false;
        *p = b + off;
        off += *len;
        return true;
    }
};

int parse_value(Cursor &c, Meta &m) {
    if (m.type == T_STRING) {
        if (!c.str(&m.data, &m.str_len)) return set_error(WGML_E_INVALID, "gguf: truncated string");
        return WGML_OK;
    }
    if (m.type == T_ARRAY) {
        m.array_type = c.pod<uint32_t>();
        m.array_len = c.pod<uint64_t>();
        if (!c.ok) return set_error(WGML_E_INVALID, "gguf: truncated array header");
        if (m.array_type == T_STRING) {
            m.strings.reserve((size_t)(m.array_len < (1u << 24) ? m.array_len : (1u << 24)));
            for (uint64_t i = 0; i < m.array_len; ++i) {
                const uint8_t *p;
                uint64_t len;
                if (!c.str(&p, &len)) return set_error(WGML_E_INVALID, "gguf: truncated string array");
                m.strings.emplace_back(p, len);
            }
            return WGML_OK;
        }
        const size_t sz = scalar_size(m.array_type);
        if (!sz)
            return set_error(WGML_E_UNSUPPORTED, "gguf: array of element type %u is not supported",
                             m.array_type);
        if (m.array_len > (c.n - c.off) / sz || !c.need(m.array_len * sz))
            return set_error(WGML_E_INVALID, "gguf: truncated array");
        m.data = c.b + c.off;
        c.off += m.array_len * sz;
        return WGML_OK;
    }
    const size_t sz = scalar_size(m.type);
    if (!sz) return set_error(WGML_E_UNSUPPORTED, "gguf: metadata value type %u", m.type);
    if (!c.need(sz)) return set_error(WGML_E_INVALID, "gguf: truncated value");
    m.data = c.b + c.off;
    c.off += sz;
    return WGML_OK;
}

int parse(wgml_gguf *g) {
    Cursor c{g->bytes, g->size};
    const uint32_t magic = c.pod<uint32_t>();
    if (!c.ok || magic != kMagicLE)
        return set_error(WGML_E_INVALID, "gguf: bad magic number 0x%08x", magic);
    g->version = c.pod<uint32_t>();
    const uint64_t n_tensors = c.pod<uint64_t>();
    const uint64_t n_meta = c.pod<uint64_t>();
    if (!c.ok) return set_error(WGML_E_INVALID, "gguf: truncated header");
    // a metadata record takes at least 13 bytes of the file (key length, type, one value
    // byte), a tensor record at least 24 (name length, ndims, type, offset): counts beyond
    // what the remaining bytes can hold are refused before anything is reserved for them
    const uint64_t remaining = g->size - c.off;
    if (n_meta > remaining / 13 || n_tensors > remaining / 24)
        return set_error(WGML_E_INVALID, "gguf: implausible counts in the header");
    g->meta.reserve((size_t)n_meta);
    for (uint64_t i = 0; i < n_meta; ++i) {
        Meta m;
        const uint8_t *kp;
        uint64_t klen;
        if (!c.str(&kp, &klen)) return set_error(WGML_E_INVALID, "gguf: truncated metadata key");
        m.key.assign(reinterpret_cast<const char *>(kp), (size_t)klen);
        m.type = c.pod<uint32_t>();
        if (!c.ok) return set_error(WGML_E_INVALID, "gguf: truncated metadata");
        WGML_TRY(parse_value(c, m));
        g->meta_index[m.key] = (int)g->meta.size();
        g->meta.push_back(std::move(m));
    }
    // general.alignment (u32), else 32 (gguf.rs:455-464)
    auto it = g->meta_index.find("general.alignment");
    if (it != g->meta_index.end() && g->meta[it->second].type == T_U32) {
        std::memcpy(&g->alignment, g->meta[it->second].data, 4);
        if (g->alignment == 0) return set_error(WGML_E_INVALID, "gguf: general.alignment is zero");
    }
    g->tensors.reserve((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; ++i) {
        Tensor t;
        const uint8_t *np;
        uint64_t nlen;
        if (!c.str(&np, &nlen)) return set_error(WGML_E_INVALID, "gguf: truncated tensor name");
        t.name.assign(reinterpret_cast<const char *>(np), (size_t)nlen);
        t.ndims = c.pod<uint32_t>();
        if (!c.ok || t.ndims > 4)
            return set_error(WGML_E_UNSUPPORTED, "gguf: tensor '%s' has %u dimensions (limit 4)",
                             t.name.c_str(), t.ndims);
        for (uint32_t d = 0; d < t.ndims; ++d) t.dims[d] = c.pod<uint64_t>();
        t.type = c.pod<uint32_t>();
        t.offset = c.pod<uint64_t>();
        if (!c.ok) return set_error(WGML_E_INVALID, "gguf: truncated tensor info");
        g->tensor_index[t.name] = (int)g->tensors.size();
        g->tensors.push_back(std::move(t));
    }
    const uint64_t a = g->alignment;
    const uint64_t data_start = c.off + (a - c.off % a) % a;
    for (Tensor &t : g->tensors) {
        // element count with overflow checks: a wrapped product would pass the bounds check
        // below with dims that describe a far larger tensor
        uint64_t n = 1;
        bool wrapped = false;
        for (int d = 0; d < 4; ++d) wrapped = wrapped || __builtin_mul_overflow(n, t.dims[d], &n);
        if (wrapped || n > (uint64_t)1 << 48 || t.offset > g->size)
            return set_error(WGML_E_INVALID, "gguf: tensor '%s' has implausible dimensions or offset",
                             t.name.c_str());
        t.offset += data_start;
        t.nbytes = tensor_bytes(t.type, n);
        if (t.offset > g->size || t.nbytes > g->size - t.offset)
            return set_error(WGML_E_INVALID, "gguf: tensor '%s' lies outside the file",
                             t.name.c_str());
    }
    return WGML_OK;
}

}  // namespace

extern "C" {

int wgml_gguf_open_bytes(const void *bytes, uint64_t size, wgml_gguf **out) {
    WGML_REQUIRE(bytes && out, "wgml_gguf_open_bytes: null argument");
    *out = nullptr;
    // no C++ exception may cross the C boundary: a file that makes the tables run out of
    // memory is reported like any other unreadable file
    wgml_gguf *g = nullptr;
    int rc;
    try {
        g = new wgml_gguf();
        g->bytes = static_cast<const uint8_t *>(bytes);
        g->size = size;
        rc = parse(g);
    } catch (const std::bad_alloc &) {
        rc = set_error(WGML_E_OOM, "wgml_gguf_open: out of memory while reading the tables");
    } catch (const std::exception &e) {
        rc = set_error(WGML_E_INVALID, "wgml_gguf_open: %s", e.what());
    }
    if (rc != WGML_OK) {
        delete g;
        return rc;
    }
    *out = g;
    return WGML_OK;
}

int wgml_gguf_open(const char *path, wgml_gguf **out) {
    WGML_REQUIRE(path && out, "wgml_gguf_open: null argument");
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) return set_error(WGML_E_INVALID, "wgml_gguf_open: cannot open '%s'", path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        ::close(fd);
        return set_error(WGML_E_INVALID, "wgml_gguf_open: cannot stat '%s' (or it is empty)", path);
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map == MAP_FAILED) return set_error(WGML_E_OOM, "wgml_gguf_open: mmap of '%s' failed", path);
    wgml_gguf *g = nullptr;
    const int rc = wgml_gguf_open_bytes(map, (uint64_t)st.st_size, &g);
    if (rc != WGML_OK) {
        munmap(map, (size_t)st.st_size);
        return rc;
    }
    g->map = map;
    *out = g;
    return WGML_OK;
}

int wgml_gguf_close(wgml_gguf *g) {
    if (!g) return WGML_OK;
    if (g->map) munmap(g->map, (size_t)g->size);
    delete g;
    return WGML_OK;
}

uint32_t wgml_gguf_version(const wgml_gguf *g) { return g ? g->version : 0; }
uint32_t wgml_gguf_alignment(const wgml_gguf *g) { return g ? g->alignment : 0; }
uint64_t wgml_gguf_n_metadata(const wgml_gguf *g) { return g ? g->meta.size() : 0; }
uint64_t wgml_gguf_n_tensors(const wgml_gguf *g) { return g ? g->tensors.size() : 0; }

int64_t wgml_gguf_find_metadata(const wgml_gguf *g, const char *key) {
    if (!g || !key) return -1;
    auto it = g->meta_index.find(key);
    return it == g->meta_index.end() ? -1 : it->second;
}

int64_t wgml_gguf_find_tensor(const wgml_gguf *g, const char *name) {
    if (!g || !name) return -1;
    auto it = g->tensor_index.find(name);
    return it == g->tensor_index.end() ? -1 : it->second;
}

int wgml_gguf_metadata(const wgml_gguf *g, uint64_t i, wgml_gguf_kv *out) {
    WGML_REQUIRE(g && out, "wgml_gguf_metadata: null argument");
    WGML_REQUIRE(i < g->meta.size(), "wgml_gguf_metadata: index %llu outside %zu entries",
                 (unsigned long long)i, g->meta.size());
    const Meta &m = g->meta[(size_t)i];
    out->key = m.key.c_str();
    out->type = (int)m.type;
    out->array_type = (int)m.array_type;
    out->array_len = m.array_len;
    out->data = m.data;
    out->nbytes = m.type == T_STRING  ? m.str_len
                  : m.type == T_ARRAY ? (m.array_type == T_STRING ? 0 : m.array_len * scalar_size(m.array_type))
                                      : scalar_size(m.type);
    return WGML_OK;
}

int wgml_gguf_metadata_string(const wgml_gguf *g, uint64_t i, uint64_t k, const char **s,
                              uint64_t *len) {
    WGML_REQUIRE(g && s && len, "wgml_gguf_metadata_string: null argument");
    WGML_REQUIRE(i < g->meta.size(), "wgml_gguf_metadata_string: index outside the metadata");
    const Meta &m = g->meta[(size_t)i];
    WGML_REQUIRE(m.type == T_ARRAY && m.array_type == T_STRING && k < m.strings.size(),
                 "wgml_gguf_metadata_string: '%s' is not a string array with more than %llu elements",
                 m.key.c_str(), (unsigned long long)k);
    *s = reinterpret_cast<const char *>(m.strings[(size_t)k].first);
    *len = m.strings[(size_t)k].second;
    return WGML_OK;
}

int wgml_gguf_tensor(const wgml_gguf *g, uint64_t i, wgml_gguf_tensor_info *out) {
    WGML_REQUIRE(g && out, "wgml_gguf_tensor: null argument");
    WGML_REQUIRE(i < g->tensors.size(), "wgml_gguf_tensor: index %llu outside %zu tensors",
                 (unsigned long long)i, g->tensors.size());
    const Tensor &t = g->tensors[(size_t)i];
    out->name = t.name.c_str();
    out->type = (int)t.type;
    out->ndims = t.ndims;
    for (int d = 0; d < 4; ++d) out->dims[d] = t.dims[d];
    out->offset = t.offset;
    out->nbytes = t.nbytes;
    out->data = g->bytes + t.offset;
    return WGML_OK;
}

}  // extern "C"
