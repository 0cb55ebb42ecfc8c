// GGUF file -> HBM: the mapping and parse of GGUFLoader::from_file (src/core/loader.rs:211-320), the metadata
// conversions of MetaValue (src/core/tensor.rs:146-187), the tensor checks of checked_tensor
// (src/models/qwen3.rs:1350-1380), and the uploads that take tensor bytes straight from the mapping through the
// pinned staging pair into the repacked tile streams.  Host code only; the kernels are the upload-time repacks.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cmath>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "rmi_internal.h"

namespace {

// metadata value tags (src/core/tensor.rs:92-106)
enum : int32_t {
    kU8 = 0, kI8 = 1, kU16 = 2, kI16 = 3, kU32 = 4, kI32 = 5, kF32 = 6, kBool = 7, kStr = 8, kArr = 9, kU64 = 10,
    kI64 = 11, kF64 = 12,
};

struct MetaValue {
    int32_t type = -1;
    union {
        uint64_t u;
        int64_t i;
        double f;
    } v = {0};
    const char *str = nullptr;  // kStr: bytes in the mapping (not terminated)
    uint64_t str_len = 0;
    int32_t elem_type = -1;  // kArr
    uint64_t n_elems = 0;
    size_t arr_pos = 0;  // kArr: offset of the first element in the mapping
};

struct TensorEntry {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[8] = {0};
    int32_t ggml_type = 0;
    uint64_t offset = 0;
    uint64_t nbytes = 0;
};

// (block elements, block bytes) of src/core/tensor.rs:61-81; false for a tag the reference does not know
bool type_traits(int32_t t, uint32_t *elems, uint32_t *bytes) {
    static const struct {
        int32_t t;
        uint32_t e, b;
    } k[] = {{0, 1, 4},     {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},   {7, 32, 24},
             {8, 32, 34},   {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176},
             {14, 256, 210}, {15, 256, 292}, {16, 1, 1},     {17, 1, 2},     {18, 1, 4}};
    for (const auto &e : k)
        if (e.t == t) {
            *elems = e.e;
            *bytes = e.b;
            return true;
        }
    return false;
}

const char *type_name(int32_t t) {
    switch (t) {
        case 0: return "F32";
        case 1: return "F16";
        case 2: return "Q4_0";
        case 8: return "Q8_0";
        case 12: return "Q4K";
        case 14: return "Q6K";
        default: return "other";
    }
}

bool mul_ok(uint64_t a, uint64_t b, uint64_t *out) { return !__builtin_mul_overflow(a, b, out); }

// TensorInfo::checked_nbytes (src/core/tensor.rs:205-219)
bool checked_nbytes(const TensorEntry &t, uint64_t *out) {
    if (t.n_dims == 0) return false;
    uint64_t rows = 1;
    for (uint32_t i = 1; i < t.n_dims; i++)
        if (!mul_ok(rows, t.dims[i], &rows)) return false;
    uint32_t be, bb;
    if (!type_traits(t.ggml_type, &be, &bb)) return false;
    if (t.dims[0] % be != 0) return false;
    uint64_t n;
    return mul_ok(t.dims[0] / be, bb, &n) && mul_ok(n, rows, out);
}

// bounds-checked little-endian cursor (ByteReader, src/core/loader.rs:18-185)
struct Reader {
    const uint8_t *data;
    size_t len, pos = 0;
    std::string err;

    size_t remaining() const { return len > pos ? len - pos : 0; }
    bool fail(const std::string &m) {
        if (err.empty()) err = m;
        return false;
    }
    template <typename T>
    bool rd(T *out, const char *what) {
        if (remaining() < sizeof(T)) return fail(std::string("EOF reading ") + what);
        memcpy(out, data + pos, sizeof(T));
        pos += sizeof(T);
        return true;
    }
    bool ensure_count(uint64_t n, size_t min_item, const char *ctx) {
        if (n > remaining() / min_item) return fail(std::string(ctx) + " count exceeds remaining bytes");
        return true;
    }
    // String::from_utf8: well-formed UTF-8 only (no overlong forms, no surrogates, nothing past U+10FFFF)
    static bool utf8_ok(const uint8_t *s, size_t n) {
        for (size_t i = 0; i < n;) {
            const uint8_t c = s[i];
            size_t more;
            uint32_t cp, min;
            if (c < 0x80) {
                i++;
                continue;
            } else if ((c & 0xe0) == 0xc0) {
                more = 1, cp = c & 0x1f, min = 0x80;
            } else if ((c & 0xf0) == 0xe0) {
                more = 2, cp = c & 0x0f, min = 0x800;
            } else if ((c & 0xf8) == 0xf0) {
                more = 3, cp = c & 0x07, min = 0x10000;
            } else {
                return false;
            }
            if (n - i <= more) return false;
            for (size_t k = 1; k <= more; k++) {
                if ((s[i + k] & 0xc0) != 0x80) return false;
                cp = (cp << 6) | (s[i + k] & 0x3f);
            }
            if (cp < min || cp > 0x10ffff || (cp >= 0xd800 && cp <= 0xdfff)) return false;
            i += more + 1;
        }
        return true;
    }
    bool rd_str(const char **p, uint64_t *n) {
        if (!rd(n, "u64")) return false;
        if (*n > remaining()) return fail("EOF reading string of length " + std::to_string(*n));
        if (!utf8_ok(data + pos, size_t(*n))) return fail("Invalid UTF-8 string");
        *p = reinterpret_cast<const char *>(data + pos);
        pos += size_t(*n);
        return true;
    }
    static size_t scalar_size(int32_t t) {
        switch (t) {
            case kU8: case kI8: case kBool: return 1;
            case kU16: case kI16: return 2;
            case kU32: case kI32: case kF32: return 4;
            case kU64: case kI64: case kF64: return 8;
            default: return 0;
        }
    }
    bool rd_value(int32_t t, MetaValue *m, bool nested) {
        m->type = t;
        switch (t) {
            case kU8: { uint8_t x; if (!rd(&x, "u8")) return false; m->v.u = x; return true; }
            case kI8: { int8_t x; if (!rd(&x, "u8")) return false; m->v.i = x; return true; }
            case kU16: { uint16_t x; if (!rd(&x, "u16")) return false; m->v.u = x; return true; }
            case kI16: { int16_t x; if (!rd(&x, "u16")) return false; m->v.i = x; return true; }
            case kU32: { uint32_t x; if (!rd(&x, "u32")) return false; m->v.u = x; return true; }
            case kI32: { int32_t x; if (!rd(&x, "u32")) return false; m->v.i = x; return true; }
            case kF32: { float x; if (!rd(&x, "u32")) return false; m->v.f = x; return true; }
            case kBool: {
                uint8_t x;
                if (!rd(&x, "u8")) return false;
                if (x > 1) return fail("Invalid bool value: " + std::to_string(x));
                m->v.u = x;
                return true;
            }
            case kStr: return rd_str(&m->str, &m->str_len);
            case kU64: return rd(&m->v.u, "u64");
            case kI64: return rd(&m->v.i, "u64");
            case kF64: return rd(&m->v.f, "u64");
            case kArr: {
                if (nested) return fail("Nested metadata arrays are not supported");
                if (!rd(&m->elem_type, "u32")) return false;
                if (m->elem_type < 0 || m->elem_type > kF64)
                    return fail("Unknown meta value type: " + std::to_string(m->elem_type));
                if (!rd(&m->n_elems, "u64")) return false;
                if (m->elem_type == kArr) return fail("Nested metadata arrays are not supported");
                const size_t item = m->elem_type == kStr ? 8 : scalar_size(m->elem_type);
                if (!ensure_count(m->n_elems, item, "array")) return false;
                m->arr_pos = pos;
                if (m->elem_type == kStr) {
                    for (uint64_t i = 0; i < m->n_elems; i++) {
                        const char *p;
                        uint64_t n;
                        if (!rd_str(&p, &n)) return false;
                    }
                } else if (m->elem_type == kBool) {
                    for (uint64_t i = 0; i < m->n_elems; i++) {
                        MetaValue e;
                        if (!rd_value(kBool, &e, true)) return false;
                    }
                } else {
                    pos += size_t(m->n_elems) * item;  // fits: ensure_count
                }
                return true;
            }
            default: return fail("Unknown meta value type: " + std::to_string(t));
        }
    }
};

// Rust's float -> u64 `as`: NaN and negatives give 0, values past the range saturate
uint64_t f_to_u64(double f) {
    if (!(f > 0.0)) return 0;
    if (f >= 18446744073709551616.0) return ~uint64_t(0);
    return uint64_t(f);
}

bool scalar_to_u64(const MetaValue &m, uint64_t *out) {  // MetaValue::to_u64, src/core/tensor.rs:147-162
    switch (m.type) {
        case kU8: case kU16: case kU32: case kU64: *out = m.v.u; return true;
        case kI8: case kI16: case kI32: case kI64: *out = uint64_t(m.v.i); return true;  // sign-extended, as `as u64`
        case kF32: case kF64: *out = f_to_u64(m.v.f); return true;
        default: return false;
    }
}

bool scalar_to_f64(const MetaValue &m, double *out) {  // MetaValue::to_f64, src/core/tensor.rs:164-174
    switch (m.type) {
        case kF32: case kF64: *out = m.v.f; return true;
        case kU32: case kU64: *out = double(m.v.u); return true;
        case kI32: case kI64: *out = double(m.v.i); return true;
        default: return false;
    }
}

}  // namespace

struct rmi_hip_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    size_t len = 0;
    uint32_t version = 0;
    uint64_t alignment = 32;
    size_t data_offset = 0;
    std::vector<std::pair<std::string, MetaValue>> kv;
    std::vector<TensorEntry> tensors;
    std::unordered_map<std::string, size_t> by_name;  // first entry of a name, as the reference's linear find

    const MetaValue *meta(const char *key) const {
        for (const auto &e : kv)
            if (e.first == key) return &e.second;
        return nullptr;
    }
    const TensorEntry *tensor(const std::string &name) const {
        auto it = by_name.find(name);
        return it == by_name.end() ? nullptr : &tensors[it->second];
    }
    const uint8_t *bytes(const TensorEntry &t) const { return map + data_offset + size_t(t.offset); }
};

namespace {

bool parse(rmi_hip_gguf *g, std::string *err) {
    Reader r{g->map, g->len};
    uint32_t magic;
    if (!r.rd(&magic, "u32")) return *err = r.err, false;
    if (memcmp(&magic, "GGUF", 4) != 0) {
        const uint8_t *b = reinterpret_cast<const uint8_t *>(&magic);
        char buf[96];
        snprintf(buf, sizeof(buf), "Invalid GGUF magic: [%u, %u, %u, %u] (expected [71, 71, 85, 70])", b[0], b[1], b[2], b[3]);
        return *err = buf, false;
    }
    if (!r.rd(&g->version, "u32")) return *err = r.err, false;
    if (g->version < 2 || g->version > 3) return *err = "Unsupported GGUF version: " + std::to_string(g->version), false;
    uint64_t n_tensors, n_kv;
    if (!r.rd(&n_tensors, "u64") || !r.rd(&n_kv, "u64")) return *err = r.err, false;
    if (!r.ensure_count(n_kv, 13, "metadata")) return *err = r.err, false;
    g->kv.reserve(size_t(n_kv));
    for (uint64_t i = 0; i < n_kv; i++) {
        const char *kp;
        uint64_t kn;
        int32_t t;
        MetaValue m;
        if (!r.rd_str(&kp, &kn) || !r.rd(&t, "u32")) return *err = r.err, false;
        if (t < 0 || t > kF64) return *err = "Unknown meta value type: " + std::to_string(t), false;
        if (!r.rd_value(t, &m, false)) return *err = r.err, false;
        g->kv.emplace_back(std::string(kp, size_t(kn)), m);
    }
    if (!r.ensure_count(n_tensors, 24, "tensor")) return *err = r.err, false;
    g->tensors.reserve(size_t(n_tensors));
    for (uint64_t i = 0; i < n_tensors; i++) {
        const char *np;
        uint64_t nn;
        TensorEntry t;
        if (!r.rd_str(&np, &nn) || !r.rd(&t.n_dims, "u32")) return *err = r.err, false;
        t.name.assign(np, size_t(nn));
        if (!r.ensure_count(t.n_dims, 8, "tensor dimension")) return *err = r.err, false;
        if (t.n_dims > 8) return *err = "tensor " + t.name + " has " + std::to_string(t.n_dims) + " dimensions", false;
        for (uint32_t d = 0; d < t.n_dims; d++)
            if (!r.rd(&t.dims[d], "u64")) return *err = r.err, false;
        if (!r.rd(&t.ggml_type, "u32")) return *err = r.err, false;
        uint32_t be, bb;
        if (!type_traits(t.ggml_type, &be, &bb)) return *err = "Unknown GGML type: " + std::to_string(t.ggml_type), false;
        if (!r.rd(&t.offset, "u64")) return *err = r.err, false;
        g->tensors.push_back(std::move(t));
    }
    if (const MetaValue *a = g->meta("general.alignment")) {
        uint64_t v;
        if (scalar_to_u64(*a, &v)) g->alignment = v;
    }
    if (g->alignment == 0) return *err = "GGUF alignment must be nonzero", false;
    const size_t rem = r.pos % g->alignment;
    g->data_offset = r.pos;
    if (rem && __builtin_add_overflow(r.pos, size_t(g->alignment - rem), &g->data_offset))
        return *err = "GGUF data offset overflow", false;
    for (size_t i = 0; i < g->tensors.size(); i++) {
        TensorEntry &t = g->tensors[i];
        if (!checked_nbytes(t, &t.nbytes)) return *err = "invalid tensor shape: " + t.name, false;
        uint64_t start, end;
        if (__builtin_add_overflow(uint64_t(g->data_offset), t.offset, &start) ||
            __builtin_add_overflow(start, t.nbytes, &end))
            return *err = "tensor " + t.name + " range overflow", false;
        if (end > g->len) return *err = "tensor " + t.name + " exceeds GGUF data", false;
        g->by_name.emplace(t.name, i);
    }
    return true;
}

int weight_dtype(int32_t ggml_type) {
    switch (ggml_type) {
        case 2: return RMI_HIP_DTYPE_Q4_0;
        case 8: return RMI_HIP_DTYPE_Q8_0;
        case 12: return RMI_HIP_DTYPE_Q4_K;
        case 14: return RMI_HIP_DTYPE_Q6_K;
        default: return 0;
    }
}

std::string dims_text(const uint64_t *d, uint32_t n) {
    std::string s = "[";
    for (uint32_t i = 0; i < n; i++) s += (i ? ", " : "") + std::to_string(d[i]);
    return s + "]";
}

// checked_tensor (src/models/qwen3.rs:1350-1380): name present, dims and type as expected
const TensorEntry *expect_tensor(const rmi_hip_gguf *g, const std::string &name, const uint64_t *dims, uint32_t n_dims,
                                 int32_t ggml_type) {
    const TensorEntry *t = g->tensor(name);
    if (!t) {
        rmi_set_error("Missing tensor: %s", name.c_str());
        return nullptr;
    }
    bool same = t->n_dims == n_dims && t->ggml_type == ggml_type;
    for (uint32_t i = 0; same && i < n_dims; i++) same = t->dims[i] == dims[i];
    if (!same) {
        rmi_set_error("Invalid tensor %s: shape %s type %s; expected %s %s", name.c_str(),
                      dims_text(t->dims, t->n_dims).c_str(), type_name(t->ggml_type), dims_text(dims, n_dims).c_str(),
                      type_name(ggml_type));
        return nullptr;
    }
    return t;
}

bool get_u64(const rmi_hip_gguf *g, const std::string &key, uint64_t *out) {
    const MetaValue *m = g->meta(key.c_str());
    if (!m || !scalar_to_u64(*m, out)) {
        rmi_set_error("Missing metadata: %s", key.c_str());
        return false;
    }
    return true;
}

bool fits_u32(uint64_t v, const std::string &key, uint32_t *out) {
    if (v > 0xffffffffull) {
        rmi_set_error("%s = %llu is beyond what the device session addresses", key.c_str(), (unsigned long long)v);
        return false;
    }
    *out = uint32_t(v);
    return true;
}

}  // namespace

extern "C" {

rmi_hip_gguf *rmi_hip_gguf_open(const char *path) {
    if (!path) {
        rmi_set_error("null path");
        return nullptr;
    }
    rmi_hip_gguf *g = new rmi_hip_gguf();
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (g->fd < 0 || fstat(g->fd, &st) != 0) {
        rmi_set_error("Failed to open GGUF file: %s: %s", path, strerror(errno));
        rmi_hip_gguf_close(g);
        return nullptr;
    }
    g->len = size_t(st.st_size);
    if (g->len) {
        void *m = mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, g->fd, 0);
        if (m == MAP_FAILED) {
            rmi_set_error("Failed to mmap: %s", strerror(errno));
            rmi_hip_gguf_close(g);
            return nullptr;
        }
        g->map = static_cast<const uint8_t *>(m);
        madvise(m, g->len, MADV_SEQUENTIAL);  // the uploads walk the tensor data once, front to back
    }
    std::string err;
    if (!parse(g, &err)) {
        rmi_set_error("%s", err.c_str());
        rmi_hip_gguf_close(g);
        return nullptr;
    }
    return g;
}

void rmi_hip_gguf_close(rmi_hip_gguf *g) {
    if (!g) return;
    if (g->map) munmap(const_cast<uint8_t *>(g->map), g->len);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

uint32_t rmi_hip_gguf_version(const rmi_hip_gguf *g) { return g ? g->version : 0; }
uint64_t rmi_hip_gguf_alignment(const rmi_hip_gguf *g) { return g ? g->alignment : 0; }
uint64_t rmi_hip_gguf_data_offset(const rmi_hip_gguf *g) { return g ? g->data_offset : 0; }
uint64_t rmi_hip_gguf_n_tensors(const rmi_hip_gguf *g) { return g ? g->tensors.size() : 0; }
uint64_t rmi_hip_gguf_n_kv(const rmi_hip_gguf *g) { return g ? g->kv.size() : 0; }

const char *rmi_hip_gguf_kv_key(const rmi_hip_gguf *g, uint64_t index) {
    return g && index < g->kv.size() ? g->kv[size_t(index)].first.c_str() : nullptr;
}

int rmi_hip_gguf_meta_type(const rmi_hip_gguf *g, const char *key) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    return m ? m->type : -1;
}

int rmi_hip_gguf_meta_u64(const rmi_hip_gguf *g, const char *key, uint64_t *out) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    uint64_t v;
    if (!m || !scalar_to_u64(*m, &v)) return 0;
    if (out) *out = v;
    return 1;
}

int rmi_hip_gguf_meta_f64(const rmi_hip_gguf *g, const char *key, double *out) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    double v;
    if (!m || !scalar_to_f64(*m, &v)) return 0;
    if (out) *out = v;
    return 1;
}

int rmi_hip_gguf_meta_bool(const rmi_hip_gguf *g, const char *key, int *out) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    if (!m || m->type != kBool) return 0;
    if (out) *out = int(m->v.u);
    return 1;
}

int64_t rmi_hip_gguf_meta_str(const rmi_hip_gguf *g, const char *key, char *buf, size_t cap) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    if (!m || m->type != kStr) return -1;
    if (buf && cap) {
        const size_t n = m->str_len < cap - 1 ? size_t(m->str_len) : cap - 1;
        memcpy(buf, m->str, n);
        buf[n] = 0;
    }
    return int64_t(m->str_len);
}

int64_t rmi_hip_gguf_meta_array_len(const rmi_hip_gguf *g, const char *key, int *elem_type) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    if (!m || m->type != kArr) return -1;
    if (elem_type) *elem_type = m->elem_type;
    return int64_t(m->n_elems);
}

int rmi_hip_gguf_meta_array_u64(const rmi_hip_gguf *g, const char *key, uint64_t index, uint64_t *out) {
    const MetaValue *m = g && key ? g->meta(key) : nullptr;
    if (!m || m->type != kArr || index >= m->n_elems) return 0;
    const size_t item = Reader::scalar_size(m->elem_type);
    if (item == 0) return 0;  // strings
    Reader r{g->map, g->len};
    r.pos = m->arr_pos + size_t(index) * item;
    MetaValue e;
    uint64_t v;
    if (!r.rd_value(m->elem_type, &e, true) || !scalar_to_u64(e, &v)) return 0;
    if (out) *out = v;
    return 1;
}

int64_t rmi_hip_gguf_find_tensor(const rmi_hip_gguf *g, const char *name) {
    if (!g || !name) return -1;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? -1 : int64_t(it->second);
}

int rmi_hip_gguf_tensor_info(const rmi_hip_gguf *g, uint64_t index, const char **name, uint32_t *n_dims, uint64_t *dims,
                             uint32_t dims_cap, int *ggml_type, uint64_t *offset, uint64_t *nbytes) {
    if (!g || index >= g->tensors.size()) return rmi_fail(RMI_HIP_E_INVALID, "tensor index %llu out of range", (unsigned long long)index);
    const TensorEntry &t = g->tensors[size_t(index)];
    if (name) *name = t.name.c_str();
    if (n_dims) *n_dims = t.n_dims;
    if (dims)
        for (uint32_t i = 0; i < t.n_dims && i < dims_cap; i++) dims[i] = t.dims[i];
    if (ggml_type) *ggml_type = t.ggml_type;
    if (offset) *offset = t.offset;
    if (nbytes) *nbytes = t.nbytes;
    return RMI_HIP_OK;
}

const uint8_t *rmi_hip_gguf_tensor_data(const rmi_hip_gguf *g, uint64_t index) {
    if (!g || index >= g->tensors.size()) {
        rmi_set_error("tensor index %llu out of range", (unsigned long long)index);
        return nullptr;
    }
    return g->bytes(g->tensors[size_t(index)]);
}

rmi_hip_weight *rmi_hip_gguf_upload_stack(const rmi_hip_gguf *g, const char *const *names, int n_names) {
    if (!g || !names || n_names < 1 || n_names > 16) {
        rmi_set_error("null file or 1..16 tensor names expected");
        return nullptr;
    }
    const uint8_t *parts[16];
    uint32_t rows[16];
    int dtype = 0;
    uint64_t n_in = 0;
    for (int i = 0; i < n_names; i++) {
        const TensorEntry *t = names[i] ? g->tensor(names[i]) : nullptr;
        if (!t) {
            rmi_set_error("Missing tensor: %s", names[i] ? names[i] : "(null)");
            return nullptr;
        }
        const int dt = weight_dtype(t->ggml_type);
        if (dt == 0 || t->n_dims != 2 || t->dims[0] > 0xffffffffull || t->dims[1] > 0xffffffffull) {
            rmi_set_error("Invalid tensor %s: shape %s type %s; expected a Q8_0, Q4_0, Q4K or Q6K matrix", names[i],
                          dims_text(t->dims, t->n_dims).c_str(), type_name(t->ggml_type));
            return nullptr;
        }
        if (i == 0) {
            dtype = dt;
            n_in = t->dims[0];
        } else if (dt != dtype || t->dims[0] != n_in) {
            rmi_set_error("tensor %s does not stack under %s: type or column count differ", names[i], names[0]);
            return nullptr;
        }
        parts[i] = g->bytes(*t);
        rows[i] = uint32_t(t->dims[1]);
    }
    return rmi_upload_stack(dtype, parts, rows, n_names, uint32_t(n_in), true);
}

rmi_hip_weight *rmi_hip_gguf_upload(const rmi_hip_gguf *g, const char *name) {
    return rmi_hip_gguf_upload_stack(g, &name, 1);
}

int rmi_hip_gguf_qwen3_config(const rmi_hip_gguf *g, uint32_t capacity, int rounding, rmi_hip_qwen3_config *out) {
    if (!g || !out) return rmi_fail(RMI_HIP_E_INVALID, "null file or configuration");
    // Qwen3Config::from_source (src/models/qwen3.rs:46-94) over model_config_from_source
    // (src/core/loader.rs:379-461) and qwen3_arch_knobs (:541-582), for the architectures whose rope is rope_neox
    const MetaValue *am = g->meta("general.architecture");
    const std::string arch = am && am->type == kStr ? std::string(am->str, size_t(am->str_len)) : std::string();
    if (!am || am->type != kStr) return rmi_fail(RMI_HIP_E_INVALID, "Missing metadata: general.architecture");
    if (arch != "qwen2" && arch != "qwen3" && arch != "qwen35" && arch != "qwen3tts" && arch != "llama" &&
        arch != "hunyuan-dense")
        return rmi_fail(RMI_HIP_E_INVALID, "Unsupported Qwen3-family architecture: %s", arch.c_str());
    const std::string p = arch + ".";
    uint64_t n_embd, n_head, n_layer, n_head_kv, n_ff, n_ctx, vocab = 0, hk, hv;
    if (!get_u64(g, p + "embedding_length", &n_embd) || !get_u64(g, p + "attention.head_count", &n_head))
        return RMI_HIP_E_INVALID;
    if (n_head == 0 || n_embd % n_head != 0)
        return rmi_fail(RMI_HIP_E_INVALID, "Invalid %s head shape: embedding_length=%llu, head_count=%llu", arch.c_str(),
                        (unsigned long long)n_embd, (unsigned long long)n_head);
    if (!get_u64(g, p + "block_count", &n_layer) || !get_u64(g, p + "attention.head_count_kv", &n_head_kv) ||
        !get_u64(g, p + "feed_forward_length", &n_ff) || !get_u64(g, p + "context_length", &n_ctx))
        return RMI_HIP_E_INVALID;
    if (const MetaValue *m = g->meta((p + "vocab_size").c_str()); !m || !scalar_to_u64(*m, &vocab)) {
        const MetaValue *tok = g->meta("tokenizer.ggml.tokens");
        vocab = tok && tok->type == kArr ? tok->n_elems : 0;
    }
    hk = hv = n_embd / n_head;
    for (int which = 0; which < 2; which++) {
        const std::string key = p + (which ? "attention.value_length" : "attention.key_length");
        if (const MetaValue *m = g->meta(key.c_str())) {
            if (!scalar_to_u64(*m, which ? &hv : &hk)) return rmi_fail(RMI_HIP_E_INVALID, "Invalid metadata: %s", key.c_str());
        }
    }
    if (hk == 0 || hv == 0)
        return rmi_fail(RMI_HIP_E_INVALID, "Invalid %s attention head lengths: key=%llu, value=%llu", arch.c_str(),
                        (unsigned long long)hk, (unsigned long long)hv);
    double eps, freq_base = 1000000.0;
    {
        const std::string key = p + "attention.layer_norm_rms_epsilon";
        const MetaValue *m = g->meta(key.c_str());
        if (!m || !scalar_to_f64(*m, &eps)) return rmi_fail(RMI_HIP_E_INVALID, "Missing metadata: %s", key.c_str());
        if (const MetaValue *fb = g->meta((p + "rope.freq_base").c_str())) scalar_to_f64(*fb, &freq_base);
    }
    // checked_session_capacity (src/models/qwen3.rs:108-121)
    if (capacity > n_ctx)
        return rmi_fail(RMI_HIP_E_INVALID, "Session capacity %u exceeds model context %llu", capacity, (unsigned long long)n_ctx);
    rmi_hip_qwen3_config c{};
    if (!fits_u32(n_embd, p + "embedding_length", &c.n_embd) || !fits_u32(n_layer, p + "block_count", &c.n_layer) ||
        !fits_u32(n_head, p + "attention.head_count", &c.n_head) ||
        !fits_u32(n_head_kv, p + "attention.head_count_kv", &c.n_head_kv) ||
        !fits_u32(hk, p + "attention.key_length", &c.head_dim_k) ||
        !fits_u32(hv, p + "attention.value_length", &c.head_dim_v) ||
        !fits_u32(n_ff, p + "feed_forward_length", &c.n_ff) || !fits_u32(vocab, p + "vocab_size", &c.vocab))
        return RMI_HIP_E_INVALID;
    c.capacity = capacity;
    c.eps = float(eps);
    c.freq_base = float(freq_base);
    c.has_qk_norm = arch == "qwen3" || arch == "hunyuan-dense";
    c.rounding = rounding;
    *out = c;
    return RMI_HIP_OK;
}

rmi_hip_qwen3 *rmi_hip_qwen3_create_from_gguf(const rmi_hip_gguf *g, uint32_t capacity, int rounding) {
    rmi_hip_qwen3_config c;
    if (rmi_hip_gguf_qwen3_config(g, capacity, rounding, &c) != RMI_HIP_OK) return nullptr;
    // tensor names, shapes and types of Qwen3Model::from_source (src/models/qwen3.rs:262-349)
    const uint64_t n_q = uint64_t(c.n_head) * c.head_dim_k, n_k = uint64_t(c.n_head_kv) * c.head_dim_k,
                   n_v = uint64_t(c.n_head_kv) * c.head_dim_v, n_attn = uint64_t(c.n_head) * c.head_dim_v;
    const uint64_t d_embd[1] = {c.n_embd}, d_head[1] = {c.head_dim_k}, d_vocab[2] = {c.n_embd, c.vocab};
    rmi_hip_qwen3_weights w{};
    const TensorEntry *t;
    if (!(t = expect_tensor(g, "output_norm.weight", d_embd, 1, 0))) return nullptr;
    w.output_norm = reinterpret_cast<const float *>(g->bytes(*t));
    if (!(t = expect_tensor(g, "token_embd.weight", d_vocab, 2, 8))) return nullptr;
    w.token_embd = g->bytes(*t);
    if (g->tensor("output.weight")) {
        if (!(t = expect_tensor(g, "output.weight", d_vocab, 2, 8))) return nullptr;
        w.output = g->bytes(*t);
    }
    std::vector<const float *> norms[4];
    std::vector<const uint8_t *> mats[7];
    static const char *const norm_names[4] = {"attn_norm.weight", "ffn_norm.weight", "attn_q_norm.weight",
                                              "attn_k_norm.weight"};
    static const char *const mat_names[7] = {"attn_q.weight",   "attn_k.weight", "attn_v.weight",  "attn_output.weight",
                                             "ffn_gate.weight", "ffn_up.weight", "ffn_down.weight"};
    const uint64_t mat_dims[7][2] = {{c.n_embd, n_q},    {c.n_embd, n_k},    {c.n_embd, n_v},   {n_attn, c.n_embd},
                                     {c.n_embd, c.n_ff}, {c.n_embd, c.n_ff}, {c.n_ff, c.n_embd}};
    for (uint32_t l = 0; l < c.n_layer; l++) {
        const std::string p = "blk." + std::to_string(l) + ".";
        for (int i = 0; i < (c.has_qk_norm ? 4 : 2); i++) {
            if (!(t = expect_tensor(g, p + norm_names[i], i < 2 ? d_embd : d_head, 1, 0))) return nullptr;
            norms[i].push_back(reinterpret_cast<const float *>(g->bytes(*t)));
        }
        for (int i = 0; i < 7; i++) {
            if (!(t = expect_tensor(g, p + mat_names[i], mat_dims[i], 2, 8))) return nullptr;
            mats[i].push_back(g->bytes(*t));
        }
    }
    w.attn_norm = norms[0].data();
    w.ffn_norm = norms[1].data();
    w.q_norm = c.has_qk_norm ? norms[2].data() : nullptr;
    w.k_norm = c.has_qk_norm ? norms[3].data() : nullptr;
    w.wq = mats[0].data();
    w.wk = mats[1].data();
    w.wv = mats[2].data();
    w.wo = mats[3].data();
    w.w_gate = mats[4].data();
    w.w_up = mats[5].data();
    w.w_down = mats[6].data();
    return rmi_hip_qwen3_create(&c, &w);
}

}  // extern "C"
