// GGUF (v2 / v3) reader: header, metadata table, tensor table, and host
// dequantizers for the unquantized and 32-element block types.  The file is
// memory-mapped; tensor data is handed out as pointers into the mapping.
//
// Mirrors Gguf::open and its accessors (crates/ksearch_gguf/src/gguf_impl.rs:
// 217-420) and the F32 / F16 / BF16 / Q4_0 / Q4_1 / Q5_1 / Q8_0 arms of
// dequant_blocks (:577-689).  Where the reference panics on a malformed file,
// this returns an error; every read is bounds-checked against the mapping.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "ksh_internal.hpp"

namespace {

constexpr uint32_t kMagic = 0x46554747;   // "GGUF"

struct MetaValue {
    int type = -1;           // GGUF value type of the scalar, or of the elements of an array
    bool is_array = false;
    uint64_t u = 0;          // integers and bools
    double f = 0.0;          // floats
    std::string s;
    std::vector<uint64_t> au;
    std::vector<double> af;
    std::vector<std::string> as;
    size_t count = 0;
};

struct TensorInfo {
    std::string name;
    uint32_t type = 0;
    std::vector<uint64_t> dims;
    uint64_t offset = 0;
};

bool ggml_block(uint32_t t, size_t &elems, size_t &bytes)
{
    switch (t) {
    case KSH_GGML_F32: elems = 1; bytes = 4; return true;
    case KSH_GGML_F16: case KSH_GGML_BF16: elems = 1; bytes = 2; return true;
    case KSH_GGML_Q4_0: elems = 32; bytes = 18; return true;
    case KSH_GGML_Q4_1: elems = 32; bytes = 20; return true;
    case KSH_GGML_Q5_1: elems = 32; bytes = 24; return true;
    case KSH_GGML_Q8_0: elems = 32; bytes = 34; return true;
    case KSH_GGML_Q4_K: elems = 256; bytes = 144; return true;
    case KSH_GGML_Q5_K: elems = 256; bytes = 176; return true;
    case KSH_GGML_Q6_K: elems = 256; bytes = 210; return true;
    }
    return false;
}

struct Cursor {
    const uint8_t *buf;
    size_t size, pos = 0;
    bool ok = true;
    bool need(size_t n)
    {
        if (!ok || n > size - pos) { ok = false; return false; }
        return true;
    }
    template <class T>
    T get()
    {
        T v{};
        if (need(sizeof(T))) { memcpy(&v, buf + pos, sizeof(T)); pos += sizeof(T); }
        return v;
    }
    std::string str()
    {
        const uint64_t n = get<uint64_t>();
        if (!need(n)) return {};
        std::string s((const char *)buf + pos, (size_t)n);
        pos += n;
        return s;
    }
};

// one scalar of GGUF value type vt into `m` (as the element of an array when `arr`)
bool read_scalar(Cursor &c, uint32_t vt, MetaValue &m, bool arr)
{
    uint64_t u = 0;
    double f = 0;
    switch (vt) {
    case 0: u = c.get<uint8_t>(); break;
    case 1: u = (uint64_t)(int64_t)c.get<int8_t>(); break;
    case 2: u = c.get<uint16_t>(); break;
    case 3: u = (uint64_t)(int64_t)c.get<int16_t>(); break;
    case 4: u = c.get<uint32_t>(); break;
    case 5: u = (uint64_t)(int64_t)c.get<int32_t>(); break;
    case 6: f = c.get<float>(); break;
    case 7: u = c.get<uint8_t>() != 0; break;
    case 8: {
        std::string s = c.str();
        if (arr) m.as.push_back(std::move(s)); else m.s = std::move(s);
        return c.ok;
    }
    case 10: u = c.get<uint64_t>(); break;
    case 11: u = (uint64_t)c.get<int64_t>(); break;
    case 12: f = c.get<double>(); break;
    default: return false;
    }
    const bool is_f = vt == 6 || vt == 12;
    if (arr) { if (is_f) m.af.push_back(f); else m.au.push_back(u); }
    else { m.u = u; m.f = f; }
    return c.ok;
}

}  // namespace

struct ksh_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    std::map<std::string, MetaValue> meta;
    std::map<std::string, TensorInfo> tensors;
    std::vector<std::string> order;   // tensor names in file order
    size_t data_offset = 0;
    ~ksh_gguf()
    {
        if (map) munmap((void *)map, size);
        if (fd >= 0) close(fd);
    }
};

using namespace ksh;

extern "C" {

int ksh_gguf_open(const char *path, ksh_gguf **out)
{
    if (!path || !out) return set_error("ksh_gguf_open: bad arguments");
    *out = nullptr;
    auto g = std::make_unique<ksh_gguf>();
    g->fd = open(path, O_RDONLY);
    if (g->fd < 0) return set_error("failed to open gguf file %s", path);
    struct stat st;
    if (fstat(g->fd, &st) || st.st_size < 24) return set_error("%s: not a GGUF file (too short)", path);
    g->size = (size_t)st.st_size;
    void *p = mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (p == MAP_FAILED) return set_error("failed to mmap gguf file %s", path);
    g->map = (const uint8_t *)p;
    Cursor c{g->map, g->size};
    if (c.get<uint32_t>() != kMagic) return set_error("not a GGUF file (bad magic)");
    g->version = c.get<uint32_t>();
    if (g->version != 2 && g->version != 3) return set_error("unsupported GGUF version %u", g->version);
    const uint64_t n_tensors = c.get<uint64_t>(), n_kv = c.get<uint64_t>();
    if (n_tensors > (1u << 24) || n_kv > (1u << 24)) return set_error("GGUF header: implausible counts");
    for (uint64_t i = 0; i < n_kv && c.ok; i++) {
        std::string key = c.str();
        const uint32_t vt = c.get<uint32_t>();
        MetaValue m;
        if (vt == 9) {
            m.is_array = true;
            m.type = (int)c.get<uint32_t>();
            const uint64_t n = c.get<uint64_t>();
            if (n > g->size) return set_error("GGUF metadata %s: array longer than the file", key.c_str());
            m.count = (size_t)n;
            for (uint64_t k = 0; k < n; k++)
                if (!read_scalar(c, (uint32_t)m.type, m, true))
                    return c.ok ? set_error("GGUF metadata %s: bad array element type %d", key.c_str(), m.type)
                                : set_error("GGUF file is truncated inside its header");
        } else {
            m.type = (int)vt;
            if (!read_scalar(c, vt, m, false))
                return c.ok ? set_error("GGUF metadata %s: unexpected value type %u", key.c_str(), vt)
                            : set_error("GGUF file is truncated inside its header");
        }
        g->meta[key] = std::move(m);
    }
    for (uint64_t i = 0; i < n_tensors && c.ok; i++) {
        TensorInfo t;
        t.name = c.str();
        const uint32_t nd = c.get<uint32_t>();
        if (nd > 8) return set_error("GGUF tensor %s: %u dims", t.name.c_str(), nd);
        for (uint32_t d = 0; d < nd; d++) t.dims.push_back(c.get<uint64_t>());
        t.type = c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        g->order.push_back(t.name);
        g->tensors[t.name] = std::move(t);
    }
    if (!c.ok) return set_error("GGUF file is truncated inside its header");
    size_t align = 32;
    auto it = g->meta.find("general.alignment");
    if (it != g->meta.end() && !it->second.is_array && (it->second.type == 4 || it->second.type == 10) && it->second.u) align = (size_t)it->second.u;
    g->data_offset = (c.pos + align - 1) / align * align;
    // every tensor must lie inside the file
    for (const auto &kv : g->tensors) {
        const TensorInfo &t = kv.second;
        size_t e, b;
        if (!ggml_block(t.type, e, b)) continue;   // unknown types are refused when asked for
        uint64_t n = 1;
        for (uint64_t d : t.dims) {
            // (a product that does not fit 64 bits cannot be a tensor of this file)
            if (d && n > (uint64_t)g->size * 256 / d) return set_error("tensor %s lies outside the file", t.name.c_str());
            n *= d;
        }
        if (n % e) return set_error("tensor %s elems %llu not divisible by block %zu", t.name.c_str(), (unsigned long long)n, e);
        const uint64_t bytes = n / e * b;
        if (g->data_offset > g->size || t.offset > g->size - g->data_offset || bytes > g->size - g->data_offset - t.offset)
            return set_error("tensor %s lies outside the file", t.name.c_str());
    }
    *out = g.release();
    return 0;
}

void ksh_gguf_close(ksh_gguf *g) { delete g; }

int ksh_gguf_version(const ksh_gguf *g) { return g ? (int)g->version : -1; }
int64_t ksh_gguf_n_tensors(const ksh_gguf *g) { return g ? (int64_t)g->order.size() : -1; }

int ksh_gguf_tensor_name(const ksh_gguf *g, int64_t index, char *dst, size_t n)
{
    if (!g || !dst || !n || index < 0 || index >= (int64_t)g->order.size()) return set_error("ksh_gguf_tensor_name: bad arguments");
    snprintf(dst, n, "%s", g->order[(size_t)index].c_str());
    return 0;
}

int ksh_gguf_tensor(const ksh_gguf *g, const char *name, int32_t *ggml_type, int64_t *dims, int32_t *n_dims, const void **data,
                    size_t *bytes)
{
    if (!g || !name) return set_error("ksh_gguf_tensor: bad arguments");
    auto it = g->tensors.find(name);
    if (it == g->tensors.end()) return set_error("tensor not found: %s", name);
    const TensorInfo &t = it->second;
    size_t e, b;
    if (!ggml_block(t.type, e, b)) return set_error("tensor %s: unsupported ggml type id %u", name, t.type);
    uint64_t n = 1;
    for (uint64_t d : t.dims) n *= d;
    if (ggml_type) *ggml_type = (int32_t)t.type;
    if (n_dims) *n_dims = (int32_t)t.dims.size();
    if (dims)
        for (size_t i = 0; i < 4; i++) dims[i] = i < t.dims.size() ? (int64_t)t.dims[i] : 1;
    if (data) *data = g->map + g->data_offset + t.offset;
    if (bytes) *bytes = (size_t)(n / e * b);
    return 0;
}

int ksh_gguf_has_tensor(const ksh_gguf *g, const char *name) { return g && name && g->tensors.count(name) ? 1 : 0; }

// get_u32 / get_f32 / get_str / get_arr_* (gguf_impl.rs:330-420): return 1 (no error text) when the key is absent
// or of another type, like the reference's None
int ksh_gguf_get_u32(const ksh_gguf *g, const char *key, uint32_t *out)
{
    if (!g || !key || !out) return 1;
    auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.is_array) return 1;
    const int t = it->second.type;
    if (t != 4 && t != 5 && t != 10 && t != 2) return 1;
    *out = (uint32_t)it->second.u;
    return 0;
}

int ksh_gguf_get_f32(const ksh_gguf *g, const char *key, float *out)
{
    if (!g || !key || !out) return 1;
    auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.is_array || (it->second.type != 6 && it->second.type != 12)) return 1;
    *out = (float)it->second.f;
    return 0;
}

int ksh_gguf_get_str(const ksh_gguf *g, const char *key, char *dst, size_t n)
{
    if (!g || !key || !dst || !n) return 1;
    auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.is_array || it->second.type != 8) return 1;
    snprintf(dst, n, "%s", it->second.s.c_str());
    return 0;
}

// integer (u32 / i32) and bool arrays; a scalar integer reads as a list of one (get_usize_list, :396-405)
int ksh_gguf_get_arr_u32(const ksh_gguf *g, const char *key, uint32_t *dst, int cap, int *n)
{
    if (!g || !key || !n) return 1;
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return 1;
    const MetaValue &m = it->second;
    if (!m.is_array) {
        if (m.type != 4 && m.type != 5 && m.type != 10) return 1;
        *n = 1;
        if (dst && cap >= 1) dst[0] = (uint32_t)m.u;
        return 0;
    }
    if (m.type != 4 && m.type != 5 && m.type != 7) return 1;
    *n = (int)m.au.size();
    if (dst)
        for (int i = 0; i < *n && i < cap; i++) dst[i] = (uint32_t)m.au[(size_t)i];
    return 0;
}

int ksh_gguf_arr_is_bool(const ksh_gguf *g, const char *key)
{
    if (!g || !key) return 0;
    auto it = g->meta.find(key);
    return it != g->meta.end() && it->second.is_array && it->second.type == 7;
}

// dequant_blocks for the types a loader converts on the host (gguf_impl.rs:577-689).  The K-quants go through the
// device kernels (KSH_DEQUANT), which are bit-exact with the same loops.
int ksh_gguf_dequant_host(int32_t ggml_type, const void *src, size_t n_elems, float *out)
{
    if (!src || !out) return set_error("ksh_gguf_dequant_host: bad arguments");
    const uint8_t *d = (const uint8_t *)src;
    auto h16 = [](const uint8_t *p) {
        // f16_to_f32, crates/ksearch_gguf/src/lib.rs:20-35: exact, subnormals included
        const uint32_t h = (uint32_t)p[0] | ((uint32_t)p[1] << 8), sign = (h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3FFu;
        uint32_t bits;
        if (exp == 0) {
            if (man == 0) bits = sign;
            else {
                int e = -1;
                uint32_t m = man;
                do { e++; m <<= 1; } while (!(m & 0x400u));
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3FFu) << 13);
            }
        } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
        else bits = sign | ((exp + 112u) << 23) | (man << 13);
        float f;
        memcpy(&f, &bits, 4);
        return f;
    };
    switch (ggml_type) {
    case KSH_GGML_F32: memcpy(out, d, n_elems * 4); return 0;
    case KSH_GGML_F16:
        for (size_t i = 0; i < n_elems; i++) out[i] = h16(d + 2 * i);
        return 0;
    case KSH_GGML_BF16:
        for (size_t i = 0; i < n_elems; i++) {
            const uint32_t bits = ((uint32_t)d[2 * i] | ((uint32_t)d[2 * i + 1] << 8)) << 16;
            memcpy(&out[i], &bits, 4);
        }
        return 0;
    case KSH_GGML_Q4_0:
        for (size_t b = 0; b < n_elems / 32; b++) {
            const uint8_t *blk = d + b * 18;
            const float dd = h16(blk);
            for (int i = 0; i < 16; i++) {
                out[b * 32 + i] = (float)((int)(blk[2 + i] & 0x0F) - 8) * dd;
                out[b * 32 + i + 16] = (float)((int)(blk[2 + i] >> 4) - 8) * dd;
            }
        }
        return 0;
    case KSH_GGML_Q4_1:
        for (size_t b = 0; b < n_elems / 32; b++) {
            const uint8_t *blk = d + b * 20;
            const float dd = h16(blk), m = h16(blk + 2);
            for (int i = 0; i < 16; i++) {
                out[b * 32 + i] = (float)(blk[4 + i] & 0x0F) * dd + m;
                out[b * 32 + i + 16] = (float)(blk[4 + i] >> 4) * dd + m;
            }
        }
        return 0;
    case KSH_GGML_Q5_1:
        for (size_t b = 0; b < n_elems / 32; b++) {
            const uint8_t *blk = d + b * 24;
            const float dd = h16(blk), m = h16(blk + 2);
            uint32_t qh;
            memcpy(&qh, blk + 4, 4);
            for (int i = 0; i < 16; i++) {
                const float x0 = (float)(blk[8 + i] & 0x0F) + (float)(((qh >> i) << 4) & 0x10);
                const float x1 = (float)(blk[8 + i] >> 4) + (float)((qh >> (i + 12)) & 0x10);
                out[b * 32 + i] = x0 * dd + m;
                out[b * 32 + i + 16] = x1 * dd + m;
            }
        }
        return 0;
    case KSH_GGML_Q8_0:
        for (size_t b = 0; b < n_elems / 32; b++) {
            const uint8_t *blk = d + b * 34;
            const float dd = h16(blk);
            for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * dd;
        }
        return 0;
    }
    return set_error("ksh_gguf_dequant_host: ggml type %d is converted on the device (K-quants) or not built", ggml_type);
}

}  // extern "C"
