// GGUF file -> resident weights: the loader side of the path (host code only, no kernels).
//
// Stands in for crates/strix-models/src/gguf.rs (header, metadata and tensor index of a memory-mapped
// GGUF v2/v3 file, :113-238) and for the upload loops of the models' attach_accel (e.g.
// crates/strix-backend-cpu/src/mellum.rs:460-535, gemma.rs:415-470): every quantised matrix the
// decode path can serve goes to smx_upload_*, every layer's stacked expert tensors to
// smx_upload_moe_*.  Also the host quantisers the reference uses to bring a tensor into a served
// format (crates/strix-models/src/ggml_quant.rs:193-237: quantize_q8_0, quantize_q4_0) and the
// dequantisers they are fed from (:239-262, 401-430).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <thread>

#include "smx_internal.h"

struct smx_gguf {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t len = 0;
    size_t data_offset = 0;
    struct Meta {
        uint32_t type;      // GGUF value type
        uint64_t u = 0;     // integers and bool, widened
        bool neg = false;   // a negative signed integer
        double f = 0;       // f32 / f64
        std::string s;      // string
        uint64_t count = 0; // array length (elements are skipped)
    };
    struct Tensor {
        std::string name;
        uint32_t type;
        std::vector<uint64_t> dims;
        uint64_t offset;
        size_t nbytes;
    };
    std::map<std::string, Meta> meta;
    std::vector<Tensor> tensors;
    std::map<std::string, size_t> index;
};

namespace {

struct BlockFormat {
    uint32_t type;
    size_t elems, bytes;
};
// ggml tensor encodings and their block shapes (ggml_quant.rs:26-124)
const BlockFormat kFormats[] = {
    {0, 1, 4},     {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},    {7, 32, 24},   {8, 32, 34},
    {9, 32, 36},   {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292},
    {24, 1, 1},    {25, 1, 2},     {26, 1, 4},     {27, 1, 8},     {28, 1, 8},     {30, 1, 2},
};
const BlockFormat* format_of(uint32_t type) {
    for (const BlockFormat& f : kFormats)
        if (f.type == type) return &f;
    return nullptr;
}

int set_err(char* err, size_t cap, int code, const char* fmt, ...) {
    if (err && cap) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, cap, fmt, ap);
        va_end(ap);
    }
    return code;
}

// little-endian cursor with bounds checks (gguf.rs:283-340)
struct Cursor {
    const uint8_t* p;
    size_t len, pos = 0;
    bool ok = true;
    const uint8_t* take(size_t n) {
        if (!ok || n > len - pos) {
            ok = false;
            return nullptr;
        }
        const uint8_t* r = p + pos;
        pos += n;
        return r;
    }
    template <class T>
    T get() {
        T v{};
        const uint8_t* b = take(sizeof(T));
        if (b) memcpy(&v, b, sizeof(T));
        return v;
    }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (!ok || n > len - pos) {
            ok = false;
            return std::string();
        }
        const uint8_t* b = take((size_t)n);
        return b ? std::string((const char*)b, (size_t)n) : std::string();
    }
};

size_t scalar_size(uint32_t t) {
    switch (t) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
        default: return 0;
    }
}

bool read_value(Cursor& c, uint32_t type, smx_gguf::Meta* m, int depth) {
    m->type = type;
    switch (type) {
        case 0: m->u = c.get<uint8_t>(); break;
        case 1: { int8_t v = c.get<int8_t>(); m->neg = v < 0; m->u = (uint64_t)(int64_t)v; break; }
        case 2: m->u = c.get<uint16_t>(); break;
        case 3: { int16_t v = c.get<int16_t>(); m->neg = v < 0; m->u = (uint64_t)(int64_t)v; break; }
        case 4: m->u = c.get<uint32_t>(); break;
        case 5: { int32_t v = c.get<int32_t>(); m->neg = v < 0; m->u = (uint64_t)(int64_t)v; break; }
        case 6: m->f = c.get<float>(); break;
        case 7: m->u = c.get<uint8_t>() != 0; break;
        case 8: m->s = c.str(); break;
        case 9: {
            if (depth > 0) return false;  // nested arrays do not occur in model files
            const uint32_t et = c.get<uint32_t>();
            m->count = c.get<uint64_t>();
            if (!c.ok) return false;
            if (et == 8) {
                for (uint64_t i = 0; i < m->count && c.ok; i++) (void)c.str();
            } else {
                const size_t sz = scalar_size(et);
                if (sz == 0 || m->count > (c.len - c.pos) / sz) return false;
                c.take((size_t)m->count * sz);
            }
            break;
        }
        case 10: m->u = c.get<uint64_t>(); break;
        case 11: { int64_t v = c.get<int64_t>(); m->neg = v < 0; m->u = (uint64_t)v; break; }
        case 12: m->f = c.get<double>(); break;
        default: return false;
    }
    return c.ok;
}

// ---- f16 <-> f32 (IEEE, round to nearest even), host side ----
float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff, bits;
    if (e == 0) {
        if (m == 0) {
            bits = sign;
        } else {
            e = 127 - 15 + 1;
            while (!(m & 0x400)) { m <<= 1; e--; }
            bits = sign | (e << 23) | ((m & 0x3ff) << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 127 - 15) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000);
    const uint32_t a = x & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00);  // NaN
    if (a == 0x7f800000u) return (uint16_t)(sign | 0x7c00);
    if (a <= 0x33000000u) return sign;  // at most half the smallest subnormal: rounds (ties to even) to zero
    int e = (int)(a >> 23) - 127;
    const uint32_t m = (a & 0x7fffffu) | 0x800000u;  // 24-bit significand
    const int shift = e < -14 ? 13 + (-14 - e) : 13;
    uint32_t r = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (r & 1))) r++;
    if (e < -14) return (uint16_t)(sign | r);  // subnormal; a carry to 0x400 is the smallest normal
    if (r == 0x800) {                          // significand carried: 2.0 -> 1.0 of the next binade
        r = 0x400;
        e++;
    }
    if (e > 15) return (uint16_t)(sign | 0x7c00);
    return (uint16_t)(sign | ((uint32_t)(e + 15) << 10) | (r & 0x3ff));
}

bool ends_with(const std::string& s, const char* suffix) {
    const size_t n = strlen(suffix);
    return s.size() >= n && s.compare(s.size() - n, n, suffix) == 0;
}

}  // namespace

extern "C" {

int smx_gguf_open(const char* path, smx_gguf** out, char* err, size_t err_cap) {
    if (!path || !out) return set_err(err, err_cap, SMX_ERR_ARG, "gguf_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return set_err(err, err_cap, SMX_ERR_ARG, "gguf_open: cannot open %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 24) {
        close(fd);
        return set_err(err, err_cap, SMX_ERR_ARG, "gguf_open: %s is not a GGUF file (too short)", path);
    }
    void* map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_SHARED, fd, 0);
    if (map == MAP_FAILED) {
        close(fd);
        return set_err(err, err_cap, SMX_ERR_NOMEM, "gguf_open: mmap of %s failed: %s", path, strerror(errno));
    }
    smx_gguf* g = new (std::nothrow) smx_gguf();
    if (!g) {
        munmap(map, (size_t)st.st_size);
        close(fd);
        return set_err(err, err_cap, SMX_ERR_NOMEM, "gguf_open: out of host memory");
    }
    g->fd = fd;
    g->map = (const uint8_t*)map;
    g->len = (size_t)st.st_size;
    try {
    auto bail = [&](int code, const char* what) {
        const int rc = set_err(err, err_cap, code, "gguf_open: %s: %s", path, what);
        smx_gguf_close(g);
        return rc;
    };
    Cursor c{g->map, g->len};
    if (c.get<uint32_t>() != 0x46554747u) return bail(SMX_ERR_ARG, "not a GGUF file (bad magic)");  // gguf.rs:20
    const uint32_t version = c.get<uint32_t>();
    if (version != 2 && version != 3) return bail(SMX_ERR_LIMIT, "unsupported GGUF version");      // gguf.rs:128-131
    const uint64_t tensor_count = c.get<uint64_t>(), kv_count = c.get<uint64_t>();
    if (tensor_count > g->len / 16 || kv_count > g->len / 12) return bail(SMX_ERR_ARG, "counts exceed the file size");
    for (uint64_t i = 0; i < kv_count; i++) {
        std::string key = c.str();
        const uint32_t type = c.get<uint32_t>();
        smx_gguf::Meta m;
        if (!c.ok || !read_value(c, type, &m, 0)) return bail(SMX_ERR_ARG, "truncated or unknown metadata value");
        g->meta.emplace(std::move(key), std::move(m));
    }
    g->tensors.reserve((size_t)tensor_count);
    for (uint64_t i = 0; i < tensor_count; i++) {
        smx_gguf::Tensor t;
        t.name = c.str();
        const uint32_t nd = c.get<uint32_t>();
        if (!c.ok || nd > 8) return bail(SMX_ERR_ARG, "truncated tensor index");
        uint64_t numel = 1;
        for (uint32_t d = 0; d < nd; d++) {
            t.dims.push_back(c.get<uint64_t>());
            if (t.dims.back() != 0 && numel > UINT64_MAX / t.dims.back()) return bail(SMX_ERR_ARG, "tensor size overflows");
            numel *= t.dims.back();
        }
        t.type = c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (!c.ok) return bail(SMX_ERR_ARG, "truncated tensor index");
        const BlockFormat* f = format_of(t.type);
        if (!f) return bail(SMX_ERR_LIMIT, "unknown tensor encoding");
        if (numel / f->elems > SIZE_MAX / f->bytes) return bail(SMX_ERR_ARG, "tensor size overflows");
        t.nbytes = (size_t)(numel / f->elems) * f->bytes;  // gguf.rs:223
        g->index[t.name] = g->tensors.size();
        g->tensors.push_back(std::move(t));
    }
    size_t alignment = 32;  // gguf.rs:21, 165-169
    auto it = g->meta.find("general.alignment");
    if (it != g->meta.end() && it->second.type != 6 && it->second.type != 12 && it->second.type != 8 && !it->second.neg &&
        it->second.u > 0)
        alignment = (size_t)it->second.u;
    g->data_offset = (c.pos + alignment - 1) / alignment * alignment;
    if (g->data_offset > g->len) return bail(SMX_ERR_ARG, "tensor data offset past the end of the file");
    for (const smx_gguf::Tensor& t : g->tensors)
        if (t.offset > g->len - g->data_offset || t.nbytes > g->len - g->data_offset - t.offset)
            return bail(SMX_ERR_ARG, "a tensor's data lies past the end of the file");  // gguf.rs:225-231
    } catch (const std::bad_alloc&) {   // a crafted count or string length: no exception crosses the C ABI
        smx_gguf_close(g);
        return set_err(err, err_cap, SMX_ERR_NOMEM, "gguf_open: %s: out of host memory while reading the index", path);
    } catch (const std::exception& e) {
        smx_gguf_close(g);
        return set_err(err, err_cap, SMX_ERR_ARG, "gguf_open: %s: %s", path, e.what());
    }
    *out = g;
    return SMX_OK;
}

void smx_gguf_close(smx_gguf* g) {
    if (!g) return;
    if (g->map) munmap((void*)g->map, g->len);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

size_t smx_gguf_tensor_count(const smx_gguf* g) { return g ? g->tensors.size() : 0; }

int smx_gguf_tensor(const smx_gguf* g, size_t index, const char** name, int* ggml_type, size_t* n_dims, size_t* dims,
                    size_t dims_cap, const void** data, size_t* nbytes) {
    if (!g || index >= g->tensors.size()) return SMX_ERR_ARG;
    const smx_gguf::Tensor& t = g->tensors[index];
    if (name) *name = t.name.c_str();
    if (ggml_type) *ggml_type = (int)t.type;
    if (n_dims) *n_dims = t.dims.size();
    if (dims)
        for (size_t d = 0; d < t.dims.size() && d < dims_cap; d++) dims[d] = (size_t)t.dims[d];
    if (data) *data = g->map + g->data_offset + t.offset;
    if (nbytes) *nbytes = t.nbytes;
    return SMX_OK;
}

int smx_gguf_find(const smx_gguf* g, const char* name, size_t* index) {
    if (!g || !name || !index) return SMX_ERR_ARG;
    auto it = g->index.find(name);
    if (it == g->index.end()) return SMX_NOT_RESIDENT;
    *index = it->second;
    return SMX_OK;
}

// MetaValue::as_u64 / as_f32 / as_str, gguf.rs:43-72
int smx_gguf_meta_u64(const smx_gguf* g, const char* key, uint64_t* value) {
    if (!g || !key || !value) return SMX_ERR_ARG;
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return SMX_NOT_RESIDENT;
    const smx_gguf::Meta& m = it->second;
    if (m.type == 6 || m.type == 12 || m.type == 8 || m.type == 9 || m.type == 7 || m.neg) return SMX_ERR_ARG;
    *value = m.u;
    return SMX_OK;
}

int smx_gguf_meta_f32(const smx_gguf* g, const char* key, float* value) {
    if (!g || !key || !value) return SMX_ERR_ARG;
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return SMX_NOT_RESIDENT;
    const smx_gguf::Meta& m = it->second;
    if (m.type == 6 || m.type == 12) *value = (float)m.f;
    else if (m.type == 8 || m.type == 9 || m.type == 7 || m.neg) return SMX_ERR_ARG;
    else *value = (float)m.u;
    return SMX_OK;
}

int smx_gguf_meta_str(const smx_gguf* g, const char* key, const char** value) {
    if (!g || !key || !value) return SMX_ERR_ARG;
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return SMX_NOT_RESIDENT;
    if (it->second.type != 8) return SMX_ERR_ARG;
    *value = it->second.s.c_str();
    return SMX_OK;
}

// The upload loop of attach_accel: matrices under their GGUF names, expert triples by layer number.
int smx_gguf_attach(smx_ctx* c, const smx_gguf* g, size_t* n_weights, size_t* n_expert_layers) {
    if (!c) return SMX_ERR_ARG;
    if (!g) return smx::fail(c, SMX_ERR_ARG, "gguf_attach: null file");
    return smx::guarded(c, "gguf_attach", [&]() -> int {
    size_t nw = 0, nl = 0;
    for (const smx_gguf::Tensor& t : g->tensors) {
        if (t.dims.size() < 2 || !ends_with(t.name, ".weight") || ends_with(t.name, "_exps.weight")) continue;
        if (t.type != 2 && t.type != 8 && t.type != 14) continue;  // not a served encoding: the caller's CPU path keeps it
        const size_t in_dim = (size_t)t.dims[0];
        size_t out_dim = 1;
        for (size_t d = 1; d < t.dims.size(); d++) out_dim *= (size_t)t.dims[d];  // mellum.rs:493-494
        const void* bytes = g->map + g->data_offset + t.offset;
        int rc = t.type == 2   ? smx_upload_q4_0(c, t.name.c_str(), bytes, t.nbytes, in_dim, out_dim)
                 : t.type == 8 ? smx_upload_q8_0(c, t.name.c_str(), bytes, t.nbytes, in_dim, out_dim)
                               : smx_upload_q6_k(c, t.name.c_str(), bytes, t.nbytes, in_dim, out_dim);
        if (rc != SMX_OK) return rc;
        nw++;
    }
    for (const smx_gguf::Tensor& t : g->tensors) {
        // blk.<il>.ffn_gate_exps.weight [hidden, eff, ne] with its up and down siblings (mellum.rs:512-535)
        unsigned il = 0;
        int consumed = 0;
        if (sscanf(t.name.c_str(), "blk.%u.ffn_gate_exps.weight%n", &il, &consumed) != 1 || (size_t)consumed != t.name.size())
            continue;
        if (t.dims.size() != 3 || (t.type != 8 && t.type != 14)) continue;
        const std::string base = "blk." + std::to_string(il) + ".";
        auto iu = g->index.find(base + "ffn_up_exps.weight"), id = g->index.find(base + "ffn_down_exps.weight");
        if (iu == g->index.end() || id == g->index.end()) continue;
        const smx_gguf::Tensor &u = g->tensors[iu->second], &d = g->tensors[id->second];
        const size_t hidden = (size_t)t.dims[0], eff = (size_t)t.dims[1], ne = (size_t)t.dims[2];
        if (u.type != t.type || d.type != t.type || u.dims != t.dims || d.dims.size() != 3 || d.dims[0] != eff ||
            d.dims[1] != hidden || d.dims[2] != ne)
            continue;
        const uint8_t* base_p = g->map + g->data_offset;
        int rc = t.type == 8 ? smx_upload_moe_q8(c, il, base_p + t.offset, t.nbytes, base_p + u.offset, u.nbytes,
                                                 base_p + d.offset, d.nbytes, hidden, eff, ne)
                             : smx_upload_moe_q6(c, il, base_p + t.offset, t.nbytes, base_p + u.offset, u.nbytes,
                                                 base_p + d.offset, d.nbytes, hidden, eff, ne);
        if (rc != SMX_OK) return rc;
        nl++;
    }
    if (n_weights) *n_weights = nw;
    if (n_expert_layers) *n_expert_layers = nl;
    return SMX_OK;
    });
}

// One tensor re-encoded on the host and uploaded: the reference's repacks of a tensor whose encoding
// the device path does not serve (gemma3n.rs:455-470: a Q4_K token_embd becomes a Q8_0 lm_head) or
// that the caller wants lighter (qwen35.rs:741-760: Q8_0 -> Q4_0).  Rows are converted in slabs so
// that the fp32 form of a large tensor never exists as a whole.
int smx_gguf_upload_as(smx_ctx* c, const smx_gguf* g, const char* tensor, const char* key, int target_type) {
    if (!c) return SMX_ERR_ARG;
    if (!g || !tensor) return smx::fail(c, SMX_ERR_ARG, "gguf_upload_as: null argument");
    if (target_type != 2 && target_type != 8)
        return smx::fail(c, SMX_ERR_ARG, "gguf_upload_as: target type %d (2 = Q4_0 or 8 = Q8_0)", target_type);
    return smx::guarded(c, "gguf_upload_as", [&]() -> int {
    auto it = g->index.find(tensor);
    if (it == g->index.end()) return SMX_NOT_RESIDENT;
    const smx_gguf::Tensor& t = g->tensors[it->second];
    if (t.dims.size() < 2) return smx::fail(c, SMX_ERR_ARG, "gguf_upload_as: %s is not a matrix", tensor);
    const BlockFormat* f = format_of(t.type);
    const size_t in_dim = (size_t)t.dims[0];
    size_t out_dim = 1;
    for (size_t d = 1; d < t.dims.size(); d++) out_dim *= (size_t)t.dims[d];
    if (!f || in_dim % f->elems != 0 || in_dim % 32 != 0)
        return smx::fail(c, SMX_ERR_ARG, "gguf_upload_as: %s has row length %zu in encoding %u", tensor, in_dim, t.type);
    const uint8_t* src = g->map + g->data_offset + t.offset;
    const char* name = key ? key : tensor;
    if ((int)t.type == target_type)
        return target_type == 2 ? smx_upload_q4_0(c, name, src, t.nbytes, in_dim, out_dim)
                                : smx_upload_q8_0(c, name, src, t.nbytes, in_dim, out_dim);
    const size_t row_src = in_dim / f->elems * f->bytes, row_dst = in_dim / 32 * (target_type == 2 ? 18 : 34);
    // slabs of rows (1 MB of floats each) shared out over the host's cores; every worker has its own fp32 slab
    const size_t slab = std::max<size_t>(1, (size_t(1) << 18) / in_dim);
    const size_t nslabs = (out_dim + slab - 1) / slab;
    std::vector<uint8_t> enc(out_dim * row_dst);
    std::atomic<size_t> next{0};
    std::atomic<int> err_deq{SMX_OK}, err_q{SMX_OK};
    auto work = [&]() {
        std::vector<float> tmp(std::min(slab, out_dim) * in_dim);
        for (size_t i; (i = next.fetch_add(1)) < nslabs;) {
            const size_t r0 = i * slab, rows = std::min(slab, out_dim - r0);
            int rc = smx_host_dequantize((int)t.type, src + r0 * row_src, rows * in_dim, tmp.data());
            if (rc != SMX_OK) { err_deq = rc; return; }
            rc = target_type == 2 ? smx_host_quantize_q4_0(tmp.data(), rows * in_dim, enc.data() + r0 * row_dst)
                                  : smx_host_quantize_q8_0(tmp.data(), rows * in_dim, enc.data() + r0 * row_dst);
            if (rc != SMX_OK) { err_q = rc; return; }
        }
    };
    {
        const size_t hw = std::max(1u, std::thread::hardware_concurrency());
        const size_t nthreads = std::min<size_t>({hw, 16, nslabs});
        auto safe_work = [&]() {   // nothing may leave a worker thread
            try { work(); } catch (...) { err_q = SMX_ERR_NOMEM; }
        };
        std::vector<std::thread> pool;
        try {
            pool.reserve(nthreads);
            for (size_t i = 1; i < nthreads; i++) pool.emplace_back(safe_work);
        } catch (...) {
            // fewer workers than asked for: the ones that started and this thread finish the slabs
        }
        safe_work();
        for (auto& th : pool) th.join();
    }
    if (err_deq != SMX_OK) return smx::fail(c, err_deq, "gguf_upload_as: encoding %u of %s has no dequantiser", t.type, tensor);
    if (err_q != SMX_OK) return smx::fail(c, err_q, "gguf_upload_as: quantiser failed on %s", tensor);
    return target_type == 2 ? smx_upload_q4_0(c, name, enc.data(), enc.size(), in_dim, out_dim)
                            : smx_upload_q8_0(c, name, enc.data(), enc.size(), in_dim, out_dim);
    });
}

// ---- host quantisers / dequantisers (n a multiple of the block size) ----

// ggml_quant.rs:193-207
int smx_host_quantize_q8_0(const float* x, size_t n, void* out) {
    if (!x || !out || n % 32 != 0) return SMX_ERR_ARG;
    uint8_t* o = (uint8_t*)out;
    for (size_t b = 0; b < n / 32; b++, o += 34) {
        const float* v = x + b * 32;
        float amax = 0.f;
        for (int i = 0; i < 32; i++) amax = std::fmax(amax, std::fabs(v[i]));
        const float d = amax / 127.0f, id = d > 0.f ? 1.0f / d : 0.f;
        const uint16_t h = f32_to_f16(d);
        o[0] = (uint8_t)(h & 0xff);
        o[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; i++) {
            float r = std::round(v[i] * id);  // half away from zero, as f32::round
            r = r < -127.f ? -127.f : (r > 127.f ? 127.f : r);
            o[2 + i] = (uint8_t)(int8_t)r;
        }
    }
    return SMX_OK;
}

// ggml_quant.rs:212-237 (ggml_quantize_row_q4_0: the signed value of largest magnitude maps to -8)
int smx_host_quantize_q4_0(const float* x, size_t n, void* out) {
    if (!x || !out || n % 32 != 0) return SMX_ERR_ARG;
    uint8_t* o = (uint8_t*)out;
    for (size_t b = 0; b < n / 32; b++, o += 18) {
        const float* v = x + b * 32;
        float amax = 0.f, vmax = 0.f;
        for (int i = 0; i < 32; i++)
            if (std::fabs(v[i]) > amax) {
                amax = std::fabs(v[i]);
                vmax = v[i];
            }
        const float d = vmax / -8.0f, id = d != 0.f ? 1.0f / d : 0.f;
        const uint16_t h = f32_to_f16(d);
        o[0] = (uint8_t)(h & 0xff);
        o[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 16; j++) {
            int q0 = (int)(v[j] * id + 8.5f), q1 = (int)(v[j + 16] * id + 8.5f);
            q0 = q0 < 0 ? 0 : (q0 > 15 ? 15 : q0);
            q1 = q1 < 0 ? 0 : (q1 > 15 ? 15 : q1);
            o[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
    return SMX_OK;
}

// ggml_quant.rs:239-262 (Q8_0, Q4_0), 401-430 (Q6_K), F32 / F16 pass-through
int smx_host_dequantize(int ggml_type, const void* bytes, size_t n, float* out) {
    if (!bytes || !out) return SMX_ERR_ARG;
    const uint8_t* p = (const uint8_t*)bytes;
    if (ggml_type == 0) {
        memcpy(out, p, n * 4);
    } else if (ggml_type == 1) {
        for (size_t i = 0; i < n; i++) out[i] = f16_to_f32((uint16_t)(p[2 * i] | (p[2 * i + 1] << 8)));
    } else if (ggml_type == 8) {
        if (n % 32) return SMX_ERR_ARG;
        for (size_t b = 0; b < n / 32; b++, p += 34) {
            const float d = f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
            for (int i = 0; i < 32; i++) out[b * 32 + i] = d * (float)(int8_t)p[2 + i];
        }
    } else if (ggml_type == 2) {
        if (n % 32) return SMX_ERR_ARG;
        for (size_t b = 0; b < n / 32; b++, p += 18) {
            const float d = f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
            for (int j = 0; j < 16; j++) {
                out[b * 32 + j] = (float)((int)(p[2 + j] & 0x0f) - 8) * d;
                out[b * 32 + j + 16] = (float)((int)(p[2 + j] >> 4) - 8) * d;
            }
        }
    } else if (ggml_type == 14) {
        if (n % 256) return SMX_ERR_ARG;
        for (size_t b = 0; b < n / 256; b++, p += 210) {
            const uint8_t *ql = p, *qh = p + 128;
            const int8_t* sc = (const int8_t*)(p + 192);
            const float d = f16_to_f32((uint16_t)(p[208] | (p[209] << 8)));
            float* y = out + b * 256;
            for (int half = 0; half < 2; half++) {  // 128 values per half: ql 64 B, qh 32 B, sc 8
                for (int l = 0; l < 32; l++) {
                    const int is = l / 16;
                    const int q1 = (int)((ql[l] & 0xf) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    const int q2 = (int)((ql[l + 32] & 0xf) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    const int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    y[l] = d * (float)sc[is] * (float)q1;
                    y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                    y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                    y[l + 96] = d * (float)sc[is + 6] * (float)q4;
                }
                y += 128;
                ql += 64;
                qh += 32;
                sc += 8;
            }
        }
    } else if (ggml_type == 3 || ggml_type == 6 || ggml_type == 7) {
        // Q4_1 (d, m, nibbles), Q5_0 (d, 32 fifth bits, nibbles), Q5_1 (d, m, fifth bits, nibbles):
        // ggml_quant.rs:265-311.  Value i of the block: nibble i % 16 of byte i % 16's low (i < 16) or high half.
        if (n % 32) return SMX_ERR_ARG;
        const bool has_m = ggml_type != 6, has_h = ggml_type != 3;
        const size_t bb = 2 + (has_m ? 2 : 0) + (has_h ? 4 : 0) + 16;
        for (size_t b = 0; b < n / 32; b++, p += bb) {
            const uint8_t* q = p + 2;
            const float d = f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
            float m = 0.f;
            uint32_t hbits = 0;
            if (has_m) { m = f16_to_f32((uint16_t)(q[0] | (q[1] << 8))); q += 2; }
            if (has_h) { hbits = (uint32_t)q[0] | ((uint32_t)q[1] << 8) | ((uint32_t)q[2] << 16) | ((uint32_t)q[3] << 24); q += 4; }
            for (int i = 0; i < 32; i++) {
                const int nib = i < 16 ? (q[i] & 0x0f) : (q[i - 16] >> 4);
                const int v = nib | (int)(((hbits >> i) & 1u) << 4);
                if (ggml_type == 6) out[b * 32 + i] = (float)(v - 16) * d;   // symmetric: no min
                else out[b * 32 + i] = (ggml_type == 3 ? d * (float)v : (float)v * d) + m;
            }
        }
    } else if (ggml_type == 12 || ggml_type == 13) {
        // Q4_K / Q5_K superblocks (ggml_quant.rs:328-400): d, dmin, 12 bytes holding eight 6-bit
        // (scale, min) pairs, [Q5_K: 32 bytes of fifth bits,] 128 nibble bytes.  Sub-block s (32 values)
        // takes the low (s even) or high (s odd) nibbles of bytes 32 * (s / 2) .. + 31, bit s of the
        // fifth-bit byte l, and y = (d * sc_s) * q - dmin * m_s.
        if (n % 256) return SMX_ERR_ARG;
        const bool k5 = ggml_type == 13;
        for (size_t b = 0; b < n / 256; b++, p += k5 ? 176 : 144) {
            const float d = f16_to_f32((uint16_t)(p[0] | (p[1] << 8))), dmin = f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
            const uint8_t *pk = p + 4, *hb = p + 16, *qs = p + (k5 ? 48 : 16);
            for (int s = 0; s < 8; s++) {
                int sc, mn;
                if (s < 4) {
                    sc = pk[s] & 63;
                    mn = pk[s + 4] & 63;
                } else {  // low four bits in bytes 8..11, the upper two in the top bits of bytes 0..7
                    sc = (pk[s + 4] & 0x0f) | ((pk[s - 4] >> 6) << 4);
                    mn = (pk[s + 4] >> 4) | ((pk[s] >> 6) << 4);
                }
                const float ds = d * (float)sc, ms = dmin * (float)mn;
                const uint8_t* q = qs + 32 * (s >> 1);
                float* y = out + b * 256 + s * 32;
                for (int l = 0; l < 32; l++) {
                    float v = (float)((s & 1) ? (q[l] >> 4) : (q[l] & 0x0f));
                    if (k5 && ((hb[l] >> s) & 1)) v += 16.0f;
                    y[l] = ds * v - ms;
                }
            }
        }
    } else {
        return SMX_ERR_LIMIT;
    }
    return SMX_OK;
}

}  // extern "C"
