// Context, weight residency (upload + repack to planar HBM layout), scratch and profiling.
#include <cstring>

#include "smx_internal.h"

namespace smx {

static thread_local std::string g_create_err;

int fail(smx_ctx* c, int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (c) c->err = buf; else g_create_err = buf;
    return code;
}

int hip_fail(smx_ctx* c, hipError_t e, const char* what) {
    (void)hipGetLastError();  // clear the sticky error so the next call reports its own
    return fail(c, SMX_ERR_HIP, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

int ensure(smx_ctx* c, DevBuf& b, size_t bytes) {
    if (bytes <= b.cap) return SMX_OK;
    if (c->capturing)
        return fail(c, SMX_ERR_ARG, "scratch would grow to %zu bytes during graph capture: run the call once outside capture first", bytes);
    if (b.p) {
        SMX_HIP(c, hipStreamSynchronize(c->stream));
        release_device(c, b.p);
        b.p = nullptr;
        b.cap = 0;
    }
    size_t cap = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    hipError_t e = hipMalloc((void**)&b.p, cap);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        b.p = nullptr;
        return fail(c, SMX_ERR_NOMEM, "device allocation of %zu bytes failed: %s", cap, hipGetErrorString(e));
    }
    b.cap = cap;
    return SMX_OK;
}

void release_device(smx_ctx* c, char* p) {
    if (!p) return;
    if (c->live_graphs > 0) {
        try {
            c->retired.push_back(p);  // a graph may still name this allocation
            return;
        } catch (const std::bad_alloc&) {
            // cannot record it: leak rather than free memory a replay may read
            return;
        }
    }
    (void)hipFree(p);
}

int ensure_host(smx_ctx* c, DevBuf& b, size_t bytes) {
    if (bytes <= b.cap) return SMX_OK;
    if (b.p) {
        SMX_HIP(c, hipStreamSynchronize(c->stream));
        SMX_HIP(c, hipHostFree(b.p));
        b.p = nullptr;
        b.cap = 0;
    }
    const size_t cap = (bytes + (size_t(1) << 16) - 1) & ~((size_t(1) << 16) - 1);
    hipError_t e = hipHostMalloc((void**)&b.p, cap, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        b.p = nullptr;
        return fail(c, SMX_ERR_NOMEM, "pinned host allocation of %zu bytes failed: %s", cap, hipGetErrorString(e));
    }
    b.cap = cap;
    return SMX_OK;
}

ProfScope::ProfScope(smx_ctx* c_, const char* name) : c(c_) {
    if (!c->prof_on || c->capturing) return;
    hipEvent_t e0, e1;
    if (!c->ev_pool.empty()) {
        e0 = c->ev_pool.back().first;
        e1 = c->ev_pool.back().second;
        c->ev_pool.pop_back();
    } else {
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return;
    }
    c->prof.push_back(ProfRec{name, e0, e1});
    idx = (int)c->prof.size() - 1;
    (void)hipEventRecord(e0, c->stream);
}

ProfScope::~ProfScope() {
    if (idx >= 0) (void)hipEventRecord(c->prof[idx].e1, c->stream);
}

static size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

// at context teardown (no graph can run any more)
static void free_weight(Weight& w) {
    if (w.base) (void)hipFree(w.base);
    w.base = nullptr;
}
// while the context lives: a captured graph may hold the weight's plane pointers
static void drop_weight(smx_ctx* c, Weight& w) {
    release_device(c, w.base);
    w.base = nullptr;
}

// ---- repack of raw GGUF blocks into the planar layout, on the device.  (The reference repacks on the host,
//      decode.rs:2500-2509, 2639-2664, 2693-2700; so did this library at first, at 4 GB/s of one host core: the raw
//      bytes now cross PCIe as they are, 30 GB/s from pageable memory, and a kernel of a few microseconds per 100 MB splits them
//      into planes.)  A workgroup copies a run of whole blocks into LDS with 16-byte loads -- 8 blocks of every format are a
//      multiple of 16 bytes -- and writes every plane with 16-byte stores; block fields are only 2-byte aligned, so LDS
//      is read in 16-bit pieces. ----
constexpr int kRepackBlocks = 256;   // blocks per workgroup (Q6_K: 128)
__device__ __forceinline__ uint4 lds_bytes16(const uint16_t* l16, int byte_off) {   // 16 bytes at an even offset
    const uint16_t* p = l16 + (byte_off >> 1);
    return make_uint4(p[0] | ((unsigned)p[1] << 16), p[2] | ((unsigned)p[3] << 16), p[4] | ((unsigned)p[5] << 16),
                      p[6] | ((unsigned)p[7] << 16));
}
// BB = 18 (Q4_0) or 34 (Q8_0): f16 scale, then 16 or 32 bytes of quants
template <int BB>
__global__ __launch_bounds__(256) void repack_q4q8_kernel(const uint4* __restrict__ raw, size_t total, uint16_t* __restrict__ scales,
                                                          uint4* __restrict__ quants) {
    __shared__ __align__(16) uint16_t lds[kRepackBlocks * BB / 2];
    const size_t b0 = (size_t)blockIdx.x * kRepackBlocks;
    const int nblk = (int)min((size_t)kRepackBlocks, total - b0);
    const int n16 = (nblk * BB + 15) / 16;   // the raw buffer is padded to a multiple of 16 bytes
    for (int i = threadIdx.x; i < n16; i += 256) ((uint4*)lds)[i] = raw[b0 * BB / 16 + i];
    __syncthreads();
    constexpr int QV = (BB - 2) / 16;   // 16-byte pieces of quants per block
    if ((int)threadIdx.x < nblk) scales[b0 + threadIdx.x] = lds[threadIdx.x * (BB / 2)];
    for (int i = threadIdx.x; i < nblk * QV; i += 256)
        quants[b0 * QV + i] = lds_bytes16(lds, (i / QV) * BB + 2 + (i % QV) * 16);
}
// Q6_K block: ql 128 | qh 64 | 16 sub-block scales | f16 d (210 bytes)
__global__ __launch_bounds__(256) void repack_q6k_kernel(const uint4* __restrict__ raw, size_t total, uint4* __restrict__ ql,
                                                         uint4* __restrict__ qh, uint4* __restrict__ sc, uint16_t* __restrict__ d) {
    constexpr int NB = kRepackBlocks / 2;
    __shared__ __align__(16) uint16_t lds[NB * 105];
    const size_t b0 = (size_t)blockIdx.x * NB;
    const int nblk = (int)min((size_t)NB, total - b0);
    const int n16 = (nblk * 210 + 15) / 16;
    for (int i = threadIdx.x; i < n16; i += 256) ((uint4*)lds)[i] = raw[b0 * 210 / 16 + i];
    __syncthreads();
    for (int i = threadIdx.x; i < nblk * 8; i += 256) ql[b0 * 8 + i] = lds_bytes16(lds, (i >> 3) * 210 + (i & 7) * 16);
    for (int i = threadIdx.x; i < nblk * 4; i += 256) qh[b0 * 4 + i] = lds_bytes16(lds, (i >> 2) * 210 + 128 + (i & 3) * 16);
    for (int i = threadIdx.x; i < nblk; i += 256) {
        sc[b0 + i] = lds_bytes16(lds, i * 210 + 192);
        d[b0 + i] = lds[i * 105 + 104];
    }
}

static int build_weight(smx_ctx* c, QType type, const uint8_t* bytes, size_t nbytes, size_t K, size_t N,
                        Weight* out) {
    const size_t be = type == kQ6_K ? 256 : 32;
    const size_t bb = type == kQ4_0 ? 18 : (type == kQ8_0 ? 34 : 210);
    if (!bytes) return fail(c, SMX_ERR_ARG, "upload: null bytes");
    if (K == 0 || N == 0 || K % be != 0)
        return fail(c, SMX_ERR_ARG, "upload: in_dim %zu is not a positive multiple of %zu", K, be);
    const size_t nblk = K / be, total = nblk * N;
    if (nbytes != total * bb)
        return fail(c, SMX_ERR_ARG, "upload: got %zu bytes, [%zu x %zu] needs %zu", nbytes, N, K, total * bb);
    if (c->capturing) return fail(c, SMX_ERR_ARG, "upload: not during graph capture");
    Weight w;
    w.type = type;
    w.K = K;
    w.N = N;
    w.nblk = nblk;
    size_t off_scales = 0, off_quants = 0, off_qh = 0, off_sc = 0;
    if (type == kQ4_0) {
        off_quants = align256(total * 2);
        w.bytes = off_quants + total * 16;
    } else if (type == kQ8_0) {
        off_quants = align256(total * 2);
        w.bytes = off_quants + total * 32;
    } else {
        off_quants = 0;  // ql
        off_qh = align256(total * 128);
        off_sc = off_qh + align256(total * 64);
        off_scales = off_sc + align256(total * 16);
        w.bytes = off_scales + total * 2;
    }
    // The raw blocks, padded to whole 16-byte pieces, next to the planes they are split into.  The staging buffer belongs to
    // the context and is reused by the next upload (a model's tensors arrive one after the other: no allocation and release
    // per tensor); one of more than kRawKeepBytes is given back at once.
    constexpr size_t kRawKeepBytes = size_t(256) << 20;
    const size_t raw_bytes = (nbytes + 15) & ~size_t(15);
    int rc0 = ensure(c, c->raw, raw_bytes);
    if (rc0 != SMX_OK) return rc0;
    char* raw = c->raw.p;
    auto drop_raw = [&]() {
        if (c->raw.cap > kRawKeepBytes) {
            (void)hipFree(c->raw.p);
            c->raw.p = nullptr;
            c->raw.cap = 0;
        }
    };
    hipError_t e = hipMalloc((void**)&w.base, w.bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        drop_raw();
        return fail(c, SMX_ERR_NOMEM, "upload: device allocation of %zu bytes failed: %s", w.bytes, hipGetErrorString(e));
    }
    auto bail = [&](hipError_t err, const char* what) {
        (void)hipStreamSynchronize(c->stream);
        drop_raw();
        (void)hipFree(w.base);
        return hip_fail(c, err, what);
    };
    if ((e = hipMemcpyAsync(raw, bytes, nbytes, hipMemcpyHostToDevice, c->stream)) != hipSuccess) return bail(e, "hipMemcpy(weight)");
    // the alignment gaps behind the planes (up to 255 bytes each) read as zero
    {
        const size_t ends[3][2] = {{type == kQ6_K ? total * 128 : total * 2, type == kQ6_K ? off_qh : off_quants},
                                   {off_qh + total * 64, off_sc}, {off_sc + total * 16, off_scales}};
        for (int i = 0; i < (type == kQ6_K ? 3 : 1); i++)
            if (ends[i][1] > ends[i][0] &&
                (e = hipMemsetAsync(w.base + ends[i][0], 0, ends[i][1] - ends[i][0], c->stream)) != hipSuccess)
                return bail(e, "hipMemset(weight)");
    }
    uint16_t* scales = (uint16_t*)(w.base + off_scales);
    if (type == kQ6_K) {
        const unsigned grid = (unsigned)((total + kRepackBlocks / 2 - 1) / (kRepackBlocks / 2));
        hipLaunchKernelGGL(repack_q6k_kernel, dim3(grid), dim3(256), 0, c->stream, (const uint4*)raw, total, (uint4*)(w.base + off_quants),
                           (uint4*)(w.base + off_qh), (uint4*)(w.base + off_sc), scales);
    } else {
        const unsigned grid = (unsigned)((total + kRepackBlocks - 1) / kRepackBlocks);
        if (type == kQ4_0)
            hipLaunchKernelGGL(repack_q4q8_kernel<18>, dim3(grid), dim3(256), 0, c->stream, (const uint4*)raw, total, scales,
                               (uint4*)(w.base + off_quants));
        else
            hipLaunchKernelGGL(repack_q4q8_kernel<34>, dim3(grid), dim3(256), 0, c->stream, (const uint4*)raw, total, scales,
                               (uint4*)(w.base + off_quants));
    }
    if ((e = hipGetLastError()) != hipSuccess) return bail(e, "repack launch");
    if ((e = hipStreamSynchronize(c->stream)) != hipSuccess) return bail(e, "repack");
    drop_raw();
    w.scales = scales;
    w.quants = w.base + off_quants;
    w.qh = type == kQ6_K ? w.base + off_qh : nullptr;
    w.sc = type == kQ6_K ? (const int8_t*)(w.base + off_sc) : nullptr;
    *out = w;
    return SMX_OK;
}

static int upload(smx_ctx* c, QType type, const char* key, const void* bytes, size_t nbytes, size_t K,
                  size_t N) {
    if (!c) return SMX_ERR_ARG;
    if (!key) return fail(c, SMX_ERR_ARG, "upload: null key");
    SMX_HIP(c, hipSetDevice(c->device));
    Weight w;
    int rc = build_weight(c, type, (const uint8_t*)bytes, nbytes, K, N, &w);
    if (rc != SMX_OK) return rc;
    return guarded(c, "upload", [&]() -> int {
        auto it = c->weights.find(key);
        if (it != c->weights.end()) {
            (void)hipStreamSynchronize(c->stream);
            drop_weight(c, it->second);
            it->second = w;
        } else {
            try {
                c->weights.emplace(key, w);
            } catch (...) {
                free_weight(w);
                throw;
            }
        }
        return SMX_OK;
    });
}

}  // namespace smx

using namespace smx;

extern "C" {

int smx_create(int device, smx_ctx** out) {
    if (!out) return fail(nullptr, SMX_ERR_ARG, "smx_create: null out pointer");
    *out = nullptr;
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev <= 0) {
        (void)hipGetLastError();
        return fail(nullptr, SMX_ERR_HIP, "smx_create: no HIP device (%s)", hipGetErrorString(e));
    }
    if (device < 0 || device >= ndev) return fail(nullptr, SMX_ERR_ARG, "smx_create: device %d of %d", device, ndev);
    e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail(nullptr, e, "hipSetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_fail(nullptr, e, "hipGetDeviceProperties");
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(nullptr, SMX_ERR_ARG, "smx_create: device %d is %s; this library is built for gfx950 only",
                    device, prop.gcnArchName);
    smx_ctx* c = new (std::nothrow) smx_ctx();
    if (!c) return fail(nullptr, SMX_ERR_NOMEM, "smx_create: out of host memory");
    c->device = device;
    c->num_cu = prop.multiProcessorCount;
    c->name = std::string(prop.name) + " (" + prop.gcnArchName + ", strix-mi355)";
    e = hipStreamCreate(&c->stream);  // default priority
    if (e != hipSuccess) {
        delete c;
        return hip_fail(nullptr, e, "hipStreamCreate");
    }
    if (hipEventCreate(&c->t0) != hipSuccess || hipEventCreate(&c->t1) != hipSuccess) {
        (void)hipStreamDestroy(c->stream);
        delete c;
        return fail(nullptr, SMX_ERR_HIP, "smx_create: hipEventCreate failed");
    }
    if (noalloc_init(c) != SMX_OK) {   // the static scratch array of the allocation-free entry point, on this device
        g_create_err = c->err;
        (void)hipEventDestroy(c->t0);
        (void)hipEventDestroy(c->t1);
        (void)hipStreamDestroy(c->stream);
        delete c;
        return SMX_ERR_HIP;
    }
    *out = c;
    return SMX_OK;
}

void smx_destroy(smx_ctx* c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    (void)hipStreamSynchronize(c->stream);
    for (auto& kv : c->weights) free_weight(kv.second);
    for (auto& kv : c->moe) {
        free_weight(kv.second.gate);
        free_weight(kv.second.up);
        free_weight(kv.second.down);
    }
    for (DevBuf* b : {&c->xf32, &c->xq, &c->xd, &c->xs, &c->yf32, &c->work, &c->work2, &c->tab, &c->raw})
        if (b->p) (void)hipFree(b->p);
    for (char* p : c->retired) (void)hipFree(p);
    for (DevBuf* b : {&c->hx, &c->hy, &c->htab})
        if (b->p) (void)hipHostFree(b->p);
    if (c->htab_done) (void)hipEventDestroy(c->htab_done);
    for (auto& r : c->prof) {
        (void)hipEventDestroy(r.e0);
        (void)hipEventDestroy(r.e1);
    }
    for (auto& p : c->ev_pool) {
        (void)hipEventDestroy(p.first);
        (void)hipEventDestroy(p.second);
    }
    (void)hipEventDestroy(c->t0);
    (void)hipEventDestroy(c->t1);
    (void)hipStreamDestroy(c->stream);
    delete c;
}

const char* smx_last_error(const smx_ctx* c) { return c ? c->err.c_str() : g_create_err.c_str(); }
const char* smx_name(const smx_ctx* c) { return c ? c->name.c_str() : ""; }
size_t smx_resident_count(const smx_ctx* c) { return c ? c->weights.size() + c->moe.size() : 0; }

size_t smx_resident_bytes(const smx_ctx* c) {
    if (!c) return 0;
    size_t n = 0;
    for (auto& kv : c->weights) n += kv.second.bytes;
    for (auto& kv : c->moe) n += kv.second.gate.bytes + kv.second.up.bytes + kv.second.down.bytes;
    return n;
}

int smx_upload_q4_0(smx_ctx* c, const char* key, const void* bytes, size_t nbytes, size_t in_dim, size_t out_dim) {
    return upload(c, kQ4_0, key, bytes, nbytes, in_dim, out_dim);
}
int smx_upload_q8_0(smx_ctx* c, const char* key, const void* bytes, size_t nbytes, size_t in_dim, size_t out_dim) {
    return upload(c, kQ8_0, key, bytes, nbytes, in_dim, out_dim);
}
int smx_upload_q6_k(smx_ctx* c, const char* key, const void* bytes, size_t nbytes, size_t in_dim, size_t out_dim) {
    return upload(c, kQ6_K, key, bytes, nbytes, in_dim, out_dim);
}

static int upload_moe(smx_ctx* c, QType type, const char* who, size_t layer, const void* gate, size_t gate_n, const void* up,
                      size_t up_n, const void* down, size_t down_n, size_t hidden, size_t eff, size_t ne) {
    if (!c) return SMX_ERR_ARG;
    if (!gate || !up || !down) return fail(c, SMX_ERR_ARG, "%s: null tensor", who);
    const size_t be = type == kQ6_K ? 256 : 32, bb = type == kQ6_K ? 210 : 34;
    if (hidden == 0 || eff == 0 || ne == 0 || hidden % be != 0 || eff % be != 0)
        return fail(c, SMX_ERR_ARG, "%s: hidden %zu / eff %zu must be positive multiples of %zu", who, hidden, eff, be);
    const size_t gate_eb = (hidden / be) * bb * eff, down_eb = (eff / be) * bb * hidden;  // decode.rs:2730-2731, 2806-2807
    if (gate_n != gate_eb * ne || up_n != gate_eb * ne || down_n != down_eb * ne)
        return fail(c, SMX_ERR_ARG, "%s: byte lengths (%zu, %zu, %zu) do not match %zu experts of %zu/%zu", who, gate_n, up_n,
                    down_n, ne, gate_eb, down_eb);
    SMX_HIP(c, hipSetDevice(c->device));
    MoeLayer L;
    L.type = type;
    L.hidden = hidden;
    L.eff = eff;
    L.ne = ne;
    int rc = build_weight(c, type, (const uint8_t*)gate, gate_n, hidden, ne * eff, &L.gate);
    if (rc != SMX_OK) return rc;
    rc = build_weight(c, type, (const uint8_t*)up, up_n, hidden, ne * eff, &L.up);
    if (rc != SMX_OK) {
        free_weight(L.gate);
        return rc;
    }
    rc = build_weight(c, type, (const uint8_t*)down, down_n, eff, ne * hidden, &L.down);
    if (rc != SMX_OK) {
        free_weight(L.gate);
        free_weight(L.up);
        return rc;
    }
    return guarded(c, who, [&]() -> int {
        auto it = c->moe.find(layer);
        if (it != c->moe.end()) {
            (void)hipStreamSynchronize(c->stream);
            drop_weight(c, it->second.gate);
            drop_weight(c, it->second.up);
            drop_weight(c, it->second.down);
            it->second = L;
        } else {
            try {
                c->moe.emplace(layer, L);
            } catch (...) {
                free_weight(L.gate);
                free_weight(L.up);
                free_weight(L.down);
                throw;
            }
        }
        return SMX_OK;
    });
}

int smx_upload_moe_q8(smx_ctx* c, size_t layer, const void* gate, size_t gate_n, const void* up, size_t up_n,
                      const void* down, size_t down_n, size_t hidden, size_t eff, size_t ne) {
    return upload_moe(c, kQ8_0, "upload_moe_q8", layer, gate, gate_n, up, up_n, down, down_n, hidden, eff, ne);
}

int smx_upload_moe_q6(smx_ctx* c, size_t layer, const void* gate, size_t gate_n, const void* up, size_t up_n,
                      const void* down, size_t down_n, size_t hidden, size_t eff, size_t ne) {
    return upload_moe(c, kQ6_K, "upload_moe_q6", layer, gate, gate_n, up, up_n, down, down_n, hidden, eff, ne);
}

int smx_evict(smx_ctx* c, const char* key) {
    if (!c || !key) return SMX_ERR_ARG;
    return guarded(c, "evict", [&]() -> int {
        auto it = c->weights.find(key);
        if (it == c->weights.end()) return SMX_NOT_RESIDENT;
        SMX_HIP(c, hipStreamSynchronize(c->stream));
        drop_weight(c, it->second);   // kept until the context closes while a captured graph may name it
        c->weights.erase(it);
        return SMX_OK;
    });
}

int smx_weight_dims(const smx_ctx* c, const char* key, size_t* in_dim, size_t* out_dim) {
    if (!c || !key) return SMX_ERR_ARG;
    for (const auto& kv : c->weights)   // no temporary std::string: this call allocates nothing
        if (kv.first == key) {
            if (in_dim) *in_dim = kv.second.K;
            if (out_dim) *out_dim = kv.second.N;
            return SMX_OK;
        }
    return SMX_NOT_RESIDENT;
}

int smx_dev_alloc(smx_ctx* c, size_t nbytes, void** dptr) {
    if (!c || !dptr) return SMX_ERR_ARG;
    SMX_HIP(c, hipSetDevice(c->device));
    hipError_t e = hipMalloc(dptr, nbytes ? nbytes : 1);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(c, SMX_ERR_NOMEM, "smx_dev_alloc: %zu bytes: %s", nbytes, hipGetErrorString(e));
    }
    return SMX_OK;
}

int smx_dev_free(smx_ctx* c, void* dptr) {
    if (!c) return SMX_ERR_ARG;
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    SMX_HIP(c, hipFree(dptr));
    return SMX_OK;
}

int smx_h2d(smx_ctx* c, void* dst, const void* src, size_t n) {
    if (!c || !dst || !src) return SMX_ERR_ARG;
    SMX_HIP(c, hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

int smx_d2h(smx_ctx* c, void* dst, const void* src, size_t n) {
    if (!c || !dst || !src) return SMX_ERR_ARG;
    SMX_HIP(c, hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

int smx_sync(smx_ctx* c) {
    if (!c) return SMX_ERR_ARG;
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

struct smx_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

int smx_graph_begin(smx_ctx* c) {
    if (!c) return SMX_ERR_ARG;
    if (c->capturing) return fail(c, SMX_ERR_ARG, "graph_begin: already capturing");
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    SMX_HIP(c, hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal));
    c->capturing = true;
    return SMX_OK;
}

int smx_graph_end(smx_ctx* c, smx_graph** out) {
    if (!c || !out) return SMX_ERR_ARG;
    if (!c->capturing) return fail(c, SMX_ERR_ARG, "graph_end: not capturing");
    c->capturing = false;
    smx_graph* g = new (std::nothrow) smx_graph();
    if (!g) return fail(c, SMX_ERR_NOMEM, "graph_end: out of host memory");
    hipError_t e = hipStreamEndCapture(c->stream, &g->graph);
    if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        return hip_fail(c, e, "hipStreamEndCapture/hipGraphInstantiate");
    }
    c->live_graphs++;
    *out = g;
    return SMX_OK;
}

int smx_graph_launch(smx_ctx* c, smx_graph* g) {
    if (!c || !g) return SMX_ERR_ARG;
    SMX_HIP(c, hipGraphLaunch(g->exec, c->stream));
    return SMX_OK;
}

void smx_graph_destroy(smx_ctx* c, smx_graph* g) {
    if (!g) return;
    if (c) (void)hipStreamSynchronize(c->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    if (c && c->live_graphs > 0) c->live_graphs--;
    delete g;
}

int smx_tune(smx_ctx* c, const char* knob, int value) {
    if (!c || !knob) return SMX_ERR_ARG;
    if (value < 0) return fail(c, SMX_ERR_ARG, "tune: negative value for %s", knob);
    const std::string k = knob;
    if (k == "gemv_rpw") {
        if (value != 0 && value != 1 && value != 2 && value != 4) return fail(c, SMX_ERR_ARG, "tune: gemv_rpw must be 0, 1, 2 or 4");
        c->tune_gemv_rpw = value;
    } else if (k == "gemv_ks") {
        if (value != 0 && value != 1 && value != 2 && value != 4) return fail(c, SMX_ERR_ARG, "tune: gemv_ks must be 0, 1, 2 or 4");
        c->tune_gemv_ks = value;
    } else if (k == "gemv_lpr") {
        if (value != 0 && value != 16 && value != 32 && value != 64) return fail(c, SMX_ERR_ARG, "tune: gemv_lpr must be 0, 16, 32 or 64");
        c->tune_gemv_lpr = value;
    } else if (k == "gemv_wpc") {
        if (value > 32) return fail(c, SMX_ERR_ARG, "tune: gemv_wpc must be 0..32");
        c->tune_gemv_wpc = value;
    } else if (k == "gemm_splitk") {
        if (value > 16) return fail(c, SMX_ERR_ARG, "tune: gemm_splitk must be 0..16");
        c->tune_gemm_splitk = value;
    } else if (k == "gemm_tile_m") {
        if (value != 0 && value != 64 && value != 128) return fail(c, SMX_ERR_ARG, "tune: gemm_tile_m must be 0, 64 or 128");
        c->tune_gemm_tile_m = value;
    } else if (k == "gemm_walk") {
        if (value > 64) return fail(c, SMX_ERR_ARG, "tune: gemm_walk must be 0..64");
        c->tune_gemm_walk = value;   // token-tile groups of the GEMM's tile walk (0: chosen from the L2 size)
    } else if (k == "gemm_narrow") {
        if (value > 1025) return fail(c, SMX_ERR_ARG, "tune: gemm_narrow must be 0 (rule), 1 (none) or 1 + the number of 96-row strips");
        c->tune_gemm_narrow = value;
    } else if (k == "host_io") {
        if (value > 2) return fail(c, SMX_ERR_ARG, "tune: host_io must be 0 (kernels on the pinned buffers), 1 (copy commands both ways) or 2 (copy in, result direct)");
        c->tune_host_io = value;
    } else {
        return fail(c, SMX_ERR_ARG, "tune: unknown knob %s", knob);
    }
    return SMX_OK;
}

int smx_prof_enable(smx_ctx* c, int on) {
    if (!c) return SMX_ERR_ARG;
    c->prof_on = on != 0;
    return SMX_OK;
}

int smx_prof_reset(smx_ctx* c) {
    if (!c) return SMX_ERR_ARG;
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    for (auto& r : c->prof) c->ev_pool.emplace_back(r.e0, r.e1);
    c->prof.clear();
    return SMX_OK;
}

int smx_prof_read(smx_ctx* c, const char* prefix, double* total_ms, size_t* launches) {
    if (!c || !prefix || !total_ms || !launches) return SMX_ERR_ARG;
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    double tot = 0;
    size_t n = 0;
    const size_t pl = strlen(prefix);
    for (auto& r : c->prof) {
        if (r.name.compare(0, pl, prefix) != 0) continue;
        float ms = 0;
        SMX_HIP(c, hipEventElapsedTime(&ms, r.e0, r.e1));
        tot += ms;
        n++;
    }
    *total_ms = tot;
    *launches = n;
    return SMX_OK;
}

const char* smx_prof_names(smx_ctx* c) {
    if (!c) return "";
    c->prof_names.clear();
    for (auto& r : c->prof)
        if (("," + c->prof_names + ",").find("," + r.name + ",") == std::string::npos)
            c->prof_names += (c->prof_names.empty() ? "" : ",") + r.name;
    return c->prof_names.c_str();
}

int smx_timer_begin(smx_ctx* c) {
    if (!c) return SMX_ERR_ARG;
    SMX_HIP(c, hipEventRecord(c->t0, c->stream));
    return SMX_OK;
}

int smx_timer_end(smx_ctx* c, float* ms) {
    if (!c || !ms) return SMX_ERR_ARG;
    SMX_HIP(c, hipEventRecord(c->t1, c->stream));
    SMX_HIP(c, hipEventSynchronize(c->t1));
    SMX_HIP(c, hipEventElapsedTime(ms, c->t0, c->t1));
    return SMX_OK;
}

}  // extern "C"
