// extern "C" entry points of the matmul path: host-pointer calls (copy in, run, copy out, sync)
// and device-pointer calls (enqueue only).
#include <algorithm>
#include <cstring>

#include "detmath.h"
#include "smx_internal.h"

using namespace smx;

namespace {

const Weight* find_weight(smx_ctx* c, const char* key) {
    auto it = c->weights.find(key);
    return it == c->weights.end() ? nullptr : &it->second;
}

// Scratch for m quantised rows of length K.
int ensure_act(smx_ctx* c, size_t m, size_t K) {
    int rc;
    if ((rc = ensure(c, c->xq, m * K)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->xd, m * (K / 32) * 4)) != SMX_OK) return rc;
    return ensure(c, c->xs, m * (K / 32) * 4);
}

// argmax per row of y[m][N], lowest index on ties (strict '>' scan order of decode.rs:3677-3683), in two launches:
// workgroup (chunk, row) finds the best of kArgmaxChunk consecutive logits, one workgroup per row then takes the best of
// the chunks.  (One workgroup scanning a 262144-entry row alone took 265 us, more than the lm_head GEMV in front of it.)
constexpr int kArgmaxChunk = 2048;
struct Best { float v; unsigned i; };
// the better of two candidates: larger value, lower index on equal values; index 0xffffffff = none yet
__device__ __forceinline__ Best better(Best a, Best b) {
    const bool take = b.i != 0xffffffffu && (a.i == 0xffffffffu || b.v > a.v || (b.v == a.v && b.i < a.i));
    return take ? b : a;
}
__device__ __forceinline__ Best workgroup_best(Best me) {   // 256 threads; valid in thread 0
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) me = better(me, Best{__shfl_xor(me.v, o), (unsigned)__shfl_xor((int)me.i, o)});
    __shared__ float sv[4];
    __shared__ unsigned si[4];
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = me.v; si[threadIdx.x >> 6] = me.i; }
    __syncthreads();
    Best r = Best{sv[0], si[0]};
#pragma unroll
    for (int w = 1; w < 4; w++) r = better(r, Best{sv[w], si[w]});
    return r;
}
__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ y, size_t N, int nchunks,
                                                            float* __restrict__ pv, unsigned* __restrict__ pi) {
    const float* row = y + (size_t)blockIdx.y * N;
    const size_t base = (size_t)blockIdx.x * kArgmaxChunk;
    float v[kArgmaxChunk / 256];
#pragma unroll
    for (int j = 0; j < kArgmaxChunk / 256; j++) {   // all loads first
        const size_t i = base + j * 256 + threadIdx.x;
        v[j] = i < N ? row[i] : 0.f;
    }
    Best me = Best{0.f, 0xffffffffu};
#pragma unroll
    for (int j = 0; j < kArgmaxChunk / 256; j++) {
        const size_t i = base + j * 256 + threadIdx.x;
        if (i < N && !(v[j] != v[j])) me = better(me, Best{v[j], (unsigned)i});   // NaN never wins
    }
    const Best r = workgroup_best(me);
    if (threadIdx.x == 0) {
        pv[(size_t)blockIdx.y * nchunks + blockIdx.x] = r.v;
        pi[(size_t)blockIdx.y * nchunks + blockIdx.x] = r.i;
    }
}
__global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ pv, const unsigned* __restrict__ pi,
                                                           int nchunks, unsigned* __restrict__ out) {
    Best me = Best{0.f, 0xffffffffu};
    for (int c = threadIdx.x; c < nchunks; c += 256)
        me = better(me, Best{pv[(size_t)blockIdx.x * nchunks + c], pi[(size_t)blockIdx.x * nchunks + c]});
    const Best r = workgroup_best(me);
    if (threadIdx.x == 0) out[blockIdx.x] = r.i == 0xffffffffu ? 0u : r.i;   // a row of NaNs: index 0
}

// ids[m] (device) = argmax of each row of y[m][N]; `part`: m * ceil(N / kArgmaxChunk) * 8 bytes of device scratch
static size_t argmax_scratch_bytes(size_t m, size_t N) { return m * ((N + kArgmaxChunk - 1) / kArgmaxChunk) * 8; }
static int launch_argmax_rows(smx_ctx* c, const float* y, size_t m, size_t N, void* part, unsigned* ids) {
    if (N >= 0xffffffffull) return fail(c, SMX_ERR_LIMIT, "argmax: %zu entries per row exceed the 32-bit index", N);
    const int nchunks = (int)((N + kArgmaxChunk - 1) / kArgmaxChunk);
    float* pv = (float*)part;
    unsigned* pi = (unsigned*)(pv + m * (size_t)nchunks);
    ProfScope ps(c, "argmax_rows");
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3((unsigned)nchunks, (unsigned)m), dim3(256), 0, c->stream, y, N, nchunks, pv, pi);
    SMX_HIP(c, hipGetLastError());
    hipLaunchKernelGGL(argmax_final_kernel, dim3((unsigned)m), dim3(256), 0, c->stream, (const float*)pv, (const unsigned*)pi, nchunks, ids);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

// quantise m device rows and run the right matmul kernel into y_dev
// Which kernel serves m rows: the small-batch MFMA kernel for 5..32 rows of a Q8_0 / Q4_0 weight (17..32 rows: weights of up
// to 32768 rows) and 5..16 rows of a Q6_K weight (skinny_serves); otherwise the dot4 GEMV up to SMX_GEMV_MAX_M rows (4 of a
// Q6_K weight), the tiled GEMM beyond.
}  // namespace

namespace smx {
// sc (optional): room for the m quantised rows instead of the context's growable scratch; only for calls
// the GEMV or the small-batch kernel serves (m <= SMX_SKINNY_MAX_M).
int run_matmul_dev(smx_ctx* c, const Weight& w, const float* xs_dev, size_t m, float* y_dev, bool force_gemm,
                   int32_t* dump, const ActScratch* sc) {
    const bool skinny = skinny_serves(w, m);
    // Q6_K with 5..8 rows of a weight the small-batch kernel declines (rows shorter than 128 elements): the tiled GEMM, whose
    // sparse tiles share their rows out over the waves; a caller that brings its own scratch keeps the dot4 GEMV there (the
    // GEMM sizes its scratch itself).
    const bool gemv_rows = m <= SMX_GEMV_MAX_M && (w.type != kQ6_K || m <= 4 || sc != nullptr);
    if (!skinny && gemv_rows && !force_gemm) return launch_gemv(c, w, xs_dev, m, y_dev, dump, sc);  // quantiser fused
    if (sc && !skinny) return fail(c, SMX_ERR_LIMIT, "%zu rows of this weight need the tiled GEMM, which sizes its scratch from the call", m);
    ActScratch a;
    int rc;
    if (sc) {
        a = *sc;   // m <= 8 rows: the fragment-ordered quants take 8 * K bytes, what m = 8 plain rows take
    } else {
        if ((rc = ensure_act(c, std::max(m, skinny ? skinny_xq_bytes(m, w.K) / w.K : m), w.K)) != SMX_OK) return rc;
        if (skinny && (rc = ensure(c, c->xd, skinny_xd_bytes(m, w.K))) != SMX_OK) return rc;
        a = ActScratch{(int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p};
    }
    if (skinny) return launch_skinny(c, w, xs_dev, m, y_dev, dump, a);
    rc = launch_actquant(c, xs_dev, m, w.K, a.xq, a.xd, a.xs);
    if (rc != SMX_OK) return rc;
    return launch_gemm(c, w, a.xq, a.xd, m, y_dev, dump);
}
}  // namespace smx

namespace {

int matmul_host(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, float* y, size_t y_cap,
                bool force_gemm, const char* who) {
    if (!c) return SMX_ERR_ARG;
    if (!key) return fail(c, SMX_ERR_ARG, "%s: null key", who);
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;  // a decline comes before any look at the buffers (the caller may not know out_dim)
    if (!xs || !y) return fail(c, SMX_ERR_ARG, "%s: null argument", who);
    if (in_dim != w->K) return fail(c, SMX_ERR_ARG, "%s: activation length %zu, weight in_dim %zu", who, in_dim, w->K);
    if (m == 0) return fail(c, SMX_ERR_ARG, "%s: zero rows", who);
    if (y_cap < m * w->N) return fail(c, SMX_ERR_ARG, "%s: output capacity %zu < %zu", who, y_cap, m * w->N);
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, m * w->K * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, m * w->N * 4)) != SMX_OK) return rc;
    // small transfers go through pinned staging: a pageable hipMemcpyAsync costs ~10 us each way
    const size_t xb = m * w->K * 4, yb = m * w->N * 4;
    const bool pinned = xb + yb <= (size_t(8) << 20);
    if (pinned) {
        if ((rc = ensure_host(c, c->hx, xb)) != SMX_OK) return rc;
        if ((rc = ensure_host(c, c->hy, yb)) != SMX_OK) return rc;
        memcpy(c->hx.p, xs, xb);
    }
    // Up to 4 rows on the GEMV kernels (plain loads of x, plain stores of y): the kernel reads the pinned staging and writes the
    // pinned result itself.  A copy command each way costs more than the kernel (measured per call with one synchronisation:
    // kernel alone 13 us, + host-to-device copy 16, + device-to-host copy 25; kernel on the pinned buffers 17).
    const bool gemv_path = m <= 4 && !force_gemm && !skinny_serves(*w, m);
    // (x: one row of up to 64 KB; every workgroup reads the whole row, and several long rows read over the bus by 256
    // workgroups cost more than the copy command: Q8_0 2560 x 9728, 3 rows, 39 - 45 us against 34)
    const bool x_direct = pinned && gemv_path && m == 1 && xb <= (size_t(64) << 10) && c->tune_host_io != 1 && c->tune_host_io != 2;
    const bool y_direct = pinned && gemv_path && c->tune_host_io != 1;
    if (!x_direct)
        SMX_HIP(c, hipMemcpyAsync(c->xf32.p, pinned ? (const void*)c->hx.p : (const void*)xs, xb, hipMemcpyHostToDevice, c->stream));
    rc = run_matmul_dev(c, *w, x_direct ? (const float*)c->hx.p : (const float*)c->xf32.p, m, y_direct ? (float*)c->hy.p : (float*)c->yf32.p,
                        force_gemm, nullptr, nullptr);
    if (rc != SMX_OK) return rc;
    if (!y_direct) SMX_HIP(c, hipMemcpyAsync(pinned ? (void*)c->hy.p : (void*)y, c->yf32.p, yb, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    if (pinned) memcpy(y, c->hy.p, yb);
    return SMX_OK;
}

}  // namespace

extern "C" {

int smx_gemv(smx_ctx* c, const char* key, const float* x, size_t in_len, float* y, size_t out_cap) {
    return matmul_host(c, key, x, 1, in_len, y, out_cap, false, "gemv");
}

int smx_gemv_rows(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, float* y, size_t y_cap) {
    if (c && m > SMX_GEMV_ROWS_MAX) return fail(c, SMX_ERR_LIMIT, "gemv_rows: %zu rows (limit %d)", m, SMX_GEMV_ROWS_MAX);
    return matmul_host(c, key, xs, m, in_dim, y, y_cap, false, "gemv_rows");
}

int smx_gemm(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, float* y, size_t y_cap) {
    return matmul_host(c, key, xs, m, in_dim, y, y_cap, true, "gemm");
}

// One device job and one synchronisation for n host-pointer GEMVs.  f32: every item runs the fp32-activation kernel
// (one launch per item, back to back); otherwise consecutive items of one format and row length share a launch.
static int gemv_batch_host(smx_ctx* c, size_t n, const char* const* keys, const float* const* xs, const size_t* in_lens,
                           float* const* ys, const size_t* out_caps, int* status, bool f32) {
    if (!c) return SMX_ERR_ARG;
    if (!keys || !xs || !in_lens || !ys || !out_caps || !status) return fail(c, SMX_ERR_ARG, "gemv_batch: null argument");
    return guarded(c, "gemv_batch", [&]() -> int {
    SMX_HIP(c, hipSetDevice(c->device));
    // Pass 1: validate and size one scratch region per item so the whole batch is one device job.
    std::vector<const Weight*> ws(n, nullptr);
    size_t xbytes = 0, ybytes = 0, qbytes = 0, dbytes = 0;
    for (size_t i = 0; i < n; i++) {
        status[i] = SMX_NOT_RESIDENT;
        if (!keys[i] || !xs[i] || !ys[i]) {
            status[i] = fail(c, SMX_ERR_ARG, "gemv_batch: item %zu has a null pointer", i);
            continue;
        }
        const Weight* w = find_weight(c, keys[i]);
        if (!w) continue;
        if (in_lens[i] != w->K) {
            status[i] = fail(c, SMX_ERR_ARG, "gemv_batch: item %zu activation length %zu, in_dim %zu", i, in_lens[i], w->K);
            continue;
        }
        if (out_caps[i] < w->N) {
            status[i] = fail(c, SMX_ERR_ARG, "gemv_batch: item %zu output capacity %zu < %zu", i, out_caps[i], w->N);
            continue;
        }
        ws[i] = w;
        xbytes += (w->K * 4 + 255) & ~size_t(255);
        ybytes += (w->N * 4 + 255) & ~size_t(255);
        qbytes += (w->K + 255) & ~size_t(255);
        dbytes += ((w->K / 32) * 4 + 255) & ~size_t(255);
    }
    int rc;
    if ((rc = ensure(c, c->xf32, xbytes)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, ybytes)) != SMX_OK) return rc;
    (void)qbytes; (void)dbytes;
    // small batches travel as ONE pinned transfer each way instead of two pageable copies per item
    const bool pinned = xbytes + ybytes <= (size_t(8) << 20);
    if (pinned) {
        if ((rc = ensure_host(c, c->hx, xbytes)) != SMX_OK) return rc;
        if ((rc = ensure_host(c, c->hy, ybytes)) != SMX_OK) return rc;
    }
    size_t xo = 0, yo = 0;
    std::vector<size_t> yoff(n, 0);
    std::vector<float*> xdev(n, nullptr), ydev(n, nullptr);
    for (size_t i = 0; i < n; i++) {
        const Weight* w = ws[i];
        if (!w) continue;
        xdev[i] = (float*)(c->xf32.p + xo);
        ydev[i] = (float*)(c->yf32.p + yo);
        yoff[i] = yo;
        if (pinned) memcpy(c->hx.p + xo, xs[i], w->K * 4);
        else SMX_HIP(c, hipMemcpyAsync(xdev[i], xs[i], w->K * 4, hipMemcpyHostToDevice, c->stream));
        xo += (w->K * 4 + 255) & ~size_t(255);
        yo += (w->N * 4 + 255) & ~size_t(255);
    }
    // small batches: the kernels read the pinned staging and write the pinned results themselves (see matmul_host)
    // (every item's row is read by that item's workgroups only: rows of up to 64 KB each)
    size_t x_longest = 0;
    for (size_t i = 0; i < n; i++)
        if (ws[i]) x_longest = std::max(x_longest, ws[i]->K * 4);
    const bool x_direct = pinned && x_longest <= (size_t(64) << 10) && c->tune_host_io != 1 && c->tune_host_io != 2;
    const bool y_direct = pinned && c->tune_host_io != 1;
    for (size_t i = 0; i < n; i++) {
        if (!ws[i]) continue;
        if (x_direct) xdev[i] = (float*)(c->hx.p + ((char*)xdev[i] - c->xf32.p));
        if (y_direct) ydev[i] = (float*)(c->hy.p + yoff[i]);
    }
    if (pinned && xo && !x_direct) SMX_HIP(c, hipMemcpyAsync(c->xf32.p, c->hx.p, xo, hipMemcpyHostToDevice, c->stream));
    // consecutive items of one format and row length share a launch (up to 8 per launch)
    for (size_t i = 0; i < n;) {
        if (!ws[i]) { i++; continue; }
        if (f32) {
            status[i] = launch_gemv_f32(c, *ws[i], xdev[i], ydev[i]);
            i++;
            continue;
        }
        const Weight* gw[8];
        const float* gx[8];
        float* gy[8];
        size_t idx[8];
        int g = 0;
        size_t j = i;
        while (j < n && g < 8 && ws[j] && ws[j]->type == ws[i]->type && ws[j]->K == ws[i]->K) {
            gw[g] = ws[j]; gx[g] = xdev[j]; gy[g] = ydev[j]; idx[g] = j;
            g++; j++;
        }
        rc = launch_gemv_group(c, gw, gx, gy, g);
        for (int k = 0; k < g; k++) status[idx[k]] = rc;
        i = j;
    }
    if (pinned) {
        if (yo && !y_direct) SMX_HIP(c, hipMemcpyAsync(c->hy.p, c->yf32.p, yo, hipMemcpyDeviceToHost, c->stream));
    } else {
        for (size_t i = 0; i < n; i++)
            if (ws[i] && status[i] == SMX_OK)
                SMX_HIP(c, hipMemcpyAsync(ys[i], c->yf32.p + yoff[i], ws[i]->N * 4, hipMemcpyDeviceToHost, c->stream));
    }
    SMX_HIP(c, hipStreamSynchronize(c->stream));  // the batch's single sync (decode.rs:3247)
    if (pinned)
        for (size_t i = 0; i < n; i++)
            if (ws[i] && status[i] == SMX_OK) memcpy(ys[i], c->hy.p + yoff[i], ws[i]->N * 4);
    return SMX_OK;
    });
}

int smx_gemv_batch(smx_ctx* c, size_t n, const char* const* keys, const float* const* xs, const size_t* in_lens,
                   float* const* ys, const size_t* out_caps, int* status) {
    return gemv_batch_host(c, n, keys, xs, in_lens, ys, out_caps, status, false);
}

int smx_gemv_f32_batch(smx_ctx* c, size_t n, const char* const* keys, const float* const* xs, const size_t* in_lens,
                       float* const* ys, const size_t* out_caps, int* status) {
    return gemv_batch_host(c, n, keys, xs, in_lens, ys, out_caps, status, true);
}

int smx_lm_head_argmax_rows(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, uint32_t* out) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !xs || !out) return fail(c, SMX_ERR_ARG, "lm_head_argmax_rows: null argument");
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (in_dim != w->K) return fail(c, SMX_ERR_ARG, "lm_head_argmax_rows: activation length %zu, in_dim %zu", in_dim, w->K);
    if (m == 0) return fail(c, SMX_ERR_ARG, "lm_head_argmax_rows: zero rows");
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, m * w->K * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, m * w->N * 4)) != SMX_OK) return rc;
    const size_t ids_bytes = (m * 4 + 255) & ~size_t(255);   // ids, then the chunk candidates
    if ((rc = ensure(c, c->tab, ids_bytes + argmax_scratch_bytes(m, w->N))) != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(c->xf32.p, xs, m * w->K * 4, hipMemcpyHostToDevice, c->stream));
    rc = run_matmul_dev(c, *w, (const float*)c->xf32.p, m, (float*)c->yf32.p, false, nullptr, nullptr);
    if (rc != SMX_OK) return rc;
    rc = launch_argmax_rows(c, (const float*)c->yf32.p, m, w->N, (char*)c->tab.p + ids_bytes, (unsigned*)c->tab.p);
    if (rc != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(out, c->tab.p, m * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

int smx_gemv_dev(smx_ctx* c, const char* key, const float* xs_dev, size_t m, float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !xs_dev || !y_dev) return fail(c, SMX_ERR_ARG, "gemv_dev: null argument");
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (m == 0 || m > SMX_GEMV_ROWS_MAX) return fail(c, SMX_ERR_LIMIT, "gemv_dev: %zu rows (1..%d)", m, SMX_GEMV_ROWS_MAX);
    return run_matmul_dev(c, *w, xs_dev, m, y_dev, false, nullptr, nullptr);
}

int smx_gemv_batch_dev(smx_ctx* c, size_t n, const char* const* keys, const float* const* xs_dev, float* const* ys_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!keys || !xs_dev || !ys_dev) return fail(c, SMX_ERR_ARG, "gemv_batch_dev: null argument");
    if (n == 0 || n > 8) return fail(c, SMX_ERR_LIMIT, "gemv_batch_dev: %zu items (1..8 per launch)", n);
    const Weight* ws[8];
    for (size_t i = 0; i < n; i++) {
        if (!keys[i] || !xs_dev[i] || !ys_dev[i]) return fail(c, SMX_ERR_ARG, "gemv_batch_dev: item %zu has a null pointer", i);
        ws[i] = find_weight(c, keys[i]);
        if (!ws[i]) return SMX_NOT_RESIDENT;
    }
    return launch_gemv_group(c, ws, xs_dev, ys_dev, (int)n);
}

// Activation producer + quantiser + GEMV(s) in one launch.
static int gemv_fused_check(smx_ctx* c, int act, const float* a, const float* b, const char* who) {
    if (act < SMX_ACT_NONE || act > SMX_ACT_GEGLU) return fail(c, SMX_ERR_ARG, "%s: unknown activation producer %d", who, act);
    if (!a) return fail(c, SMX_ERR_ARG, "%s: null activation", who);
    if ((act == SMX_ACT_SILU_MUL || act == SMX_ACT_GEGLU) && !b) return fail(c, SMX_ERR_ARG, "%s: the producer needs its second operand", who);
    if (act == SMX_ACT_NONE && b) return fail(c, SMX_ERR_ARG, "%s: second operand without a producer", who);
    return SMX_OK;
}

int smx_gemv_fused_dev(smx_ctx* c, size_t n, const char* const* keys, int act, const float* a_dev, const float* b_dev,
                       float eps, float* const* ys_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!keys || !ys_dev) return fail(c, SMX_ERR_ARG, "gemv_fused_dev: null argument");
    if (n == 0 || n > SMX_GEMV_GROUP_MAX) return fail(c, SMX_ERR_LIMIT, "gemv_fused_dev: %zu weights (1..%d per launch)", n, SMX_GEMV_GROUP_MAX);
    int rc = gemv_fused_check(c, act, a_dev, b_dev, "gemv_fused_dev");
    if (rc != SMX_OK) return rc;
    const Weight* ws[SMX_GEMV_GROUP_MAX];
    const float* xs[SMX_GEMV_GROUP_MAX];
    for (size_t i = 0; i < n; i++) {
        if (!keys[i] || !ys_dev[i]) return fail(c, SMX_ERR_ARG, "gemv_fused_dev: item %zu has a null pointer", i);
        ws[i] = find_weight(c, keys[i]);
        if (!ws[i]) return SMX_NOT_RESIDENT;
        xs[i] = a_dev;
    }
    const ActProd prod = {act, b_dev, eps};
    return launch_gemv_group(c, ws, xs, ys_dev, (int)n, nullptr, &prod);
}

// h[i] = act(g[i]) * u[i], the arithmetic of the paired GEMV's tail (for shapes the paired launch does not serve)
__global__ __launch_bounds__(256) void act_mul_kernel(const float* __restrict__ g, const float* __restrict__ u, float* __restrict__ h,
                                                      int n, int act) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) h[i] = (act == SMX_ACT_GEGLU ? det_gelu_tanh(g[i]) : det_silu(g[i])) * u[i];
}

int smx_ffn_gate_up_dev(smx_ctx* c, const char* gate_key, const char* up_key, int act, const float* x_dev, int norm,
                        const float* norm_w_dev, float eps, float* h_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!gate_key || !up_key || !x_dev || !h_dev) return fail(c, SMX_ERR_ARG, "ffn_gate_up_dev: null argument");
    if (act != SMX_ACT_SILU_MUL && act != SMX_ACT_GEGLU)
        return fail(c, SMX_ERR_ARG, "ffn_gate_up_dev: activation %d (SMX_ACT_SILU_MUL or SMX_ACT_GEGLU)", act);
    if (norm != 0 && norm != 1) return fail(c, SMX_ERR_ARG, "ffn_gate_up_dev: norm %d (0 or 1)", norm);
    if (!norm && norm_w_dev) return fail(c, SMX_ERR_ARG, "ffn_gate_up_dev: norm weight without norm");
    const Weight* wg = find_weight(c, gate_key);
    const Weight* wu = find_weight(c, up_key);
    if (!wg || !wu) return SMX_NOT_RESIDENT;
    if (wg->type != wu->type || wg->K != wu->K || wg->N != wu->N)
        return fail(c, SMX_ERR_ARG, "ffn_gate_up_dev: gate is %zu x %zu (type %d), up %zu x %zu (type %d)", wg->N, wg->K,
                    (int)wg->type, wu->N, wu->K, (int)wu->type);
    const ActProd prod = {norm ? SMX_ACT_RMSNORM : SMX_ACT_NONE, norm_w_dev, eps};
    const float* xs[2] = {x_dev, x_dev};
    float* hs[1] = {h_dev};
    bool served = false;
    int rc = launch_gemv_dual(c, &wg, &wu, xs, nullptr, nullptr, hs, 1, act, &prod, nullptr, &served);
    if (rc != SMX_OK || served) return rc;
    // other shapes: the pair in one launch, then the product
    if ((rc = ensure(c, c->work2, 2 * wg->N * 4)) != SMX_OK) return rc;
    float* g = (float*)c->work2.p;
    float* u = g + wg->N;
    const Weight* ws[2] = {wg, wu};
    float* ys[2] = {g, u};
    if ((rc = launch_gemv_group(c, ws, xs, ys, 2, nullptr, &prod)) != SMX_OK) return rc;
    ProfScope ps(c, "act_mul");
    hipLaunchKernelGGL(act_mul_kernel, dim3((unsigned)((wg->N + 255) / 256)), dim3(256), 0, c->stream, (const float*)g, (const float*)u,
                       h_dev, (int)wg->N, act);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

int smx_gemv_fused(smx_ctx* c, const char* key, int act, const float* a, const float* b, size_t in_len, float eps,
                   float* y, size_t out_cap) {
    if (!c) return SMX_ERR_ARG;
    if (!key) return fail(c, SMX_ERR_ARG, "gemv_fused: null key");
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (!y) return fail(c, SMX_ERR_ARG, "gemv_fused: null output");
    int rc = gemv_fused_check(c, act, a, b, "gemv_fused");
    if (rc != SMX_OK) return rc;
    if (in_len != w->K) return fail(c, SMX_ERR_ARG, "gemv_fused: activation length %zu, weight in_dim %zu", in_len, w->K);
    if (out_cap < w->N) return fail(c, SMX_ERR_ARG, "gemv_fused: output capacity %zu < %zu", out_cap, w->N);
    SMX_HIP(c, hipSetDevice(c->device));
    if ((rc = ensure(c, c->xf32, 2 * w->K * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, w->N * 4)) != SMX_OK) return rc;
    float* a_dev = (float*)c->xf32.p;
    float* b_dev = b ? a_dev + w->K : nullptr;
    const size_t xb = (b ? 2 : 1) * w->K * 4, yb = w->N * 4;
    if ((rc = ensure_host(c, c->hx, xb)) != SMX_OK) return rc;
    if ((rc = ensure_host(c, c->hy, yb)) != SMX_OK) return rc;
    memcpy(c->hx.p, a, w->K * 4);
    if (b) memcpy(c->hx.p + w->K * 4, b, w->K * 4);
    // the kernel reads the pinned staging and writes the pinned result itself (see matmul_host)
    const bool x_direct = xb <= (size_t(64) << 10) && c->tune_host_io != 1 && c->tune_host_io != 2, y_direct = c->tune_host_io != 1;
    if (x_direct) {
        a_dev = (float*)c->hx.p;
        b_dev = b ? a_dev + w->K : nullptr;
    } else {
        SMX_HIP(c, hipMemcpyAsync(a_dev, c->hx.p, xb, hipMemcpyHostToDevice, c->stream));
    }
    const float* xs[1] = {a_dev};
    float* ys[1] = {y_direct ? (float*)c->hy.p : (float*)c->yf32.p};
    const ActProd prod = {act, b_dev, eps};
    if ((rc = launch_gemv_group(c, &w, xs, ys, 1, nullptr, &prod)) != SMX_OK) return rc;
    if (!y_direct) SMX_HIP(c, hipMemcpyAsync(c->hy.p, c->yf32.p, yb, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    memcpy(y, c->hy.p, yb);
    return SMX_OK;
}

// Prefill form of smx_gemv_fused_dev: the producer runs over m rows in the quantiser launch.
int smx_gemm_fused_dev(smx_ctx* c, const char* key, int act, const float* a_dev, const float* b_dev, size_t m, float eps,
                       float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !y_dev) return fail(c, SMX_ERR_ARG, "gemm_fused_dev: null argument");
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (m == 0) return fail(c, SMX_ERR_ARG, "gemm_fused_dev: zero rows");
    int rc = gemv_fused_check(c, act, a_dev, b_dev, "gemm_fused_dev");
    if (rc != SMX_OK) return rc;
    if (act == SMX_ACT_NONE) return run_matmul_dev(c, *w, a_dev, m, y_dev, true, nullptr, nullptr);
    if ((rc = ensure_act(c, m, w->K)) != SMX_OK) return rc;
    rc = launch_rows_prod_quant(c, act, a_dev, b_dev, m, w->K, eps, (int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p);
    if (rc != SMX_OK) return rc;
    return launch_gemm(c, *w, (const int8_t*)c->xq.p, (const float*)c->xd.p, m, y_dev, nullptr);
}

int smx_gemm_dev(smx_ctx* c, const char* key, const float* xs_dev, size_t m, float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !xs_dev || !y_dev) return fail(c, SMX_ERR_ARG, "gemm_dev: null argument");
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (m == 0) return fail(c, SMX_ERR_ARG, "gemm_dev: zero rows");
    return run_matmul_dev(c, *w, xs_dev, m, y_dev, true, nullptr, nullptr);
}

int smx_quantize(smx_ctx* c, const float* x, size_t m, size_t k, int8_t* xq, float* xd, int16_t* xs16) {
    if (!c) return SMX_ERR_ARG;
    if (!x || !xq || !xd) return fail(c, SMX_ERR_ARG, "quantize: null argument");
    if (m == 0 || k == 0 || k % 32 != 0) return fail(c, SMX_ERR_ARG, "quantize: bad shape %zu x %zu", m, k);
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, m * k * 4)) != SMX_OK) return rc;
    if ((rc = ensure_act(c, m, k)) != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(c->xf32.p, x, m * k * 4, hipMemcpyHostToDevice, c->stream));
    rc = launch_actquant(c, (const float*)c->xf32.p, m, k, (int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p);
    if (rc != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(xq, c->xq.p, m * k, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipMemcpyAsync(xd, c->xd.p, m * (k / 32) * 4, hipMemcpyDeviceToHost, c->stream));
    // the packed dword (lo16 | hi16 << 16) is two consecutive little-endian i16: xs16[m][k/16]
    if (xs16) SMX_HIP(c, hipMemcpyAsync(xs16, c->xs.p, m * (k / 32) * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

static int block_dots(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, int32_t* out,
                      size_t out_cap, bool gemm, const char* who) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !xs || !out) return fail(c, SMX_ERR_ARG, "%s: null argument", who);
    const Weight* w = find_weight(c, key);
    if (!w) return SMX_NOT_RESIDENT;
    if (in_dim != w->K) return fail(c, SMX_ERR_ARG, "%s: activation length %zu, in_dim %zu", who, in_dim, w->K);
    const size_t per = w->type == kQ6_K ? w->K / 16 : w->K / 32;
    const size_t need = m * w->N * per;
    if (out_cap < need) return fail(c, SMX_ERR_ARG, "%s: output capacity %zu < %zu", who, out_cap, need);
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, m * w->K * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, m * w->N * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->work, need * 4)) != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(c->xf32.p, xs, m * w->K * 4, hipMemcpyHostToDevice, c->stream));
    rc = run_matmul_dev(c, *w, (const float*)c->xf32.p, m, (float*)c->yf32.p, gemm, (int32_t*)c->work.p, nullptr);
    if (rc != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(out, c->work.p, need * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

int smx_gemv_block_dots(smx_ctx* c, const char* key, const float* x, size_t in_len, int32_t* out, size_t out_cap) {
    return block_dots(c, key, x, 1, in_len, out, out_cap, false, "gemv_block_dots");
}

int smx_gemm_block_dots(smx_ctx* c, const char* key, const float* xs, size_t m, size_t in_dim, int32_t* out,
                        size_t out_cap) {
    return block_dots(c, key, xs, m, in_dim, out, out_cap, true, "gemm_block_dots");
}

}  // extern "C"
