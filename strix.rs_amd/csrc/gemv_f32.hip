// GEMV with fp32 activations: y = dequant(W) . x, the arithmetic of the reference's per-weight `gemv`
// (crates/strix-backend-rocm/src/kernels.rs:41-69 q4_gemv, :646-668 q8_0_gemv, :607-640 q6_gemv; launched
// by decode.rs:3827-3898) and of strix-backend-cpu (dequantise a row, f32 dot).  No activation
// quantiser, no integer dots: every weight is widened to fp32 in registers and multiplied with the
// fp32 activation staged in LDS.  The decode path proper is the Q8-activation GEMV (gemv.hip); this
// form serves callers that hold the accelerator to the CPU result at fp32 accuracy.
//
// Two kernels.  gemv_f32_flat_kernel (rows of up to 16384 elements that are a whole number of unit groups: every shape
// of the models) has the memory side of the flat Q8-activation GEMV: the activation row is requested first, a
// workgroup's rows are one flat sequence of 64-unit loads, three loads per wave in flight, group sums through LDS.
// A weight element costs two vector operations: one conversion (v_cvt_f32_ubyteN on the unsigned quants of Q4_0 and
// Q6_K, the sign-extending byte select on Q8_0) and one FMA; the offsets (q - 8, q - 32) are taken out per
// 16-element half through the sums of the activation that the staging leaves in LDS.
// gemv_f32_kernel (any other shape up to 32768 elements): a wave serves RPW rows at a time, one load per row and lane
// in flight, DPP reduction per row.
// HBM-bound by bytes.
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "gemv_body.h"
#include "smx_internal.h"

namespace smx {

// The activation lives in LDS as 32-element blocks padded to 36 floats, so that lanes reading
// consecutive blocks with 16-byte loads fall into different bank groups.
__device__ __forceinline__ int xpad(int e) { return e + (e >> 5) * 4; }

// sum over the unit's elements of (weight value / block scale) * x, times the scale
__device__ __forceinline__ float unit_dot_f32(OpsQ4_0, const OpsQ4_0::Regs& r, const float* xs, int u) {
    const float* xb = xs + u * 36;
    const unsigned w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 xl = *(const float4*)(xb + 4 * g), xh = *(const float4*)(xb + 16 + 4 * g);
        const float xlo[4] = {xl.x, xl.y, xl.z, xl.w}, xhi[4] = {xh.x, xh.y, xh.z, xh.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float lo = (float)((w[g] >> (8 * k)) & 0xfu) - 8.f;       // element 4g + k
            const float hi = (float)((w[g] >> (8 * k + 4)) & 0xfu) - 8.f;   // element 16 + 4g + k
            s = fmaf(lo, xlo[k], s);
            s = fmaf(hi, xhi[k], s);
        }
    }
    return h2f(r.s) * s;
}

// Q8_0: unit u = half (u & 1) of block u >> 1
__device__ __forceinline__ float unit_dot_f32(OpsQ8_0, const OpsQ8_0::Regs& r, const float* xs, int u) {
    const float* xb = xs + (u >> 1) * 36 + (u & 1) * 16;
    const int w[4] = {(int)r.q.x, (int)r.q.y, (int)r.q.z, (int)r.q.w};
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 xv = *(const float4*)(xb + 4 * g);
        const float x4[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int k = 0; k < 4; k++) s = fmaf((float)(signed char)((w[g] >> (8 * k)) & 0xff), x4[k], s);
    }
    return h2f(r.s) * s;
}

// Q6_K: unit u = 64 elements: sub-blocks 2j + c (j = 0..3) of 128-element half g = u >> 1, c = u & 1
// (element map crates/strix-models/src/ggml_quant.rs:417-426); value d * sc * (q - 32)
__device__ __forceinline__ float unit_dot_f32(OpsQ6_K, const OpsQ6_K::Regs& r, const float* xs, int u) {
    const int g = u >> 1, c = u & 1;
    const unsigned a4[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
    const unsigned b4[4] = {r.b.x, r.b.y, r.b.z, r.b.w};
    const unsigned h4[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
    const unsigned long long scw = ((unsigned long long)r.sc.y << 32) | r.sc.x;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float* xb = xs + xpad(g * 128 + (2 * j + c) * 16);   // 16 consecutive elements, inside one 32-block
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            unsigned q;
            if (j == 0) q = (a4[i] & 0x0f0f0f0fu) | ((h4[i] << 4) & 0x30303030u);
            else if (j == 1) q = (b4[i] & 0x0f0f0f0fu) | ((h4[i] << 2) & 0x30303030u);
            else if (j == 2) q = ((a4[i] >> 4) & 0x0f0f0f0fu) | (h4[i] & 0x30303030u);
            else q = ((b4[i] >> 4) & 0x0f0f0f0fu) | ((h4[i] >> 2) & 0x30303030u);
            const float4 xv = *(const float4*)(xb + 4 * i);
            const float x4[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int k = 0; k < 4; k++) s = fmaf((float)((q >> (8 * k)) & 0xffu) - 32.f, x4[k], s);
        }
        const float sc = (float)(int)(signed char)((scw >> (8 * (2 * j + c))) & 0xff);
        acc = fmaf(sc, s, acc);
    }
    return h2f(r.d) * acc;
}

// Wave `wid` of `nwaves` serves row chunks wid, wid + nwaves, ... of RPW rows; a lane walks the units of
// a row 64 apart, the RPW loads of a pass requested together.
template <class Ops, int RPW>
__global__ __launch_bounds__(1024) void gemv_f32_kernel(const GemvW W, const float* __restrict__ x, float* __restrict__ y,
                                                        int nblk, int N) {
    extern __shared__ __align__(16) char smem[];
    float* xs = (float*)smem;
    const int K4 = Ops::nb32(nblk) * 8;   // float4 items of the row
    for (int i = threadIdx.x; i < K4; i += blockDim.x) *(float4*)(xs + xpad(4 * i)) = ((const float4*)x)[i];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), nwaves = gridDim.x * (blockDim.x >> 6);
    const int U = Ops::units_per_row(nblk);
    const int nchunks = (N + RPW - 1) / RPW;
    for (int ch = wid; ch < nchunks; ch += nwaves) {
        float acc[RPW];
#pragma unroll
        for (int r = 0; r < RPW; r++) acc[r] = 0.f;
        for (int u0 = 0; u0 < U; u0 += 64) {
            const int uu = u0 + lane;
            const bool act = uu < U;
            const int u = act ? uu : U - 1;   // clamped: the loads stay unconditional
            typename Ops::Regs regs[RPW];
#pragma unroll
            for (int r = 0; r < RPW; r++) Ops::load(regs[r], W, (size_t)min(ch * RPW + r, N - 1), nblk, u);
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                const float t = unit_dot_f32(Ops(), regs[r], xs, u);
                acc[r] += act ? t : 0.f;
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const float s = group_sum<64>(acc[r]);
            const int row = ch * RPW + r;
            if (lane == 63 && row < N) y[row] = s;
        }
    }
}

// ---- flat form ----
// LDS: the row as 32-blocks padded to 36 floats | hs[nb32 * 2]: the sums of its 16-element halves | group sums.
__device__ __forceinline__ float ubyte_f(unsigned w, int k) { return (float)((w >> (8 * k)) & 0xffu); }                  // v_cvt_f32_ubyteK
__device__ __forceinline__ float sbyte_f(unsigned w, int k) { return (float)(int)(signed char)((w >> (8 * k)) & 0xffu); }  // byte select, sign-extended

// Q4_0, unit = block u: sum((q - 8) x) = sum(q x) - 8 sum(x); the high nibbles are converted in place (16 q) and rescaled once
__device__ __forceinline__ float unit_dot_flat(OpsQ4_0, const OpsQ4_0::Regs& r, const float* xs, const float* hs, int u) {
    const float* xb = xs + u * 36;
    const unsigned w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    float sl = 0.f, sh = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        unsigned lo = w[g] & 0x0f0f0f0fu, hi = w[g] & 0xf0f0f0f0u;
        asm("" : "+v"(lo), "+v"(hi));   // keep the masked dwords: the byte conversions then need no extraction of their own
        const float4 xl = *(const float4*)(xb + 4 * g), xh = *(const float4*)(xb + 16 + 4 * g);
        const float xlo[4] = {xl.x, xl.y, xl.z, xl.w}, xhi[4] = {xh.x, xh.y, xh.z, xh.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            sl = fmaf(ubyte_f(lo, k), xlo[k], sl);   // element 4g + k
            sh = fmaf(ubyte_f(hi, k), xhi[k], sh);   // 16 x element 16 + 4g + k
        }
    }
    const float2 h = *(const float2*)(hs + 2 * u);
    return h2f(r.s) * (fmaf(sh, 0.0625f, sl) - 8.f * (h.x + h.y));
}

// Q8_0, unit u = half (u & 1) of block u >> 1
__device__ __forceinline__ float unit_dot_flat(OpsQ8_0, const OpsQ8_0::Regs& r, const float* xs, const float*, int u) {
    const float* xb = xs + (u >> 1) * 36 + (u & 1) * 16;
    const unsigned w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 xv = *(const float4*)(xb + 4 * g);
        s0 = fmaf(sbyte_f(w[g], 0), xv.x, s0);
        s1 = fmaf(sbyte_f(w[g], 1), xv.y, s1);
        s0 = fmaf(sbyte_f(w[g], 2), xv.z, s0);
        s1 = fmaf(sbyte_f(w[g], 3), xv.w, s1);
    }
    return h2f(r.s) * (s0 + s1);
}

// Q6_K, unit u = 64 elements: sub-blocks 2j + c (j = 0..3) of 128-element half g = u >> 1, c = u & 1; a sub-block is
// one 16-element half of the row: sum((q - 32) x) = sum(q x) - 32 hs
__device__ __forceinline__ float unit_dot_flat(OpsQ6_K, const OpsQ6_K::Regs& r, const float* xs, const float* hs, int u) {
    const int g = u >> 1, c = u & 1;
    const unsigned a4[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
    const unsigned b4[4] = {r.b.x, r.b.y, r.b.z, r.b.w};
    const unsigned h4[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
    const unsigned long long scw = ((unsigned long long)r.sc.y << 32) | r.sc.x;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float* xb = xs + xpad(g * 128 + (2 * j + c) * 16);
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            unsigned q;
            if (j == 0) q = (a4[i] & 0x0f0f0f0fu) | ((h4[i] << 4) & 0x30303030u);
            else if (j == 1) q = (b4[i] & 0x0f0f0f0fu) | ((h4[i] << 2) & 0x30303030u);
            else if (j == 2) q = ((a4[i] >> 4) & 0x0f0f0f0fu) | (h4[i] & 0x30303030u);
            else q = ((b4[i] >> 4) & 0x0f0f0f0fu) | ((h4[i] >> 2) & 0x30303030u);
            asm("" : "+v"(q));   // as above
            const float4 xv = *(const float4*)(xb + 4 * i);
            s0 = fmaf(ubyte_f(q, 0), xv.x, s0);
            s1 = fmaf(ubyte_f(q, 1), xv.y, s1);
            s0 = fmaf(ubyte_f(q, 2), xv.z, s0);
            s1 = fmaf(ubyte_f(q, 3), xv.w, s1);
        }
        const float sc = (float)(int)(signed char)((scw >> (8 * (2 * j + c))) & 0xff);
        acc = fmaf(sc, (s0 + s1) - 32.f * hs[g * 8 + 2 * j + c], acc);
    }
    return h2f(r.d) * acc;
}

// blockIdx.x of n_wgs workgroups share the rows; magic_u = ceil(2^32 / units per row).  Every argument lies in the
// first 64-byte line of the kernel-argument segment.
template <class Ops, int PRE, int GL>
__global__ __launch_bounds__(1024) void gemv_f32_flat_kernel(const GemvW W, const float* __restrict__ x, float* __restrict__ y,
                                                             int nblk, int N, int n_wgs, unsigned magic_u) {
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wg = blockIdx.x;
    const int U = Ops::units_per_row(nblk), nb32 = Ops::nb32(nblk);
    float* xs = (float*)smem;
    float* hs = xs + nb32 * 36;
    float* part = hs + nb32 * 2;   // [units of the workgroup / GL]
    // rows split evenly: the first N % n_wgs workgroups take one row more
    const unsigned rbase = (unsigned)N / (unsigned)n_wgs, rrem = (unsigned)N - rbase * (unsigned)n_wgs;
    const int r0 = wg * (int)rbase + min(wg, (int)rrem), r1 = r0 + (int)rbase + (wg < (int)rrem ? 1 : 0);
    const int nunits = (r1 - r0) * U;          // < 2^16 (launcher)
    const int nloads = (nunits + 63) >> 6;
    const size_t f_base = nunits > 0 ? (size_t)r0 * U : 0;   // a workgroup without rows re-reads the first unit

    // the row first (a wave's loads complete in order), a 16-element half per thread
    const int hb = threadIdx.x;
    float4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = hb < nb32 * 2 ? ((const float4*)x)[hb * 4 + j] : make_float4(0.f, 0.f, 0.f, 0.f);

    typename Ops::Regs ring[PRE];
    int l_t = wave, c_t = wave;
    auto request = [&]() {
#pragma unroll
        for (int k = 0; k < PRE; k++) {
            const int fl = min(l_t * 64 + lane, max(nunits - 1, 0));
            Ops::load_flat(ring[k], W, f_base + fl);
            l_t += 16;
        }
    };
    auto consume = [&]() {
#pragma unroll
        for (int k = 0; k < PRE; k++) {
            if (c_t < nloads) {   // wave-uniform
                const int fl = c_t * 64 + lane;
                const bool act = fl < nunits;
                const int flc = act ? fl : nunits - 1;
                const int rl = (int)__umulhi((unsigned)flc, magic_u);   // flc / U: row within the workgroup
                const int u = flc - rl * U;
                const float t = unit_dot_flat(Ops(), ring[k], xs, hs, u);
                const float s = small_group_sum<GL>(act ? t : 0.f);
                if (act && (lane & (GL - 1)) == GL - 1) part[fl / GL] = s;
            }
            c_t += 16;
        }
    };
    // a long row's loads lead the memory queue: the waves meet once before the first weight request (gemv_body_flat has the
    // measurements; Q8_0 2560 x 9728 here 7.7 -> 7.2 us)
    if (nb32 >= 256) __builtin_amdgcn_s_barrier();
    request();
    if (hb < nb32 * 2) {
        float* dst = xs + (hb >> 1) * 36 + (hb & 1) * 16;
#pragma unroll
        for (int j = 0; j < 4; j++) *(float4*)(dst + 4 * j) = v[j];
        hs[hb] = ((v[0].x + v[0].y) + (v[0].z + v[0].w)) + ((v[1].x + v[1].y) + (v[1].z + v[1].w)) +
                 (((v[2].x + v[2].y) + (v[2].z + v[2].w)) + ((v[3].x + v[3].y) + (v[3].z + v[3].w)));
    }
    __syncthreads();
    consume();
    while (c_t < nloads) {
        request();
        consume();
    }
    __syncthreads();
    // a row's G group sums: 8 lanes take them in ascending order, then a fixed DPP tree
    const int G = U / GL;
    for (int i8 = threadIdx.x; i8 < (r1 - r0) * 8; i8 += 1024) {
        const int r = i8 >> 3, l = i8 & 7;
        float s = 0.f;
        for (int j = l; j < G; j += 8) s += part[r * G + j];
        s = small_group_sum<8>(s);
        if (l == 0) y[r0 + r] = s;
    }
}

// The flat form's geometry (as for the Q8-activation GEMV): whole further rounds of workgroups when a CU's share of
// the rows is too large for the 16-bit unit index or for LDS.  Returns false when the shape is not served.
struct F32Flat { int gl; unsigned grid, magic; size_t lds; };
static bool f32_flat_geom(const smx_ctx* c, const Weight& w, F32Flat& g) {
    const size_t upb = w.type == kQ6_K ? 4 : (w.type == kQ8_0 ? 2 : 1);
    const size_t units = w.nblk * upb, nb32 = w.K / 32;
    if (w.K > 16384 || units == 0) return false;
    g.gl = units % 16 == 0 ? 16 : (units % 8 == 0 ? 8 : (w.type == kQ6_K && units % 4 == 0 ? 4 : 0));
    if (!g.gl) return false;
    const size_t cus = (size_t)c->num_cu, xbytes = nb32 * (36 + 2) * 4;
    const size_t share = (w.N + cus - 1) / cus * units;
    size_t rounds = share < 65536 ? 1 : (share + 59999) / 60000;
    size_t fwgs, rows, lds;
    for (;; rounds++) {
        fwgs = std::min(w.N, cus * rounds);
        rows = (w.N + fwgs - 1) / fwgs;
        lds = xbytes + rows * units / g.gl * 4;
        if (lds <= 128 * 1024 || fwgs == w.N) break;
    }
    if (rows * units >= 65536 || lds > 160 * 1024) return false;
    g.grid = (unsigned)fwgs;
    g.lds = lds;
    g.magic = (unsigned)(((1ull << 32) + units - 1) / units);
    return true;
}

template <class Ops, int PRE>
static int launch_f32_flat(smx_ctx* c, const Weight& w, const float* x, float* y, const F32Flat& g) {
    const GemvW W = {w.scales, (const uint4*)w.quants, (const uint4*)w.qh, (const uint2*)w.sc};
    auto go = [&](auto kern) -> int {
        int rc = set_dyn_lds(c, kern, g.lds);
        if (rc != SMX_OK) return rc;
        hipLaunchKernelGGL(kern, dim3(g.grid), dim3(1024), g.lds, c->stream, W, x, y, (int)w.nblk, (int)w.N, (int)g.grid, g.magic);
        SMX_HIP(c, hipGetLastError());
        return SMX_OK;
    };
    if (g.gl == 16) return go(gemv_f32_flat_kernel<Ops, PRE, 16>);
    if (g.gl == 8) return go(gemv_f32_flat_kernel<Ops, PRE, 8>);
    if constexpr (std::is_same<Ops, OpsQ6_K>::value) {
        if (g.gl == 4) return go(gemv_f32_flat_kernel<Ops, PRE, 4>);
    }
    return fail(c, SMX_ERR_ARG, "gemv_f32: no flat variant for %d-unit groups", g.gl);
}

template <class Ops>
static int launch_f32_type(smx_ctx* c, const Weight& w, const float* x, float* y) {
    const GemvW W = {w.scales, (const uint4*)w.quants, (const uint4*)w.qh, (const uint2*)w.sc};
    const size_t lds = (w.K / 32) * 36 * 4;
    const size_t waves = (size_t)c->num_cu * 16;
    const int rpw = w.N >= waves * 4 ? 4 : (w.N >= waves * 2 ? 2 : 1);
    const size_t chunks = (w.N + rpw - 1) / rpw;
    const unsigned grid = (unsigned)std::min<size_t>((chunks + 15) / 16, (size_t)c->num_cu);
    auto go = [&](auto kern) -> int {
        int rc = set_dyn_lds(c, kern, lds);
        if (rc != SMX_OK) return rc;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(1024), lds, c->stream, W, x, y, (int)w.nblk, (int)w.N);
        SMX_HIP(c, hipGetLastError());
        return SMX_OK;
    };
    if (rpw == 4) return go(gemv_f32_kernel<Ops, 4>);
    if (rpw == 2) return go(gemv_f32_kernel<Ops, 2>);
    return go(gemv_f32_kernel<Ops, 1>);
}

int launch_gemv_f32(smx_ctx* c, const Weight& w, const float* x, float* y) {
    if (w.K > SMX_GEMV_F32_MAX_IN_DIM)
        return fail(c, SMX_ERR_LIMIT, "gemv_f32: in_dim %zu (the fp32 activation is staged in LDS: at most %d)", w.K,
                    SMX_GEMV_F32_MAX_IN_DIM);
    if (w.N > 0x7fffffffu / 4) return fail(c, SMX_ERR_LIMIT, "gemv_f32: %zu rows exceed the kernel's index range", w.N);
    F32Flat fg;
    const bool flat = f32_flat_geom(c, w, fg);
    if (w.type == kQ4_0) {
        ProfScope ps(c, "gemv_f32_q4_0");
        return flat ? launch_f32_flat<OpsQ4_0, 3>(c, w, x, y, fg) : launch_f32_type<OpsQ4_0>(c, w, x, y);
    }
    if (w.type == kQ8_0) {
        ProfScope ps(c, "gemv_f32_q8_0");
        return flat ? launch_f32_flat<OpsQ8_0, 3>(c, w, x, y, fg) : launch_f32_type<OpsQ8_0>(c, w, x, y);
    }
    ProfScope ps(c, "gemv_f32_q6_k");
    return flat ? launch_f32_flat<OpsQ6_K, 1>(c, w, x, y, fg) : launch_f32_type<OpsQ6_K>(c, w, x, y);
}

}  // namespace smx

using namespace smx;

extern "C" {

int smx_gemv_f32_dev(smx_ctx* c, const char* key, const float* x_dev, float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !x_dev || !y_dev) return fail(c, SMX_ERR_ARG, "gemv_f32_dev: null argument");
    return guarded(c, "gemv_f32_dev", [&]() -> int {
        auto it = c->weights.find(key);
        if (it == c->weights.end()) return SMX_NOT_RESIDENT;
        return launch_gemv_f32(c, it->second, x_dev, y_dev);
    });
}

int smx_gemv_f32(smx_ctx* c, const char* key, const float* x, size_t in_len, float* y, size_t out_cap) {
    if (!c) return SMX_ERR_ARG;
    if (!key) return fail(c, SMX_ERR_ARG, "gemv_f32: null key");
    return guarded(c, "gemv_f32", [&]() -> int {
        auto it = c->weights.find(key);
        if (it == c->weights.end()) return SMX_NOT_RESIDENT;
        const Weight& w = it->second;
        if (!x || !y) return fail(c, SMX_ERR_ARG, "gemv_f32: null argument");
        if (in_len != w.K) return fail(c, SMX_ERR_ARG, "gemv_f32: activation length %zu, weight in_dim %zu", in_len, w.K);
        if (out_cap < w.N) return fail(c, SMX_ERR_ARG, "gemv_f32: output capacity %zu < %zu", out_cap, w.N);
        SMX_HIP(c, hipSetDevice(c->device));
        int rc;
        const size_t xb = w.K * 4, yb = w.N * 4;
        if ((rc = ensure(c, c->xf32, xb)) != SMX_OK) return rc;
        if ((rc = ensure(c, c->yf32, yb)) != SMX_OK) return rc;
        if ((rc = ensure_host(c, c->hx, xb)) != SMX_OK) return rc;
        if ((rc = ensure_host(c, c->hy, yb)) != SMX_OK) return rc;
        std::memcpy(c->hx.p, x, xb);
        // the kernel reads the pinned staging and writes the pinned result itself (see smx_gemv)
        const bool x_direct = xb <= (size_t(64) << 10) && c->tune_host_io != 1 && c->tune_host_io != 2, y_direct = c->tune_host_io != 1;
        if (!x_direct) SMX_HIP(c, hipMemcpyAsync(c->xf32.p, c->hx.p, xb, hipMemcpyHostToDevice, c->stream));
        if ((rc = launch_gemv_f32(c, w, x_direct ? (const float*)c->hx.p : (const float*)c->xf32.p,
                                  y_direct ? (float*)c->hy.p : (float*)c->yf32.p)) != SMX_OK) return rc;
        if (!y_direct) SMX_HIP(c, hipMemcpyAsync(c->hy.p, c->yf32.p, yb, hipMemcpyDeviceToHost, c->stream));
        SMX_HIP(c, hipStreamSynchronize(c->stream));
        std::memcpy(y, c->hy.p, yb);
        return SMX_OK;
    });
}

}  // extern "C"
