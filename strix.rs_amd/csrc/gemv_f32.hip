// GEMV with fp32 activations: y = dequant(W) . x, the arithmetic of the reference's per-weight `gemv`
// (crates/strix-backend-rocm/src/kernels.rs:41-69 q4_gemv, :646-668 q8_0_gemv, :607-640 q6_gemv; launched
// by decode.rs:3827-3898) and of strix-backend-cpu (dequantise a row, f32 dot).  No activation
// quantiser, no integer dots: every weight is widened to fp32 in registers and multiplied with the
// fp32 activation staged in LDS.  The decode path proper is the Q8-activation GEMV (gemv.hip); this
// form serves callers that hold the accelerator to the CPU result at fp32 accuracy.
//
// Same memory side as the other GEMVs: planar weights streamed as 16-byte units, 16-wave workgroups,
// a wave serves RPW rows at a time with one load per row and lane in flight, DPP reduction per row.
// HBM-bound by bytes, VALU-bound in practice (about three operations per weight element).
#include <algorithm>
#include <cstring>

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
    if (w.type == kQ4_0) {
        ProfScope ps(c, "gemv_f32_q4_0");
        return launch_f32_type<OpsQ4_0>(c, w, x, y);
    }
    if (w.type == kQ8_0) {
        ProfScope ps(c, "gemv_f32_q8_0");
        return launch_f32_type<OpsQ8_0>(c, w, x, y);
    }
    ProfScope ps(c, "gemv_f32_q6_k");
    return launch_f32_type<OpsQ6_K>(c, w, x, y);
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
        SMX_HIP(c, hipMemcpyAsync(c->xf32.p, c->hx.p, xb, hipMemcpyHostToDevice, c->stream));
        if ((rc = launch_gemv_f32(c, w, (const float*)c->xf32.p, (float*)c->yf32.p)) != SMX_OK) return rc;
        SMX_HIP(c, hipMemcpyAsync(c->hy.p, c->yf32.p, yb, hipMemcpyDeviceToHost, c->stream));
        SMX_HIP(c, hipStreamSynchronize(c->stream));
        std::memcpy(y, c->hy.p, yb);
        return SMX_OK;
    });
}

}  // extern "C"
