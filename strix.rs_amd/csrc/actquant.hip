// Activation quantiser: fp32 rows -> per-32-block Q8 (int8 quants + f32 scale + 16-element sums).
//
// Arithmetic of the reference's device quantisers (crates/strix-backend-rocm/src/kernels.rs:75-96,
// 864-876, 1000-1013): d = amax/127, inv = d > 0 ? 1/d : 0, q = clamp(rint(x*inv), -127, 127).
// Layout differs: quants stay contiguous int8 [m][K]; the block sum the reference keeps per 32
// (kernels.rs:93) is kept as two 16-element sums packed in one dword, which also serves the
// 16-wide sub-blocks of Q6_K.
#include <algorithm>

#include "detmath.h"
#include "smx_internal.h"

namespace smx {

// Up to SMX_GEMV_GROUP_MAX rows, each the product of an activation function of one operand and a
// second operand (SwiGLU: silu(a) * b, GeGLU: gelu_tanh(a) * b; kernels.rs:151-226), quantised like
// actquant_kernel below.  Row j goes to xq + j*K, xd / xs + j*K/32.  The arithmetic is the one the
// GEMV staging performs when it runs the producer itself, operation for operation.
struct ProdRows {
    const float4* a[SMX_GEMV_GROUP_MAX];
    const float4* b[SMX_GEMV_GROUP_MAX];
};
__global__ __launch_bounds__(256) void actprod_quant_kernel(const ProdRows R, int kind, int* __restrict__ xq4,
                                                            float* __restrict__ xd, int* __restrict__ xs, int nb32) {
#pragma clang fp contract(off)
    const int j = blockIdx.y;
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int blk = gid >> 3;
    const bool live = blk < nb32;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f), g = v;
    if (live) {
        v = R.a[j][gid];
        g = R.b[j][gid];
    }
    float4 w;
    if (kind == SMX_ACT_SILU_MUL) {
        w.x = det_silu(v.x) * g.x; w.y = det_silu(v.y) * g.y; w.z = det_silu(v.z) * g.z; w.w = det_silu(v.w) * g.w;
    } else {
        w.x = det_gelu_tanh(v.x) * g.x; w.y = det_gelu_tanh(v.y) * g.y;
        w.z = det_gelu_tanh(v.z) * g.z; w.w = det_gelu_tanh(v.w) * g.w;
    }
    float a = fmaxf(fmaxf(fabsf(w.x), fabsf(w.y)), fmaxf(fabsf(w.z), fabsf(w.w)));
    a = fmaxf(a, __shfl_xor(a, 1));
    a = fmaxf(a, __shfl_xor(a, 2));
    a = fmaxf(a, __shfl_xor(a, 4));
    const float d = a / 127.f;
    const float inv = d > 0.f ? 1.f / d : 0.f;
    const int q0 = max(-127, min(127, (int)rintf(w.x * inv)));
    const int q1 = max(-127, min(127, (int)rintf(w.y * inv)));
    const int q2 = max(-127, min(127, (int)rintf(w.z * inv)));
    const int q3 = max(-127, min(127, (int)rintf(w.w * inv)));
    int s = q0 + q1 + q2 + q3;
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    const int other = __shfl_xor(s, 4);
    if (live) {
        xq4[(size_t)j * nb32 * 8 + gid] = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | ((q3 & 0xff) << 24);
        if ((gid & 7) == 0) {
            xd[(size_t)j * nb32 + blk] = d;
            xs[(size_t)j * nb32 + blk] = (s & 0xffff) | (other << 16);
        }
    }
}

// m rows through an activation producer and the quantiser: the prefill form of the producers (kernels.rs:101-147
// rmsnorm_xquant per row, :1174-1187 silu_quant_rows).  b: rmsnorm weight [K] (or null) shared by the rows
// (b_stride 0), or the second operand [m][K] of silu / gelu.  Workgroup (row, part) takes the 256-item slices
// part, part + gridDim.y, ... of its row: rmsnorm needs the whole row's sum of squares and runs one workgroup per
// row; the exp-based producers have independent blocks and spread a row over one workgroup per slice (a single
// workgroup per 9728-element row left 64 rows on 64 of the 256 CUs, ten exp-heavy rounds each).
__global__ __launch_bounds__(256) void rows_prod_quant_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                              size_t b_stride, int kind, float eps, int* __restrict__ xq4,
                                                              float* __restrict__ xd, int* __restrict__ xs, int nb32) {
#pragma clang fp contract(off)
    __shared__ double red[4];
    const size_t row = blockIdx.x;
    const float* ar = a + row * (size_t)nb32 * 32;
    const float* br = b ? b + row * b_stride : nullptr;
    float rs = 1.f;
    if (kind == SMX_ACT_RMSNORM) rs = rms_scale((char*)red, ar, nb32 * 32, eps);
    const int items = nb32 * 8;
    for (int i0 = blockIdx.y * 256; i0 < items; i0 += gridDim.y * 256) {  // whole 8-lane groups stay together: items % 8 == 0
        const int i = i0 + threadIdx.x;
        const bool live = i < items;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f), g = make_float4(1.f, 1.f, 1.f, 1.f);
        if (live) {
            v = ((const float4*)ar)[i];
            if (br) g = ((const float4*)br)[i];
        }
        float4 w;
        if (kind == SMX_ACT_RMSNORM) {
            w.x = (v.x * rs) * g.x; w.y = (v.y * rs) * g.y; w.z = (v.z * rs) * g.z; w.w = (v.w * rs) * g.w;
        } else if (kind == SMX_ACT_SILU_MUL) {
            w.x = det_silu(v.x) * g.x; w.y = det_silu(v.y) * g.y; w.z = det_silu(v.z) * g.z; w.w = det_silu(v.w) * g.w;
        } else {
            w.x = det_gelu_tanh(v.x) * g.x; w.y = det_gelu_tanh(v.y) * g.y;
            w.z = det_gelu_tanh(v.z) * g.z; w.w = det_gelu_tanh(v.w) * g.w;
        }
        float am = fmaxf(fmaxf(fabsf(w.x), fabsf(w.y)), fmaxf(fabsf(w.z), fabsf(w.w)));
        am = fmaxf(am, __shfl_xor(am, 1));
        am = fmaxf(am, __shfl_xor(am, 2));
        am = fmaxf(am, __shfl_xor(am, 4));
        const float d = am / 127.f;
        const float inv = d > 0.f ? 1.f / d : 0.f;
        const int q0 = max(-127, min(127, (int)rintf(w.x * inv)));
        const int q1 = max(-127, min(127, (int)rintf(w.y * inv)));
        const int q2 = max(-127, min(127, (int)rintf(w.z * inv)));
        const int q3 = max(-127, min(127, (int)rintf(w.w * inv)));
        int s = q0 + q1 + q2 + q3;
        s += __shfl_xor(s, 1);
        s += __shfl_xor(s, 2);
        const int other = __shfl_xor(s, 4);
        if (live) {
            xq4[row * (size_t)items + i] = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | ((q3 & 0xff) << 24);
            if ((i & 7) == 0) {
                xd[row * (size_t)nb32 + (i >> 3)] = d;
                xs[row * (size_t)nb32 + (i >> 3)] = (s & 0xffff) | (other << 16);
            }
        }
    }
}

int launch_rows_prod_quant(smx_ctx* c, int kind, const float* a, const float* b, size_t m, size_t K, float eps, int8_t* xq,
                           float* xd, int32_t* xs) {
    if (K % 32 != 0 || m == 0 || m > 0x7fffffffu) return fail(c, SMX_ERR_ARG, "producer quantiser: %zu rows of %zu", m, K);
    if (kind != SMX_ACT_RMSNORM && kind != SMX_ACT_SILU_MUL && kind != SMX_ACT_GEGLU)
        return fail(c, SMX_ERR_ARG, "producer quantiser: kind %d", kind);
    ProfScope ps(c, "rows_prod_quant");
    const unsigned parts = kind == SMX_ACT_RMSNORM ? 1u : (unsigned)std::min<size_t>((K / 4 + 255) / 256, 65535);
    hipLaunchKernelGGL(rows_prod_quant_kernel, dim3((unsigned)m, parts), dim3(256), 0, c->stream, a, b,
                       kind == SMX_ACT_RMSNORM ? (size_t)0 : K, kind, eps, (int*)xq, xd, (int*)xs, (int)(K / 32));
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

int launch_actprod_quant(smx_ctx* c, int kind, const float* const* as, const float* const* bs, int n, size_t K,
                         int8_t* xq, float* xd, int32_t* xs) {
    if (K % 32 != 0 || n < 1 || n > SMX_GEMV_GROUP_MAX) return fail(c, SMX_ERR_ARG, "producer quantiser: %d rows of %zu", n, K);
    if (kind != SMX_ACT_SILU_MUL && kind != SMX_ACT_GEGLU) return fail(c, SMX_ERR_ARG, "producer quantiser: kind %d", kind);
    ProdRows R = {};
    for (int j = 0; j < n; j++) {
        R.a[j] = (const float4*)as[j];
        R.b[j] = (const float4*)bs[j];
    }
    const int nb32 = (int)(K / 32);
    ProfScope ps(c, "actprod_quant");
    hipLaunchKernelGGL(actprod_quant_kernel, dim3((unsigned)((nb32 * 8 + 255) / 256), (unsigned)n), dim3(256), 0, c->stream, R,
                       kind, (int*)xq, xd, (int*)xs, nb32);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

// 8 lanes per 32-block, one float4 each: 128-bit loads, 32-bit packed stores.
__global__ __launch_bounds__(256) void actquant_kernel(const float4* __restrict__ x, int* __restrict__ xq4,
                                                       float* __restrict__ xd, int* __restrict__ xs,
                                                       size_t nblocks) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t blk = gid >> 3;
    const bool live = blk < nblocks;
    float4 v = live ? x[gid] : make_float4(0.f, 0.f, 0.f, 0.f);
    float a = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    a = fmaxf(a, __shfl_xor(a, 1));
    a = fmaxf(a, __shfl_xor(a, 2));
    a = fmaxf(a, __shfl_xor(a, 4));
    const float d = a / 127.f;
    const float inv = d > 0.f ? 1.f / d : 0.f;
    int q0 = max(-127, min(127, (int)rintf(v.x * inv)));
    int q1 = max(-127, min(127, (int)rintf(v.y * inv)));
    int q2 = max(-127, min(127, (int)rintf(v.z * inv)));
    int q3 = max(-127, min(127, (int)rintf(v.w * inv)));
    int s = q0 + q1 + q2 + q3;
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);                 // sum over this lane's 16-element half
    const int other = __shfl_xor(s, 4);    // the other half's sum
    if (live) {
        xq4[gid] = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | ((q3 & 0xff) << 24);
        if ((gid & 7) == 0) {
            xd[blk] = d;
            xs[blk] = (s & 0xffff) | (other << 16);
        }
    }
}

int launch_actquant(smx_ctx* c, const float* x, size_t m, size_t K, int8_t* xq, float* xd, int32_t* xs) {
    if (K % 32 != 0) return fail(c, SMX_ERR_ARG, "quantise: row length %zu is not a multiple of 32", K);
    const size_t nblocks = m * (K / 32);
    if (nblocks == 0) return SMX_OK;
    const size_t threads = nblocks * 8;
    const size_t grid = (threads + 255) / 256;
    if (grid > 0x7fffffffu) return fail(c, SMX_ERR_LIMIT, "quantise: %zu blocks exceed the grid limit", nblocks);
    ProfScope ps(c, "actquant");
    hipLaunchKernelGGL(actquant_kernel, dim3((unsigned)grid), dim3(256), 0, c->stream, (const float4*)x, (int*)xq,
                       xd, (int*)xs, nblocks);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

}  // namespace smx

extern "C" int smx_dev_copy(smx_ctx* c, void* dst, const void* src, size_t nbytes) {
    using namespace smx;
    if (!c) return SMX_ERR_ARG;
    if (!dst || !src || nbytes % 16 != 0 || ((uintptr_t)dst | (uintptr_t)src) % 16 != 0)
        return fail(c, SMX_ERR_ARG, "dev_copy: pointers and size must be 16-byte aligned");
    if (nbytes == 0) return SMX_OK;
    const size_t n16 = nbytes / 16;
    const unsigned grid = (unsigned)std::min<size_t>((n16 + 255) / 256, (size_t)c->num_cu * 32);
    ProfScope ps(c, "copy");
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, c->stream, (const uint4*)src, (uint4*)dst, n16);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}
