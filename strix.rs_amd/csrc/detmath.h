// Elementary functions as fixed sequences of IEEE fp32 operations (no FMA contraction), restated
// operation for operation by the CPU oracle, so that activations built from them quantise to the
// same int8 values on any conforming implementation.
#pragma once
#include <hip/hip_runtime.h>

namespace smx {

// exp() as a fixed sequence of IEEE fp32 operations (no contraction), so that the quantised
// silu(g)*u is reproducible bit for bit on any conforming implementation.
__device__ __forceinline__ float det_expf(float x) {
#pragma clang fp contract(off)
    x = x > 88.0f ? 88.0f : x;
    x = x < -87.0f ? -87.0f : x;
    const float n = rintf(x * 1.44269504088896341f);
    float r = x - n * 0.693359375f;
    r = r - n * -2.12194440e-4f;
    float p = 1.9875691500e-4f;
    p = p * r + 1.3981999507e-3f;
    p = p * r + 8.3334519073e-3f;
    p = p * r + 4.1665795894e-2f;
    p = p * r + 1.6666665459e-1f;
    p = p * r + 5.0000001201e-1f;
    const float r2 = r * r;
    p = p * r2;
    p = p + r;
    p = p + 1.0f;
    return ldexpf(p, (int)n);
}

// silu(x) = x / (1 + exp(-x)), crates/strix-backend-cpu/src/ops.rs:73-76
__device__ __forceinline__ float det_silu(float x) {
#pragma clang fp contract(off)
    return x / (1.0f + det_expf(-x));
}

// tanh(z) = 1 - 2/(exp(2z) + 1); saturates to +-1 through det_expf's clamps
__device__ __forceinline__ float det_tanhf(float z) {
#pragma clang fp contract(off)
    return 1.0f - 2.0f / (det_expf(2.0f * z) + 1.0f);
}

// 0.5*x*(1 + tanh(sqrt(2/pi)*(x + 0.044715 x^3))), crates/strix-backend-cpu/src/ops.rs:110-113,
// crates/strix-backend-rocm/src/kernels.rs:162-163
__device__ __forceinline__ float det_gelu_tanh(float x) {
#pragma clang fp contract(off)
    const float x3 = x * x * x;
    const float inner = 0.7978845608f * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + det_tanhf(inner));
}

// 1/sqrt(mean(x^2) + eps) of one row for the rmsnorm producer (kernels.rs:101-113).  The squares are
// summed in double by the whole workgroup (per thread, per wave, then over the waves in index order)
// and the scale is rounded to fp32 once, so it does not depend on the workgroup's shape.  `scratch`
// is LDS the caller has not written yet; every thread of the workgroup must call this.
__device__ __forceinline__ float rms_scale(char* scratch, const float* x, int n, float eps) {
#pragma clang fp contract(off)
    double ss = 0.0;
    for (int i = threadIdx.x; i < n / 4; i += blockDim.x) {
        const float4 v = ((const float4*)x)[i];
        ss += (double)v.x * (double)v.x;
        ss += (double)v.y * (double)v.y;
        ss += (double)v.z * (double)v.z;
        ss += (double)v.w * (double)v.w;
    }
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    double* red = (double*)scratch;
    const int nwaves = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    double tot = 0.0;
    for (int w = 0; w < nwaves; w++) tot += red[w];
    __syncthreads();  // the caller overwrites the scratch next
    return (float)(1.0 / sqrt(tot / (double)n + (double)eps));
}

}  // namespace smx
