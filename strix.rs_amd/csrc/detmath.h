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

}  // namespace smx
