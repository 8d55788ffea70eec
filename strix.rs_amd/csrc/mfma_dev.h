// Device helpers shared by the int8 matrix-core kernels (tiled GEMMs, small-batch matmul).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace smx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// An MFMA that accumulates onto MAGIC_I leaves 12582912 + I in every accumulator when its bits are
// read as a float (|I| < 2^22), so fl(dw * I) is one FMA with the exactly representable -dw * 12582912.
constexpr float MAGIC_F = 12582912.f;  // 1.5 * 2^23
constexpr int MAGIC_I = 0x4B400000;

__device__ __forceinline__ float h2f_(uint16_t h) { return __half2float(__ushort_as_half(h)); }
// four nibbles (one per byte) -> four signed bytes nibble - 8 (kernels.rs:458-462)
__device__ __forceinline__ unsigned sub8(unsigned x) { return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u; }

// 64 lanes x 16 bytes from global memory straight into LDS (no register round trip): lane i's
// bytes land at LDS byte address lds_base + 16 * i; lds_base is wave-uniform (M0).  Completion is
// counted by vmcnt.  Written as inline assembly so that the compiler's wait-count insertion does
// not put vmcnt(0) in front of every later LDS read (it cannot tell stage buffers apart); the
// kernels wait for the loads themselves before the barrier that publishes a stage.
__device__ __forceinline__ void load_to_lds16(const void* g, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(g)
                 : "memory", "m0");
}
// The same with a wave-uniform base pointer and a 32-bit per-lane byte offset (no 64-bit address arithmetic).
__device__ __forceinline__ void load_to_lds16(const void* sbase, unsigned voff, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)p;
}

// acc[I] += dx(token of accumulator I) * fl(dw * dot I).  In the 32x32 MFMA output, accumulator i of
// lane half h is token (i/4)*8 + h*4 + i%4, so the 16 activation scales a lane needs differ between the
// two halves; they are kept ONE per lane -- lane n of every 16-lane row holds the scale of accumulator n
// for that row's half -- and the multiply-add reads it through a row broadcast (DPP row_newbcast:n):
// one LDS dword and one register per lane and block instead of 16.
#define SMX_FMAC_BC(I)                                                                      \
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #I " row_mask:0xf bank_mask:0xf"        \
        : "+v"(accv[I])                                                                     \
        : "v"(dxv), "v"(t[I]))
__device__ __forceinline__ void scale_accumulate(float (&accv)[16], const v16i& dn, float dw, float ndw, float dxv) {
    float t[16];
#pragma unroll
    for (int i = 0; i < 16; i++) t[i] = fmaf(dw, __int_as_float(dn[i]), ndw);
    SMX_FMAC_BC(0); SMX_FMAC_BC(1); SMX_FMAC_BC(2); SMX_FMAC_BC(3); SMX_FMAC_BC(4); SMX_FMAC_BC(5); SMX_FMAC_BC(6);
    SMX_FMAC_BC(7); SMX_FMAC_BC(8); SMX_FMAC_BC(9); SMX_FMAC_BC(10); SMX_FMAC_BC(11); SMX_FMAC_BC(12);
    SMX_FMAC_BC(13); SMX_FMAC_BC(14); SMX_FMAC_BC(15);
}
#undef SMX_FMAC_BC

}  // namespace smx
