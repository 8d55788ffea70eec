// Device bodies of the fused block-dequant GEMV (shared by the dense and the MoE launches): the
// persistent form described next (gemv_body) and the flat form (gemv_body_flat, further down).
//
// One wavefront serves RPW consecutive output rows at a time ("chunk") and walks the rows in
// 64-lane passes; every lane streams one 16-byte unit of packed quants per row and pass:
//     Q4_0  unit = one 32-block   (16 B nibbles + f16 scale)
//     Q8_0  unit = half a block   (16 B int8; lanes 2i, 2i+1 share block i and its scale)
//     Q6_K  unit = 64 elements    (2 x 16 B ql + 16 B qh + 8 B sub-scales + f16 d; lanes 2i, 2i+1
//                                  hold the two 16-element halves of four 32-wide blocks)
// The (chunk, pass) items of a wave form one sequence that is software-pipelined PRE items deep:
// the first PRE items are requested before the activation is staged, and each consumed item's
// registers are refilled at once with the item PRE steps ahead, so HBM requests never wait for
// arithmetic.  Waves are persistent: chunk ids advance by the total number of waves.
//
// The activation is staged once per workgroup in LDS, either from pre-quantised int8 rows or,
// fused, straight from the fp32 rows through the path's quantiser (d = amax/127,
// q = clamp(rint(x/d)), crates/strix-backend-rocm/src/kernels.rs:75-96).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/strix_mi355.h"
#include "detmath.h"

namespace smx {

// Optional per-wave timeline stamps (development builds only; compiled out of the library).
#ifdef SMX_TRACE
extern __device__ unsigned long long* g_smx_trace;
#define SMX_STAMP_DECL unsigned long long smx_ts[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define SMX_STAMP(slot) smx_ts[slot] = wall_clock64()
#define SMX_STAMP_FLUSH()                                                                                 \
    do {                                                                                                  \
        if ((threadIdx.x & 63) == 0 && g_smx_trace) {                                                     \
            unsigned long long* o_ = g_smx_trace + ((size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 8; \
            for (int s_ = 0; s_ < 8; s_++) o_[s_] = smx_ts[s_];                                           \
        }                                                                                                 \
    } while (0)
#else
#define SMX_STAMP_DECL do { } while (0)
#define SMX_STAMP(slot) do { } while (0)
#define SMX_STAMP_FLUSH() do { } while (0)
#endif

__device__ __forceinline__ float h2f(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }
// value of the neighbouring lane (lane ^ 1)
__device__ __forceinline__ int swap1(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false); }

// Cross-lane moves on the DPP path (no LDS round trip).  CTRL: 0xB1 = lane^1, 0x4E = lane^2 (quad
// permutes), 0x141 = mirror within 8 lanes, 0x140 = mirror within a 16-lane row, 0x142 / 0x143 =
// broadcast of lane 15 / 31 into the following row(s).
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}

// Sum over groups of LPR (16, 32 or 64) adjacent lanes in a fixed order; the last lane of each group
// (lane % LPR == LPR - 1) ends up holding the group's total.
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);                         // all lanes of a 16-lane row hold the row's sum
    if (LPR >= 32) v += dpp_f<0x142, 0xa>(v);     // rows 1, 3 += rows 0, 2
    if (LPR == 64) v += dpp_f<0x143, 0xc>(v);     // rows 2, 3 += rows 0+1
    return v;
}

// The same moves for a double (both halves), and the sum over the 64 lanes of a wave in a fixed order: lane 63 ends up
// holding the total.  (__shfl_xor on a double is two LDS permutes per step, six steps one after the other.)
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_d(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)b, CTRL, ROW_MASK, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, ROW_MASK, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}
__device__ __forceinline__ double wave_sum_d(double v) {
    v += dpp_d<0xB1>(v);
    v += dpp_d<0x4E>(v);
    v += dpp_d<0x141>(v);
    v += dpp_d<0x140>(v);
    v += dpp_d<0x142, 0xa>(v);
    v += dpp_d<0x143, 0xc>(v);
    return v;
}

// Pointers of one resident weight (planar layout) and of the activation.
struct GemvW {
    const uint16_t* scales;  // Q4_0/Q8_0: f16 per block; Q6_K: f16 d per superblock
    const uint4* quants;     // Q4_0: 1 uint4/block; Q8_0: 2 uint4/block; Q6_K: ql, 8 uint4/superblock
    const uint4* qh;         // Q6_K: 4 uint4/superblock
    const uint2* sc;         // Q6_K: 2 uint2/superblock
};
struct GemvX {
    const float* x;      // fp32 rows [m][K] (fused quantiser) or null
    const int8_t* xq;    // pre-quantised rows [m][K]
    const float* xd;     // [m][K/32]
    const int* xs;       // [m][K/32] packed 16-element sums
    // activation producer applied to x before the fused quantiser (one row only):
    const float* x2;     // rmsnorm: weight or null; silu_mul / geglu: the `up` operand
    int prod;            // SMX_ACT_*
    float eps;           // rmsnorm
};

// ---------------------------------------------------------------------------------------------
// Per-format pieces.  `U` = units per row, `nb32` = 32-blocks per row.

struct OpsQ4_0 {
    struct Regs { uint4 q; uint16_t s; };
    static __device__ __forceinline__ int units_per_row(int nblk) { return nblk; }
    static __device__ __forceinline__ int nb32(int nblk) { return nblk; }
    static __device__ __forceinline__ int tok_bytes(int nblk) { return (nblk * 40 + 15) & ~15; }
    // LDS per token: lo[nb] uint4 | hi[nb] uint4 | {f32 d, i32 8*sum(q)}[nb]
    static __device__ __forceinline__ int* xq_dword(char* tok, int nblk, int blk, int sub) {
        uint4* lo = (uint4*)tok;
        return (int*)((sub < 4 ? lo : lo + nblk) + blk) + (sub & 3);
    }
    static __device__ __forceinline__ void put_scale(char* tok, int nblk, int blk, float d, int s_lo, int s_hi) {
        int2* p = (int2*)(tok + nblk * 32) + blk;
        *p = make_int2(__float_as_int(d), 8 * (s_lo + s_hi));
    }
    static constexpr bool kNeedsSums = true;
    static __device__ __forceinline__ void load(Regs& r, const GemvW& w, size_t row, int nblk, int u) {
        r.q = w.quants[row * nblk + u];
        r.s = w.scales[row * nblk + u];
    }
    // unit f of the flat [row][unit] sequence (rows are contiguous)
    static __device__ __forceinline__ void load_flat(Regs& r, const GemvW& w, size_t f) {
        r.q = w.quants[f];
        r.s = w.scales[f];
    }
    // move the planes b0 blocks further (to another expert of a stacked tensor)
    static __device__ __forceinline__ void advance(GemvW& w, size_t b0) {
        w.scales += b0;
        w.quants += b0;
    }
};

struct OpsQ8_0 {
    struct Regs { uint4 q; uint16_t s; };
    static __device__ __forceinline__ int units_per_row(int nblk) { return nblk * 2; }
    static __device__ __forceinline__ int nb32(int nblk) { return nblk; }
    static __device__ __forceinline__ int tok_bytes(int nblk) { return (nblk * 36 + 15) & ~15; }
    // LDS per token: xq[2nb] uint4 | sd[nb] f32
    static __device__ __forceinline__ int* xq_dword(char* tok, int, int blk, int sub) {
        return (int*)tok + blk * 8 + sub;
    }
    static __device__ __forceinline__ void put_scale(char* tok, int nblk, int blk, float d, int, int) {
        ((float*)(tok + nblk * 32))[blk] = d;
    }
    static constexpr bool kNeedsSums = false;
    static __device__ __forceinline__ void load(Regs& r, const GemvW& w, size_t row, int nblk, int u) {
        r.q = w.quants[row * nblk * 2 + u];
        r.s = w.scales[row * nblk + (u >> 1)];
    }
    static __device__ __forceinline__ void load_flat(Regs& r, const GemvW& w, size_t f) {
        r.q = w.quants[f];
        r.s = w.scales[f >> 1];   // two units per block, an even number of units per row
    }
    static __device__ __forceinline__ void advance(GemvW& w, size_t b0) {
        w.scales += b0;
        w.quants += b0 * 2;
    }
};

// Q8_0 with a whole 32-byte block per lane: used for several activation rows, where the per-row
// scale arithmetic and LDS scale read of a unit are paid once per block instead of once per half block.
struct OpsQ8_0W : OpsQ8_0 {
    struct Regs { uint4 q0, q1; uint16_t s; };
    static __device__ __forceinline__ int units_per_row(int nblk) { return nblk; }
    // LDS per token: first halves [nb] uint4 | second halves [nb] uint4 | sd[nb] f32 -- a lane reads both
    // halves of its block, and consecutive lanes read consecutive 16-byte chunks of a plane
    static __device__ __forceinline__ int* xq_dword(char* tok, int nblk, int blk, int sub) {
        uint4* lo = (uint4*)tok;
        return (int*)((sub < 4 ? lo : lo + nblk) + blk) + (sub & 3);
    }
    static __device__ __forceinline__ void load(Regs& r, const GemvW& w, size_t row, int nblk, int u) {
        r.q0 = w.quants[(row * nblk + u) * 2];
        r.q1 = w.quants[(row * nblk + u) * 2 + 1];
        r.s = w.scales[row * nblk + u];
    }
    static __device__ __forceinline__ void load_flat(Regs& r, const GemvW& w, size_t f) {
        r.q0 = w.quants[f * 2];
        r.q1 = w.quants[f * 2 + 1];
        r.s = w.scales[f];
    }
};

struct OpsQ6_K {
    struct Regs { uint4 a, b, h; uint2 sc; uint16_t d; };
    static __device__ __forceinline__ int units_per_row(int nsb) { return nsb * 4; }
    static __device__ __forceinline__ int nb32(int nsb) { return nsb * 8; }
    static constexpr int kPad = 10;  // 16-byte chunks per 128 elements in LDS (8 used)
    static __device__ __forceinline__ int tok_bytes(int nsb) { return nsb * 2 * (kPad * 16 + 16 + 16); }
    // LDS per token: xq 16-byte chunks, 8 per 128 elements padded to kPad (lanes 2g, 2g + 1 read chunks
    // kPad * g + 2j + {0, 1}: with 10, eight consecutive lanes fall into eight different 16-byte bank groups) |
    // sd float4[2nsb] | ss int4[2nsb]
    static __device__ __forceinline__ int* xq_dword(char* tok, int, int blk, int sub) {
        const int ci = blk * 2 + (sub >> 2);
        return (int*)((uint4*)tok + (ci >> 3) * kPad + (ci & 7)) + (sub & 3);
    }
    static __device__ __forceinline__ void put_scale(char* tok, int nsb, int blk, float d, int s_lo, int s_hi) {
        ((float*)(tok + nsb * 2 * kPad * 16))[blk] = d;
        ((int*)(tok + nsb * 2 * (kPad * 16 + 16)))[blk] = (s_lo & 0xffff) | (s_hi << 16);
    }
    static constexpr bool kNeedsSums = true;
    static __device__ __forceinline__ void load(Regs& r, const GemvW& w, size_t row, int nsb, int u) {
        const size_t sb0 = row * nsb;
        r.a = w.quants[sb0 * 8 + (u >> 1) * 4 + (u & 1)];
        r.b = w.quants[sb0 * 8 + (u >> 1) * 4 + (u & 1) + 2];
        r.h = w.qh[sb0 * 4 + u];
        r.sc = w.sc[sb0 * 2 + (u >> 1)];
        r.d = w.scales[sb0 + (u >> 2)];
    }
    // unit f of the flat [row][unit] sequence: four units per superblock, superblocks contiguous
    static __device__ __forceinline__ void load_flat(Regs& r, const GemvW& w, size_t f) {
        const size_t q = (f >> 2) * 8 + ((f & 3) >> 1) * 4 + (f & 1);
        r.a = w.quants[q];
        r.b = w.quants[q + 2];
        r.h = w.qh[f];
        r.sc = w.sc[f >> 1];
        r.d = w.scales[f >> 2];
    }
    static __device__ __forceinline__ void advance(GemvW& w, size_t sb0) {
        w.scales += sb0;
        w.quants += sb0 * 8;
        w.qh += sb0 * 4;
        w.sc += sb0 * 2;
    }
};

// Q4_0: whole-block i32 = sum(nibble*xq) - 8*sum(xq)  (kernels.rs:241-250), then (dw*dx)*float(isum)
template <int MT, bool DUMP>
__device__ __forceinline__ void compute_unit(OpsQ4_0, const OpsQ4_0::Regs& r, const char* smem, int tokb, int nblk,
                                             int u, bool act, float* acc, int* dump_row) {
    unsigned lo4[4], hi4[4];
    const unsigned w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int g = 0; g < 4; g++) {
        lo4[g] = w[g] & 0x0f0f0f0fu;         // elements 4g..4g+3
        hi4[g] = (w[g] >> 4) & 0x0f0f0f0fu;  // elements 16+4g..
    }
    const float dw = act ? h2f(r.s) : 0.f;
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const char* tok = smem + t * tokb;
        const uint4 xl = ((const uint4*)tok)[u], xh = ((const uint4*)tok)[nblk + u];
        const int2 ds = ((const int2*)(tok + nblk * 32))[u];
        const float dx = __int_as_float(ds.x);
        int isum = 0;
        isum = dot4((int)lo4[0], (int)xl.x, isum);
        isum = dot4((int)hi4[0], (int)xh.x, isum);
        isum = dot4((int)lo4[1], (int)xl.y, isum);
        isum = dot4((int)hi4[1], (int)xh.y, isum);
        isum = dot4((int)lo4[2], (int)xl.z, isum);
        isum = dot4((int)hi4[2], (int)xh.z, isum);
        isum = dot4((int)lo4[3], (int)xl.w, isum);
        isum = dot4((int)hi4[3], (int)xh.w, isum);
        isum -= ds.y;  // sum((q-8)x) = sum(qx) - 8 sum(x)
        if (DUMP) {
            if (act && t == 0 && dump_row) dump_row[u] = isum;
        }
        acc[t] += (dw * dx) * (float)isum;
    }
}

// Q8_0: the two half-block lanes add their i32 halves (DPP), the even lane carries the block
template <int MT, bool DUMP>
__device__ __forceinline__ void compute_unit(OpsQ8_0, const OpsQ8_0::Regs& r, const char* smem, int tokb, int nblk,
                                             int u, bool act, float* acc, int* dump_row) {
    const float dw = (act && !(u & 1)) ? h2f(r.s) : 0.f;
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const char* tok = smem + t * tokb;
        const uint4 xv = ((const uint4*)tok)[u];
        const float dx = ((const float*)(tok + nblk * 32))[u >> 1];
        int isum = dot4((int)r.q.x, (int)xv.x, 0);
        isum = dot4((int)r.q.y, (int)xv.y, isum);
        isum = dot4((int)r.q.z, (int)xv.z, isum);
        isum = dot4((int)r.q.w, (int)xv.w, isum);
        isum += swap1(isum);  // whole-block i32
        if (DUMP) {
            if (act && !(u & 1) && t == 0 && dump_row) dump_row[u >> 1] = isum;
        }
        acc[t] += (dw * dx) * (float)isum;
    }
}

template <int MT, bool DUMP>
__device__ __forceinline__ void compute_unit(OpsQ8_0W, const OpsQ8_0W::Regs& r, const char* smem, int tokb, int nblk,
                                             int u, bool act, float* acc, int* dump_row) {
    const float dw = act ? h2f(r.s) : 0.f;
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const char* tok = smem + t * tokb;
        const uint4 x0 = ((const uint4*)tok)[u], x1 = ((const uint4*)tok)[nblk + u];
        const float dx = ((const float*)(tok + nblk * 32))[u];
        int isum = dot4((int)r.q0.x, (int)x0.x, 0);
        isum = dot4((int)r.q0.y, (int)x0.y, isum);
        isum = dot4((int)r.q0.z, (int)x0.z, isum);
        isum = dot4((int)r.q0.w, (int)x0.w, isum);
        isum = dot4((int)r.q1.x, (int)x1.x, isum);
        isum = dot4((int)r.q1.y, (int)x1.y, isum);
        isum = dot4((int)r.q1.z, (int)x1.z, isum);
        isum = dot4((int)r.q1.w, (int)x1.w, isum);
        if (DUMP) {
            if (act && t == 0 && dump_row) dump_row[u] = isum;
        }
        acc[t] += (dw * dx) * (float)isum;
    }
}

// Q6_K: four 16-element sub-block dots per lane (sub-blocks 8h + 2j + c of the superblock, element
// map crates/strix-models/src/ggml_quant.rs:417-426); t_j = sc*isum summed over the lane pair is the
// scaled i32 of 32-block 4h + j; acc += (d*dx_j)*float(t_j).
template <int MT, bool DUMP>
__device__ __forceinline__ void compute_unit(OpsQ6_K, const OpsQ6_K::Regs& r, const char* smem, int tokb, int nsb,
                                             int u, bool act, float* acc, int* dump_row) {
    const int g = u >> 1, c = u & 1;
    const unsigned a4[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
    const unsigned b4[4] = {r.b.x, r.b.y, r.b.z, r.b.w};
    const unsigned h4[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
    unsigned q[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        q[0][i] = (a4[i] & 0x0f0f0f0fu) | ((h4[i] << 4) & 0x30303030u);
        q[1][i] = (b4[i] & 0x0f0f0f0fu) | ((h4[i] << 2) & 0x30303030u);
        q[2][i] = ((a4[i] >> 4) & 0x0f0f0f0fu) | (h4[i] & 0x30303030u);
        q[3][i] = ((b4[i] >> 4) & 0x0f0f0f0fu) | ((h4[i] >> 2) & 0x30303030u);
    }
    const float d = (act && c == 0) ? h2f(r.d) : 0.f;  // even lane carries the 32-blocks
    const unsigned long long scw = ((unsigned long long)r.sc.y << 32) | r.sc.x;
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const char* tok = smem + t * tokb;
        const uint4* sq = (const uint4*)tok;
        const float4 dx4 = ((const float4*)(tok + nsb * 2 * OpsQ6_K::kPad * 16))[g];
        const int4 sp4 = ((const int4*)(tok + nsb * 2 * (OpsQ6_K::kPad * 16 + 16)))[g];
        const float dxs[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
        const int sps[4] = {sp4.x, sp4.y, sp4.z, sp4.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint4 xv = sq[g * OpsQ6_K::kPad + 2 * j + c];
            int is = dot4((int)q[j][0], (int)xv.x, 0);
            is = dot4((int)q[j][1], (int)xv.y, is);
            is = dot4((int)q[j][2], (int)xv.z, is);
            is = dot4((int)q[j][3], (int)xv.w, is);
            const int xs16 = c ? (sps[j] >> 16) : (int)(short)(sps[j] & 0xffff);
            const int isum = is - 32 * xs16;  // sum((q-32)x) = sum(qx) - 32 sum(x)
            if (DUMP) {
                if (act && t == 0 && dump_row) dump_row[(u >> 2) * 16 + ((u >> 1) & 1) * 8 + 2 * j + c] = isum;
            }
            const int s8 = (int)(signed char)((scw >> (8 * (2 * j + c))) & 0xff);
            int tj = s8 * isum;
            tj += swap1(tj);
            acc[t] += (d * dxs[j]) * (float)tj;
        }
    }
}

// One item of an activation row on its way into LDS: 8 lanes share a 32-block, each holds one float4
// (fused quantiser) or one packed dword (pre-quantised row); reductions inside the 8 lanes go over DPP.
// With the quantiser fused, an activation producer (X.prod: rmsnorm(x)*x2, silu(x)*x2, gelu_tanh(x)*x2;
// kernels.rs:101-226) runs on the values first.  Whole 8-lane groups are live or not together.
// FQ: 0 the row is pre-quantised, 1 fp32 row quantised here, 2 the same behind an activation producer.
template <class Ops, int FQ>
__device__ __forceinline__ void stage_item(char* tok, int nblk, const GemvX& X, int t, int i, bool live, bool zero,
                                           float4 w, float4 g, int packed, float rs) {
    const int nb32 = Ops::nb32(nblk);
    const int blk = i >> 3, sub = i & 7;
    int s_lo = 0, s_hi = 0;
    float d = 0.f;
    if (FQ != 0) {
        if (FQ == 2 && X.prod != SMX_ACT_NONE) {
#pragma clang fp contract(off)
            if (X.prod == SMX_ACT_RMSNORM) {
                w.x = (w.x * rs) * g.x; w.y = (w.y * rs) * g.y; w.z = (w.z * rs) * g.z; w.w = (w.w * rs) * g.w;
            } else if (X.prod == SMX_ACT_SILU_MUL) {
                w.x = det_silu(w.x) * g.x; w.y = det_silu(w.y) * g.y; w.z = det_silu(w.z) * g.z; w.w = det_silu(w.w) * g.w;
            } else {
                w.x = det_gelu_tanh(w.x) * g.x; w.y = det_gelu_tanh(w.y) * g.y;
                w.z = det_gelu_tanh(w.z) * g.z; w.w = det_gelu_tanh(w.w) * g.w;
            }
        }
        float a = fmaxf(fmaxf(fabsf(w.x), fabsf(w.y)), fmaxf(fabsf(w.z), fabsf(w.w)));
        a = fmaxf(a, dpp_f<0xB1>(a));
        a = fmaxf(a, dpp_f<0x4E>(a));
        a = fmaxf(a, dpp_f<0x141>(a));
        d = a / 127.f;
        const float inv = d > 0.f ? 1.f / d : 0.f;
        const int q0 = max(-127, min(127, (int)rintf(w.x * inv)));
        const int q1 = max(-127, min(127, (int)rintf(w.y * inv)));
        const int q2 = max(-127, min(127, (int)rintf(w.z * inv)));
        const int q3 = max(-127, min(127, (int)rintf(w.w * inv)));
        packed = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | ((q3 & 0xff) << 24);
        if (Ops::kNeedsSums) {
            int s = q0 + q1 + q2 + q3;
            s += dpp_i<0xB1>(s);
            s += dpp_i<0x4E>(s);          // sum over this lane's 16-element half
            s_lo = s;
            s_hi = dpp_i<0x141>(s);       // the other half's sum (valid in lanes 0..3 of the group)
        }
    } else if (live && !zero && sub == 0) {
        d = X.xd[(size_t)t * nb32 + blk];
        if (Ops::kNeedsSums) {
            const int sp = X.xs[(size_t)t * nb32 + blk];
            s_lo = (int)(short)(sp & 0xffff);
            s_hi = sp >> 16;
        }
    }
    if (live) {
        *Ops::xq_dword(tok, nblk, blk, sub) = packed;
        if (sub == 0) Ops::put_scale(tok, nblk, blk, d, s_lo, s_hi);
    }
}

// Stage one activation row into LDS (stage_item over the row, two items per thread in flight).
template <class Ops, int FQ>
__device__ __forceinline__ void stage_token(char* tok, int nblk, const GemvX& X, int t, bool zero) {
    const int nb32 = Ops::nb32(nblk);
    const int items = nb32 * 8;
    constexpr int SB = 2;  // items per thread requested before any is consumed
    float rs = 1.f;
    constexpr bool FUSEQ = FQ != 0;
    if (FQ == 2 && X.prod == SMX_ACT_RMSNORM) rs = rms_scale(tok, X.x + (size_t)t * nb32 * 32, nb32 * 32, X.eps);
    for (int i0 = threadIdx.x; i0 < items; i0 += blockDim.x * SB) {
        float4 v[SB], v2[SB];
        int pk[SB];
#pragma unroll
        for (int j = 0; j < SB; j++) {
            const int i = i0 + j * blockDim.x;
            const bool live = i < items && !zero;
            v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            v2[j] = make_float4(1.f, 1.f, 1.f, 1.f);
            pk[j] = 0;
            if (FUSEQ) {
                if (live) {
                    v[j] = ((const float4*)(X.x + (size_t)t * nb32 * 32))[i];
                    if (FQ == 2 && X.x2) v2[j] = ((const float4*)(X.x2 + (size_t)t * nb32 * 32))[i];
                }
            } else {
                if (live) pk[j] = ((const int*)(X.xq + (size_t)t * nb32 * 32))[i];
            }
        }
#pragma unroll
        for (int j = 0; j < SB; j++) {
            const int i = i0 + j * blockDim.x;
            stage_item<Ops, FQ>(tok, nblk, X, t, i, i < items, zero, v[j], v2[j], pk[j], rs);
        }
    }
}

// Stage m pre-quantised activation rows, 16 bytes (half a block) per thread and load: every global
// load of all rows is requested before the first LDS write, so the staging costs one memory round
// trip, not one per row.  All formats keep a block's two 16-byte halves whole in LDS (xq_dword(.., 0)
// and (.., 4) are 16-byte aligned), so a half moves as one 128-bit load and one 128-bit store.
template <class Ops, int MT>
__device__ __forceinline__ void stage_prequant_all(char* smem, int tokb, int nblk, const GemvX& X, int m) {
    const int nb32 = Ops::nb32(nblk);
    const int items = nb32 * 2;
    for (int i = threadIdx.x; i < items; i += blockDim.x) {
        uint4 pk[MT];
        int sp[MT];
        float d[MT];
        const bool head = (i & 1) == 0;
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const bool live = t < m;
            pk[t] = live ? ((const uint4*)(X.xq + (size_t)t * nb32 * 32))[i] : make_uint4(0, 0, 0, 0);
            d[t] = (live && head) ? X.xd[(size_t)t * nb32 + (i >> 1)] : 0.f;
            sp[t] = (live && head && Ops::kNeedsSums) ? X.xs[(size_t)t * nb32 + (i >> 1)] : 0;
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            char* tok = smem + t * tokb;
            *(uint4*)Ops::xq_dword(tok, nblk, i >> 1, (i & 1) * 4) = pk[t];
            if (head) Ops::put_scale(tok, nblk, i >> 1, d[t], (int)(short)(sp[t] & 0xffff), sp[t] >> 16);
        }
    }
}

// The GEMV proper.  rows [0, N) of weight W against m <= MT activation rows; y[t*ldy + row].
//
// Lane mapping: LPR (16, 32 or 64) lanes walk one row, so a wave serves RS = 64/LPR rows side by
// side ("slot") and RPW slots per chunk; a row of U units takes ceil(U/LPR) passes.  LPR is chosen
// by the launcher to waste the fewest lanes (80-unit rows: LPR 16, five full passes for four rows).
// `wave_id` / `n_waves`: this wave's index among all waves sharing the row range, and their number.
// KS adjacent waves (same workgroup) form a group that shares each chunk: wave j of the group takes
// passes j, j+KS, ...; with KS > 1 every group owns at most one chunk (the launcher guarantees
// nchunks <= n_waves / KS) and the KS partial sums meet in LDS behind the staged activation.
template <class Ops, int MT, int RPW, int PRE, int KS, int LPR, int FQ, bool DUMP>
__device__ __forceinline__ void gemv_body(const GemvW W, const GemvX X, float* __restrict__ y, int ldy, int nblk, int N,
                                          int m, int* __restrict__ dump, int dump_per_row, int wave_id, int n_waves) {
    extern __shared__ __align__(16) char smem[];
    SMX_STAMP_DECL;
    SMX_STAMP(0);
    constexpr int RS = 64 / LPR;                 // rows side by side in a wave
    constexpr int RC = RPW * RS;                 // rows per chunk
    const int lane = threadIdx.x & 63;
    const int sub = lane & (LPR - 1), rsub = lane / LPR;
    const int U = Ops::units_per_row(nblk);
    const int P = (U + LPR - 1) / LPR;           // passes per chunk
    const int nchunks = (N + RC - 1) / RC;
    const int group = KS == 1 ? wave_id : wave_id / KS, ks = KS == 1 ? 0 : wave_id % KS;
    const int n_groups = KS == 1 ? n_waves : n_waves / KS;
    const int tokb = Ops::tok_bytes(nblk);

    typename Ops::Regs ring[PRE][RPW];
    // loader cursor (runs PRE items ahead of the consumer)
    int l_chunk = group, l_pass = ks;
    if (KS > 1 && l_pass >= P) l_chunk = nchunks;  // more waves in the group than passes
    auto issue = [&](int slot) {
        const int u = min(l_pass * LPR + sub, U - 1);
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const size_t row = (size_t)min(l_chunk * RC + r * RS + rsub, N - 1);
            Ops::load(ring[slot][r], W, row, nblk, u);
        }
        l_pass += KS;
        if (l_pass >= P) {
            l_pass = ks;
            l_chunk += n_groups;
        }
    };
#pragma unroll
    for (int k = 0; k < PRE; k++)
        if (l_chunk < nchunks) issue(k);
    SMX_STAMP(1);

    if (FQ != 0) {
        for (int t = 0; t < MT; t++) stage_token<Ops, FQ>(smem + t * tokb, nblk, X, t, t >= m);
    } else {
        stage_prequant_all<Ops, MT>(smem, tokb, nblk, X, m);
    }
    SMX_STAMP(2);
    __syncthreads();
    SMX_STAMP(3);

    float acc[RPW][MT];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[r][t] = 0.f;
    int c_chunk = group, c_pass = ks;
    if (KS > 1 && c_pass >= P) c_chunk = nchunks;
    float* part = (float*)(smem + MT * tokb);  // [waves of the workgroup][RC][MT], KS > 1 only
    const int wave_in_wg = threadIdx.x >> 6;
    while (c_chunk < nchunks) {
#pragma unroll
        for (int k = 0; k < PRE; k++) {
            if (c_chunk < nchunks) {
                const int uu = c_pass * LPR + sub;
                const bool act = uu < U;
                const int u = act ? uu : U - 1;
#pragma unroll
                for (int r = 0; r < RPW; r++) {
                    const int row = c_chunk * RC + r * RS + rsub;
                    int* drow = (DUMP && row < N) ? dump + (size_t)row * dump_per_row : nullptr;
                    compute_unit<MT, DUMP>(Ops(), ring[k][r], smem, tokb, nblk, u, act, acc[r], drow);
                }
                if (l_chunk < nchunks) issue(k);
                if (k == 0) SMX_STAMP(4);
                c_pass += KS;
                if (c_pass >= P) {
#pragma unroll
                    for (int r = 0; r < RPW; r++)
#pragma unroll
                        for (int t = 0; t < MT; t++) {
                            const float s = group_sum<LPR>(acc[r][t]);
                            const int row = c_chunk * RC + r * RS + rsub;
                            if (sub == LPR - 1) {  // the lane holding the group's total
                                if (KS == 1) {
                                    if (row < N && t < m) y[(size_t)t * ldy + row] = s;
                                } else {
                                    part[wave_in_wg * (RC * MT) + (r * RS + rsub) * MT + t] = s;
                                }
                            }
                            acc[r][t] = 0.f;
                        }
                    c_pass = ks;
                    c_chunk += n_groups;
                }
            }
        }
    }
    if (KS > 1) {
        __syncthreads();
        // the group's first wave adds the KS partials in slice order
        if (ks == 0 && group < nchunks && lane < RC * MT) {
            const int rr = lane / MT, t = lane % MT;
            const int row = group * RC + rr;
            float s = 0.f;
            for (int j = 0; j < KS && j < P; j++) s += part[(wave_in_wg + j) * (RC * MT) + lane];
            if (row < N && t < m) y[(size_t)t * ldy + row] = s;
        }
    }
    SMX_STAMP(5);
    SMX_STAMP_FLUSH();
}

// Sum over groups of GL = 2, 4, 8 or 16 adjacent lanes (all lanes of a group end up with the total).
template <int GL>
__device__ __forceinline__ float small_group_sum(float v) {
    v += dpp_f<0xB1>(v);
    if (GL >= 4) v += dpp_f<0x4E>(v);
    if (GL >= 8) v += dpp_f<0x141>(v);
    if (GL >= 16) v += dpp_f<0x140>(v);
    return v;
}

// One half block (16 fp32 values in v[0..3]) of an activation row on its way into LDS, as item `hb` of the row at `tok`
// (hb / 2 = block, hb % 2 = half): d = amax / 127 over the block (the other half sits in the neighbouring lane),
// q = rint(x / d) (kernels.rs:75-96).  Whole lane pairs are live or not together; every lane of the wave calls this.
template <class Ops>
__device__ __forceinline__ void quantize_half_block(char* tok, int nblk, int hb, bool live, const float4 (&v)[4]) {
    const float f[16] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w,
                         v[2].x, v[2].y, v[2].z, v[2].w, v[3].x, v[3].y, v[3].z, v[3].w};
    float a = 0.f;
#pragma unroll
    for (int k = 0; k < 16; k++) a = fmaxf(a, fabsf(f[k]));
    a = fmaxf(a, dpp_f<0xB1>(a));   // the block's other half: the neighbouring lane
    const float d = a / 127.f;
    const float inv = d > 0.f ? 1.f / d : 0.f;
    unsigned pkw[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        unsigned pk = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) pk |= (unsigned)(max(-127, min(127, (int)rintf(f[4 * w + k] * inv))) & 0xff) << (8 * k);
        pkw[w] = pk;
    }
    int s_half = 0;
    if (Ops::kNeedsSums) {
#pragma unroll
        for (int w = 0; w < 4; w++) s_half = dot4((int)pkw[w], 0x01010101, s_half);
    }
    const int s_other = Ops::kNeedsSums ? dpp_i<0xB1>(s_half) : 0;
    if (live) {
        *(uint4*)Ops::xq_dword(tok, nblk, hb >> 1, (hb & 1) * 4) = make_uint4(pkw[0], pkw[1], pkw[2], pkw[3]);
        if ((hb & 1) == 0) Ops::put_scale(tok, nblk, hb >> 1, d, s_half, s_other);
    }
}

// The activation row of the flat form: every global load is requested up front (before the weight
// stream, so that waiting for the row does not wait for the weights: a wave's loads complete in
// order), the values are quantised and written to LDS later.  Thread t holds items t, t + 1024, ...
// Holds rows of up to 16384 elements (the launcher's bound for this form).
template <class Ops, int FQ>
struct FlatX {
    static constexpr int XI = FQ == 0 ? 2 : 4;
    float4 v[XI], v2[XI];
    uint4 pk[XI];
    float d[XI];
    int sp[XI];

    // FQ == 1: a thread takes a whole half block (16 values), so that the per-block part of the quantiser (two
    // divisions, the 16-element sums, the scale's LDS write) runs once per 2 lanes instead of once per 8: with
    // one float4 per thread the staging held every CU for 1 us before it could touch its weights on a
    // 9728-element row, and Q6_K 15360 x 3840 ran 0.6 us longer.  Same arithmetic per element, same results.
    // rmsnorm in front of the quantiser (FQ == 2) uses the same mapping; the exp-based producers keep one float4 per thread
    // (their per-element work is what counts, and it spreads over four times as many threads).
    static __device__ __forceinline__ bool wide(const GemvX& X) { return FQ == 1 || (FQ == 2 && X.prod == SMX_ACT_RMSNORM); }

    __device__ __forceinline__ void request(const GemvX& X, int nblk) {
        const int nb32 = Ops::nb32(nblk);
        const int items = FQ == 0 ? nb32 * 2 : nb32 * 8;
        if (wide(X)) {
            const int i = threadIdx.x;   // half block
#pragma unroll
            for (int j = 0; j < XI; j++) {
                v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                v2[j] = make_float4(1.f, 1.f, 1.f, 1.f);
                if (i < nb32 * 2) {
                    v[j] = ((const float4*)X.x)[i * 4 + j];
                    if (FQ == 2 && X.x2) v2[j] = ((const float4*)X.x2)[i * 4 + j];
                }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < XI; j++) {
            const int i = threadIdx.x + j * 1024;
            v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            v2[j] = make_float4(1.f, 1.f, 1.f, 1.f);
            pk[j] = make_uint4(0, 0, 0, 0);
            d[j] = 0.f;
            sp[j] = 0;
            if (i < items) {
                if (FQ == 0) {
                    pk[j] = ((const uint4*)X.xq)[i];
                    if ((i & 1) == 0) {
                        d[j] = X.xd[i >> 1];
                        if (Ops::kNeedsSums) sp[j] = X.xs[i >> 1];
                    }
                } else {
                    v[j] = ((const float4*)X.x)[i];
                    if (FQ == 2 && X.x2) v2[j] = ((const float4*)X.x2)[i];
                }
            }
        }
    }

    // `tok`: the row's LDS area (the rmsnorm reduction's scratch are the 128 bytes behind it); every thread of the
    // 1024-thread workgroup calls this.
    __device__ __forceinline__ void store(char* tok, int nblk, const GemvX& X) {
        const int nb32 = Ops::nb32(nblk);
        if (FQ == 0) {
#pragma unroll
            for (int j = 0; j < XI; j++) {
                const int i = threadIdx.x + j * 1024;
                if (i < nb32 * 2) {
                    *(uint4*)Ops::xq_dword(tok, nblk, i >> 1, (i & 1) * 4) = pk[j];
                    if ((i & 1) == 0) Ops::put_scale(tok, nblk, i >> 1, d[j], (int)(short)(sp[j] & 0xffff), sp[j] >> 16);
                }
            }
            return;
        }
        if constexpr (FQ == 1) {
            const int i = threadIdx.x;
            if ((i & ~63) >= nb32 * 2) return;   // whole waves
            quantize_half_block<Ops>(tok, nblk, i, i < nb32 * 2, v);
            return;
        }
        if constexpr (FQ == 2) {
            if (X.prod == SMX_ACT_RMSNORM) {   // workgroup-uniform
#pragma clang fp contract(off)
                const int i = threadIdx.x;
                // mean of squares in double over the values already in registers (threads past the row hold zeros), rounded to
                // fp32 once: independent of the summation order
                double ss = 0.0;
#pragma unroll
                for (int j = 0; j < XI; j++) {
                    ss += (double)v[j].x * (double)v[j].x;
                    ss += (double)v[j].y * (double)v[j].y;
                    ss += (double)v[j].z * (double)v[j].z;
                    ss += (double)v[j].w * (double)v[j].w;
                }
                ss = wave_sum_d(ss);
                // the sixteen wave sums meet behind the row's own LDS area (where the group sums go once the weights are
                // consumed): nothing the quantiser writes below touches them, so one barrier is enough
                double* red = (double*)(tok + Ops::tok_bytes(nblk));
                if ((i & 63) == 63) red[i >> 6] = ss;
                __syncthreads();
                double tot = 0.0;
                for (int w = 0; w < 16; w++) tot += red[w];
                const float rs = (float)(1.0 / sqrt(tot / (double)(nb32 * 32) + (double)X.eps));
                if ((i & ~63) >= nb32 * 2) return;   // whole waves
                float4 w4[4];
#pragma unroll
                for (int j = 0; j < XI; j++)
                    w4[j] = make_float4((v[j].x * rs) * v2[j].x, (v[j].y * rs) * v2[j].y, (v[j].z * rs) * v2[j].z, (v[j].w * rs) * v2[j].w);
                quantize_half_block<Ops>(tok, nblk, i, i < nb32 * 2, w4);
                return;
            }
        }
        const int items = nb32 * 8;
        const float rs = 1.f;   // (rmsnorm is handled above)
#pragma unroll
        for (int j = 0; j < XI; j++) {
            const int i = threadIdx.x + j * 1024;
            // whole waves are live or not together (items is a multiple of 8, i of a wave spans 64)
            if ((i & ~63) < items) stage_item<Ops, FQ>(tok, nblk, X, 0, i, i < items, false, v[j], v2[j], 0, rs);
        }
    }
};

// The same for m <= MT pre-quantised rows (several activation rows per weight pass): one 16-byte
// half block per row and thread, rows of up to 16384 elements.
template <class Ops, int MT>
struct FlatXRows {
    uint4 pk[MT];
    float d[MT];
    int sp[MT];

    __device__ __forceinline__ void request(const GemvX& X, int nblk, int m) {
        const int nb32 = Ops::nb32(nblk);
        const int i = threadIdx.x;
#pragma unroll
        for (int t = 0; t < MT; t++) {
            pk[t] = make_uint4(0, 0, 0, 0);
            d[t] = 0.f;
            sp[t] = 0;
            if (i < nb32 * 2 && t < m) {
                pk[t] = ((const uint4*)(X.xq + (size_t)t * nb32 * 32))[i];
                if ((i & 1) == 0) {
                    d[t] = X.xd[(size_t)t * nb32 + (i >> 1)];
                    if (Ops::kNeedsSums) sp[t] = X.xs[(size_t)t * nb32 + (i >> 1)];
                }
            }
        }
    }
    // rows past m are staged as zeros (their results are not written)
    __device__ __forceinline__ void store(char* smem, int tokb, int nblk) {
        const int i = threadIdx.x;
        if (i < Ops::nb32(nblk) * 2) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                char* tok = smem + t * tokb;
                *(uint4*)Ops::xq_dword(tok, nblk, i >> 1, (i & 1) * 4) = pk[t];
                if ((i & 1) == 0) Ops::put_scale(tok, nblk, i >> 1, d[t], (int)(short)(sp[t] & 0xffff), sp[t] >> 16);
            }
        }
    }
};

// The same for up to MT fp32 rows that are quantised here (FQ = 1 with MT > 1): item i = half block i % hb of row i / hb,
// hb = half blocks per row; a thread takes items threadIdx.x, threadIdx.x + 1024 and threadIdx.x + 2048, MT * hb <= 3072 (the
// launcher's bound: 49152 values in all, e.g. 4 rows of up to 12288 elements).  Saves the quantiser launch in front of a
// 2..4-row GEMV (2.5 of the 7.6 us Q4_0 9728 x 2560 takes at 2 rows).
template <class Ops, int MT>
struct FlatXRowsF {
    static_assert(MT <= 4, "row = number of row boundaries at or below the item index");
    static constexpr int NP = 3;   // items per thread
    float4 v[NP][4];
    int t[NP], h[NP];

    __device__ __forceinline__ void request(const GemvX& X, int nblk, int m) {
        const int hb = Ops::nb32(nblk) * 2;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int i = threadIdx.x + p * 1024;
            t[p] = (i >= hb ? 1 : 0) + (i >= 2 * hb ? 1 : 0) + (i >= 3 * hb ? 1 : 0);
            h[p] = i - t[p] * hb;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[p][j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (t[p] < m && i < MT * hb) v[p][j] = ((const float4*)(X.x + (size_t)t[p] * hb * 16))[h[p] * 4 + j];
            }
        }
    }
    // rows past m are staged as zeros (their results are not written)
    __device__ __forceinline__ void store(char* smem, int tokb, int nblk) {
        const int hb = Ops::nb32(nblk) * 2;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int i = threadIdx.x + p * 1024;
            if ((i & ~63) >= MT * hb) return;   // whole waves
            quantize_half_block<Ops>(smem + min(t[p], MT - 1) * tokb, nblk, h[p], i < MT * hb, v[p]);
        }
    }
};

// Flat form for weight rows that are a whole number of GL-lane groups (GL = 16, 8 or 4 units).  Rows are contiguous in the planar layout, so the units of a workgroup's rows [r0, r1) are
// one flat sequence: a wave load covers 64 consecutive units of it (1 KB of quants, whatever the row
// length), wave w takes loads w, w + 16, ...  Every GL-lane group lies inside one row; its sum goes
// to LDS, and after a barrier the groups of a row are added in ascending order.  All waves of a
// workgroup carry the same number of loads, issued without conditions (lanes past the end re-read the
// last unit) so that the wait for ring slot k is exactly "all but the loads issued after it" instead
// of "all loads".  A round requests PRE loads and consumes them; the activation is staged during the
// first round, after its weight loads are out.
//
// MT > 1: m <= MT pre-quantised activation rows (FQ = 0) share every weight load; y[t * ldy + row].
//
// DUMP (one activation row): every unit also writes its exact integer block dot(s) to
// dump[row * dump_per_row + ...], the same integers that enter the fp32 combination.
//
// DUAL (one activation row): the workgroup walks the same rows of a second weight W1 (the `up` projection next to `gate`)
// after those of W -- the loads of the two weights form one sequence, whole 64-unit loads each -- and its tail has both
// dots of a row: y[r] (optional), y1[r] (optional) and hout[r] = act2(y[r]) * y1[r] (SMX_ACT_SILU_MUL / SMX_ACT_GEGLU).
// A row's sums are formed exactly as without DUAL, so y and y1 have the bits of two separate launches.
template <class Ops, int MT, int PRE, int GL, int FQ, bool DUMP = false, bool DUAL = false>
__device__ __forceinline__ void gemv_body_flat(const GemvW W, const GemvX X, float* __restrict__ y, int ldy, int nblk,
                                               int N, int m, int wg, int n_wgs, unsigned magic_u,
                                               int* __restrict__ dump = nullptr, int dump_per_row = 0,
                                               const GemvW W1 = GemvW{}, float* __restrict__ y1 = nullptr,
                                               float* __restrict__ hout = nullptr, int act2 = 0) {
    static_assert(MT == 1 || FQ == 0 || FQ == 1, "several activation rows: staged from quantised rows or quantised here");
    static_assert(!DUMP || MT == 1, "the block-dot dump covers one activation row");
    static_assert(!DUAL || (MT == 1 && !DUMP), "the paired form serves one activation row");
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int U = Ops::units_per_row(nblk);
    // rows split evenly: the first N % n_wgs workgroups take one row more
    const unsigned rbase = (unsigned)N / (unsigned)n_wgs, rrem = (unsigned)N - rbase * (unsigned)n_wgs;
    const int r0 = wg * (int)rbase + min(wg, (int)rrem), r1 = r0 + (int)rbase + (wg < (int)rrem ? 1 : 0);
    const int nunits = (r1 - r0) * U;          // < 2^16 (launcher)
    const int nloads1 = (nunits + 63) >> 6;          // loads per weight
    const int nloads = DUAL ? 2 * nloads1 : nloads1;
    const int tokb = Ops::tok_bytes(nblk);
    float* part = (float*)(smem + MT * tokb);  // [nunits / GL][MT]; DUAL: the second weight's groups follow the first's
    // a job with fewer rows than the launch has workgroups leaves some without rows: their (unused)
    // loads go to the weight's first unit
    const size_t f_base = nunits > 0 ? (size_t)r0 * U : 0;

    FlatX<Ops, MT == 1 ? FQ : 0> xs;
    FlatXRows<Ops, MT> xr;
    FlatXRowsF<Ops, MT <= 4 ? MT : 4> xf;
    constexpr bool kRowsF = MT > 1 && MT <= 4 && FQ == 1;
    if (MT == 1) xs.request(X, nblk);
    else if (kRowsF) xf.request(X, nblk, m);
    else xr.request(X, nblk, m);

    typename Ops::Regs ring[PRE];
    int l_t = wave, c_t = wave;
    auto request = [&]() {
#pragma unroll
        for (int k = 0; k < PRE; k++) {
            const bool second = DUAL && l_t >= nloads1;   // wave-uniform
            const int fl = min((second ? l_t - nloads1 : l_t) * 64 + lane, max(nunits - 1, 0));
            Ops::load_flat(ring[k], second ? W1 : W, f_base + fl);
            l_t += 16;
        }
    };
    auto consume = [&]() {
#pragma unroll
        for (int k = 0; k < PRE; k++) {
            if (c_t < nloads) {   // wave-uniform
                const bool second = DUAL && c_t >= nloads1;
                const int fl = (second ? c_t - nloads1 : c_t) * 64 + lane;
                const bool act = fl < nunits;
                const int flc = act ? fl : nunits - 1;
                const int rl = (int)__umulhi((unsigned)flc, magic_u);            // flc / U: row within the workgroup
                const int u = flc - rl * U;                                      // flc mod U
                float acc[MT];
#pragma unroll
                for (int t = 0; t < MT; t++) acc[t] = 0.f;
                int* drow = (DUMP && dump) ? dump + (size_t)(r0 + rl) * dump_per_row : nullptr;
                compute_unit<MT, DUMP>(Ops(), ring[k], smem, tokb, nblk, u, act, acc, drow);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float s = small_group_sum<GL>(acc[t]);
                    if (act && (lane & (GL - 1)) == GL - 1) part[((second ? nunits / GL : 0) + fl / GL) * MT + t] = s;
                }
            }
            c_t += 16;
        }
    };
    // A long activation row (8192 elements or more) is several loads per thread on the first ten waves, and the weight loads
    // of the waves that carry none of it would reach the CU's memory pipeline first and hold the row back behind cold HBM
    // traffic (the staging barrier then fell 2.8 us after the launch instead of 1.4): there the waves meet once before the
    // first weight request, so that the row's loads lead the queue.  Q4_0 / Q8_0 2560 x 9728 5.98 / 7.71 -> 5.4 / 7.3 us; on
    // shorter rows the wait for the last wave to start costs more than it brings (cfg1 +0.15 us) and is left out.
    if (MT == 1 && Ops::nb32(nblk) >= 256) __builtin_amdgcn_s_barrier();
    request();
    if (MT == 1) xs.store(smem, nblk, X);
    else if (kRowsF) xf.store(smem, tokb, nblk);
    else xr.store(smem, tokb, nblk);
    __syncthreads();
    consume();
    while (c_t < nloads) {
        request();
        consume();
    }
    __syncthreads();
    // A row's G group sums are added by 8 lanes (lane l takes groups l, l + 8, ... in ascending order, then a
    // fixed DPP tree): one thread per row would pay the LDS latency once per group, one after the other.
    const int G = U / GL;
    if constexpr (DUAL) {
#pragma clang fp contract(off)
        const float* part1 = part + nunits / GL;
        for (int i8 = threadIdx.x; i8 < (r1 - r0) * 8; i8 += 1024) {
            const int r = i8 >> 3, l = i8 & 7;
            float s0 = 0.f, s1 = 0.f;
            for (int j = l; j < G; j += 8) {
                s0 += part[r * G + j];
                s1 += part1[r * G + j];
            }
            s0 = small_group_sum<8>(s0);
            s1 = small_group_sum<8>(s1);
            if (l == 0) {
                if (y) y[r0 + r] = s0;
                if (y1) y1[r0 + r] = s1;
                hout[r0 + r] = (act2 == SMX_ACT_GEGLU ? det_gelu_tanh(s0) : det_silu(s0)) * s1;
            }
        }
        return;
    }
    for (int i8 = threadIdx.x; i8 < (r1 - r0) * MT * 8; i8 += 1024) {   // 1024: the form's workgroup size
        const int i = i8 >> 3, l = i8 & 7;
        const int r = i / MT, t = i % MT;
        float s = 0.f;
        for (int j = l; j < G; j += 8) s += part[(r * G + j) * MT + t];
        s = small_group_sum<8>(s);
        if (l == 0 && t < m) y[(size_t)t * ldy + r0 + r] = s;
    }
}

}  // namespace smx
