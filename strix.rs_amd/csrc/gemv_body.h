// Device bodies of the fused block-dequant GEMV (shared by the dense and the MoE launches).
// Each body serves the RPW consecutive rows starting at `row0` for the calling wavefront; every
// wave of the workgroup must call it (the activation staging ends in a workgroup barrier).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace smx {

__device__ __forceinline__ float h2f(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }
// value of the neighbouring lane (lane ^ 1)
__device__ __forceinline__ int swap1(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ------------------------------------------------------------------ Q4_0
// LDS: per token  lo[nb] uint4 | hi[nb] uint4 | xd[nb] f32 | xs[nb] i32
template <int MT, int RPW, bool DUMP>
__device__ __forceinline__ void gemv_q4_0_body(const uint16_t* __restrict__ scales,
                                                         const uint4* __restrict__ quants,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         const int* __restrict__ xs, float* __restrict__ y, int nb,
                                                         int N, int m, int* __restrict__ dump, const int row0) {
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int tok_bytes = (nb * 40 + 15) & ~15;

    // first pass of weight loads goes out before the activation is staged
    uint4 wq[RPW];
    uint16_t wsc[RPW];
    size_t rbase[RPW];
    {
        const int bc = min(lane, nb - 1);
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            rbase[r] = (size_t)min(row0 + r, N - 1) * nb;
            wq[r] = quants[rbase[r] + bc];
            wsc[r] = scales[rbase[r] + bc];
        }
    }
    for (int t = 0; t < MT; t++) {
        uint4* lo = (uint4*)(smem + t * tok_bytes);
        uint4* hi = lo + nb;
        float* sd = (float*)(hi + nb);
        int* ss = (int*)(sd + nb);
        if (t < m) {
            const uint4* src = (const uint4*)(xq + (size_t)t * nb * 32);
            for (int i = tid; i < nb * 2; i += blockDim.x) ((i & 1) ? hi : lo)[i >> 1] = src[i];
            for (int i = tid; i < nb; i += blockDim.x) {
                sd[i] = xd[(size_t)t * nb + i];
                ss[i] = xs[(size_t)t * nb + i];
            }
        } else {
            for (int i = tid; i < nb; i += blockDim.x) {
                lo[i] = make_uint4(0, 0, 0, 0);
                hi[i] = make_uint4(0, 0, 0, 0);
                sd[i] = 0.f;
                ss[i] = 0;
            }
        }
    }
    __syncthreads();

    float acc[RPW][MT];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[r][t] = 0.f;

    for (int b0 = 0; b0 < nb; b0 += 64) {
        const int b = b0 + lane;
        const bool act = b < nb;
        const int bc = act ? b : nb - 1;
        uint4 nq[RPW];
        uint16_t nsc[RPW];
        const bool more = b0 + 64 < nb;
        if (more) {
            const int bn = min(b + 64, nb - 1);
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                nq[r] = quants[rbase[r] + bn];
                nsc[r] = scales[rbase[r] + bn];
            }
        }
        unsigned lo4[RPW][4], hi4[RPW][4];
        float dw[RPW];
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const unsigned w[4] = {wq[r].x, wq[r].y, wq[r].z, wq[r].w};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                lo4[r][g] = w[g] & 0x0f0f0f0fu;         // elements 4g..4g+3
                hi4[r][g] = (w[g] >> 4) & 0x0f0f0f0fu;  // elements 16+4g..
            }
            dw[r] = act ? h2f(wsc[r]) : 0.f;
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const uint4* lo = (const uint4*)(smem + t * tok_bytes);
            const uint4* hi = lo + nb;
            const float* sd = (const float*)(hi + nb);
            const int* ss = (const int*)(sd + nb);
            const uint4 xl = lo[bc], xh = hi[bc];
            const float dx = sd[bc];
            const int sp = ss[bc];
            const int xsum = (int)(short)(sp & 0xffff) + (sp >> 16);
            const int xlw[4] = {(int)xl.x, (int)xl.y, (int)xl.z, (int)xl.w};
            const int xhw[4] = {(int)xh.x, (int)xh.y, (int)xh.z, (int)xh.w};
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                int isum = 0;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    isum = dot4((int)lo4[r][g], xlw[g], isum);
                    isum = dot4((int)hi4[r][g], xhw[g], isum);
                }
                isum -= 8 * xsum;  // sum((q-8)x) = sum(qx) - 8 sum(x)
                if (DUMP) {
                    if (act && t == 0 && row0 + r < N) dump[(size_t)(row0 + r) * nb + b] = isum;
                }
                acc[r][t] += (dw[r] * dx) * (float)isum;
            }
        }
        if (more) {
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                wq[r] = nq[r];
                wsc[r] = nsc[r];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float s = wave_sum(acc[r][t]);
            if (lane == 0 && row0 + r < N && t < m) y[(size_t)t * N + row0 + r] = s;
        }
}

// ------------------------------------------------------------------ Q8_0
// A lane owns a 16-byte half block; lanes 2i and 2i+1 share block i and add their i32 halves.
// LDS: per token  xq[nb*2] uint4 | xd[nb] f32
template <int MT, int RPW, bool DUMP>
__device__ __forceinline__ void gemv_q8_0_body(const uint16_t* __restrict__ scales,
                                                         const uint4* __restrict__ quants,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         float* __restrict__ y, int nb, int N, int m,
                                                         int* __restrict__ dump, const int row0) {
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int cpr = nb * 2;  // 16-byte chunks per row
    const int tok_bytes = (nb * 36 + 15) & ~15;

    uint4 wq[RPW];
    uint16_t wsc[RPW];
    size_t rbase[RPW];
    {
        const int cc = min(lane, cpr - 1);
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            rbase[r] = (size_t)min(row0 + r, N - 1) * nb;
            wq[r] = quants[rbase[r] * 2 + cc];
            wsc[r] = scales[rbase[r] + (cc >> 1)];
        }
    }
    for (int t = 0; t < MT; t++) {
        uint4* sq = (uint4*)(smem + t * tok_bytes);
        float* sd = (float*)(sq + cpr);
        if (t < m) {
            const uint4* src = (const uint4*)(xq + (size_t)t * nb * 32);
            for (int i = tid; i < cpr; i += blockDim.x) sq[i] = src[i];
            for (int i = tid; i < nb; i += blockDim.x) sd[i] = xd[(size_t)t * nb + i];
        } else {
            for (int i = tid; i < cpr; i += blockDim.x) sq[i] = make_uint4(0, 0, 0, 0);
            for (int i = tid; i < nb; i += blockDim.x) sd[i] = 0.f;
        }
    }
    __syncthreads();

    float acc[RPW][MT];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[r][t] = 0.f;

    for (int c0 = 0; c0 < cpr; c0 += 64) {
        const int ch = c0 + lane;
        const bool act = ch < cpr;
        const int cc = act ? ch : cpr - 1;
        const int b = cc >> 1;
        uint4 nq[RPW];
        uint16_t nsc[RPW];
        const bool more = c0 + 64 < cpr;
        if (more) {
            const int cn = min(ch + 64, cpr - 1);
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                nq[r] = quants[rbase[r] * 2 + cn];
                nsc[r] = scales[rbase[r] + (cn >> 1)];
            }
        }
        float dw[RPW];
#pragma unroll
        for (int r = 0; r < RPW; r++) dw[r] = (act && !(cc & 1)) ? h2f(wsc[r]) : 0.f;  // even lane carries the block
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const uint4* sq = (const uint4*)(smem + t * tok_bytes);
            const float* sd = (const float*)(sq + cpr);
            const uint4 xv = sq[cc];
            const float dx = sd[b];
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                int isum = dot4((int)wq[r].x, (int)xv.x, 0);
                isum = dot4((int)wq[r].y, (int)xv.y, isum);
                isum = dot4((int)wq[r].z, (int)xv.z, isum);
                isum = dot4((int)wq[r].w, (int)xv.w, isum);
                isum += swap1(isum);  // whole-block i32
                if (DUMP) {
                    if (act && !(cc & 1) && t == 0 && row0 + r < N) dump[(size_t)(row0 + r) * nb + b] = isum;
                }
                acc[r][t] += (dw[r] * dx) * (float)isum;
            }
        }
        if (more) {
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                wq[r] = nq[r];
                wsc[r] = nsc[r];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float s = wave_sum(acc[r][t]);
            if (lane == 0 && row0 + r < N && t < m) y[(size_t)t * N + row0 + r] = s;
        }
}

// ------------------------------------------------------------------ Q6_K
// A lane owns a 64-element task (superblock sb, half h, 16-lane column c): two 16-byte ql chunks
// (c and c+2 of the half), one 16-byte qh chunk, i.e. four 16-element sub-blocks 8h + 2j + c.
// Lanes 2i / 2i+1 (c = 0 / 1) hold the two halves of the same four 32-wide activation blocks.
// Element map: crates/strix-models/src/ggml_quant.rs:417-426.
// LDS: xq as 16-byte chunks, 8 per 128 elements padded to 9 | xd[K/32] f32 | xs[K/32] i32
template <int RPW, bool DUMP>
__device__ __forceinline__ void gemv_q6_k_body(const uint4* __restrict__ ql, const uint4* __restrict__ qh,
                                                         const uint2* __restrict__ sc,
                                                         const uint16_t* __restrict__ dsb,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         const int* __restrict__ xs, float* __restrict__ y, int nsb,
                                                         int N, int* __restrict__ dump, const int row0) {
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int tpr = nsb * 4;   // tasks per row
    const int ngrp = nsb * 2;  // 128-element groups
    uint4* sq = (uint4*)smem;
    float4* sd = (float4*)(sq + ngrp * 9);
    int4* ss = (int4*)(sd + ngrp);

    uint4 wa[RPW], wb[RPW], wh[RPW];
    uint2 wsc[RPW];
    uint16_t wd[RPW];
    size_t rsb[RPW];
    {
        const int tk = min(lane, tpr - 1);
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            rsb[r] = (size_t)min(row0 + r, N - 1) * nsb;
            wa[r] = ql[rsb[r] * 8 + (tk >> 1) * 4 + (tk & 1)];
            wb[r] = ql[rsb[r] * 8 + (tk >> 1) * 4 + (tk & 1) + 2];
            wh[r] = qh[rsb[r] * 4 + tk];
            wsc[r] = sc[rsb[r] * 2 + (tk >> 1)];
            wd[r] = dsb[rsb[r] + (tk >> 2)];
        }
    }
    {
        const uint4* src = (const uint4*)xq;
        for (int i = tid; i < ngrp * 8; i += blockDim.x) sq[(i >> 3) * 9 + (i & 7)] = src[i];
        const float4* srcd = (const float4*)xd;
        const int4* srcs = (const int4*)xs;
        for (int i = tid; i < ngrp; i += blockDim.x) {
            sd[i] = srcd[i];
            ss[i] = srcs[i];
        }
    }
    __syncthreads();

    float acc[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) acc[r] = 0.f;

    for (int t0 = 0; t0 < tpr; t0 += 64) {
        const int tku = t0 + lane;
        const bool act = tku < tpr;
        const int tk = act ? tku : tpr - 1;
        const int g = tk >> 1, c = tk & 1;
        uint4 na[RPW], nbq[RPW], nh[RPW];
        uint2 nsc[RPW];
        uint16_t nd[RPW];
        const bool more = t0 + 64 < tpr;
        if (more) {
            const int tn = min(tku + 64, tpr - 1);
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                na[r] = ql[rsb[r] * 8 + (tn >> 1) * 4 + (tn & 1)];
                nbq[r] = ql[rsb[r] * 8 + (tn >> 1) * 4 + (tn & 1) + 2];
                nh[r] = qh[rsb[r] * 4 + tn];
                nsc[r] = sc[rsb[r] * 2 + (tn >> 1)];
                nd[r] = dsb[rsb[r] + (tn >> 2)];
            }
        }
        // activation: four 16-byte pieces (32-block j of the half, 16-half c), their scales and sums
        uint4 xv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) xv[j] = sq[g * 9 + 2 * j + c];
        const float4 dx4 = sd[g];
        const int4 sp4 = ss[g];
        const float dxs[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
        const int sps[4] = {sp4.x, sp4.y, sp4.z, sp4.w};
        int xs16[4];
#pragma unroll
        for (int j = 0; j < 4; j++) xs16[j] = c ? (sps[j] >> 16) : (int)(short)(sps[j] & 0xffff);
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const unsigned a4[4] = {wa[r].x, wa[r].y, wa[r].z, wa[r].w};
            const unsigned b4[4] = {wb[r].x, wb[r].y, wb[r].z, wb[r].w};
            const unsigned h4[4] = {wh[r].x, wh[r].y, wh[r].z, wh[r].w};
            int is[4] = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const unsigned q0 = (a4[i] & 0x0f0f0f0fu) | ((h4[i] << 4) & 0x30303030u);
                const unsigned q1 = (b4[i] & 0x0f0f0f0fu) | ((h4[i] << 2) & 0x30303030u);
                const unsigned q2 = ((a4[i] >> 4) & 0x0f0f0f0fu) | (h4[i] & 0x30303030u);
                const unsigned q3 = ((b4[i] >> 4) & 0x0f0f0f0fu) | ((h4[i] >> 2) & 0x30303030u);
                const int x0 = (int)(&xv[0].x)[i], x1 = (int)(&xv[1].x)[i], x2 = (int)(&xv[2].x)[i],
                          x3 = (int)(&xv[3].x)[i];
                is[0] = dot4((int)q0, x0, is[0]);
                is[1] = dot4((int)q1, x1, is[1]);
                is[2] = dot4((int)q2, x2, is[2]);
                is[3] = dot4((int)q3, x3, is[3]);
            }
            const float d = (act && c == 0) ? h2f(wd[r]) : 0.f;  // even lane carries the 32-block
            const unsigned long long scw = ((unsigned long long)wsc[r].y << 32) | wsc[r].x;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int isum = is[j] - 32 * xs16[j];  // sum((q-32)x) = sum(qx) - 32 sum(x)
                if (DUMP) {
                    if (act && row0 + r < N)
                        dump[(size_t)(row0 + r) * nsb * 16 + (size_t)(tk >> 2) * 16 + ((tk >> 1) & 1) * 8 + 2 * j + c] =
                            isum;
                }
                const int s8 = (int)(signed char)((scw >> (8 * (2 * j + c))) & 0xff);
                int tj = s8 * isum;
                tj += swap1(tj);  // both 16-element halves of the 32-block
                acc[r] += (d * dxs[j]) * (float)tj;
            }
        }
        if (more) {
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                wa[r] = na[r];
                wb[r] = nbq[r];
                wh[r] = nh[r];
                wsc[r] = nsc[r];
                wd[r] = nd[r];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) y[row0 + r] = s;
    }
}


}  // namespace smx
