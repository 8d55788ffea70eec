/*
 * strix_oracle.c — CPU restatement of the Strix.rs quantized-matmul path.
 * TEST INFRASTRUCTURE ONLY (see strix_oracle.h for scope and parity status).
 *
 * Build with -ffp-contract=off: the Rust reference never fuses a*b+c.
 */
#include "strix_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ f16 */

/* IEEE binary16 -> binary32, exact (half::f16::to_f32, call sites
 * ggml_quant.rs:164, 186-188; subnormal case as kernels.rs:9-15). */
float orc_f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h >> 15) & 1u, e = (uint32_t)(h >> 10) & 0x1fu, m = h & 0x3ffu;
    uint32_t bits;
    if (e == 0) {
        if (m == 0) {
            bits = s << 31;
        } else { /* subnormal: m * 2^-24, renormalise */
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3ffu;
            bits = (s << 31) | ((uint32_t)(113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        bits = (s << 31) | 0x7f800000u | (m << 13);
    } else {
        bits = (s << 31) | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (half::f16::from_f32,
 * ggml_quant.rs:201, 228). */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t mant = x & 0x7fffffu;
    int exp = (int)((x >> 23) & 0xffu);
    if (exp == 255) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u | (mant >> 13) : 0));
    int e = exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign;
        mant |= 0x800000u;
        int sh = 14 - e; /* 14..24 */
        uint32_t h = mant >> sh;
        uint32_t rem = mant & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++; /* may carry into exponent: correct */
    return (uint16_t)(sign | h);
}

/* -------------------------------------------------------- block formats */

int orc_block_elems(int type) {
    switch (type) {
        case ORC_Q4_0: case ORC_Q8_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: return 32;
        case ORC_Q6_K: case ORC_Q4_K: case ORC_Q5_K: return 256;
        default: return 0;
    }
}

int orc_block_bytes(int type) {
    switch (type) {
        case ORC_Q4_0: return 18;  /* ggml_quant.rs:111 */
        case ORC_Q8_0: return 34;  /* :115 */
        case ORC_Q6_K: return 210; /* :121 */
        case ORC_Q4_1: return 20;  /* :112 */
        case ORC_Q5_0: return 22;  /* :113 */
        case ORC_Q5_1: return 24;  /* :114 */
        case ORC_Q4_K: return 144; /* :119 */
        case ORC_Q5_K: return 176; /* :120 */
        default: return 0;
    }
}

static inline float rd_f16(const uint8_t* b) { return orc_f16_to_f32((uint16_t)(b[0] | (b[1] << 8))); }

/* ggml_quant.rs:240-247 */
static void dequant_q8_0(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 34;
        float d = rd_f16(blk);
        for (int i = 0; i < 32; i++) out[b * 32 + i] = d * (float)(int8_t)blk[2 + i];
    }
}

/* ggml_quant.rs:251-262 */
static void dequant_q4_0(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 18;
        float d = rd_f16(blk);
        const uint8_t* qs = blk + 2;
        for (int j = 0; j < 16; j++) {
            int lo = (int)(qs[j] & 0x0F) - 8, hi = (int)(qs[j] >> 4) - 8;
            out[b * 32 + j] = d * (float)lo;
            out[b * 32 + j + 16] = d * (float)hi;
        }
    }
}

/* The four 6-bit quants addressed by (half, l), ggml_quant.rs:417-422. */
static inline void q6k_quad(const uint8_t* blk, int half, int l, int q[4]) {
    const uint8_t* ql = blk + half * 64;
    const uint8_t* qh = blk + 128 + half * 32;
    q[0] = (int)((ql[l] & 0x0F) | ((qh[l] & 3) << 4)) - 32;
    q[1] = (int)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
    q[2] = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
    q[3] = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
}

/* ggml_quant.rs:404-430 */
static void dequant_q6_k(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 210;
        const int8_t* sc = (const int8_t*)(blk + 192);
        float d = rd_f16(blk + 208);
        float* ob = out + b * 256;
        for (int half = 0; half < 2; half++) {
            const int8_t* sch = sc + half * 8;
            int ybase = half * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16, q[4];
                q6k_quad(blk, half, l, q);
                ob[ybase + l] = d * (float)sch[is] * (float)q[0];
                ob[ybase + l + 32] = d * (float)sch[is + 2] * (float)q[1];
                ob[ybase + l + 64] = d * (float)sch[is + 4] * (float)q[2];
                ob[ybase + l + 96] = d * (float)sch[is + 6] * (float)q[3];
            }
        }
    }
}

/* ggml_quant.rs:265-275 */
static void dequant_q4_1(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 20;
        float d = rd_f16(blk), m = rd_f16(blk + 2);
        const uint8_t* qs = blk + 4;
        for (int j = 0; j < 16; j++) {
            out[b * 32 + j] = d * (float)(qs[j] & 0x0F) + m;
            out[b * 32 + j + 16] = d * (float)(qs[j] >> 4) + m;
        }
    }
}

/* the fifth bits of values j and j + 16 of a Q5 block, ggml_quant.rs:284-285 */
static inline void q5_high_bits(uint32_t qh, int j, int* h0, int* h1) {
    *h0 = (int)(((qh >> j) << 4) & 0x10);
    *h1 = (int)((qh >> (j + 12)) & 0x10);
}

/* ggml_quant.rs:278-292 */
static void dequant_q5_0(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 22;
        float d = rd_f16(blk);
        uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
        const uint8_t* qs = blk + 6;
        for (int j = 0; j < 16; j++) {
            int h0, h1;
            q5_high_bits(qh, j, &h0, &h1);
            out[b * 32 + j] = (float)((int)((qs[j] & 0x0F) | h0) - 16) * d;
            out[b * 32 + j + 16] = (float)((int)((qs[j] >> 4) | h1) - 16) * d;
        }
    }
}

/* ggml_quant.rs:295-311 */
static void dequant_q5_1(const uint8_t* bytes, float* out, size_t nblocks) {
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * 24;
        float d = rd_f16(blk), m = rd_f16(blk + 2);
        uint32_t qh = (uint32_t)blk[4] | ((uint32_t)blk[5] << 8) | ((uint32_t)blk[6] << 16) | ((uint32_t)blk[7] << 24);
        const uint8_t* qs = blk + 8;
        for (int j = 0; j < 16; j++) {
            int h0, h1;
            q5_high_bits(qh, j, &h0, &h1);
            out[b * 32 + j] = (float)((qs[j] & 0x0F) | h0) * d + m;
            out[b * 32 + j + 16] = (float)((qs[j] >> 4) | h1) * d + m;
        }
    }
}

/* 6-bit scale and min of sub-block j out of the 12 packed bytes, ggml_quant.rs:316-324 */
static inline void scale_min_k4(int j, const uint8_t* q, int* sc, int* mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
        *mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

/* ggml_quant.rs:328-359 (fifth = 0) and :365-400 (fifth = 1: Q5_K, 32 more bytes of high bits) */
static void dequant_q45_k(const uint8_t* bytes, float* out, size_t nblocks, int fifth) {
    const size_t bb = fifth ? 176 : 144;
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t* blk = bytes + b * bb;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t* scales = blk + 4;
        const uint8_t* qh = blk + 16;
        const uint8_t* qs = blk + (fifth ? 48 : 16);
        float* ob = out + b * 256;
        for (int chunk = 0; chunk < 4; chunk++) {
            int sc1, m1, sc2, m2;
            scale_min_k4(2 * chunk, scales, &sc1, &m1);
            scale_min_k4(2 * chunk + 1, scales, &sc2, &m2);
            float d1 = d * (float)sc1, min1 = dmin * (float)m1, d2 = d * (float)sc2, min2 = dmin * (float)m2;
            const uint8_t* q = qs + chunk * 32;
            for (int l = 0; l < 32; l++) {
                float lo = (float)(q[l] & 0x0F), hi = (float)(q[l] >> 4);
                if (fifth) {
                    if (qh[l] & (1u << (2 * chunk))) lo += 16.0f;
                    if (qh[l] & (2u << (2 * chunk))) hi += 16.0f;
                }
                ob[chunk * 64 + l] = d1 * lo - min1;
                ob[chunk * 64 + 32 + l] = d2 * hi - min2;
            }
        }
    }
}

int orc_dequantize(int type, const uint8_t* bytes, size_t nbytes, float* out, size_t n) {
    int be = orc_block_elems(type);
    if (be == 0 || n % (size_t)be != 0) return -1; /* ggml_quant.rs:142-146 */
    size_t nblocks = n / (size_t)be;
    if (nbytes < nblocks * (size_t)orc_block_bytes(type)) return -1; /* :149-154 */
    switch (type) {
        case ORC_Q8_0: dequant_q8_0(bytes, out, nblocks); break;
        case ORC_Q4_0: dequant_q4_0(bytes, out, nblocks); break;
        case ORC_Q6_K: dequant_q6_k(bytes, out, nblocks); break;
        case ORC_Q4_1: dequant_q4_1(bytes, out, nblocks); break;
        case ORC_Q5_0: dequant_q5_0(bytes, out, nblocks); break;
        case ORC_Q5_1: dequant_q5_1(bytes, out, nblocks); break;
        case ORC_Q4_K: dequant_q45_k(bytes, out, nblocks, 0); break;
        case ORC_Q5_K: dequant_q45_k(bytes, out, nblocks, 1); break;
        default: return -1;
    }
    return 0;
}

/* ggml_quant.rs:193-207.  Rust's f32::round is ties-away = roundf. */
void orc_quantize_q8_0(const float* x, size_t n, uint8_t* out) {
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; b++) {
        const float* blk = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(blk[i]));
        float d = amax / 127.0f;
        float id = d > 0.0f ? 1.0f / d : 0.0f;
        uint16_t h = orc_f32_to_f16(d);
        uint8_t* o = out + b * 34;
        o[0] = (uint8_t)(h & 0xff);
        o[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; i++) {
            float r = roundf(blk[i] * id);
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            o[2 + i] = (uint8_t)(int8_t)r;
        }
    }
}

/* ggml_quant.rs:212-237 */
void orc_quantize_q4_0(const float* x, size_t n, uint8_t* out) {
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; b++) {
        const float* blk = x + b * 32;
        float amax = 0.0f, vmax = 0.0f;
        for (int i = 0; i < 32; i++)
            if (fabsf(blk[i]) > amax) { amax = fabsf(blk[i]); vmax = blk[i]; }
        float d = vmax / -8.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint16_t h = orc_f32_to_f16(d);
        uint8_t* o = out + b * 18;
        o[0] = (uint8_t)(h & 0xff);
        o[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 16; j++) {
            int q0 = (int)(blk[j] * id + 8.5f), q1 = (int)(blk[j + 16] * id + 8.5f);
            q0 = q0 < 0 ? 0 : (q0 > 15 ? 15 : q0);
            q1 = q1 < 0 ? 0 : (q1 > 15 ? 15 : q1);
            o[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

/* ----------------------------------------------------------- f32 oracle */

/* gemma.rs:323-326 */
static float dot_seq(const float* a, const float* b, int n) {
    float acc = 0.0f;
    for (int i = 0; i < n; i++) acc += a[i] * b[i];
    return acc;
}

/* mellum.rs:278-293 */
static float dot_lane8(const float* a, const float* b, int n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int chunks = n / 8;
    for (int c = 0; c < chunks; c++) {
        int i = c * 8;
        for (int k = 0; k < 8; k++) acc[k] += a[i + k] * b[i + k];
    }
    float s = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    for (int i = chunks * 8; i < n; i++) s += a[i] * b[i];
    return s;
}

int orc_matmul_f32(int type, const uint8_t* w, int K, int N, const float* x, int m, float* y,
                   int order, int nthreads) {
    int be = orc_block_elems(type);
    if (be == 0 || K % be != 0) return -1;
    size_t bpr = (size_t)(K / be) * (size_t)orc_block_bytes(type);
    int err = 0;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel num_threads(nthreads)
    {
        float* buf = (float*)malloc((size_t)K * sizeof(float)); /* per-thread scratch, gemma.rs:319 */
#pragma omp for schedule(static)
        for (int o = 0; o < N; o++) {
            if (!buf || orc_dequantize(type, w + (size_t)o * bpr, bpr, buf, (size_t)K) != 0) {
                err = 1;
                continue;
            }
            for (int t = 0; t < m; t++) {
                const float* xt = x + (size_t)t * K;
                y[(size_t)t * N + o] = order ? dot_lane8(buf, xt, K) : dot_seq(buf, xt, K);
            }
        }
        free(buf);
    }
    return err ? -1 : 0;
}

/* ------------------------------------------------------------ Q8 oracle */

/* kernels.rs:75-96 (single row) / :1000-1013 (rows) */
void orc_actquant(const float* x, int m, int K, int8_t* xq, float* xd, int16_t* xs16) {
    int nb = K / 32;
    for (int t = 0; t < m; t++) {
        for (int b = 0; b < nb; b++) {
            const float* xb = x + (size_t)t * K + (size_t)b * 32;
            float amax = 0.0f;
            for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(xb[i]));
            float d = amax / 127.0f;
            float inv = d > 0.0f ? 1.0f / d : 0.0f;
            int s0 = 0, s1 = 0;
            for (int i = 0; i < 32; i++) {
                int q = (int)rintf(xb[i] * inv); /* ties to even, as the device's rintf */
                q = q < -127 ? -127 : (q > 127 ? 127 : q);
                xq[(size_t)t * K + (size_t)b * 32 + i] = (int8_t)q;
                if (i < 16) s0 += q; else s1 += q;
            }
            xd[(size_t)t * nb + b] = d;
            if (xs16) {
                xs16[((size_t)t * nb + b) * 2] = (int16_t)s0;
                xs16[((size_t)t * nb + b) * 2 + 1] = (int16_t)s1;
            }
        }
    }
}

/* kernels.rs:241-250: sum(nibble*xq) - 8*sum(xq) == sum((nibble-8)*xq). */
static inline int32_t bdot_q4_0(const uint8_t* blk, const int8_t* xq) {
    const uint8_t* qs = blk + 2;
    int32_t s = 0;
    for (int j = 0; j < 16; j++) {
        s += ((int32_t)(qs[j] & 0x0F) - 8) * (int32_t)xq[j];
        s += ((int32_t)(qs[j] >> 4) - 8) * (int32_t)xq[j + 16];
    }
    return s;
}

/* kernels.rs:903-909, summed over the whole block */
static inline int32_t bdot_q8_0(const uint8_t* blk, const int8_t* xq) {
    int32_t s = 0;
    for (int i = 0; i < 32; i++) s += (int32_t)(int8_t)blk[2 + i] * (int32_t)xq[i];
    return s;
}

/* 16 sub-block dots of one Q6_K superblock; element map ggml_quant.rs:417-426 */
static inline void bdot_q6_k(const uint8_t* blk, const int8_t* xq, int32_t out[16]) {
    for (int i = 0; i < 16; i++) out[i] = 0;
    for (int half = 0; half < 2; half++)
        for (int l = 0; l < 32; l++) {
            int q[4];
            q6k_quad(blk, half, l, q);
            for (int j = 0; j < 4; j++) {
                int e = half * 128 + l + 32 * j;
                out[e / 16] += q[j] * (int32_t)xq[e];
            }
        }
}

int orc_block_dots(int type, const uint8_t* w, int K, int N, const int8_t* xq, int32_t* out) {
    int be = orc_block_elems(type);
    if (be == 0 || K % be != 0) return -1;
    int nblk = K / be;
    size_t bb = (size_t)orc_block_bytes(type);
    for (int o = 0; o < N; o++)
        for (int b = 0; b < nblk; b++) {
            const uint8_t* blk = w + ((size_t)o * nblk + b) * bb;
            if (type == ORC_Q4_0) out[(size_t)o * nblk + b] = bdot_q4_0(blk, xq + (size_t)b * 32);
            else if (type == ORC_Q8_0) out[(size_t)o * nblk + b] = bdot_q8_0(blk, xq + (size_t)b * 32);
            else bdot_q6_k(blk, xq + (size_t)b * 256, out + ((size_t)o * nblk + b) * 16);
        }
    return 0;
}

int orc_matmul_q8(int type, const uint8_t* w, int K, int N, const int8_t* xq, const float* xd, int m,
                  float* y, int nthreads) {
    int be = orc_block_elems(type);
    if (be == 0 || K % be != 0) return -1;
    int nblk = K / be, nb32 = K / 32;
    size_t bb = (size_t)orc_block_bytes(type);
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int o = 0; o < N; o++) {
        const uint8_t* row = w + (size_t)o * nblk * bb;
        for (int t = 0; t < m; t++) {
            const int8_t* xt = xq + (size_t)t * K;
            const float* dt = xd + (size_t)t * nb32;
            float acc = 0.0f;
            if (type == ORC_Q6_K) {
                for (int b = 0; b < nblk; b++) {
                    const uint8_t* blk = row + (size_t)b * 210;
                    const int8_t* sc = (const int8_t*)(blk + 192);
                    float d = rd_f16(blk + 208);
                    int32_t is16[16];
                    bdot_q6_k(blk, xt + (size_t)b * 256, is16);
                    for (int j = 0; j < 8; j++) {
                        int32_t tj = (int32_t)sc[2 * j] * is16[2 * j] + (int32_t)sc[2 * j + 1] * is16[2 * j + 1];
                        acc += (d * dt[b * 8 + j]) * (float)tj;
                    }
                }
            } else {
                for (int b = 0; b < nblk; b++) {
                    const uint8_t* blk = row + (size_t)b * bb;
                    float dw = rd_f16(blk);
                    int32_t isum = type == ORC_Q4_0 ? bdot_q4_0(blk, xt + (size_t)b * 32)
                                                    : bdot_q8_0(blk, xt + (size_t)b * 32);
                    acc += (dw * dt[b]) * (float)isum; /* kernels.rs:251, 522 */
                }
            }
            y[(size_t)t * N + o] = acc;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ MoE */

/* exp(x) as a fixed sequence of IEEE fp32 operations (Cephes-style range
 * reduction and degree-6 polynomial); the device code performs the same
 * operations in the same order with contraction disabled. */
float orc_expf(float x) {
    if (x > 88.0f) x = 88.0f;
    if (x < -87.0f) x = -87.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = x - n * 0.693359375f;
    r = r - n * -2.12194440e-4f;
    float p = 1.9875691500e-4f;
    p = p * r + 1.3981999507e-3f;
    p = p * r + 8.3334519073e-3f;
    p = p * r + 4.1665795894e-2f;
    p = p * r + 1.6666665459e-1f;
    p = p * r + 5.0000001201e-1f;
    float r2 = r * r;
    p = p * r2;
    p = p + r;
    p = p + 1.0f;
    return ldexpf(p, (int)n);
}

float orc_silu(float x) { return x / (1.0f + orc_expf(-x)); }

/* tanh(z) = 1 - 2/(exp(2z) + 1) on the fixed-sequence exp above (saturates to +-1 through its clamps) */
float orc_tanhf(float z) { return 1.0f - 2.0f / (orc_expf(2.0f * z) + 1.0f); }

/* 0.5*x*(1 + tanh(sqrt(2/pi)*(x + 0.044715 x^3))), ops.rs:110-113; kernels.rs:162-163 */
float orc_gelu_tanh(float x) {
    float x3 = x * x * x;
    float inner = 0.7978845608f * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + orc_tanhf(inner));
}

/* Activation producers of the step before a GEMV (kernels.rs:101-226; ops.rs:15-27, 74-87, 110-121).
 *   ORC_ACT_RMSNORM : out = (a * scale) * b, scale = 1/sqrt(mean(a^2) + eps); b == NULL: unit weight.
 *                     The mean and the scale are formed in double and rounded once, so the result does
 *                     not depend on the order in which the squares are summed.
 *   ORC_ACT_SILU_MUL: out = silu(a) * b
 *   ORC_ACT_GEGLU   : out = gelu_tanh(a) * b */
int orc_act_produce(int act, const float* a, const float* b, int n, float eps, float* out) {
    if (act == ORC_ACT_NONE) {
        for (int i = 0; i < n; i++) out[i] = a[i];
    } else if (act == ORC_ACT_RMSNORM) {
        double ss = 0.0;
        for (int i = 0; i < n; i++) ss += (double)a[i] * (double)a[i];
        float scale = (float)(1.0 / sqrt(ss / (double)n + (double)eps));
        for (int i = 0; i < n; i++) {
            float v = a[i] * scale;
            out[i] = b ? v * b[i] : v;
        }
    } else if (act == ORC_ACT_SILU_MUL) {
        if (!b) return -1;
        for (int i = 0; i < n; i++) out[i] = orc_silu(a[i]) * b[i];
    } else if (act == ORC_ACT_GEGLU) {
        if (!b) return -1;
        for (int i = 0; i < n; i++) out[i] = orc_gelu_tanh(a[i]) * b[i];
    } else {
        return -1;
    }
    return 0;
}

int orc_moe_ffn_q8(const uint8_t* gate, const uint8_t* up, const uint8_t* down, int hidden, int eff,
                   int ne, const int32_t* ids, const float* wexp, int k, const float* x, float* y,
                   float* gu, int8_t* aq, float* ad, const int8_t* aq_in, const float* ad_in) {
    return orc_moe_ffn(ORC_Q8_0, gate, up, down, hidden, eff, ne, ids, wexp, k, x, y, gu, aq, ad, aq_in, ad_in);
}

int orc_moe_ffn(int type, const uint8_t* gate, const uint8_t* up, const uint8_t* down, int hidden, int eff,
                int ne, const int32_t* ids, const float* wexp, int k, const float* x, float* y,
                float* gu, int8_t* aq, float* ad, const int8_t* aq_in, const float* ad_in) {
    if (type != ORC_Q8_0 && type != ORC_Q6_K) return -1;
    const int be = type == ORC_Q6_K ? 256 : 32, bb = type == ORC_Q6_K ? 210 : 34;
    if (hidden % be || eff % be) return -1;
    size_t gate_eb = (size_t)(hidden / be) * bb * (size_t)eff; /* decode.rs:2730, 2806 */
    size_t down_eb = (size_t)(eff / be) * bb * (size_t)hidden; /* decode.rs:2731, 2807 */
    int8_t* xq = (int8_t*)malloc((size_t)hidden);
    float* xd = (float*)malloc((size_t)(hidden / 32) * 4);
    float* g = (float*)malloc((size_t)eff * 4);
    float* u = (float*)malloc((size_t)eff * 4);
    float* a = (float*)malloc((size_t)eff * 4);
    int8_t* aqk = (int8_t*)malloc((size_t)eff);
    float* adk = (float*)malloc((size_t)(eff / 32) * 4);
    float* dy = (float*)malloc((size_t)hidden * 4);
    orc_actquant(x, 1, hidden, xq, xd, NULL);
    for (int i = 0; i < hidden; i++) y[i] = 0.0f;
    int rc = 0;
    for (int kk = 0; kk < k; kk++) {
        int e = ids[kk];
        if (e < 0 || e >= ne) { rc = -1; break; }
        orc_matmul_q8(type, gate + (size_t)e * gate_eb, hidden, eff, xq, xd, 1, g, 1);
        orc_matmul_q8(type, up + (size_t)e * gate_eb, hidden, eff, xq, xd, 1, u, 1);
        if (gu) {
            memcpy(gu + ((size_t)kk * 2) * eff, g, (size_t)eff * 4);
            memcpy(gu + ((size_t)kk * 2 + 1) * eff, u, (size_t)eff * 4);
        }
        for (int i = 0; i < eff; i++) a[i] = orc_silu(g[i]) * u[i]; /* mellum.rs:1650-1652 */
        orc_actquant(a, 1, eff, aqk, adk, NULL);                     /* kernels.rs:879-892 */
        if (aq) memcpy(aq + (size_t)kk * eff, aqk, (size_t)eff);
        if (ad) memcpy(ad + (size_t)kk * (eff / 32), adk, (size_t)(eff / 32) * 4);
        const int8_t* q = aq_in ? aq_in + (size_t)kk * eff : aqk;
        const float* d = ad_in ? ad_in + (size_t)kk * (eff / 32) : adk;
        orc_matmul_q8(type, down + (size_t)e * down_eb, eff, hidden, q, d, 1, dy, 1);
        for (int i = 0; i < hidden; i++) y[i] += wexp[kk] * dy[i]; /* mellum.rs:1666-1668; kernels.rs:1880 */
    }
    free(xq); free(xd); free(g); free(u); free(a); free(aqk); free(adk); free(dy);
    return rc;
}

/* mellum.rs:1180-1191.  The reference sorts indices by descending probability
 * with a stable sort, so equal probabilities keep ascending index order. */
void orc_route_topk(const float* logits, int ne, int k, int32_t* ids, float* w) {
    float* probs = (float*)malloc((size_t)ne * 4);
    char* used = (char*)calloc((size_t)ne, 1);
    float mx = -3.40282347e+38f; /* f32::MIN */
    for (int e = 0; e < ne; e++) mx = fmaxf(mx, logits[e]);
    float sum = 0.0f;
    for (int e = 0; e < ne; e++) { probs[e] = expf(logits[e] - mx); sum += probs[e]; }
    for (int e = 0; e < ne; e++) probs[e] /= sum;
    float wsum = 0.0f;
    for (int i = 0; i < k; i++) {
        int best = -1;
        for (int e = 0; e < ne; e++)
            if (!used[e] && (best < 0 || probs[e] > probs[best])) best = e;
        used[best] = 1;
        ids[i] = best;
        wsum += probs[best];
    }
    for (int i = 0; i < k; i++) w[i] = probs[ids[i]] / wsum;
    free(probs);
    free(used);
}

/* ------------------------------------------------------------ generator */

void orc_lcg_fill(uint64_t* seed, uint32_t* out, size_t n) {
    uint64_t s = *seed;
    for (size_t i = 0; i < n; i++) {
        s = s * 6364136223846793005ULL + 1ULL;
        out[i] = (uint32_t)(s >> 33);
    }
    *seed = s;
}
