// Fused block-dequant -> GEMV for Q4_0 / Q8_0 / Q6_K weights against Q8-quantised activations.
//
// Stands in for the reference's decode GEMVs (crates/strix-backend-rocm/src/kernels.rs:259-287
// q4_gemv_dp, :894-912 q8i_gemv, :1016-1045 q8i_gemm_rows32, :607-640 q6_gemv) on gfx950:
//   * one wavefront (64 lanes) per output row, RPW rows per wave, NW waves per workgroup;
//   * every lane streams 128-bit chunks of the row's packed quants straight from HBM, the next
//     pass is issued before the current one is consumed;
//   * the quantised activation (int8 + scales + 16-element sums) is staged once per workgroup in LDS;
//   * v_dot4_i32_i8 integer block dots, exact i32 per block, then acc += (dw*dx)*float(isum);
//   * cross-lane (DPP) combination of lanes that share a block, wave-wide reduction at the end.
// HBM-bound: algorithmic bytes per row are K/32 * {18, 34} (Q4_0, Q8_0) or K/256 * 210 (Q6_K).
#include "gemv_body.h"
#include "smx_internal.h"

namespace smx {


template <int MT, int RPW, bool DUMP>
__global__ __launch_bounds__(1024) void gemv_q4_0_kernel(const uint16_t* __restrict__ scales,
                                                         const uint4* __restrict__ quants,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         const int* __restrict__ xs, float* __restrict__ y, int nb,
                                                         int N, int m, int* __restrict__ dump) {
    const int row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RPW;
    gemv_q4_0_body<MT, RPW, DUMP>(scales, quants, xq, xd, xs, y, nb, N, m, dump, row0);
}

template <int MT, int RPW, bool DUMP>
__global__ __launch_bounds__(1024) void gemv_q8_0_kernel(const uint16_t* __restrict__ scales,
                                                         const uint4* __restrict__ quants,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         float* __restrict__ y, int nb, int N, int m,
                                                         int* __restrict__ dump) {
    const int row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RPW;
    gemv_q8_0_body<MT, RPW, DUMP>(scales, quants, xq, xd, y, nb, N, m, dump, row0);
}

template <int RPW, bool DUMP>
__global__ __launch_bounds__(1024) void gemv_q6_k_kernel(const uint4* __restrict__ ql, const uint4* __restrict__ qh,
                                                         const uint2* __restrict__ sc,
                                                         const uint16_t* __restrict__ dsb,
                                                         const int8_t* __restrict__ xq, const float* __restrict__ xd,
                                                         const int* __restrict__ xs, float* __restrict__ y, int nsb,
                                                         int N, int* __restrict__ dump) {
    const int row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RPW;
    gemv_q6_k_body<RPW, DUMP>(ql, qh, sc, dsb, xq, xd, xs, y, nsb, N, dump, row0);
}

// ---------------------------------------------------------------- launch

template <typename Kern>
static int set_lds(smx_ctx* c, Kern kern, size_t lds) {
    if (lds > 160 * 1024) return fail(c, SMX_ERR_LIMIT, "gemv: activation needs %zu bytes of LDS (limit 163840)", lds);
    if (lds > 48 * 1024)
        SMX_HIP(c, hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    return SMX_OK;
}

struct GemvGeom {
    int rpw, nw;
    unsigned grid;
};

// Rows per wave and waves per workgroup.  Small activations: 4-wave groups (many groups per CU);
// large staged activations: 16-wave groups so one LDS copy serves a whole CU's worth of waves.
static GemvGeom pick_geom(const smx_ctx* c, size_t N, size_t lds, size_t row_bytes, int max_rpw) {
    GemvGeom g;
    g.nw = lds > 40 * 1024 ? 16 : 4;
    // keep >= ~8 waves per CU in flight when the matrix allows it, and give short rows more per wave
    int rpw = 1;
    const size_t want_waves = (size_t)c->num_cu * 8;
    while (rpw < max_rpw && N / (size_t)(rpw * 2) >= want_waves && row_bytes * (size_t)rpw < 8192) rpw *= 2;
    g.rpw = rpw;
    const size_t rows_per_wg = (size_t)g.nw * g.rpw;
    g.grid = (unsigned)((N + rows_per_wg - 1) / rows_per_wg);
    return g;
}

#define LAUNCH_Q4(MT, RPW, DUMP)                                                                                   \
    do {                                                                                                           \
        auto k = gemv_q4_0_kernel<MT, RPW, DUMP>;                                                                  \
        int rc = set_lds(c, k, lds);                                                                               \
        if (rc != SMX_OK) return rc;                                                                               \
        hipLaunchKernelGGL(k, dim3(g.grid), dim3(g.nw * 64), lds, c->stream, w.scales, (const uint4*)w.quants, xq, \
                           xd, (const int*)xs, y, (int)w.nblk, (int)w.N, (int)m, (int*)dump);                      \
    } while (0)

#define LAUNCH_Q8(MT, RPW, DUMP)                                                                                   \
    do {                                                                                                           \
        auto k = gemv_q8_0_kernel<MT, RPW, DUMP>;                                                                  \
        int rc = set_lds(c, k, lds);                                                                               \
        if (rc != SMX_OK) return rc;                                                                               \
        hipLaunchKernelGGL(k, dim3(g.grid), dim3(g.nw * 64), lds, c->stream, w.scales, (const uint4*)w.quants, xq, \
                           xd, y, (int)w.nblk, (int)w.N, (int)m, (int*)dump);                                      \
    } while (0)

#define LAUNCH_Q6(RPW, DUMP)                                                                                      \
    do {                                                                                                          \
        auto k = gemv_q6_k_kernel<RPW, DUMP>;                                                                     \
        int rc = set_lds(c, k, lds);                                                                              \
        if (rc != SMX_OK) return rc;                                                                              \
        hipLaunchKernelGGL(k, dim3(g.grid), dim3(g.nw * 64), lds, c->stream, (const uint4*)w.quants,              \
                           (const uint4*)w.qh, (const uint2*)w.sc, w.scales, xq, xd, (const int*)xs, y,           \
                           (int)w.nblk, (int)w.N, (int*)dump);                                                    \
    } while (0)

#define DISPATCH_MT_RPW(L)                                  \
    do {                                                    \
        if (mt == 1) {                                      \
            if (g.rpw == 1) L(1, 1, false);                 \
            else if (g.rpw == 2) L(1, 2, false);            \
            else L(1, 4, false);                            \
        } else if (mt == 2) {                               \
            if (g.rpw == 1) L(2, 1, false);                 \
            else L(2, 2, false);                            \
        } else if (mt == 4) {                               \
            if (g.rpw == 1) L(4, 1, false);                 \
            else L(4, 2, false);                            \
        } else {                                            \
            if (g.rpw == 1) L(8, 1, false);                 \
            else L(8, 2, false);                            \
        }                                                   \
    } while (0)

int launch_gemv(smx_ctx* c, const Weight& w, const int8_t* xq, const float* xd, const int32_t* xs, size_t m,
                float* y, int32_t* dump) {
    if (m == 0 || m > SMX_GEMV_MAX_M) return fail(c, SMX_ERR_LIMIT, "gemv: %zu rows (1..%d supported)", m, SMX_GEMV_MAX_M);
    if (w.N > 0x7fffffffu / 4 || w.K > (size_t(1) << 20))
        return fail(c, SMX_ERR_LIMIT, "gemv: shape %zu x %zu exceeds the kernel's index range", w.N, w.K);
    const int mt = m == 1 ? 1 : (m == 2 ? 2 : (m <= 4 ? 4 : 8));
    if (w.type == kQ4_0) {
        const size_t lds = (size_t)mt * ((w.nblk * 40 + 15) & ~size_t(15));
        GemvGeom g = pick_geom(c, w.N, lds, w.nblk * 18, mt == 1 ? 4 : 2);
        ProfScope ps(c, "gemv_q4_0");
        if (dump) {
            g.rpw = 1;
            g.grid = (unsigned)((w.N + g.nw - 1) / g.nw);
            LAUNCH_Q4(1, 1, true);
        } else {
            DISPATCH_MT_RPW(LAUNCH_Q4);
        }
    } else if (w.type == kQ8_0) {
        const size_t lds = (size_t)mt * ((w.nblk * 36 + 15) & ~size_t(15));
        GemvGeom g = pick_geom(c, w.N, lds, w.nblk * 34, mt == 1 ? 4 : 2);
        ProfScope ps(c, "gemv_q8_0");
        if (dump) {
            g.rpw = 1;
            g.grid = (unsigned)((w.N + g.nw - 1) / g.nw);
            LAUNCH_Q8(1, 1, true);
        } else {
            DISPATCH_MT_RPW(LAUNCH_Q8);
        }
    } else {
        if (m != 1) return fail(c, SMX_ERR_LIMIT, "gemv: Q6_K weights take one activation row per call");
        const size_t ngrp = w.nblk * 2;
        const size_t lds = ngrp * 9 * 16 + ngrp * 16 + ngrp * 16;
        GemvGeom g = pick_geom(c, w.N, lds, w.nblk * 210, 4);
        ProfScope ps(c, "gemv_q6_k");
        if (dump) {
            g.rpw = 1;
            g.grid = (unsigned)((w.N + g.nw - 1) / g.nw);
            LAUNCH_Q6(1, true);
        } else if (g.rpw == 1) {
            LAUNCH_Q6(1, false);
        } else if (g.rpw == 2) {
            LAUNCH_Q6(2, false);
        } else {
            LAUNCH_Q6(4, false);
        }
    }
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

}  // namespace smx
