// The router's arithmetic as a device function run by one wave (kernels.rs:1846-1872 topk_router; crates/strix-backend-cpu/src/
// mellum.rs:1178-1192): shared by the routing kernel and by the expert gate/up launch that routes in its own prologue.
#pragma once
#include "detmath.h"

namespace smx {

constexpr int kRouterPerLane = 16;   // ne <= 1024
template <int CTRL>
__device__ __forceinline__ float rb_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double rb_dpp_d(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)b, CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xf, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}
__device__ __forceinline__ float rb_lane(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
__device__ __forceinline__ double rb_lane_d(double v, int l) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)b, l), hi = __builtin_amdgcn_readlane((int)(b >> 32), l);
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}
// Up to 64 experts, one per lane: the softmax probability of this lane's expert (-1 for a lane past ne).  x: the expert's
// logit (-FLT_MAX past ne).  Every cross-lane step is a DPP move or a lane read into a scalar register (no LDS round trips).
__device__ __forceinline__ float router_prob_lane(float x, bool live) {
#pragma clang fp contract(off)
    // maximum and (double) sum over the wave: a DPP tree inside each 16-lane row, then the four rows in ascending order
    float rm = x;
    rm = fmaxf(rm, rb_dpp<0xB1>(rm));
    rm = fmaxf(rm, rb_dpp<0x4E>(rm));
    rm = fmaxf(rm, rb_dpp<0x141>(rm));
    rm = fmaxf(rm, rb_dpp<0x140>(rm));
    const float mx = fmaxf(fmaxf(rb_lane(rm, 0), rb_lane(rm, 16)), fmaxf(rb_lane(rm, 32), rb_lane(rm, 48)));
    const float e = live ? det_expf(x - mx) : 0.f;
    double rs = (double)e;
    rs += rb_dpp_d<0xB1>(rs);
    rs += rb_dpp_d<0x4E>(rs);
    rs += rb_dpp_d<0x141>(rs);
    rs += rb_dpp_d<0x140>(rs);
    const double sum = ((rb_lane_d(rs, 0) + rb_lane_d(rs, 16)) + rb_lane_d(rs, 32)) + rb_lane_d(rs, 48);
    return live ? e / (float)sum : -1.f;
}
// The part of a lane's rank that the experts j0 <= j < j1 contribute: how many of them precede this lane's expert in
// (probability descending, index ascending) order.  The parts over all j add up to the rank; rank r < k is pick r.
__device__ __forceinline__ int router_rank_part(float p, int j0, int j1) {
    const int lane = threadIdx.x & 63;
    int rank = 0;
    for (int j = j0; j < j1; j++) {   // wave-uniform bounds
        const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), j));
        rank += (pj > p || (pj == p && j < lane)) ? 1 : 0;
    }
    return rank;
}

// The router's arithmetic, run by ONE wave: v[j] = logit of expert lane + 64 j (-FLT_MAX past ne); sel: 64 floats of LDS.
template <int PL>
__device__ __forceinline__ void topk_router_wave(float (&v)[PL], int ne, int k, int* __restrict__ ids, float* __restrict__ w,
                                                 float* sel) {
#pragma clang fp contract(off)
    constexpr int kRouterPerLane = PL;
    const int lane = threadIdx.x & 63;
    if constexpr (PL == 1) {
        // Up to 64 experts, one per lane.  A lane's rank = the number of experts that precede it in (probability descending,
        // index ascending) order; rank r < k is pick r.
        const bool live = lane < ne;
        const float p = router_prob_lane(v[0], live);
        int rank = 0;
#pragma unroll
        for (int j = 0; j < 64; j++) {
            const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), j));
            rank += (pj > p || (pj == p && j < lane)) ? 1 : 0;
        }
        if (live && rank < k) {
            sel[rank] = p;
            ids[rank] = lane;
        }
        // one wave: its own LDS writes, read back by its other lanes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float wsum = 0.f;   // in pick order, as the reference sums the chosen probabilities
        for (int i = 0; i < k; i++) wsum += sel[i];
        if (lane < k) w[lane] = sel[lane] / wsum;
        return;
    }
    float mx = -3.40282347e+38f;
#pragma unroll
    for (int j = 0; j < kRouterPerLane; j++) mx = fmaxf(mx, v[j]);
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < kRouterPerLane; j++) {
        const int e = lane + 64 * j;
        v[j] = e < ne ? det_expf(v[j] - mx) : -1.f;   // probabilities are >= 0: -1 marks "absent or taken"
        if (e < ne) sum += (double)v[j];
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    const float fsum = (float)sum;
#pragma unroll
    for (int j = 0; j < kRouterPerLane; j++)
        if (v[j] >= 0.f) v[j] = v[j] / fsum;
    float wsum = 0.f;
    float mine = 0.f;   // lane i keeps the probability of pick i (k <= 64)
    for (int i = 0; i < k; i++) {
        float b = -1.f;
        int bi = 1 << 30;
#pragma unroll
        for (int j = 0; j < kRouterPerLane; j++)
            if (v[j] > b) { b = v[j]; bi = lane + 64 * j; }   // ascending index within the lane: '>' keeps the lowest
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(b, off);
            const int oi = __shfl_xor(bi, off);
            if (ob > b || (ob == b && oi < bi)) { b = ob; bi = oi; }
        }
#pragma unroll
        for (int j = 0; j < kRouterPerLane; j++)
            if (lane + 64 * j == bi) v[j] = -1.f;
        if (lane == i) mine = b;
        if (lane == 0) ids[i] = bi;
        wsum += b;   // in pick order, as the reference sums the chosen probabilities
    }
    if (lane < k) w[lane] = mine / wsum;
}

}  // namespace smx
