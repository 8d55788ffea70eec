// Mixture-of-experts FFN on resident Q8_0 experts: decode (one token, k routed experts, grouped
// GEMVs) and prefill (m tokens grouped by expert, one table-driven MFMA GEMM launch per stage).
//
// Stands in for crates/strix-backend-rocm/src/decode.rs:1923-2128 (moe_launches: q8i_moe_gu ->
// silu_quant -> q8i_moe_down -> moe_wsum, kernels.rs:942-996, 879-892, 1875-1882) and
// decode.rs:1608-1739 (moe_layer_dev_inner: xquant8_rows -> gather_xq8 -> per-expert GEMMs ->
// silu_quant_rows -> per-expert GEMMs -> scatter_add_w, kernels.rs:1162-1198).
// Differences by design: the gather is an index indirection inside the GEMM's loader, all experts
// of a stage share one launch (tile table) instead of one launch per expert, and the weighted
// combine walks each token's slots in ascending slot order instead of fp32 atomics, so results do
// not depend on scheduling.
#include <algorithm>
#include <cstring>
#include <vector>

#include "detmath.h"
#include "gemv_body.h"
#include "router_body.h"
#include "smx_internal.h"

namespace smx {

// a = silu(g)*u for 4 consecutive elements, then the activation quantiser over the 32-block that
// 8 adjacent lanes hold (kernels.rs:879-892, 1174-1187): packed quants and the block scale.
// the activation quantiser over the 32-block that 8 adjacent lanes hold, 4 consecutive elements per lane
__device__ __forceinline__ void quant4(float4 v, int* packed, float* scale);
__device__ __forceinline__ void silu_mul_quant4(float4 gv, float4 uv, int* packed, float* scale) {
    float4 v;
    {
#pragma clang fp contract(off)
        v.x = det_silu(gv.x) * uv.x;
        v.y = det_silu(gv.y) * uv.y;
        v.z = det_silu(gv.z) * uv.z;
        v.w = det_silu(gv.w) * uv.w;
    }
    quant4(v, packed, scale);
}
__device__ __forceinline__ void quant4(float4 v, int* packed, float* scale) {
    float a = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    a = fmaxf(a, __shfl_xor(a, 1));
    a = fmaxf(a, __shfl_xor(a, 2));
    a = fmaxf(a, __shfl_xor(a, 4));
    const float d = a / 127.f;
    const float inv = d > 0.f ? 1.f / d : 0.f;
    const int q0 = max(-127, min(127, (int)rintf(v.x * inv)));
    const int q1 = max(-127, min(127, (int)rintf(v.y * inv)));
    const int q2 = max(-127, min(127, (int)rintf(v.z * inv)));
    const int q3 = max(-127, min(127, (int)rintf(v.w * inv)));
    *packed = (q0 & 0xff) | ((q1 & 0xff) << 8) | ((q2 & 0xff) << 16) | ((q3 & 0xff) << 24);
    *scale = d;
}

// Rows of `eff` floats g, u at stride ldg -> quantised silu(g)*u; 8 lanes per 32-block.
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                             size_t ldg, int eff, int* __restrict__ xq4,
                                                             float* __restrict__ xd, size_t nblocks) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t blk = gid >> 3;
    const bool live = blk < nblocks;
    float4 gv = make_float4(0.f, 0.f, 0.f, 0.f), uv = gv;
    if (live) {
        const int bpr = eff / 32;
        const size_t row = blk / bpr, e0 = (blk % bpr) * 32 + (gid & 7) * 4;
        gv = *(const float4*)(g + row * ldg + e0);
        uv = *(const float4*)(u + row * ldg + e0);
    }
    int packed;
    float d;
    silu_mul_quant4(gv, uv, &packed, &d);
    if (live) {
        xq4[gid] = packed;
        if ((gid & 7) == 0) xd[blk] = d;
    }
}

// Routed expert ids and weights travel as kernel arguments (no table upload on the decode path), or,
// when the router ran on the device, are read from its output at run time (ids_dev / w_dev non-null):
// a captured graph then serves every token's own routing.
struct MoeRoute {
    int ids[64];
    float w[64];
    const int* ids_dev;
    const float* w_dev;
    int ne;   // expert ids read from the device are clamped to 0 .. ne - 1
};
__device__ __forceinline__ int route_id(const MoeRoute& r, int i) {
    return r.ids_dev ? min(max(r.ids_dev[i], 0), r.ne - 1) : r.ids[i];
}
__device__ __forceinline__ float route_w(const MoeRoute& r, int i) { return r.w_dev ? r.w_dev[i] : r.w[i]; }

// Router (kernels.rs:1846-1872 topk_router; crates/strix-backend-cpu/src/mellum.rs:1178-1192): softmax over
// all ne logits, the k largest probabilities in descending order (equal probabilities: lowest index
// first, the order of the reference's stable sort), weights renormalised over the chosen k.  Experts more
// than 87 below the largest logit all get the probability exp(-87) (the fixed-sequence exp clamps its
// argument) and tie to the lowest index; their weight is below 2e-38 either way.  One wave;
// lane l holds experts l, l + 64, ... (PL of them: 1 for up to 64 experts, which keeps the k selection
// rounds at one compare each).  The softmax denominator is summed in double in a fixed order.
template <int PL>
__global__ __launch_bounds__(64) void topk_router_kernel(const float* __restrict__ logits, int ne, int k,
                                                         int* __restrict__ ids, float* __restrict__ w) {
    __shared__ float sel[64];
    float v[PL];
#pragma unroll
    for (int j = 0; j < PL; j++) {
        const int e = (int)threadIdx.x + 64 * j;
        v[j] = e < ne ? logits[e] : -3.40282347e+38f;
    }
    topk_router_wave<PL>(v, ne, k, ids, w, sel);
}

// Decode, second half, in one launch: a_k = quantised silu(g_k)*u_k is rebuilt in LDS by every
// workgroup (k*eff elements; measured faster than a launch of its own), then each wave computes
// output rows y[r] = sum_k w_k * sum_b dw*dx*I over the k routed experts' down-projection rows,
// k ascending (the roles of silu_quant, q8i_moe_down and moe_wsum, kernels.rs:879-892, 972-996,
// 1875-1882).  A lane owns 16-byte half blocks; the k*eff/16 units of a row are walked 64*UNR at
// a time with all UNR loads issued before the first use.  Workgroup 0 also writes the quantised
// activation out for the stage-by-stage checks.
template <int UNR>
__global__ __launch_bounds__(1024) void moe_down_fused_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                             const uint16_t* __restrict__ scales,
                                                             const uint4* __restrict__ quants, const MoeRoute route,
                                                             int k, int eff, int hidden, float* __restrict__ y,
                                                             int* __restrict__ aq_out, float* __restrict__ ad_out) {
    extern __shared__ __align__(16) char smem[];
    const int nbe = eff / 32;  // blocks per expert row
    int* sxq = (int*)smem;                          // [k][eff] int8
    float* sxd = (float*)(smem + (size_t)k * eff);  // [k][nbe]
    int* sid = (int*)(sxd + k * nbe);               // [k] expert ids
    float* sw = (float*)(sid + k);                  // [k] routing weights
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < k) {
        sid[tid] = route_id(route, tid);
        sw[tid] = route_w(route, tid);
    }
    __syncthreads();

    const int upe = eff / 16;  // 16-byte units per expert row
    const int units = k * upe;
    uint4 q[UNR];
    uint16_t sc[UNR];
    int uu[UNR];
    auto load_chunk = [&](int r, int base) {
#pragma unroll
        for (int j = 0; j < UNR; j++) {
            const int uidx = base + j * 64 + lane;
            const int uc = min(uidx, units - 1);
            const int kk = uc / upe, j16 = uc - kk * upe;
            const size_t rowblk = ((size_t)sid[kk] * hidden + r) * nbe;
            q[j] = quants[rowblk * 2 + j16];
            sc[j] = scales[rowblk + (j16 >> 1)];
            uu[j] = uidx < units ? uc : -1;
        }
    };
    const int items = k * eff / 4;  // float4 items, 8 per block; whole 8-lane groups are live or dead together
    for (int it0 = 0; it0 < items; it0 += 1024 * 2) {
        float4 gv[2], uv[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int it = it0 + j * 1024 + tid;
            gv[j] = uv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (it < items) {
                gv[j] = ((const float4*)g)[it];
                uv[j] = ((const float4*)u)[it];
            }
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int it = it0 + j * 1024 + tid;
            int packed;
            float d;
            silu_mul_quant4(gv[j], uv[j], &packed, &d);
            if (it < items) {
                sxq[it] = packed;
                if ((it & 7) == 0) sxd[it >> 3] = d;
                if (blockIdx.x == 0 && aq_out) {
                    aq_out[it] = packed;
                    if ((it & 7) == 0) ad_out[it >> 3] = d;
                }
            }
        }
    }
    __syncthreads();
    if (wave >= 8) return;  // waves 8..15 only help with the staging above
    int r = blockIdx.x * 8 + wave;
    if (r < hidden) load_chunk(r, 0);

    const uint4* sx16 = (const uint4*)smem;
    for (; r < hidden; r += gridDim.x * 8) {
        float acc = 0.f;
        for (int base = 0; base < units; base += 64 * UNR) {
            if (base > 0) load_chunk(r, base);
#pragma unroll
            for (int j = 0; j < UNR; j++) {
                const int uc = max(uu[j], 0);
                const int kk = uc / upe, j16 = uc - kk * upe;
                const uint4 xv = sx16[uc];
                int isum = dot4((int)q[j].x, (int)xv.x, 0);
                isum = dot4((int)q[j].y, (int)xv.y, isum);
                isum = dot4((int)q[j].z, (int)xv.z, isum);
                isum = dot4((int)q[j].w, (int)xv.w, isum);
                isum += swap1(isum);  // the other half of the block sits in the neighbouring lane
                const float dx = sxd[kk * nbe + (j16 >> 1)];
                const float term = sw[kk] * ((h2f(sc[j]) * dx) * (float)isum);
                acc += (uu[j] >= 0 && (lane & 1) == 0) ? term : 0.f;
            }
        }
        acc = group_sum<64>(acc);
        if (lane == 63) y[r] = acc;
        if (r + (int)gridDim.x * 8 < hidden) load_chunk(r + gridDim.x * 8, 0);
    }
}

// The same work in the flat form of the dense GEMV, for layers whose k*eff intermediate values fit four
// float4 items per thread: the units (16-byte half blocks) of a workgroup's rows, k experts side by
// side per row, form one sequence that the 16 waves walk in 64-unit loads, three loads per round.
// g and u are requested first and the weight loads follow without conditions, so waiting for g and u
// does not wait for the weights (a wave's loads complete in order) and every later wait is exact.
// Every GL-lane group lies inside one expert's row segment; its weighted sum goes to LDS and the groups
// of a row are added in ascending order (expert k ascending, blocks ascending).
// u == nullptr: g holds the finished products silu(g_k) * u_k (the paired gate/up launch wrote them) and only the
// quantiser runs here.
template <int GL>
__global__ __launch_bounds__(1024) void moe_down_flat_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                            const uint16_t* __restrict__ scales,
                                                            const uint4* __restrict__ quants, const MoeRoute route,
                                                            int k, int eff, int hidden, float* __restrict__ y,
                                                            int* __restrict__ aq_out, float* __restrict__ ad_out,
                                                            unsigned magic_units, unsigned magic_upe, int n_wgs) {
    extern __shared__ __align__(16) char smem[];
    constexpr int PRE = 3, XI = 4;
    const int nbe = eff / 32, upe = eff / 16, units = k * upe;
    int* sxq = (int*)smem;                          // [k][eff] int8
    float* sxd = (float*)(smem + (size_t)k * eff);  // [k][nbe]
    int* sid = (int*)(sxd + k * nbe);               // [k] expert ids
    float* sw = (float*)(sid + k);                  // [k] routing weights
    float* part = sw + k;                           // [rows * units / GL]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // g and u first: they do not depend on the routing, and the routing (read from the router's output when it ran
    // on the device) is a memory round trip of its own that the weight addresses have to wait for
    const int items = k * eff / 4;                  // float4 items, 8 per block; <= XI * 1024 (launcher)
    float4 gv[XI], uv[XI];
#pragma unroll
    for (int j = 0; j < XI; j++) {
        const int it = tid + j * 1024;
        gv[j] = uv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (it < items) {
            gv[j] = ((const float4*)g)[it];
            if (u) uv[j] = ((const float4*)u)[it];
        }
    }
    if (tid < k) {
        sid[tid] = route_id(route, tid);
        sw[tid] = route_w(route, tid);
    }
    __syncthreads();
    // (n_wgs = gridDim.x as an argument: the built-in is a load from the hidden arguments)
    const unsigned rbase = (unsigned)hidden / (unsigned)n_wgs, rrem = (unsigned)hidden - rbase * (unsigned)n_wgs;
    const int r0 = blockIdx.x * (int)rbase + min((int)blockIdx.x, (int)rrem);
    const int rows = (int)rbase + ((int)blockIdx.x < (int)rrem ? 1 : 0);
    const int nv = rows * units;                    // < 2^16 (launcher)
    const int nloads = (nv + 63) >> 6;

    uint4 q[PRE];
    uint16_t sc[PRE];
    int l_t = wave, c_t = wave;
    // virtual unit v of the workgroup -> (row, expert, half block)
    auto locate = [&](int v, int& rl, int& e, int& j16, int& uidx) {
        rl = (int)__umulhi((unsigned)v, magic_units);
        uidx = v - rl * units;
        e = (int)__umulhi((unsigned)uidx, magic_upe);
        j16 = uidx - e * upe;
    };
    auto request = [&]() {
#pragma unroll
        for (int s = 0; s < PRE; s++) {
            int rl, e, j16, uidx;
            locate(min(l_t * 64 + lane, max(nv - 1, 0)), rl, e, j16, uidx);
            const size_t rowblk = ((size_t)sid[e] * hidden + min(r0 + rl, hidden - 1)) * nbe;
            q[s] = quants[rowblk * 2 + j16];
            sc[s] = scales[rowblk + (j16 >> 1)];
            l_t += 16;
        }
    };
    const uint4* sx16 = (const uint4*)smem;
    auto consume = [&]() {
#pragma unroll
        for (int s = 0; s < PRE; s++) {
            if (c_t < nloads) {   // wave-uniform
                const int v = c_t * 64 + lane;
                const bool act = v < nv;
                int rl, e, j16, uidx;
                locate(act ? v : nv - 1, rl, e, j16, uidx);
                const uint4 xv = sx16[uidx];
                int isum = dot4((int)q[s].x, (int)xv.x, 0);
                isum = dot4((int)q[s].y, (int)xv.y, isum);
                isum = dot4((int)q[s].z, (int)xv.z, isum);
                isum = dot4((int)q[s].w, (int)xv.w, isum);
                isum += swap1(isum);  // the other half of the block sits in the neighbouring lane
                const float dx = sxd[e * nbe + (j16 >> 1)];
                const float term = sw[e] * ((h2f(sc[s]) * dx) * (float)isum);
                const float gs = small_group_sum<GL>((act && (lane & 1) == 0) ? term : 0.f);
                if (act && (lane & (GL - 1)) == GL - 1) part[v / GL] = gs;
            }
            c_t += 16;
        }
    };
    request();
#pragma unroll
    for (int j = 0; j < XI; j++) {
        const int it = tid + j * 1024;
        if ((it & ~63) < items) {   // whole waves are live or not together
            int packed;
            float d;
            if (u) silu_mul_quant4(gv[j], uv[j], &packed, &d);   // (workgroup-uniform)
            else quant4(gv[j], &packed, &d);
            if (it < items) {
                sxq[it] = packed;
                if ((it & 7) == 0) sxd[it >> 3] = d;
                if (blockIdx.x == 0 && aq_out) {
                    aq_out[it] = packed;
                    if ((it & 7) == 0) ad_out[it >> 3] = d;
                }
            }
        }
    }
    __syncthreads();
    consume();
    while (c_t < nloads) {
        request();
        consume();
    }
    __syncthreads();
    // a row's G group sums: 8 lanes take groups l, l + 8, ... (ascending), then a fixed DPP tree -- one thread per
    // row would pay the LDS latency G times in a row
    const int G = units / GL;
    for (int i8 = tid; i8 < rows * 8; i8 += 1024) {
        const int r = i8 >> 3, l = i8 & 7;
        float s = 0.f;
        for (int j = l; j < G; j += 8) s += part[r * G + j];
        s = small_group_sum<8>(s);
        if (l == 0) y[r0 + r] = s;
    }
}

// The same for Q6_K experts, in terms of the GEMV's per-format pieces (gemv_body.h): h holds the k * eff products
// silu(g_k) * u_k (the paired gate/up launch wrote them); every workgroup quantises them into the k experts' activation
// areas in LDS (a half block per thread), then walks its rows' units -- k experts side by side per row, four 64-element
// units per superblock -- one load round at a time.  A GL-lane group lies inside one expert's row segment.
template <int GL>
__global__ __launch_bounds__(1024) void moe_down_flat_q6_kernel(const float* __restrict__ h, const GemvW D, const MoeRoute route,
                                                               int k, int eff, int hidden, float* __restrict__ y,
                                                               unsigned magic_units, unsigned magic_upe, int n_wgs) {
    extern __shared__ __align__(16) char smem[];
    const int nsb = eff / 256, upe = nsb * 4, units = k * upe;   // superblocks and units per expert row
    const int tokb = OpsQ6_K::tok_bytes(nsb);
    int* sid = (int*)(smem + (size_t)k * tokb);   // [k] expert ids
    float* sw = (float*)(sid + k);                // [k] routing weights
    float* part = sw + k;                         // [rows * units / GL]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the products first: a 16-element half per thread (k * eff <= 16384, the launcher's bound)
    const int hbe = eff / 16, nhb = k * hbe;
    float4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = tid < nhb ? ((const float4*)h)[tid * 4 + j] : make_float4(0.f, 0.f, 0.f, 0.f);
    if (tid < k) {
        sid[tid] = route_id(route, tid);
        sw[tid] = route_w(route, tid);
    }
    __syncthreads();
    const unsigned rbase = (unsigned)hidden / (unsigned)n_wgs, rrem = (unsigned)hidden - rbase * (unsigned)n_wgs;
    const int r0 = blockIdx.x * (int)rbase + min((int)blockIdx.x, (int)rrem);
    const int rows = (int)rbase + ((int)blockIdx.x < (int)rrem ? 1 : 0);
    const int nv = rows * units;                  // < 2^16 (launcher)
    const int nloads = (nv + 63) >> 6;
    auto locate = [&](int vv, int& rl, int& e, int& u) {
        rl = (int)__umulhi((unsigned)vv, magic_units);
        const int uidx = vv - rl * units;
        e = (int)__umulhi((unsigned)uidx, magic_upe);
        u = uidx - e * upe;
    };
    OpsQ6_K::Regs regs;
    int l_t = wave, c_t = wave;
    auto request = [&]() {
        int rl, e, u;
        locate(min(l_t * 64 + lane, max(nv - 1, 0)), rl, e, u);
        OpsQ6_K::load_flat(regs, D, ((size_t)sid[e] * hidden + min(r0 + rl, hidden - 1)) * upe + u);
        l_t += 16;
    };
    auto consume = [&]() {
        if (c_t < nloads) {   // wave-uniform
            const int vv = c_t * 64 + lane;
            const bool act = vv < nv;
            int rl, e, u;
            locate(act ? vv : nv - 1, rl, e, u);
            float acc[1] = {0.f};
            compute_unit<1, false>(OpsQ6_K(), regs, smem + (size_t)e * tokb, tokb, nsb, u, act, acc, nullptr);
            const float gs = small_group_sum<GL>(act ? sw[e] * acc[0] : 0.f);
            if (act && (lane & (GL - 1)) == GL - 1) part[vv / GL] = gs;
        }
        c_t += 16;
    };
    request();
    if ((tid & ~63) < nhb) {   // whole waves
        const int e = tid / hbe;
        quantize_half_block<OpsQ6_K>(smem + (size_t)min(e, k - 1) * tokb, nsb, tid - e * hbe, tid < nhb, v);
    }
    __syncthreads();
    consume();
    while (c_t < nloads) {
        request();
        consume();
    }
    __syncthreads();
    const int G = units / GL;
    for (int i8 = tid; i8 < rows * 8; i8 += 1024) {
        const int r = i8 >> 3, l = i8 & 7;
        float s = 0.f;
        for (int j = l; j < G; j += 8) s += part[r * G + j];
        s = small_group_sum<8>(s);
        if (l == 0) y[r0 + r] = s;
    }
}

// y[t][i] = sum over the token's slots (ascending slot index) of wslot[s]*dy[s][i].  Eight slots at a
// time: their indices, weights and rows are requested together (clamped, not conditional, so the
// loads of a batch are in flight at once instead of one dependent round trip per slot).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ dy, const int* __restrict__ tok_ptr,
                                                          const int* __restrict__ tok_slots,
                                                          const float* __restrict__ wslot, float* __restrict__ y,
                                                          int hidden, bool y_vec) {
    const int t = blockIdx.y, i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= hidden) return;
    const int j0 = tok_ptr[t], j1 = tok_ptr[t + 1];
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int jb = j0; jb < j1; jb += 8) {
        int sl[8];
        float w[8];
        float4 v[8];
#pragma unroll
        for (int q = 0; q < 8; q++) sl[q] = tok_slots[min(jb + q, j1 - 1)];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            w[q] = wslot[sl[q]];
            v[q] = *(const float4*)(dy + (size_t)sl[q] * hidden + i);
        }
#pragma unroll
        for (int q = 0; q < 8; q++) {
            if (jb + q < j1) {
                s.x += w[q] * v[q].x;
                s.y += w[q] * v[q].y;
                s.z += w[q] * v[q].z;
                s.w += w[q] * v[q].w;
            }
        }
    }
    float* o = y + (size_t)t * hidden + i;
    if (y_vec) {   // the caller's buffer is 16-byte aligned
        *(float4*)o = s;
    } else {
        o[0] = s.x; o[1] = s.y; o[2] = s.z; o[3] = s.w;
    }
}

static int silu_mul_quant(smx_ctx* c, const float* g, const float* u, size_t ldg, size_t rows, size_t eff, int8_t* xq,
                          float* xd) {
    const size_t nblocks = rows * (eff / 32);
    ProfScope ps(c, "silu_mul_quant");
    hipLaunchKernelGGL(silu_mul_quant_kernel, dim3((unsigned)((nblocks * 8 + 255) / 256)), dim3(256), 0, c->stream, g, u,
                       ldg, (int)eff, (int*)xq, xd, nblocks);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

// out[o] = sum_k wexp[k]*dy[k][o], k ascending (kernels.rs:1875-1882); used by the Q6_K expert path
__global__ __launch_bounds__(256) void moe_wsum_kernel(const float* __restrict__ dy, const MoeRoute route,
                                                       float* __restrict__ out, int n, int k) {
    const int o = blockIdx.x * 256 + threadIdx.x;
    if (o >= n) return;
    float s = 0.f;
    for (int e = 0; e < k; e++) s += route_w(route, e) * dy[(size_t)e * n + o];
    out[o] = s;
}

// Rows [e*rows, (e+1)*rows) of a stacked expert tensor as a weight of its own (planes are row-major).
static Weight expert_view(const Weight& src, size_t e, size_t rows) {
    Weight v = src;
    v.N = rows;
    const size_t b0 = e * rows * src.nblk;  // first block / superblock of the expert
    v.scales = src.scales + b0;
    if (src.type == kQ6_K) {
        v.quants = (const char*)src.quants + b0 * 128;
        v.qh = (const char*)src.qh + b0 * 64;
        v.sc = src.sc + b0 * 16;
    } else {
        v.quants = (const char*)src.quants + b0 * (src.type == kQ4_0 ? 16 : 32);
    }
    return v;
}

// Scratch carve-up helper: 256-byte aligned bump allocation inside one DevBuf.
struct Carver {
    size_t off = 0;
    size_t take(size_t bytes) {
        const size_t o = off;
        off += (bytes + 255) & ~size_t(255);
        return o;
    }
};

// One token through k routed experts; x_dev fp32 [hidden] on the device, y_dev fp32 [hidden].
// Intermediates live in c->work: g[k][eff], u[k][eff], and a copy of the quantised activation
// aq[k][eff], ad[k][eff/32] for the stage-by-stage checks.
struct MoeScratch {
    float *g, *u;
    int8_t* aq;
    float* ad;
};

// ids / wexp: the routing on the host; or, with ids_dev / w_dev, device memory read when the kernels run; or, with logits_dev
// as well, the routing is computed from the router logits by the gate/up launch itself (which writes ids_dev / w_dev for
// the down launch), or by a routing launch in front where that form does not serve.
static int moe_ffn_enqueue(smx_ctx* c, const MoeLayer& L, const int32_t* ids, const float* wexp, size_t k,
                           const float* x_dev, float* y_dev, MoeScratch* out_scratch, const int32_t* ids_dev = nullptr,
                           const float* w_dev = nullptr, const float* logits_dev = nullptr) {
    if (k == 0 || k > 64) return fail(c, SMX_ERR_LIMIT, "moe_ffn: %zu routed experts (1..64 supported)", k);
    const bool routed_on_device = ids_dev != nullptr;
    bool route_pending = logits_dev != nullptr;   // the routing has not been computed yet
    for (size_t i = 0; i < k && !routed_on_device; i++)
        if (ids[i] < 0 || (size_t)ids[i] >= L.ne)
            return fail(c, SMX_ERR_ARG, "moe_ffn: expert id %d outside 0..%zu", ids[i], L.ne - 1);
    const size_t hidden = L.hidden, eff = L.eff;
    int rc;
    Carver cv;
    const size_t o_g = cv.take(k * eff * 4), o_u = cv.take(k * eff * 4), o_aq = cv.take(k * eff),
                 o_ad = cv.take(k * (eff / 32) * 4), o_dy = cv.take(L.type == kQ6_K ? k * hidden * 4 : 0),
                 o_h = cv.take(k * eff * 4);
    if ((rc = ensure(c, c->work, cv.off)) != SMX_OK) return rc;
    MoeRoute route = {};
    route.ids_dev = ids_dev;
    route.w_dev = w_dev;
    route.ne = (int)L.ne;
    for (size_t i = 0; i < k && !routed_on_device; i++) {
        route.ids[i] = ids[i];
        route.w[i] = wexp[i];
    }
    // With the routing on the device every job is a view of expert 0 and the kernel moves it to the
    // expert it reads from ids_dev (GemvIndirect).
    GemvIndirect ind = {};
    ind.ids = ids_dev;
    ind.ne = (int)L.ne;
    bool paired = false;   // the gate/up launch left silu(g) * u at o_h
    MoeScratch s;
    s.g = (float*)(c->work.p + o_g);
    s.u = (float*)(c->work.p + o_u);
    s.aq = (int8_t*)(c->work.p + o_aq);
    s.ad = (float*)(c->work.p + o_ad);
    // gate and up of every routed expert: 2k single-row GEMVs over the same activation, grouped
    // SMX_GEMV_GROUP_MAX to a launch (the activation quantiser runs inside the GEMV's staging)
    {
        std::vector<Weight> views(2 * k);
        std::vector<const Weight*> ws(2 * k);
        std::vector<const float*> xs(2 * k, x_dev);
        std::vector<float*> ys(2 * k);
        for (size_t i = 0; i < k; i++)
            for (int z = 0; z < 2; z++) {
                views[2 * i + z] = expert_view(z ? L.up : L.gate, routed_on_device ? 0 : (size_t)ids[i], eff);
                ws[2 * i + z] = &views[2 * i + z];
                ys[2 * i + z] = (z ? s.u : s.g) + i * eff;
            }
        ind.blocks_per_expert = eff * L.gate.nblk;
        // gate and up of an expert as one paired job with silu(g) * u in the kernel's tail (g and u are still
        // written: the stage-by-stage checks read them); the down kernel then only quantises the products
        {
            std::vector<const Weight*> wgp(k), wup(k);
            std::vector<float*> ygp(k), yup(k), hp(k);
            for (size_t i = 0; i < k; i++) {
                wgp[i] = ws[2 * i]; wup[i] = ws[2 * i + 1];
                ygp[i] = ys[2 * i]; yup[i] = ys[2 * i + 1];
                hp[i] = (float*)(c->work.p + o_h) + i * eff;
            }
            constexpr int kPairs = SMX_GEMV_GROUP_MAX / 2;
            paired = true;
            // the routing inside the gate/up launch: one launch of all k pairs, up to 64 experts
            const bool route_here = route_pending && k <= (size_t)kPairs && L.ne <= 64 && k <= L.ne;
            if (route_pending && !route_here) {
                if ((rc = smx_moe_route_dev(c, logits_dev, L.ne, k, (int32_t*)ids_dev, (float*)w_dev)) != SMX_OK) return rc;
                route_pending = false;
            }
            for (size_t i = 0; i < k && paired; i += kPairs) {
                const int n = (int)std::min<size_t>(kPairs, k - i);
                for (int j = 0; j < n; j++) ind.slot[j] = (int)(i + j);
                bool served = false;
                GemvIndirect ind2 = ind;
                if (route_pending) {
                    ind2.logits = logits_dev;
                    ind2.route_k = (int)k;
                    ind2.ids_out = (int*)ids_dev;
                    ind2.w_out = (float*)w_dev;
                }
                rc = launch_gemv_dual(c, &wgp[i], &wup[i], &xs[i], &ygp[i], &yup[i], &hp[i], n, SMX_ACT_SILU_MUL, nullptr,
                                      "moe_gemv_gate_up", &served, routed_on_device ? &ind2 : nullptr);
                if (rc != SMX_OK) return rc;
                if (!served) paired = false;   // (the first chunk decides: every chunk has the same shape)
                else route_pending = false;
            }
            if (route_pending) {   // the paired form does not serve this shape: the routing launch, then the grouped launch below
                if ((rc = smx_moe_route_dev(c, logits_dev, L.ne, k, (int32_t*)ids_dev, (float*)w_dev)) != SMX_OK) return rc;
                route_pending = false;
            }
        }
        for (size_t i = 0; i < 2 * k && !paired; i += SMX_GEMV_GROUP_MAX) {
            const int n = (int)std::min<size_t>(SMX_GEMV_GROUP_MAX, 2 * k - i);
            for (int j = 0; j < n; j++) ind.slot[j] = (int)((i + j) / 2);
            rc = launch_gemv_group(c, &ws[i], &xs[i], &ys[i], n, "moe_gemv_gate_up", nullptr, nullptr,
                                   routed_on_device ? &ind : nullptr);
            if (rc != SMX_OK) return rc;
        }
    }
    bool q6_flat = false;
    if (L.type == kQ6_K && paired) {
        // Q6_K experts, second launch in the flat form: quantiser + the k down projections + the weighted sum
        const size_t nsb = eff / 256, upe = nsb * 4, units = k * upe;
        const size_t tokb = nsb * 2 * (OpsQ6_K::kPad * 16 + 32);
        const size_t fgrid = std::min<size_t>(hidden, (size_t)c->num_cu);
        const size_t frows = (hidden + fgrid - 1) / fgrid;
        const int gl = upe % 16 == 0 ? 16 : (upe % 8 == 0 ? 8 : 4);
        const size_t flds = k * tokb + k * 8 + frows * units / gl * 4;
        if (k * eff <= 16384 && frows * units < 65536 && flds <= 160 * 1024) {
            q6_flat = true;
            ProfScope ps(c, "moe_gemv_down");
            const GemvW D = {L.down.scales, (const uint4*)L.down.quants, (const uint4*)L.down.qh, (const uint2*)L.down.sc};
            const unsigned m_units = (unsigned)(((1ull << 32) + units - 1) / units), m_upe = (unsigned)(((1ull << 32) + upe - 1) / upe);
            auto launch = [&](auto kern) -> int {
                int rc2 = set_dyn_lds(c, kern, flds);
                if (rc2 != SMX_OK) return rc2;
                hipLaunchKernelGGL(kern, dim3((unsigned)fgrid), dim3(1024), flds, c->stream, (const float*)(c->work.p + o_h), D, route,
                                   (int)k, (int)eff, (int)hidden, y_dev, m_units, m_upe, (int)fgrid);
                SMX_HIP(c, hipGetLastError());
                return SMX_OK;
            };
            rc = gl == 16 ? launch(moe_down_flat_q6_kernel<16>) : (gl == 8 ? launch(moe_down_flat_q6_kernel<8>) : launch(moe_down_flat_q6_kernel<4>));
            if (rc != SMX_OK) return rc;
            if (out_scratch) {  // the quantised activation stays in LDS on this path: rebuild it for the checks
                rc = silu_mul_quant(c, s.g, s.u, eff, k, eff, s.aq, s.ad);
                if (rc != SMX_OK) return rc;
            }
        }
    }
    if (q6_flat) {
    } else if (L.type == kQ6_K) {
        // Q6_K experts (decode.rs:2839-2852, moe6_launches): the down projections are k more jobs of the
        // grouped GEMV, each quantising silu(g_k)*u_k inside its staging; then the weighted sum
        float* dy = (float*)(c->work.p + o_dy);
        std::vector<Weight> views(k);
        std::vector<const Weight*> ws(k);
        std::vector<const float*> gs(k), us(k);
        std::vector<float*> ys(k);
        for (size_t i = 0; i < k; i++) {
            views[i] = expert_view(L.down, routed_on_device ? 0 : (size_t)ids[i], hidden);
            ws[i] = &views[i];
            gs[i] = s.g + i * eff;
            us[i] = s.u + i * eff;
            ys[i] = dy + i * hidden;
        }
        const ActProd prod = {SMX_ACT_SILU_MUL, nullptr, 0.f};
        ind.blocks_per_expert = hidden * L.down.nblk;
        for (size_t i = 0; i < k; i += SMX_GEMV_GROUP_MAX) {
            const int n = (int)std::min<size_t>(SMX_GEMV_GROUP_MAX, k - i);
            for (int j = 0; j < n; j++) ind.slot[j] = (int)(i + j);
            rc = launch_gemv_group(c, &ws[i], &gs[i], &ys[i], n, "moe_gemv_down", &prod, &us[i], routed_on_device ? &ind : nullptr);
            if (rc != SMX_OK) return rc;
        }
        {
            ProfScope ps(c, "moe_wsum");
            hipLaunchKernelGGL(moe_wsum_kernel, dim3((unsigned)((hidden + 255) / 256)), dim3(256), 0, c->stream, dy, route,
                               y_dev, (int)hidden, (int)k);
            SMX_HIP(c, hipGetLastError());
        }
        if (out_scratch) {  // the quantised activation is never materialised on this path: rebuild it for the checks
            rc = silu_mul_quant(c, s.g, s.u, eff, k, eff, s.aq, s.ad);
            if (rc != SMX_OK) return rc;
        }
    } else {
        const size_t lds = k * eff + k * (eff / 32) * 4 + k * 8;
        if (lds > 160 * 1024)
            return fail(c, SMX_ERR_LIMIT, "moe_ffn: %zu experts x %zu intermediate values need %zu bytes of LDS (limit 163840)",
                        k, eff, lds);
        ProfScope ps(c, "moe_gemv_down");
        const size_t upe = eff / 16, units = k * upe;
        const size_t fgrid = std::min<size_t>(hidden, (size_t)c->num_cu);
        const size_t frows = (hidden + fgrid - 1) / fgrid;
        const int gl = upe % 16 == 0 ? 16 : (upe % 8 == 0 ? 8 : (upe % 4 == 0 ? 4 : 2));
        const size_t flds = lds + frows * units / gl * 4;
        if (k * eff <= 4 * 1024 * 4 && frows * units < 65536 && flds <= 160 * 1024) {
            const unsigned m_units = (unsigned)(((1ull << 32) + units - 1) / units), m_upe = (unsigned)(((1ull << 32) + upe - 1) / upe);
            auto launch = [&](auto kern) -> int {
                int rc2 = set_dyn_lds(c, kern, flds);
                if (rc2 != SMX_OK) return rc2;
                const float* hsrc = (const float*)(c->work.p + o_h);
                hipLaunchKernelGGL(kern, dim3((unsigned)fgrid), dim3(1024), flds, c->stream, paired ? hsrc : (const float*)s.g,
                                   paired ? (const float*)nullptr : (const float*)s.u, L.down.scales,
                                   (const uint4*)L.down.quants, route, (int)k, (int)eff, (int)hidden, y_dev, (int*)s.aq, s.ad,
                                   m_units, m_upe, (int)fgrid);
                SMX_HIP(c, hipGetLastError());
                return SMX_OK;
            };
            if (gl == 16) rc = launch(moe_down_flat_kernel<16>);
            else if (gl == 8) rc = launch(moe_down_flat_kernel<8>);
            else if (gl == 4) rc = launch(moe_down_flat_kernel<4>);
            else rc = launch(moe_down_flat_kernel<2>);
            if (rc != SMX_OK) return rc;
        } else {
            auto kern = moe_down_fused_kernel<6>;
            if ((rc = set_dyn_lds(c, kern, lds)) != SMX_OK) return rc;
            const unsigned grid = (unsigned)std::min<size_t>((hidden + 7) / 8, (size_t)c->num_cu * 2);
            hipLaunchKernelGGL(kern, dim3(grid), dim3(1024), lds, c->stream, s.g, s.u, L.down.scales, (const uint4*)L.down.quants,
                               route, (int)k, (int)eff, (int)hidden, y_dev, (int*)s.aq, s.ad);
            SMX_HIP(c, hipGetLastError());
        }
    }
    if (out_scratch) *out_scratch = s;
    return SMX_OK;
}

// out[i] += sd[i] * sgate (kernels.rs:1747-1751 shexp_add)
__global__ __launch_bounds__(256) void shexp_add_kernel(float* __restrict__ out, const float* __restrict__ sd, float sgate, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] += sd[i] * sgate;
}

// The layer's shared expert, added onto y (decode.rs:1820-1855 queue_shexp): the dense FFN
// blk.<layer>.ffn_{gate,up,down}_shexp.weight over the same activation, scaled by the caller's gate.
// Gate and up share one grouped GEMV launch; silu(g)*u is quantised inside the down GEMV's staging
// (or in a launch of its own on long rows).  Declines when the three weights are not resident.
static int shexp_enqueue(smx_ctx* c, size_t layer, size_t hidden, float sgate, const float* x_dev, float* y_dev) {
    const std::string base = "blk." + std::to_string(layer) + ".ffn_";
    const Weight* w[3];
    const char* part[3] = {"gate", "up", "down"};
    for (int i = 0; i < 3; i++) {
        auto it = c->weights.find(base + part[i] + "_shexp.weight");
        if (it == c->weights.end()) return SMX_NOT_RESIDENT;
        w[i] = &it->second;
    }
    const size_t sff = w[0]->N;
    if (w[0]->K != hidden || w[1]->K != hidden || w[1]->N != sff || w[1]->type != w[0]->type || w[2]->K != sff ||
        w[2]->N != hidden)
        return fail(c, SMX_ERR_ARG, "moe_ffn: shared expert of layer %zu has shapes %zux%zu, %zux%zu, %zux%zu for hidden %zu",
                    layer, w[0]->N, w[0]->K, w[1]->N, w[1]->K, w[2]->N, w[2]->K, hidden);
    Carver cv;
    const size_t o_g = cv.take(sff * 4), o_u = cv.take(sff * 4), o_d = cv.take(hidden * 4);
    int rc = ensure(c, c->work2, cv.off);
    if (rc != SMX_OK) return rc;
    float* g = (float*)(c->work2.p + o_g);
    float* u = (float*)(c->work2.p + o_u);
    float* sd = (float*)(c->work2.p + o_d);
    {   // gate and up with the SwiGLU product in the kernel's tail (h lands in g) where the shape takes the flat form
        const float* xs[2] = {x_dev, x_dev};
        float* hs[1] = {g};
        bool served = false;
        if ((rc = launch_gemv_dual(c, &w[0], &w[1], xs, nullptr, nullptr, hs, 1, SMX_ACT_SILU_MUL, nullptr, "shexp_gate_up", &served)) != SMX_OK)
            return rc;
        if (served) {
            const float* hx[1] = {g};
            float* ys[1] = {sd};
            if ((rc = launch_gemv_group(c, &w[2], hx, ys, 1, "shexp_down")) != SMX_OK) return rc;
        } else {
            const Weight* ws[2] = {w[0], w[1]};
            float* ys2[2] = {g, u};
            if ((rc = launch_gemv_group(c, ws, xs, ys2, 2, "shexp_gate_up")) != SMX_OK) return rc;
            const ActProd prod = {SMX_ACT_SILU_MUL, u, 0.f};
            const float* gx[1] = {g};
            float* ys[1] = {sd};
            if ((rc = launch_gemv_group(c, &w[2], gx, ys, 1, "shexp_down", &prod)) != SMX_OK) return rc;
        }
    }
    ProfScope ps(c, "shexp_add");
    hipLaunchKernelGGL(shexp_add_kernel, dim3((unsigned)((hidden + 255) / 256)), dim3(256), 0, c->stream, y_dev, sd, sgate,
                       (int)hidden);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

static int moe_ffn_host(smx_ctx* c, size_t layer, const int32_t* ids, const float* wexp, size_t k, const float* x,
                        size_t x_len, float sgate, float* y, size_t y_cap, float* gu, int8_t* aq, float* ad) {
    if (!c) return SMX_ERR_ARG;
    if (!ids || !wexp || !x || !y) return fail(c, SMX_ERR_ARG, "moe_ffn: null argument");
    return guarded(c, "moe_ffn", [&]() -> int {
    auto it = c->moe.find(layer);
    if (it == c->moe.end()) return SMX_NOT_RESIDENT;
    const MoeLayer& L = it->second;
    if (x_len != L.hidden) return fail(c, SMX_ERR_ARG, "moe_ffn: activation length %zu, hidden %zu", x_len, L.hidden);
    if (y_cap < L.hidden) return fail(c, SMX_ERR_ARG, "moe_ffn: output capacity %zu < %zu", y_cap, L.hidden);
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, L.hidden * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->yf32, L.hidden * 4)) != SMX_OK) return rc;
    // The token's row and the result travel through the context's pinned staging; the kernels read the row there themselves
    // (up to 64 KB) and, when no shared expert adds onto the result afterwards, write the result there too: a copy command
    // costs 3 us in front of the kernels and 9 - 11 us behind them (smx_gemv does the same).
    const size_t hb = L.hidden * 4;
    if ((rc = ensure_host(c, c->hx, hb)) != SMX_OK) return rc;
    if ((rc = ensure_host(c, c->hy, hb)) != SMX_OK) return rc;
    memcpy(c->hx.p, x, hb);
    const bool x_direct = hb <= (size_t(64) << 10) && c->tune_host_io == 0, y_direct = sgate == 0.0f && c->tune_host_io != 1;
    if (!x_direct) SMX_HIP(c, hipMemcpyAsync(c->xf32.p, c->hx.p, hb, hipMemcpyHostToDevice, c->stream));
    const float* x_dev = x_direct ? (const float*)c->hx.p : (const float*)c->xf32.p;
    MoeScratch s;
    rc = moe_ffn_enqueue(c, L, ids, wexp, k, x_dev, y_direct ? (float*)c->hy.p : (float*)c->yf32.p, &s);
    if (rc != SMX_OK) return rc;
    if (sgate != 0.0f) {  // decode.rs:2850, 2865: no shared expert resident -> the whole call declines
        rc = shexp_enqueue(c, layer, L.hidden, sgate, x_dev, (float*)c->yf32.p);
        if (rc != SMX_OK) {
            (void)hipStreamSynchronize(c->stream);
            return rc;
        }
    }
    if (!y_direct) SMX_HIP(c, hipMemcpyAsync(c->hy.p, c->yf32.p, hb, hipMemcpyDeviceToHost, c->stream));
    if (gu) {
        for (size_t kk = 0; kk < k; kk++) {
            SMX_HIP(c, hipMemcpyAsync(gu + (kk * 2) * L.eff, s.g + kk * L.eff, L.eff * 4, hipMemcpyDeviceToHost, c->stream));
            SMX_HIP(c, hipMemcpyAsync(gu + (kk * 2 + 1) * L.eff, s.u + kk * L.eff, L.eff * 4, hipMemcpyDeviceToHost, c->stream));
        }
    }
    if (aq) SMX_HIP(c, hipMemcpyAsync(aq, s.aq, k * L.eff, hipMemcpyDeviceToHost, c->stream));
    if (ad) SMX_HIP(c, hipMemcpyAsync(ad, s.ad, k * (L.eff / 32) * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    memcpy(y, c->hy.p, hb);
    return SMX_OK;
    });
}

// Tile table of one grouped GEMM stage: for every plan entry, ceil(cnt/128) x ceil(rows/128) tiles.
static void build_tiles(const size_t* plan, size_t nplan, size_t rows_per_expert, std::vector<GemmTile>* tiles) {
    tiles->clear();
    for (size_t i = 0; i < nplan; i++) {
        const int e = (int)plan[i * 3], off = (int)plan[i * 3 + 1], cnt = (int)plan[i * 3 + 2];
        for (int tn = 0; tn * 128 < (int)rows_per_expert; tn++)      // tiles of one weight strip are adjacent
            for (int tm = 0; tm * 128 < cnt; tm++) {
                GemmTile t;
                t.tok0 = off + tm * 128;
                t.tok_end = off + cnt;
                t.row0 = e * (int)rows_per_expert + tn * 128;
                t.row_end = (e + 1) * (int)rows_per_expert;
                t.col0 = tn * 128;
                tiles->push_back(t);
            }
    }
    // Longest first: a tile's time follows the row tiles each of its waves computes (4 with more than 64 live
    // tokens, 2 up to 64, 1 up to 32), and workgroups start in table order, so the long tiles must not be
    // the last to start.  Equal-cost tiles keep their order (tiles of one weight strip stay adjacent).
    auto cost = [](const GemmTile& t) { const int live = t.tok_end - t.tok0; return live > 64 ? 4 : live > 32 ? 2 : 1; };
    std::stable_sort(tiles->begin(), tiles->end(), [&](const GemmTile& a, const GemmTile& b) { return cost(a) > cost(b); });
}

}  // namespace smx

using namespace smx;

extern "C" {

int smx_moe_ffn(smx_ctx* c, size_t layer, const int32_t* ids, const float* wexp, size_t k, const float* x, size_t x_len,
                float sgate, float* y, size_t y_cap) {
    return moe_ffn_host(c, layer, ids, wexp, k, x, x_len, sgate, y, y_cap, nullptr, nullptr, nullptr);
}

int smx_moe_ffn_stages(smx_ctx* c, size_t layer, const int32_t* ids, const float* wexp, size_t k, const float* x,
                       size_t x_len, float* y, float* gu, int8_t* aq, float* ad) {
    return moe_ffn_host(c, layer, ids, wexp, k, x, x_len, 0.0f, y, x_len, gu, aq, ad);
}

int smx_moe_ffn_dev(smx_ctx* c, size_t layer, const int32_t* ids, const float* wexp, size_t k, const float* x_dev,
                    float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!ids || !wexp || !x_dev || !y_dev) return fail(c, SMX_ERR_ARG, "moe_ffn_dev: null argument");
    return guarded(c, "moe_ffn_dev", [&]() -> int {
        auto it = c->moe.find(layer);
        if (it == c->moe.end()) return SMX_NOT_RESIDENT;
        return moe_ffn_enqueue(c, it->second, ids, wexp, k, x_dev, y_dev, nullptr);
    });
}

int smx_moe_route_dev(smx_ctx* c, const float* logits_dev, size_t ne, size_t k, int32_t* ids_dev, float* w_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!logits_dev || !ids_dev || !w_dev) return fail(c, SMX_ERR_ARG, "moe_route_dev: null argument");
    if (ne == 0 || ne > 64 * kRouterPerLane || k == 0 || k > 64 || k > ne)
        return fail(c, SMX_ERR_LIMIT, "moe_route_dev: %zu experts, top %zu (up to %d experts, top 64)", ne, k, 64 * kRouterPerLane);
    ProfScope ps(c, "topk_router");
    auto kern = ne <= 64 ? topk_router_kernel<1> : ne <= 256 ? topk_router_kernel<4> : topk_router_kernel<kRouterPerLane>;
    hipLaunchKernelGGL(kern, dim3(1), dim3(64), 0, c->stream, logits_dev, (int)ne, (int)k, ids_dev, w_dev);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

int smx_moe_router_dev(smx_ctx* c, const char* key, const float* x_dev, size_t k, int32_t* ids_dev, float* w_dev, float* logits_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !x_dev || !ids_dev || !w_dev) return fail(c, SMX_ERR_ARG, "moe_router_dev: null argument");
    return guarded(c, "moe_router_dev", [&]() -> int {
        auto it = c->weights.find(key);
        if (it == c->weights.end()) return SMX_NOT_RESIDENT;
        const Weight& w = it->second;
        const size_t ne = w.N;
        if (ne > 64 * (size_t)kRouterPerLane || k == 0 || k > 64 || k > ne)
            return fail(c, SMX_ERR_LIMIT, "moe_router_dev: %zu experts, top %zu (up to %d experts, top 64)", ne, k, 64 * kRouterPerLane);
        int rc;
        if (!logits_dev) {   // the logits still pass through memory: the context's own room when the caller does not want them
            if ((rc = ensure(c, c->yf32, ne * 4)) != SMX_OK) return rc;
            logits_dev = (float*)c->yf32.p;
        }
        // Two launches: the GEMV over all CUs (2.4 us back to back for a 64 x 2048 Q8_0 router, launch-bound) and the one-wave
        // routing kernel (3.2 us).  ONE launch -- a single 16-wave workgroup running the flat GEMV over the whole router weight,
        // then routing the logits it just stored -- was built and gave the same bits, but took 6.6-6.9 us against 5.7-5.9 us:
        // on one CU the activation fetch, the 139 KB of weights, the row sums, the store and the routing run one after the
        // other, and together they cost more than the second launch.
        if ((rc = launch_gemv(c, w, x_dev, 1, logits_dev, nullptr)) != SMX_OK) return rc;
        return smx_moe_route_dev(c, logits_dev, ne, k, ids_dev, w_dev);
    });
}

int smx_moe_route(smx_ctx* c, const float* logits, size_t ne, size_t k, int32_t* ids, float* w) {
    if (!c) return SMX_ERR_ARG;
    if (!logits || !ids || !w) return fail(c, SMX_ERR_ARG, "moe_route: null argument");
    if (ne == 0 || k == 0 || k > 64) return fail(c, SMX_ERR_LIMIT, "moe_route: %zu experts, top %zu", ne, k);
    SMX_HIP(c, hipSetDevice(c->device));
    int rc;
    if ((rc = ensure(c, c->xf32, ne * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->tab, 2 * 64 * 4)) != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(c->xf32.p, logits, ne * 4, hipMemcpyHostToDevice, c->stream));
    rc = smx_moe_route_dev(c, (const float*)c->xf32.p, ne, k, (int32_t*)c->tab.p, (float*)(c->tab.p + 256));
    if (rc != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(ids, c->tab.p, k * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipMemcpyAsync(w, c->tab.p + 256, k * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
}

int smx_moe_ffn_routed_dev(smx_ctx* c, size_t layer, const int32_t* ids_dev, const float* w_dev, size_t k, const float* x_dev,
                           float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!ids_dev || !w_dev || !x_dev || !y_dev) return fail(c, SMX_ERR_ARG, "moe_ffn_routed_dev: null argument");
    return guarded(c, "moe_ffn_routed_dev", [&]() -> int {
        auto it = c->moe.find(layer);
        if (it == c->moe.end()) return SMX_NOT_RESIDENT;
        return moe_ffn_enqueue(c, it->second, nullptr, nullptr, k, x_dev, y_dev, nullptr, ids_dev, w_dev);
    });
}

int smx_moe_ffn_logits_dev(smx_ctx* c, size_t layer, const float* logits_dev, size_t k, const float* x_dev, float* y_dev,
                           int32_t* ids_dev, float* w_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!logits_dev || !ids_dev || !w_dev || !x_dev || !y_dev) return fail(c, SMX_ERR_ARG, "moe_ffn_logits_dev: null argument");
    return guarded(c, "moe_ffn_logits_dev", [&]() -> int {
        auto it = c->moe.find(layer);
        if (it == c->moe.end()) return SMX_NOT_RESIDENT;
        const MoeLayer& L = it->second;
        if (L.ne > 64 * (size_t)kRouterPerLane || k == 0 || k > 64 || k > L.ne)
            return fail(c, SMX_ERR_LIMIT, "moe_ffn_logits_dev: %zu experts, top %zu (up to %d experts, top 64)", L.ne, k, 64 * kRouterPerLane);
        return moe_ffn_enqueue(c, L, nullptr, nullptr, k, x_dev, y_dev, nullptr, ids_dev, w_dev, logits_dev);
    });
}

int smx_moe_shexp_dev(smx_ctx* c, size_t layer, float sgate, const float* x_dev, float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!x_dev || !y_dev) return fail(c, SMX_ERR_ARG, "moe_shexp_dev: null argument");
    return guarded(c, "moe_shexp_dev", [&]() -> int {
        auto it = c->moe.find(layer);
        if (it == c->moe.end()) return SMX_NOT_RESIDENT;
        return shexp_enqueue(c, layer, it->second.hidden, sgate, x_dev, y_dev);
    });
}

// The grouped expert FFN over a slot table: quantise the m activation rows, gate and up of every
// expert group in one GEMM launch (slot s reads activation row rowmap[s], or row s when rowmap is
// null), silu(g)*u re-quantised, down in a second GEMM launch.  dy[slots][hidden] is left in c->work.
// The two tile tables (device pointers) are those of build_tiles over the plan for eff and hidden rows.
struct SlotScratch {
    float *g, *u;   // [slots][eff] gate and up outputs
    int8_t* aq;     // [slots][eff] quantised silu(g)*u
    float* ad;      // [slots][eff/32]
    float* dy;      // [slots][hidden] unweighted down outputs
};
static int moe_slots_enqueue(smx_ctx* c, const MoeLayer& L, const float* x_dev, size_t m, const int* rowmap_dev, size_t slots,
                             const GemmTile* tiles_gu, size_t n_gu, const GemmTile* tiles_dn, size_t n_dn, SlotScratch* out) {
    const size_t hidden = L.hidden, eff = L.eff, nb = hidden / 32, enb = eff / 32;
    int rc;
    if ((rc = ensure(c, c->xq, m * hidden)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->xd, m * nb * 4)) != SMX_OK) return rc;
    if ((rc = ensure(c, c->xs, m * nb * 4)) != SMX_OK) return rc;
    Carver cv;
    const size_t o_g = cv.take(slots * eff * 4), o_u = cv.take(slots * eff * 4), o_aq = cv.take(slots * eff),
                 o_ad = cv.take(slots * enb * 4), o_dy = cv.take(slots * hidden * 4);
    if ((rc = ensure(c, c->work, cv.off)) != SMX_OK) return rc;
    float* g = (float*)(c->work.p + o_g);
    float* u = (float*)(c->work.p + o_u);
    int8_t* aq = (int8_t*)(c->work.p + o_aq);
    float* ad = (float*)(c->work.p + o_ad);
    float* dy = (float*)(c->work.p + o_dy);
    rc = launch_actquant(c, x_dev, m, hidden, (int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p);
    if (rc != SMX_OK) return rc;
    {
        GemmArgs p = {};
        p.op[0] = gemm_operand(L.gate, g);
        p.op[1] = gemm_operand(L.up, u);
        p.xq = (const int8_t*)c->xq.p;
        p.xd = (const float*)c->xd.p;
        p.a_rowmap = rowmap_dev;  // slot -> token: the gather of kernels.rs:1162-1171
        p.tiles = tiles_gu;
        p.M = (int)slots;
        p.N = (int)eff;
        p.nb = (int)nb;
        p.ldo = (int)eff;
        p.stages_per_slice = (int)((nb + 3) / 4);
        rc = launch_gemm_grouped(c, L.type, p, (int)n_gu, 2, "moe_gemm_gate_up");
        if (rc != SMX_OK) return rc;
    }
    rc = silu_mul_quant(c, g, u, eff, slots, eff, aq, ad);
    if (rc != SMX_OK) return rc;
    {
        GemmArgs p = {};
        p.op[0] = gemm_operand(L.down, dy);
        p.op[1] = p.op[0];
        p.xq = aq;
        p.xd = ad;
        p.tiles = tiles_dn;
        p.M = (int)slots;
        p.N = (int)hidden;
        p.nb = (int)enb;
        p.ldo = (int)hidden;
        p.stages_per_slice = (int)((enb + 3) / 4);
        rc = launch_gemm_grouped(c, L.type, p, (int)n_dn, 1, "moe_gemm_down");
        if (rc != SMX_OK) return rc;
    }
    *out = SlotScratch{g, u, aq, ad, dy};
    return SMX_OK;
}

// Host destinations of the stage-by-stage copy-out of a grouped layer call (any may be null).
struct LayerStagesOut {
    float* gu;    // [slots][2][eff]
    int8_t* aq;   // [slots][eff]
    float* ad;    // [slots][eff/32]
    float* dy;    // [slots][hidden]
};

// The small tables of one call, packed on the host (256-byte aligned parts) and sent to c->tab in
// ONE copy: six separate uploads cost about 4 us each.
struct TableBlob {
    std::vector<char> bytes;
    size_t add(const void* p, size_t n) {
        const size_t off = bytes.size();
        bytes.resize(off + ((n + 255) & ~size_t(255)));
        if (n) std::memcpy(bytes.data() + off, p, n);
        return off;
    }
    // Through the context's pinned staging buffer, so that the caller (and this blob) may go away while
    // the copy is still queued; an event guards the buffer against the next call's tables.
    int upload(smx_ctx* c) {
        int rc = ensure(c, c->tab, bytes.size());
        if (rc != SMX_OK) return rc;
        if (c->htab_done) SMX_HIP(c, hipEventSynchronize(c->htab_done));  // the previous copy out of htab has run
        else SMX_HIP(c, hipEventCreateWithFlags(&c->htab_done, hipEventDisableTiming));
        if ((rc = ensure_host(c, c->htab, bytes.size())) != SMX_OK) return rc;
        std::memcpy(c->htab.p, bytes.data(), bytes.size());
        SMX_HIP(c, hipMemcpyAsync(c->tab.p, c->htab.p, bytes.size(), hipMemcpyHostToDevice, c->stream));
        SMX_HIP(c, hipEventRecord(c->htab_done, c->stream));
        return SMX_OK;
    }
};

static int moe_check_shape(smx_ctx* c, const MoeLayer& L, size_t m, size_t slots) {
    if (slots > (size_t(1) << 24) || m > (size_t(1) << 24) || m * L.hidden >= (size_t(1) << 31) || slots * L.eff >= (size_t(1) << 31) ||
        slots * L.hidden >= (size_t(1) << 31) || L.ne * L.eff * L.hidden >= (size_t(1) << 31))
        return fail(c, SMX_ERR_LIMIT, "moe: m %zu / slots %zu exceed the launch limits", m, slots);
    return SMX_OK;
}

// xs / y on the host (copied in and out, one sync) or, with on_device, device pointers (enqueue only).
static int moe_layer_impl(smx_ctx* c, size_t layer, const float* xs, size_t m, const size_t* plan, size_t nplan,
                          const int32_t* slot_tok, const float* wslot, size_t slots, float* y, size_t y_cap,
                          bool on_device, const LayerStagesOut* stages = nullptr) {
    if (!c) return SMX_ERR_ARG;
    if (!xs || !plan || !slot_tok || !wslot || !y) return fail(c, SMX_ERR_ARG, "moe_layer: null argument");
    return guarded(c, "moe_layer", [&]() -> int {
    auto it = c->moe.find(layer);
    if (it == c->moe.end()) return SMX_NOT_RESIDENT;
    const MoeLayer& L = it->second;
    const size_t hidden = L.hidden;
    if (m == 0 || slots == 0) return fail(c, SMX_ERR_ARG, "moe_layer: m %zu, slots %zu", m, slots);  // decode.rs:1622
    if (y_cap < m * hidden) return fail(c, SMX_ERR_ARG, "moe_layer: output capacity %zu < %zu", y_cap, m * hidden);
    int rc = moe_check_shape(c, L, m, slots);
    if (rc != SMX_OK) return rc;
    if (m > 65535) return fail(c, SMX_ERR_LIMIT, "moe_layer: %zu tokens (the combine launch takes 65535)", m);
    // the plan must tile [0, slots) with in-range experts; every slot's token must exist
    size_t covered = 0;
    for (size_t i = 0; i < nplan; i++) {
        const size_t e = plan[i * 3], off = plan[i * 3 + 1], cnt = plan[i * 3 + 2];
        if (e >= L.ne || cnt == 0 || off != covered || off + cnt > slots)
            return fail(c, SMX_ERR_ARG, "moe_layer: plan entry %zu (expert %zu, off %zu, count %zu) is inconsistent", i, e, off, cnt);
        covered += cnt;
    }
    if (covered != slots) return fail(c, SMX_ERR_ARG, "moe_layer: plan covers %zu of %zu slots", covered, slots);
    std::vector<int> tok_ptr(m + 1, 0), tok_slots(slots);
    for (size_t s = 0; s < slots; s++) {
        if (slot_tok[s] < 0 || (size_t)slot_tok[s] >= m)
            return fail(c, SMX_ERR_ARG, "moe_layer: slot %zu names token %d of %zu", s, slot_tok[s], m);
        tok_ptr[slot_tok[s] + 1]++;
    }
    for (size_t t = 0; t < m; t++) tok_ptr[t + 1] += tok_ptr[t];
    {
        std::vector<int> fill(tok_ptr.begin(), tok_ptr.end() - 1);
        for (size_t s = 0; s < slots; s++) tok_slots[fill[slot_tok[s]]++] = (int)s;  // ascending slot order per token
    }
    SMX_HIP(c, hipSetDevice(c->device));
    if (!on_device) {
        if ((rc = ensure(c, c->xf32, m * hidden * 4)) != SMX_OK) return rc;
        if ((rc = ensure(c, c->yf32, m * hidden * 4)) != SMX_OK) return rc;
    }
    const float* x_dev = on_device ? xs : (const float*)c->xf32.p;
    float* y_dev = on_device ? y : (float*)c->yf32.p;
    std::vector<GemmTile> tiles_gu, tiles_dn;
    build_tiles(plan, nplan, L.eff, &tiles_gu);
    build_tiles(plan, nplan, hidden, &tiles_dn);
    TableBlob tb;
    const size_t o_st = tb.add(slot_tok, slots * 4), o_ws = tb.add(wslot, slots * 4), o_tp = tb.add(tok_ptr.data(), (m + 1) * 4),
                 o_ts = tb.add(tok_slots.data(), slots * 4), o_t1 = tb.add(tiles_gu.data(), tiles_gu.size() * sizeof(GemmTile)),
                 o_t2 = tb.add(tiles_dn.data(), tiles_dn.size() * sizeof(GemmTile));
    if (!on_device) SMX_HIP(c, hipMemcpyAsync(c->xf32.p, xs, m * hidden * 4, hipMemcpyHostToDevice, c->stream));
    if ((rc = tb.upload(c)) != SMX_OK) return rc;
    SlotScratch ss;
    rc = moe_slots_enqueue(c, L, x_dev, m, (const int*)(c->tab.p + o_st), slots, (const GemmTile*)(c->tab.p + o_t1), tiles_gu.size(),
                           (const GemmTile*)(c->tab.p + o_t2), tiles_dn.size(), &ss);
    if (rc != SMX_OK) return rc;
    float* dy = ss.dy;
    {
        ProfScope ps(c, "moe_combine");
        hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((hidden / 4 + 255) / 256), (unsigned)m), dim3(256), 0, c->stream,
                           dy, (const int*)(c->tab.p + o_tp), (const int*)(c->tab.p + o_ts),
                           (const float*)(c->tab.p + o_ws), y_dev, (int)hidden, ((uintptr_t)y_dev & 15) == 0);
        SMX_HIP(c, hipGetLastError());
    }
    if (!on_device) {
        SMX_HIP(c, hipMemcpyAsync(y, c->yf32.p, m * hidden * 4, hipMemcpyDeviceToHost, c->stream));
        if (stages) {
            const size_t eff = L.eff;
            if (stages->gu) {   // g and u are separate [slots][eff] planes on the device
                SMX_HIP(c, hipMemcpy2DAsync(stages->gu, 2 * eff * 4, ss.g, eff * 4, eff * 4, slots, hipMemcpyDeviceToHost, c->stream));
                SMX_HIP(c, hipMemcpy2DAsync(stages->gu + eff, 2 * eff * 4, ss.u, eff * 4, eff * 4, slots, hipMemcpyDeviceToHost, c->stream));
            }
            if (stages->aq) SMX_HIP(c, hipMemcpyAsync(stages->aq, ss.aq, slots * eff, hipMemcpyDeviceToHost, c->stream));
            if (stages->ad) SMX_HIP(c, hipMemcpyAsync(stages->ad, ss.ad, slots * (eff / 32) * 4, hipMemcpyDeviceToHost, c->stream));
            if (stages->dy) SMX_HIP(c, hipMemcpyAsync(stages->dy, ss.dy, slots * hidden * 4, hipMemcpyDeviceToHost, c->stream));
        }
        SMX_HIP(c, hipStreamSynchronize(c->stream));
    }
    return SMX_OK;
    });
}

// WeightAccel::moe_layer_ffn (accel.rs:238-246, decode.rs:3552-3629): xs holds the rows of every
// expert group back to back (expert-major, already gathered by the caller), plan = (expert, rows)
// pairs; returns the unweighted expert outputs dy[rows][hidden] for the caller's weighted scatter.
int smx_moe_layer_ffn(smx_ctx* c, size_t layer, const int32_t* plan, size_t nplan, const float* xs, size_t rows, float* dy,
                      size_t dy_cap) {
    if (!c) return SMX_ERR_ARG;
    if (!plan || !xs || !dy) return fail(c, SMX_ERR_ARG, "moe_layer_ffn: null argument");
    return guarded(c, "moe_layer_ffn", [&]() -> int {
    auto it = c->moe.find(layer);
    if (it == c->moe.end()) return SMX_NOT_RESIDENT;
    const MoeLayer& L = it->second;
    const size_t hidden = L.hidden;
    if (rows == 0 || nplan == 0) return fail(c, SMX_ERR_ARG, "moe_layer_ffn: %zu rows in %zu groups", rows, nplan);
    if (dy_cap < rows * hidden) return fail(c, SMX_ERR_ARG, "moe_layer_ffn: output capacity %zu < %zu", dy_cap, rows * hidden);
    int rc = moe_check_shape(c, L, rows, rows);
    if (rc != SMX_OK) return rc;
    std::vector<size_t> plan3(nplan * 3);
    size_t off = 0;
    for (size_t i = 0; i < nplan; i++) {
        const int e = plan[i * 2], cnt = plan[i * 2 + 1];
        if (e < 0 || (size_t)e >= L.ne || cnt <= 0)
            return fail(c, SMX_ERR_ARG, "moe_layer_ffn: group %zu (expert %d, %d rows) is inconsistent", i, e, cnt);
        plan3[i * 3] = (size_t)e; plan3[i * 3 + 1] = off; plan3[i * 3 + 2] = (size_t)cnt;
        off += (size_t)cnt;
    }
    if (off != rows) return fail(c, SMX_ERR_ARG, "moe_layer_ffn: the groups hold %zu rows, the call says %zu", off, rows);
    SMX_HIP(c, hipSetDevice(c->device));
    if ((rc = ensure(c, c->xf32, rows * hidden * 4)) != SMX_OK) return rc;
    std::vector<GemmTile> tiles_gu, tiles_dn;
    build_tiles(plan3.data(), nplan, L.eff, &tiles_gu);
    build_tiles(plan3.data(), nplan, hidden, &tiles_dn);
    TableBlob tb;
    const size_t o_t1 = tb.add(tiles_gu.data(), tiles_gu.size() * sizeof(GemmTile)),
                 o_t2 = tb.add(tiles_dn.data(), tiles_dn.size() * sizeof(GemmTile));
    if ((rc = tb.upload(c)) != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(c->xf32.p, xs, rows * hidden * 4, hipMemcpyHostToDevice, c->stream));
    SlotScratch ss;
    rc = moe_slots_enqueue(c, L, (const float*)c->xf32.p, rows, nullptr, rows, (const GemmTile*)(c->tab.p + o_t1), tiles_gu.size(),
                           (const GemmTile*)(c->tab.p + o_t2), tiles_dn.size(), &ss);
    if (rc != SMX_OK) return rc;
    SMX_HIP(c, hipMemcpyAsync(dy, ss.dy, rows * hidden * 4, hipMemcpyDeviceToHost, c->stream));
    SMX_HIP(c, hipStreamSynchronize(c->stream));
    return SMX_OK;
    });
}

// WeightAccel::moe_expert_ffn (accel.rs:220-223): one expert's FFN for m grouped rows, one sync.
int smx_moe_expert_ffn(smx_ctx* c, size_t layer, size_t expert, const float* xs, size_t m, float* y, size_t y_cap) {
    if (expert > 0x7fffffffu || m > 0x7fffffffu) return c ? fail(c, SMX_ERR_ARG, "moe_expert_ffn: expert %zu, %zu rows", expert, m) : SMX_ERR_ARG;
    const int32_t plan[2] = {(int32_t)expert, (int32_t)m};
    return smx_moe_layer_ffn(c, layer, plan, 1, xs, m, y, y_cap);
}

int smx_moe_layer(smx_ctx* c, size_t layer, const float* xs, size_t m, const size_t* plan, size_t nplan,
                  const int32_t* slot_tok, const float* wslot, size_t slots, float* y, size_t y_cap) {
    return moe_layer_impl(c, layer, xs, m, plan, nplan, slot_tok, wslot, slots, y, y_cap, false);
}

int smx_moe_layer_stages(smx_ctx* c, size_t layer, const float* xs, size_t m, const size_t* plan, size_t nplan,
                         const int32_t* slot_tok, const float* wslot, size_t slots, float* y, size_t y_cap, float* gu,
                         int8_t* aq, float* ad, float* dy) {
    const LayerStagesOut so = {gu, aq, ad, dy};
    return moe_layer_impl(c, layer, xs, m, plan, nplan, slot_tok, wslot, slots, y, y_cap, false, &so);
}

int smx_moe_layer_dev(smx_ctx* c, size_t layer, const float* xs_dev, size_t m, const size_t* plan, size_t nplan,
                      const int32_t* slot_tok, const float* wslot, size_t slots, float* y_dev) {
    if (c && c->capturing)
        return fail(c, SMX_ERR_ARG, "moe_layer_dev: the routing tables are copied from the host at every call and cannot be captured");
    return moe_layer_impl(c, layer, xs_dev, m, plan, nplan, slot_tok, wslot, slots, y_dev, SIZE_MAX, true);
}

}  // extern "C"
