// Fused block-dequant -> GEMV for Q4_0 / Q8_0 / Q6_K weights against Q8-quantised activations.
//
// Stands in for the reference's decode GEMVs (crates/strix-backend-rocm/src/kernels.rs:259-287
// q4_gemv_dp, :894-912 q8i_gemv, :1016-1045 q8i_gemm_rows32, :607-640 q6_gemv) on gfx950:
//   * 16-wave workgroups, one per CU; the quantised activation (int8 + scales + 16-element sums) is
//     staged once per workgroup in LDS, quantised on the way when it arrives as fp32;
//   * every lane streams 128-bit units of the packed quants straight from HBM;
//   * v_dot4_i32_i8 integer block dots, exact i32 per block, then acc += (dw*dx)*float(isum);
//   * cross-lane (DPP) combination of lanes that share a block and of the lanes of a row.
// Two forms (gemv_body.h): the flat form (activation requested before the weights, a workgroup's rows
// walked as one sequence of 64-unit loads, no conditional loads) for every shape whose rows are a whole
// number of unit groups, and the persistent row-per-wave form for the rest.
// HBM-bound: algorithmic bytes per row are K/32 * {18, 34} (Q4_0, Q8_0) or K/256 * 210 (Q6_K).
#include <algorithm>
#include <cstddef>
#include <type_traits>

#include "gemv_body.h"
#include "router_body.h"
#include "smx_internal.h"

namespace smx {

// One launch serves up to 8 independent GEMVs of the same format and row length (blockIdx.y picks
// the job): the gate/up pair or the q/k/v triple of a decode step, or a caller's batch of (key, x)
// pairs, share one kernel start-up.
// A job's launch scalars.  Its first 64 bytes are one line of the kernel-argument segment and hold everything the
// one-row kernels need before their first weight load, so that a wave's start costs ONE scalar-cache miss: with
// the fields spread over the segment (and the grid size taken from the hidden arguments) a workgroup paid two
// misses one after the other before it could request a weight, and a third one in its tail.
struct alignas(128) GemvJob {
    GemvW W;
    const float* x;     // fp32 activation row(s), null when they arrive quantised
    float* y;
    int N;
    int nblk;
    int n_wgs;          // flat form: workgroups that share the job's rows (the launch's gridDim.x)
    unsigned magic_u;   // flat form: ceil(2^32 / units per row)
    // second line: what only some variants read
    const int8_t* xq;   // quantised rows [m][K], their scales and packed 16-element sums
    const float* xd;
    const int* xs;
    const float* x2;    // activation producer: second operand
    int prod;           // SMX_ACT_*
    float eps;
    int m;              // activation rows
    int act2;           // paired launch: SMX_ACT_SILU_MUL or SMX_ACT_GEGLU applied to this job's dot ...
    float* h;           // ... times the next job's: h[r] = act2(y[r]) * y_next[r]
    __host__ __device__ GemvX X() const { return GemvX{x, xq, xd, xs, x2, prod, eps}; }
    void set_x(const GemvX& a) { x = a.x; xq = a.xq; xd = a.xd; xs = a.xs; x2 = a.x2; prod = a.prod; eps = a.eps; }
};
static_assert(offsetof(GemvJob, xq) == 64, "the first line ends with magic_u");
static_assert(sizeof(GemvJob) == 128, "two lines per job: 16 jobs and the routing fit the kernel-argument segment");
struct GemvJobs {
    GemvJob job[SMX_GEMV_GROUP_MAX];
    // expert indirection (MoE decode routed on the device): job j reads expert ids[slot[j]] of a stacked tensor
    const int* ids;
    int ne;
    unsigned long long blocks_per_expert;
    int slot[SMX_GEMV_GROUP_MAX];
    // routing inside the launch (paired form only): every workgroup routes the ne <= 64 router logits itself (top route_k) and
    // workgroup (0, 0) writes the routing out for the launches behind this one
    const float* logits;
    int route_k;
    int* ids_out;
    float* w_out;
};

// The planes of a job's weight; IND: moved to the expert the device-side routing names.  The indirection is
// compiled only into the kernels that a routed launch uses: with it the plane pointers are no longer
// known to be wave-uniform, which costs every other GEMV 0.2-0.3 us per launch.
template <class Ops, bool IND>
__device__ __forceinline__ GemvW job_weight(const GemvJobs& J, int j) {
    GemvW W = J.job[j].W;
    if (IND) {
        const size_t b0 = (size_t)min(max(J.ids[J.slot[j]], 0), J.ne - 1) * J.blocks_per_expert;
        Ops::advance(W, b0);
    }
    return W;
}
// the same with the expert given (routing computed inside the launch)
template <class Ops>
__device__ __forceinline__ GemvW job_weight_at(const GemvJobs& J, int j, int expert) {
    GemvW W = J.job[j].W;
    Ops::advance(W, (size_t)min(max(expert, 0), J.ne - 1) * J.blocks_per_expert);
    return W;
}

template <class Ops, int MT, int RPW, int PRE, int KS, int LPR, int FQ, bool DUMP, int NT, bool IND = false>
__global__ __launch_bounds__(NT) void gemv_kernel(const GemvJobs J, int* __restrict__ dump, int dump_per_row) {
    const int nw = NT / 64;
    const GemvJob& jb = J.job[blockIdx.y];
    gemv_body<Ops, MT, RPW, PRE, KS, LPR, FQ, DUMP>(job_weight<Ops, IND>(J, blockIdx.y), jb.X(), jb.y, jb.N, jb.nblk, jb.N, MT == 1 ? 1 : jb.m,
                                                       dump, dump_per_row, blockIdx.x * nw + (threadIdx.x >> 6), gridDim.x * nw);
}

// Flat form (one activation row): blockIdx.x of the job's n_wgs workgroups share its rows.
// DUMP: the per-block i32 dots of job 0 are also written to dump[row * dump_per_row + ...].
template <class Ops, int MT, int PRE, int GL, int FQ, bool DUMP, bool IND = false>
__global__ __launch_bounds__(1024) void gemv_flat_kernel(const GemvJobs J, int* __restrict__ dump, int dump_per_row) {
    const GemvJob& jb = J.job[blockIdx.y];
    gemv_body_flat<Ops, MT, PRE, GL, FQ, DUMP>(job_weight<Ops, IND>(J, blockIdx.y), jb.X(), jb.y, jb.N, jb.nblk, jb.N, MT == 1 ? 1 : jb.m,
                                               blockIdx.x, jb.n_wgs, jb.magic_u, dump, dump_per_row);
}

// Paired form: workgroup (x, p) serves jobs 2p (gate) and 2p + 1 (up) over the same rows and writes the product of the
// activated gate dot and the up dot (gemv_body_flat, DUAL).
// IND: 0 = the jobs' weights as given, 1 = experts read from device memory (J.ids), 2 = experts routed here: every workgroup
// runs the router (softmax + top route_k of the ne <= 64 logits, the arithmetic of topk_router_kernel) before it requests its
// weights, which saves the routing launch in front of a decode token's expert FFN (2.9 us for less than 1 us of prologue);
// workgroup (0, 0) writes ids and weights out for the down launch.
template <class Ops, int PRE, int GL, int FQ, int IND = 0>
__global__ __launch_bounds__(1024) void gemv_flat_dual_kernel(const GemvJobs J) {
    const GemvJob& jg = J.job[2 * blockIdx.y];
    const GemvJob& ju = J.job[2 * blockIdx.y + 1];
    if constexpr (IND == 2) {
        // Routing by the whole workgroup: every wave computes the 64 probabilities (the same bits everywhere), takes the rank
        // contributions of 64 / waves experts, and after one barrier every wave adds the parts up and finds the expert whose
        // rank is this workgroup's slot.  One wave doing all 64 comparisons alone costs the launch 0.6 us more.
        __shared__ int r_part[16 * 64];
        __shared__ float r_sel[64];
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;   // nwaves <= 16
        // eight waves pull the activation row through this CU's cache meanwhile (used after the barrier, so nothing waits
        // for it here): the staging that follows finds the row on its way or there
        float4 pf = make_float4(0.f, 0.f, 0.f, 0.f);
        if (wave >= 1 && wave <= 8) {
            const int i = threadIdx.x - 64;
            if (i < Ops::nb32(jg.nblk) * 8) pf = ((const float4*)jg.x)[i];
        }
        const bool live = lane < J.ne;
        const float p = router_prob_lane(live ? J.logits[lane] : -3.40282347e+38f, live);
        const int per = (64 + nwaves - 1) / nwaves;
        r_part[wave * 64 + lane] = router_rank_part(p, min(wave * per, 64), min(wave * per + per, 64));
        __syncthreads();
        int rank = 0;
        for (int w = 0; w < nwaves; w++) rank += r_part[w * 64 + lane];
        const int slot = J.slot[2 * blockIdx.y];
        const unsigned long long hit = __ballot(live && rank == slot);   // the ranks of the live lanes are a permutation
        const int e = hit ? (int)__builtin_ctzll(hit) : 0;
        if (blockIdx.x == 0 && blockIdx.y == 0 && wave == 0) {   // the routing itself, for the down launch and the caller
#pragma clang fp contract(off)
            if (live && rank < J.route_k) {
                r_sel[rank] = p;
                J.ids_out[rank] = lane;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            float wsum = 0.f;   // in pick order, as the reference sums the chosen probabilities
            for (int i = 0; i < J.route_k; i++) wsum += r_sel[i];
            if (lane < J.route_k) J.w_out[lane] = r_sel[lane] / wsum;
        }
        if (J.route_k < 0) r_sel[lane] = pf.x + pf.y + pf.z + pf.w;   // (never: keeps the loads)
        gemv_body_flat<Ops, 1, PRE, GL, FQ, false, true>(job_weight_at<Ops>(J, 2 * blockIdx.y, e), jg.X(), jg.y, jg.N, jg.nblk, jg.N, 1,
                                                          blockIdx.x, jg.n_wgs, jg.magic_u, nullptr, 0,
                                                          job_weight_at<Ops>(J, 2 * blockIdx.y + 1, e), ju.y, jg.h, jg.act2);
    } else {
        gemv_body_flat<Ops, 1, PRE, GL, FQ, false, true>(job_weight<Ops, IND == 1>(J, 2 * blockIdx.y), jg.X(), jg.y, jg.N, jg.nblk, jg.N, 1,
                                                          blockIdx.x, jg.n_wgs, jg.magic_u, nullptr, 0,
                                                          job_weight<Ops, IND == 1>(J, 2 * blockIdx.y + 1), ju.y, jg.h, jg.act2);
    }
}

namespace {

// Row length from which silu / gelu producers run in their own launch (measured on 2560 <- 9728).
constexpr size_t kProducerSplitK = 4096;

// Launch geometry: slots per wave, pipeline depth, K-split, lanes per row, threads per workgroup.
struct Geom {
    bool prod = false;  // an activation producer runs in the staging
    bool preq = false;  // the (single) activation row arrives quantised
    bool rowsf = false; // 2..4 fp32 activation rows are quantised inside the flat kernel
    int flat = 0;       // flat form: lanes per group (16 or 8), 0 = not used
    int flat_pre = 0;   // its loads per round
    int rpw, pre, ks, lpr, nt;
    unsigned grid;
    size_t lds;
};

template <class Ops, int MT, int RPW, int PRE, int KS, int LPR, int FQ, bool DUMP, int NT>
int launch_fq(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int* dump, int dump_per_row) {
    auto k = gemv_kernel<Ops, MT, RPW, PRE, KS, LPR, FQ, DUMP, NT>;
    if (J.ids) {   // experts chosen on the device: one fp32 activation row per job, no dump
        if constexpr (MT == 1 && FQ != 0 && !DUMP) k = gemv_kernel<Ops, MT, RPW, PRE, KS, LPR, FQ, DUMP, NT, true>;
        else return fail(c, SMX_ERR_ARG, "gemv: device-routed experts take one fp32 activation row per job");
    }
    int rc = set_dyn_lds(c, k, g.lds);
    if (rc != SMX_OK) return rc;
    GemvJobs JJ = J;
    for (int i = 0; i < njobs; i++) { JJ.job[i].nblk = nblk; JJ.job[i].m = m; JJ.job[i].n_wgs = (int)g.grid; JJ.job[i].magic_u = 0; }
    hipLaunchKernelGGL(k, dim3(g.grid, (unsigned)njobs), dim3(NT), g.lds, c->stream, JJ, dump, dump_per_row);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

template <class Ops, int MT, int RPW, int PRE, int KS, int LPR, bool DUMP, int NT>
int launch_one(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int* dump,
               int dump_per_row) {
    // one activation row: quantiser fused into the staging (FQ 1), behind an activation producer if the
    // caller asked for one (FQ 2: its own variant, so that the plain GEMV carries none of its code);
    // several rows: staged from rows quantised once (FQ 0)
    if (MT == 1 && !DUMP && g.preq) return launch_fq<Ops, MT, RPW, PRE, KS, LPR, 0, DUMP, NT>(c, g, J, njobs, nblk, m, dump, dump_per_row);
    if (MT == 1 && !DUMP && g.prod) return launch_fq<Ops, MT, RPW, PRE, KS, LPR, (MT == 1 && !DUMP) ? 2 : 0, DUMP, NT>(c, g, J, njobs, nblk, m, dump, dump_per_row);
    return launch_fq<Ops, MT, RPW, PRE, KS, LPR, MT == 1 ? 1 : 0, DUMP, NT>(c, g, J, njobs, nblk, m, dump, dump_per_row);
}

template <class Ops, int MT, int PRE, int GL, int FQ, bool DUMP = false>
int launch_flat_fq(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int* dump = nullptr,
                   int dump_per_row = 0) {
    auto k = gemv_flat_kernel<Ops, MT, PRE, GL, FQ, DUMP>;
    if (J.ids) {   // experts chosen on the device: one fp32 activation row per job, no dump
        if constexpr (MT == 1 && FQ != 0 && !DUMP) k = gemv_flat_kernel<Ops, MT, PRE, GL, FQ, DUMP, true>;
        else return fail(c, SMX_ERR_ARG, "gemv: device-routed experts take one fp32 activation row per job");
    }
    int rc = set_dyn_lds(c, k, g.lds);
    if (rc != SMX_OK) return rc;
    const unsigned upb = std::is_same<Ops, OpsQ6_K>::value ? 4u : (std::is_same<Ops, OpsQ8_0>::value ? 2u : 1u);
    const unsigned units = (unsigned)nblk * upb;                             // units per row
    const unsigned magic = (unsigned)(((1ull << 32) + units - 1) / units);   // floor(f * magic / 2^32) = f / units for f < 2^16
    GemvJobs JJ = J;
    for (int i = 0; i < njobs; i++) { JJ.job[i].nblk = nblk; JJ.job[i].m = m; JJ.job[i].n_wgs = (int)g.grid; JJ.job[i].magic_u = magic; }
    hipLaunchKernelGGL(k, dim3(g.grid, (unsigned)njobs), dim3(1024), g.lds, c->stream, JJ, dump, dump_per_row);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

template <class Ops, int MT>
int launch_flat(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int* dump = nullptr,
                int dump_per_row = 0) {
    constexpr bool kQ6 = std::is_same<Ops, OpsQ6_K>::value;
    if constexpr (MT == 1) {
#define SMX_FLAT(PRE, GL)                                                                            \
    if (g.flat_pre == PRE && g.flat == GL) {                                                         \
        if (dump) return launch_flat_fq<Ops, 1, PRE, GL, 1, true>(c, g, J, njobs, nblk, m, dump, dump_per_row); \
        if (g.preq) return launch_flat_fq<Ops, 1, PRE, GL, 0>(c, g, J, njobs, nblk, m);              \
        if (g.prod) return launch_flat_fq<Ops, 1, PRE, GL, 2>(c, g, J, njobs, nblk, m);              \
        return launch_flat_fq<Ops, 1, PRE, GL, 1>(c, g, J, njobs, nblk, m);                          \
    }
        if constexpr (std::is_same<Ops, OpsQ4_0>::value || std::is_same<Ops, OpsQ8_0>::value) {
            SMX_FLAT(3, 16) SMX_FLAT(3, 8) SMX_FLAT(2, 16) SMX_FLAT(4, 16)
        } else if constexpr (kQ6) {
            SMX_FLAT(1, 16) SMX_FLAT(1, 8) SMX_FLAT(1, 4)
        }
#undef SMX_FLAT
    } else if constexpr (!(kQ6 && MT == 8)) {
        if constexpr (MT <= 4 && !kQ6) {   // fp32 rows quantised by the kernel, two loads per round
            if constexpr (MT == 2 && std::is_same<Ops, OpsQ8_0>::value) {
                if (g.rowsf && g.flat == 16 && g.flat_pre == 2) return launch_flat_fq<Ops, MT, 2, 16, 1>(c, g, J, njobs, nblk, m);
            }
        }
        // several rows arrive quantised
        constexpr int PRE = 1;
        if (g.flat_pre == PRE) {
            if constexpr (MT <= 4) {
                if (g.rowsf) {   // fp32 rows, quantised by the kernel
                    if (g.flat == 16) return launch_flat_fq<Ops, MT, PRE, 16, 1>(c, g, J, njobs, nblk, m);
                    if (g.flat == 8) return launch_flat_fq<Ops, MT, PRE, 8, 1>(c, g, J, njobs, nblk, m);
                    if constexpr (kQ6) {
                        if (g.flat == 4) return launch_flat_fq<Ops, MT, PRE, 4, 1>(c, g, J, njobs, nblk, m);
                    }
                }
            }
            if (g.flat == 16) return launch_flat_fq<Ops, MT, PRE, 16, 0>(c, g, J, njobs, nblk, m);
            if (g.flat == 8) return launch_flat_fq<Ops, MT, PRE, 8, 0>(c, g, J, njobs, nblk, m);
            if constexpr (kQ6) {
                if (g.flat == 4) return launch_flat_fq<Ops, MT, PRE, 4, 0>(c, g, J, njobs, nblk, m);
            }
        }
    }
    return fail(c, SMX_ERR_ARG, "gemv: no flat variant for this geometry");
}

// The compiled variants (RPW, PRE, KS, LPR):
//   whole-wave rows   (4,2,1,64) (2,2,1,64) (1,4,1,64) (1,2,2,64) (1,2,4,64)
//   sub-wave rows     (2,2,1,32) (1,2,1,32) (2,2,1,16) (1,2,1,16)        [one activation row only]
template <class Ops, int MT>
int launch_variant(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m) {
    // sub-wave rows: the pipeline is deep enough to put a whole short row set in flight before the
    // activation is staged (Q6_K units are three times as wide, so half the depth)
    constexpr bool kWide = sizeof(typename Ops::Regs) > 32;
    if (g.flat) return launch_flat<Ops, MT>(c, g, J, njobs, nblk, m);
    if (MT == 1 && g.lpr == 32) {
        if (g.rpw == 2) return launch_one<Ops, 1, 2, kWide ? 2 : 3, 1, 32, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
        return launch_one<Ops, 1, 1, kWide ? 2 : 4, 1, 32, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    }
    if (MT == 1 && g.lpr == 16) {
        if (g.rpw == 2) return launch_one<Ops, 1, 2, kWide ? 2 : 3, 1, 16, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
        return launch_one<Ops, 1, 1, kWide ? 4 : 6, 1, 16, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    }
    if (g.ks == 4) return launch_one<Ops, MT, 1, 2, 4, 64, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    if (g.ks == 2) return launch_one<Ops, MT, 1, 2, 2, 64, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    // 8 activation rows (4 with Q6_K's wide units): a ring of 4 units spills (128 registers per lane at
    // 16 waves), and the scratch traffic costs more than the shallower pipeline: 2 fit
    constexpr int kPre1 = (MT == 8 || (kWide && MT == 4)) ? 2 : 4;
    if (g.rpw == 1) return launch_one<Ops, MT, 1, kPre1, 1, 64, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    if (g.rpw == 4 && MT == 1) return launch_one<Ops, 1, 4, 2, 1, 64, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
    return launch_one<Ops, MT, 2, 2, 1, 64, false, 1024>(c, g, J, njobs, nblk, m, nullptr, 0);
}

template <class Ops>
int launch_type(smx_ctx* c, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int mt,
                int* dump, int dump_per_row) {
    if (dump && g.flat) return launch_flat<Ops, 1>(c, g, J, njobs, nblk, m, dump, dump_per_row);
    if (dump) {
        if (g.lpr == 16) return launch_one<Ops, 1, 1, 2, 1, 16, true, 256>(c, g, J, njobs, nblk, m, dump, dump_per_row);
        return launch_one<Ops, 1, 1, 4, 1, 64, true, 256>(c, g, J, njobs, nblk, m, dump, dump_per_row);
    }
    switch (mt) {
        case 1: return launch_variant<Ops, 1>(c, g, J, njobs, nblk, m);
        case 2: return launch_variant<Ops, 2>(c, g, J, njobs, nblk, m);
        case 4: return launch_variant<Ops, 4>(c, g, J, njobs, nblk, m);
        default: return launch_variant<Ops, 8>(c, g, J, njobs, nblk, m);
    }
}

}  // namespace

// Geometry choice.  The small GEMVs of a decode step are bound by instruction issue and start-up
// latency rather than by HBM, so: 16-wave workgroups (the activation is quantised and staged once
// per 16 waves), persistent workgroups looping over chunks, lanes-per-row chosen to waste the fewest
// lanes on short rows, and for weights with few, long rows the passes of a row are split over 2 or
// 4 waves (K-split) so every SIMD has work.
// Loads per round of the flat form (Q4_0 / Q8_0, one activation row, 16-lane groups).  A wave takes L = units of the
// workgroup / 64 / 16 loads in rounds of PRE, each round one trip to memory; a last round of a single load costs as much as a
// full one.  Measured (cold, in a graph): Q4_0 8192 x 2048 gate/up pair (L = 4) 7.56 / 6.79 / 7.66 us with 3 / 2 / 4 per round
// and its single GEMV (L = 2) 4.16 / 4.10 / 4.19; Q8_0 8192 x 2048 single (L = 4) 5.68 / 5.23 / 5.37, pair (L = 8) 9.6 / 9.2 / 9.7;
// Q4_0 14336 x 4096 single (L = 7) 7.98 / 7.85 / 7.72; Q4_0 9728 x 2560 single (L = 3) 4.89 / 5.11 / 4.95, pair (L = 6) 8.47 / 8.45 / 9.26.
static int pick_flat_pre(size_t units_per_wg) {
    const int L = (int)((((units_per_wg + 63) / 64) + 15) / 16);
    if (L % 3 == 0) return 3;
    if (L % 2 == 0) return 2;
    if (L % 3 == 2) return 3;
    return L >= 7 ? 4 : 3;   // 7 = 4 + 3; a single load either way
}

static Geom pick_geom(const smx_ctx* c, QType type, size_t N, size_t nblk, int mt, bool dump, int njobs) {
    Geom g;
    size_t tokb, units;
    if (type == kQ4_0) { tokb = (nblk * 40 + 15) & ~size_t(15); units = nblk; }
    else if (type == kQ8_0) { tokb = (nblk * 36 + 15) & ~size_t(15); units = (mt >= 4 && !dump) ? nblk : nblk * 2; }
    else { tokb = nblk * 2 * (OpsQ6_K::kPad * 16 + 32); units = nblk * 4; }
    g.nt = 1024;
    g.lpr = 64;
    g.ks = 1;
    const size_t cus = std::max<size_t>(1, (size_t)c->num_cu / njobs);  // this job's share of the chip
    const size_t waves = cus * 16;
    // lanes per row: fewest wasted lanes, whole-wave rows on ties (short rows, one activation row only)
    if (mt == 1 && units < 256) {
        size_t best = ((units + 63) / 64) * 64;
        for (int lpr : {32, 16}) {
            const size_t slots = ((units + lpr - 1) / lpr) * lpr;
            // measured: with equal waste, rows of fewer than 128 units run best two to a wave
            if (slots < best || (slots == best && lpr == 32 && units < 128)) { best = slots; g.lpr = lpr; }
        }
    }
    if (c->tune_gemv_lpr > 0 && mt == 1) g.lpr = c->tune_gemv_lpr;
    const int P = (int)((units + g.lpr - 1) / g.lpr);
    if (g.lpr == 64) {
        // K-split pays for a single activation row only (batched rows are bound by their own arithmetic)
        if (mt == 1 && P >= 4 && N * 2 <= waves) g.ks = (P >= 8 && N * 4 <= waves) ? 4 : 2;
        else if (mt == 1 && P >= 4 && N <= waves) g.ks = 2;  // more wave-tasks than one round of waves: extra workgroups queue
        if (g.ks > 1) { g.rpw = 1; g.pre = 2; }
        else if (P >= 4) { g.rpw = 1; g.pre = 4; }
        else if (mt == 1 && type != kQ6_K && P <= 2 && N >= waves * 4) { g.rpw = 4; g.pre = 2; }
        else { g.rpw = 2; g.pre = 2; }
        if (c->tune_gemv_rpw > 0 || c->tune_gemv_ks > 0) {
            const int ks = c->tune_gemv_ks > 0 ? c->tune_gemv_ks : 1;
            const int rpw = c->tune_gemv_rpw > 0 ? c->tune_gemv_rpw : 1;
            if (ks > 1) { g.ks = ks; g.rpw = 1; g.pre = 2; }
            else if (rpw == 1) { g.ks = 1; g.rpw = 1; g.pre = 4; }
            else if (rpw == 4 && mt == 1) { g.ks = 1; g.rpw = 4; g.pre = 2; }
            else { g.ks = 1; g.rpw = 2; g.pre = 2; }
        }
        // register budget of the 16-wave workgroup (128 VGPRs): Q6_K units are wide, batched rows multiply accumulators
        if (g.ks == 1 && g.rpw > 1 && ((type == kQ6_K && (g.rpw > 2 || mt > 1)) || mt == 8)) {
            g.rpw = (type == kQ6_K && mt == 1) ? 2 : 1;
            g.pre = g.rpw == 1 ? 4 : 2;
        }
    } else {
        const size_t rows_per_slot = 64 / g.lpr;
        g.pre = 2;
        g.rpw = (N / rows_per_slot >= waves * 2 && type != kQ6_K) ? 2 : 1;
        if (c->tune_gemv_rpw > 0) g.rpw = c->tune_gemv_rpw >= 2 && type != kQ6_K ? 2 : 1;
    }
    if (dump) { g.rpw = 1; g.pre = g.lpr == 16 ? 2 : 4; g.ks = 1; g.nt = 256; if (g.lpr == 32) g.lpr = 64; }
    const int nw = g.nt / 64;
    const size_t rc = (size_t)g.rpw * (64 / g.lpr);
    g.lds = tokb * (size_t)mt + (g.ks > 1 ? (size_t)nw * rc * mt * 4 : 0);
    const size_t chunks = (N + rc - 1) / rc;
    const size_t wgs = (chunks * g.ks + nw - 1) / nw;
    if (g.ks > 1) {
        g.grid = (unsigned)wgs;  // one chunk per wave group
    } else {
        int wpc = c->tune_gemv_wpc > 0 ? c->tune_gemv_wpc : 1;
        if (dump) wpc = 8;
        g.grid = (unsigned)std::min<size_t>(wgs, cus * wpc);
    }
    // Flat form: one activation row of up to 16384 elements and rows of a whole number of unit groups.
    // Measured against the persistent form above: Q4_0 9728 x 2560 6.8 -> 5.4 us, eight of them in one
    // launch 24.8 -> 22.4 us, Q6_K 262144 x 3840 159 -> 144 us.
    // The block-dot dump of the parity tests runs in whichever form the shape gets.
    if (!(type == kQ6_K && mt == 8) && (units % (type == kQ6_K ? 4 : 8)) == 0 &&
        nblk * (type == kQ6_K ? 256 : 32) <= 16384) {  // the row is held in registers while the weights are requested
        // a workgroup's units are indexed with 16 bits and its group sums live in LDS: whole further
        // rounds of workgroups when a CU's share of the rows is too large for either
        g.flat = (units % 16) == 0 ? 16 : ((units % 8) == 0 ? 8 : 4);
        const size_t share = (N + cus - 1) / cus * units;   // units of a CU's share of the rows
        size_t rounds = share < 65536 ? 1 : (share + 59999) / 60000;   // margin for the rounding of rows per workgroup
        size_t fwgs, rows, lds;
        for (;; rounds++) {
            fwgs = std::min(N, cus * rounds);
            rows = (N + fwgs - 1) / fwgs;                          // of the workgroup with the most rows
            lds = tokb * (size_t)mt + std::max<size_t>(rows * units / g.flat * 4 * mt, 128);   // (128: the rmsnorm reduction's sixteen wave sums)
            if (lds <= 128 * 1024 || fwgs == N) break;
        }
        if (rows * units < 65536 && lds <= 160 * 1024) {
            // loads requested per round, measured: Q4_0 pair 8.2 / 8.0 / 7.7 / 8.1 / 8.9 us with 1 / 2 / 3 / 4 / 6,
            // Q6_K 15360 x 3840 (five load instructions per unit) 11.4 / 12.5 / 14.1 / 14.8 us with 1 / 2 / 3 / 4,
            // eight rows on Q8_0 2560 x 9728 14.1-14.6 / 14.8 / 15.8 us with 1 / 2 / 3
            g.flat_pre = type == kQ6_K ? 1 : (mt == 1 ? 3 : 1);
            if (mt == 1 && type != kQ6_K && g.flat == 16) g.flat_pre = pick_flat_pre(rows * units);
            g.nt = 1024;
            g.grid = (unsigned)fwgs;
            g.lds = lds;
        } else {
            g.flat = 0;
        }
    }
    return g;
}

static int launch_jobs(smx_ctx* c, QType type, const Geom& g, const GemvJobs& J, int njobs, int nblk, int m, int mt,
                       int32_t* dump, int dump_per_row, const char* name = nullptr) {
    if (type == kQ4_0) {
        ProfScope ps(c, name ? name : "gemv_q4_0");
        return launch_type<OpsQ4_0>(c, g, J, njobs, nblk, m, mt, dump, dump_per_row);
    }
    if (type == kQ8_0) {
        ProfScope ps(c, name ? name : "gemv_q8_0");
        // 4 or 8 activation rows: a lane takes whole blocks (the per-row scale work halves)
        if (mt >= 4 && !dump) return launch_type<OpsQ8_0W>(c, g, J, njobs, nblk, m, mt, dump, dump_per_row);
        return launch_type<OpsQ8_0>(c, g, J, njobs, nblk, m, mt, dump, dump_per_row);
    }
    ProfScope ps(c, name ? name : "gemv_q6_k");
    return launch_type<OpsQ6_K>(c, g, J, njobs, nblk, m, mt, dump, dump_per_row);
}

int launch_gemv(smx_ctx* c, const Weight& w, const float* x, size_t m, float* y, int32_t* dump, const ActScratch* sc) {
    if (m == 0 || m > SMX_GEMV_MAX_M) return fail(c, SMX_ERR_LIMIT, "gemv: %zu rows (1..%d supported)", m, SMX_GEMV_MAX_M);
    if (w.N > 0x7fffffffu / 4 || w.K > (size_t(1) << 20))
        return fail(c, SMX_ERR_LIMIT, "gemv: shape %zu x %zu exceeds the kernel's index range", w.N, w.K);
    if (w.type == kQ6_K && m > 4) {  // Q6_K keeps at most 4 activation rows in registers per launch
        int rc = launch_gemv(c, w, x, 4, y, nullptr, sc);
        if (rc != SMX_OK) return rc;
        return launch_gemv(c, w, x + 4 * w.K, m - 4, y + 4 * w.N, nullptr, sc);   // same stream: the second pass may reuse sc
    }
    const int mt = m == 1 ? 1 : (m == 2 ? 2 : (m <= 4 ? 4 : 8));
    Geom g = pick_geom(c, w.type, w.N, w.nblk, mt, dump != nullptr, 1);
    if (g.lds > 160 * 1024)
        return fail(c, SMX_ERR_LIMIT, "gemv: %zu activation rows of %zu need %zu bytes of LDS (limit 163840)", m, w.K, g.lds);
    GemvJobs J = {};
    J.job[0].W = {w.scales, (const uint4*)w.quants, (const uint4*)w.qh, (const uint2*)w.sc};
    J.job[0].x = x;
    J.job[0].y = y;
    J.job[0].N = (int)w.N;
    // 2..4 rows of at most 49152 values in all: the flat kernel quantises them itself (up to three half blocks per thread), which
    // saves the quantiser launch; longer rows are quantised once for all workgroups by their own launch
    g.rowsf = mt > 1 && mt <= 4 && g.flat && !dump && (size_t)mt * w.K <= 49152;
    // Two rows of a Q8_0 weight (a unit is one 16-byte load there): two loads per round.  Measured with 1 / 2 / 3 / 4 per round:
    // 2560 x 9728 9.60 / 9.15 / 9.15 / 9.45 us, 9728 x 2560 8.30 / 7.64 / 7.48 / 7.96, 4096 x 4096 6.76 / 6.14 / 6.63 / 6.58.  Q4_0 and three
    // or four rows (bound by the staging of the rows and the LDS reads of four rows per unit) lose 0 .. 8 % with more than one.
    if (g.rowsf && w.type == kQ8_0 && mt == 2 && g.flat == 16) g.flat_pre = 2;
    if (mt > 1 && !g.rowsf) {
        // each of the persistent workgroups would repeat the quantiser for all m rows: do it once instead
        int rc;
        ActScratch a;
        if (sc) {
            a = *sc;
        } else {
            if ((rc = ensure(c, c->xq, m * w.K)) != SMX_OK) return rc;
            if ((rc = ensure(c, c->xd, m * (w.K / 32) * 4)) != SMX_OK) return rc;
            if ((rc = ensure(c, c->xs, m * (w.K / 32) * 4)) != SMX_OK) return rc;
            a = ActScratch{(int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p};
        }
        rc = launch_actquant(c, x, m, w.K, a.xq, a.xd, a.xs);
        if (rc != SMX_OK) return rc;
        J.job[0].set_x(GemvX{nullptr, a.xq, a.xd, (const int*)a.xs});
    }
    return launch_jobs(c, w.type, g, J, 1, (int)w.nblk, (int)m, mt, dump, (int)(w.type == kQ6_K ? w.K / 16 : w.K / 32));
}

// n <= SMX_GEMV_GROUP_MAX single-row GEMVs of one format and row length in one launch.
int launch_gemv_group(smx_ctx* c, const Weight* const* ws, const float* const* xs, float* const* ys, int n,
                      const char* name, const ActProd* prod, const float* const* x2s, const GemvIndirect* ind) {
    if (n < 1 || n > SMX_GEMV_GROUP_MAX) return fail(c, SMX_ERR_ARG, "gemv group of %d", n);
    size_t maxN = 0;
    GemvJobs J = {};
    if (ind) {
        J.ids = ind->ids;
        J.ne = ind->ne;
        J.blocks_per_expert = ind->blocks_per_expert;
        for (int i = 0; i < n; i++) J.slot[i] = ind->slot[i];
    }
    for (int i = 0; i < n; i++) {
        const Weight& w = *ws[i];
        if (w.type != ws[0]->type || w.K != ws[0]->K) return fail(c, SMX_ERR_ARG, "gemv group mixes formats or row lengths");
        if (w.N > 0x7fffffffu / 4 || w.K > (size_t(1) << 20))
            return fail(c, SMX_ERR_LIMIT, "gemv: shape %zu x %zu exceeds the kernel's index range", w.N, w.K);
        maxN = std::max(maxN, w.N);
        J.job[i].W = {w.scales, (const uint4*)w.quants, (const uint4*)w.qh, (const uint2*)w.sc};
        J.job[i].x = xs[i];
        if (prod) {
            J.job[i].x2 = x2s ? x2s[i] : prod->b;
            J.job[i].prod = prod->kind;
            J.job[i].eps = prod->eps;
        }
        J.job[i].y = ys[i];
        J.job[i].N = (int)w.N;
    }
    const Weight& w0 = *ws[0];
    Geom g = pick_geom(c, w0.type, maxN, w0.nblk, 1, false, n);
    g.prod = prod && prod->kind != SMX_ACT_NONE;
    // Every workgroup runs the producer over the whole row.  For the exp-based ones on a long row
    // (an FFN's down projection) that repeated work outweighs a launch: they run once, in a
    // quantiser kernel of their own, and the GEMV stages the quantised row.
    if (g.prod && (prod->kind == SMX_ACT_SILU_MUL || prod->kind == SMX_ACT_GEGLU) && w0.K >= kProducerSplitK) {
        const float* bs[SMX_GEMV_GROUP_MAX];
        for (int i = 0; i < n; i++) bs[i] = J.job[i].x2;
        const size_t nb = w0.K / 32;
        int rc;
        if ((rc = ensure(c, c->xq, (size_t)n * w0.K)) != SMX_OK) return rc;
        if ((rc = ensure(c, c->xd, (size_t)n * nb * 4)) != SMX_OK) return rc;
        if ((rc = ensure(c, c->xs, (size_t)n * nb * 4)) != SMX_OK) return rc;
        rc = launch_actprod_quant(c, prod->kind, xs, bs, n, w0.K, (int8_t*)c->xq.p, (float*)c->xd.p, (int32_t*)c->xs.p);
        if (rc != SMX_OK) return rc;
        for (int i = 0; i < n; i++)
            J.job[i].set_x(GemvX{nullptr, (const int8_t*)c->xq.p + (size_t)i * w0.K, (const float*)c->xd.p + (size_t)i * nb,
                                 (const int*)c->xs.p + (size_t)i * nb});
        g.prod = false;
        g.preq = true;
    }
    if (g.lds > 160 * 1024) return fail(c, SMX_ERR_LIMIT, "gemv: activation of %zu needs %zu bytes of LDS", w0.K, g.lds);
    return launch_jobs(c, w0.type, g, J, n, (int)w0.nblk, 1, 1, nullptr, 0, name);
}

// npairs (gate, up) pairs of one format and shape in one launch: h[p][r] = act2(gate_p[r] . x_p) * (up_p[r] . x_p), the
// activation optionally behind rmsnorm (prod).  yg / yu (optional, per pair) also receive the two dots.  *served = false
// (and nothing launched) when the shape does not take the flat form: the caller then runs the projections and the
// product separately.
int launch_gemv_dual(smx_ctx* c, const Weight* const* wg, const Weight* const* wu, const float* const* xs, float* const* yg,
                     float* const* yu, float* const* hs, int npairs, int act2, const ActProd* prod, const char* name, bool* served,
                     const GemvIndirect* ind) {
    *served = false;
    if (npairs < 1 || 2 * npairs > SMX_GEMV_GROUP_MAX) return fail(c, SMX_ERR_ARG, "paired gemv of %d pairs", npairs);
    if (act2 != SMX_ACT_SILU_MUL && act2 != SMX_ACT_GEGLU) return fail(c, SMX_ERR_ARG, "paired gemv: activation %d", act2);
    if (prod && prod->kind != SMX_ACT_NONE && prod->kind != SMX_ACT_RMSNORM)
        return fail(c, SMX_ERR_ARG, "paired gemv: the activation row may pass through rmsnorm only");
    const Weight& w0 = *wg[0];
    GemvJobs J = {};
    if (ind) {   // experts chosen on the device: both jobs of a pair read the same routing slot
        if (prod && prod->kind != SMX_ACT_NONE) return fail(c, SMX_ERR_ARG, "paired gemv: device-routed experts take the plain activation row");
        J.ids = ind->ids;
        J.ne = ind->ne;
        J.blocks_per_expert = ind->blocks_per_expert;
        for (int p = 0; p < npairs; p++) J.slot[2 * p] = J.slot[2 * p + 1] = ind->slot[p];
        if (ind->logits) {   // routed inside this launch
            if (ind->ne > 64 || ind->route_k < 1 || ind->route_k > ind->ne || !ind->ids_out || !ind->w_out)
                return fail(c, SMX_ERR_ARG, "paired gemv: in-launch routing takes up to 64 experts and buffers for the routing");
            J.logits = ind->logits;
            J.route_k = ind->route_k;
            J.ids_out = ind->ids_out;
            J.w_out = ind->w_out;
        }
    }
    for (int p = 0; p < npairs; p++) {
        const Weight *a = wg[p], *b = wu[p];
        if (a->type != w0.type || b->type != w0.type || a->K != w0.K || b->K != w0.K || a->N != w0.N || b->N != w0.N)
            return fail(c, SMX_ERR_ARG, "paired gemv mixes formats or shapes");
        GemvJob& jg = J.job[2 * p];
        GemvJob& ju = J.job[2 * p + 1];
        jg.W = {a->scales, (const uint4*)a->quants, (const uint4*)a->qh, (const uint2*)a->sc};
        ju.W = {b->scales, (const uint4*)b->quants, (const uint4*)b->qh, (const uint2*)b->sc};
        jg.x = ju.x = xs[p];
        if (prod && prod->kind == SMX_ACT_RMSNORM) {
            jg.x2 = prod->b;
            jg.prod = prod->kind;
            jg.eps = prod->eps;
        }
        jg.y = yg ? yg[p] : nullptr;
        ju.y = yu ? yu[p] : nullptr;
        jg.h = hs[p];
        jg.act2 = act2;
        jg.N = ju.N = (int)a->N;
    }
    if (w0.N > 0x7fffffffu / 4 || w0.K > (size_t(1) << 20))
        return fail(c, SMX_ERR_LIMIT, "gemv: shape %zu x %zu exceeds the kernel's index range", w0.N, w0.K);
    Geom g = pick_geom(c, w0.type, w0.N, w0.nblk, 1, false, npairs);
    if (!g.flat) return SMX_OK;
    // the group sums of both weights live in LDS side by side
    const size_t upb = w0.type == kQ6_K ? 4 : (w0.type == kQ8_0 ? 2 : 1);
    const size_t rows = (w0.N + g.grid - 1) / g.grid;
    g.lds += rows * w0.nblk * upb / g.flat * 4;
    if (w0.type != kQ6_K && g.flat == 16) g.flat_pre = pick_flat_pre(2 * rows * w0.nblk * upb);   // both weights' units in one sequence
    if (g.lds + (ind && ind->logits ? 8192 : 0) > 160 * 1024) return SMX_OK;   // (in-launch routing keeps 4.3 KB of LDS of its own)
    const bool norm = prod && prod->kind == SMX_ACT_RMSNORM;
    const unsigned units = (unsigned)(w0.nblk * upb);
    const unsigned magic = (unsigned)(((1ull << 32) + units - 1) / units);
    for (int i = 0; i < 2 * npairs; i++) { J.job[i].nblk = (int)w0.nblk; J.job[i].m = 1; J.job[i].n_wgs = (int)g.grid; J.job[i].magic_u = magic; }
    ProfScope ps(c, name ? name : "gemv_gate_up_act");
    auto go = [&](auto kern) -> int {
        int rc = set_dyn_lds(c, kern, g.lds);
        if (rc != SMX_OK) return rc;
        hipLaunchKernelGGL(kern, dim3(g.grid, (unsigned)npairs), dim3(1024), g.lds, c->stream, J);
        SMX_HIP(c, hipGetLastError());
        *served = true;
        return SMX_OK;
    };
#define SMX_DUAL(OPS, PRE, GL)                                                                                  \
    if (g.flat_pre == PRE && g.flat == GL)                                                                      \
        return ind ? (ind->logits ? go(gemv_flat_dual_kernel<OPS, PRE, GL, 1, 2>) : go(gemv_flat_dual_kernel<OPS, PRE, GL, 1, 1>)) \
                   : (norm ? go(gemv_flat_dual_kernel<OPS, PRE, GL, 2>) : go(gemv_flat_dual_kernel<OPS, PRE, GL, 1>));
    if (w0.type == kQ4_0) { SMX_DUAL(OpsQ4_0, 3, 16) SMX_DUAL(OpsQ4_0, 3, 8) SMX_DUAL(OpsQ4_0, 2, 16) SMX_DUAL(OpsQ4_0, 4, 16) }
    else if (w0.type == kQ8_0) { SMX_DUAL(OpsQ8_0, 3, 16) SMX_DUAL(OpsQ8_0, 3, 8) SMX_DUAL(OpsQ8_0, 2, 16) SMX_DUAL(OpsQ8_0, 4, 16) }
    else { SMX_DUAL(OpsQ6_K, 1, 16) SMX_DUAL(OpsQ6_K, 1, 8) SMX_DUAL(OpsQ6_K, 1, 4) }
#undef SMX_DUAL
    return SMX_OK;   // no variant for this geometry: not served
}

}  // namespace smx
