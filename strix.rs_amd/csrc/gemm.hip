// int8 W8A8 prefill GEMM on CDNA4 matrix cores: Y[m][N] = Xq . Wq^T with per-32-block fp32 rescale.
//
// Stands in for the reference's WMMA GEMMs (crates/strix-backend-rocm/src/kernels.rs:481-537
// q4_gemm_w, :545-601 q4_gemm_w_sk, :1373-1443 q8w_gemm32) on gfx950:
//   * v_mfma_i32_32x32x32_i8: K = 32 is exactly one quant block, so each MFMA yields the exact
//     i32 block dots of a 32-token x 32-row tile (tokens on the A side, weight rows on the B side:
//     a lane then owns one weight row and 16 tokens, and stores are 128-byte row segments);
//   * workgroup tile 128 tokens x 128 rows, 4 waves, each wave 32 tokens x 128 rows;
//   * K advances 4 blocks (128 bytes per row, one full cache line) per stage, double-buffered
//     through LDS in MFMA-fragment order so every fragment read is one conflict-free 128-bit load;
//   * Q4_0 nibbles are widened to signed int8 (nibble - 8) while being staged (kernels.rs:458-462);
//   * per block and output: acc += dx * (dw * I).  The MFMA accumulates onto the constant
//     0x4B400000 so its i32 result, read as a float, is 12582912 + I exactly; one FMA with the
//     exactly representable -dw*12582912 (dw is an f16 value) gives fl(dw*I) with no int->float
//     conversion, a second FMA applies dx and accumulates: two VALU operations per output per block;
//   * split-K: grid.z slices of whole stages write fp32 partials that a second kernel sums in slice
//     order (deterministic, unlike the reference's atomicAdd, kernels.rs:597).
// Bound: dense int8 MFMA, 2*M*N*K operations.
#include <hip/hip_fp16.h>

#include <algorithm>

#include "smx_internal.h"

namespace smx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, KB = 4;
constexpr int HPLANE = 528;                 // bytes between the two k-halves of a fragment (512 + 16 pad)
constexpr int FRAG = 1040;                  // one 32 x 32 int8 fragment
constexpr int A_BYTES = KB * 4 * FRAG;      // 4 token tiles
constexpr int B_BYTES = KB * 4 * FRAG;      // 4 row tiles
constexpr int S_BYTES = KB * 128 * 4;       // one scale plane
constexpr int STAGE_BYTES = A_BYTES + B_BYTES + 2 * S_BYTES;
constexpr float MAGIC_F = 12582912.f;       // 1.5 * 2^23
constexpr int MAGIC_I = 0x4B400000;

__device__ __forceinline__ float h2f_(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ unsigned sub8(unsigned x) { return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u; }

// (moved to smx_internal.h: GemmOperand, GemmTile, GemmArgs)

template <bool Q4, bool DUMP>
__global__ __launch_bounds__(256, 2) void gemm_i8_kernel(GemmArgs p) {
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = p.nb * 32;

    // tile coordinates; consecutive logical tiles share a weight strip, and each XCD (blockIdx % 8)
    // gets a contiguous range of logical tiles so its L2 holds few strips
    int t = blockIdx.x;
    int tok0, row0, col0, M_end, N_end;
    if (p.tiles) {  // grouped (MoE): tile table, A rows are slots of one expert, B rows that expert's rows
        const GemmTile tl = p.tiles[t];
        tok0 = tl.tok0; M_end = tl.tok_end; row0 = tl.row0; N_end = tl.row_end; col0 = tl.col0;
    } else {
        const int T = p.tiles_m * p.tiles_n;
        if (p.xcd_remap) t = (t & 7) * (T >> 3) + (t >> 3);
        const int tm = t % p.tiles_m, tn = t / p.tiles_m;
        tok0 = tm * BM; row0 = tn * BN; col0 = row0; M_end = p.M; N_end = p.N;
    }
    const GemmOperand op = p.op[blockIdx.y];

    const int nstage_total = (p.nb + KB - 1) / KB;
    const int s_begin = blockIdx.z * p.stages_per_slice;
    const int s_end = min(nstage_total, s_begin + p.stages_per_slice);

    // ---- global -> register staging: branch-free (clamped addresses, masks applied when the
    //      registers are written to LDS) so the loads of stage s+1 stay in flight during stage s ----
    uint4 ra[4], rb[4];
    unsigned rsw;  // raw weight scales: two f16 (blocks 2*sh, 2*sh+1 of the stage) of row sr
    uint2 rsx;     // raw activation scales: two f32 of token sr
    // A (and Q8_0 B): lane = [chunk_hi:2][row_lo:3][chunk_lo:1], 8 rows x 128 B per wave load
    const int g_chunk = ((lane >> 4) << 1) | (lane & 1);  // 16-byte chunk 0..7 within the 128-byte stage row
    const int g_rowlo = (lane >> 1) & 7;
    // Q4_0 B: lane = [bi:2][row_lo:4]
    const int q_bi = lane >> 4, q_rowlo = lane & 15;
    const bool nb4 = (p.nb & 3) == 0;  // whole stages only, scale rows 8/16-byte aligned
    // per-thread row bases (fixed for the whole K loop)
    unsigned a_off[4], b_off[4];  // element offsets; the launcher keeps M*K and N*K below 2^31
#pragma unroll
    for (int ps = 0; ps < 4; ps++) {
        const int r = (ps * 4 + wave) * 8 + g_rowlo;
        const int ti = min(tok0 + r, M_end - 1);
        a_off[ps] = (unsigned)(p.a_rowmap ? p.a_rowmap[ti] : ti) * (unsigned)K;
        if (!Q4) {
            b_off[ps] = (unsigned)min(row0 + r, N_end - 1) * (unsigned)K;
        } else if (ps < 2) {
            const int rq = (ps * 4 + wave) * 16 + q_rowlo;
            b_off[ps] = (unsigned)min(row0 + rq, N_end - 1) * (unsigned)p.nb;
        }
    }
    // scales: thread (sr, sh) carries blocks 2*sh, 2*sh+1 of the stage for weight row sr and token sr
    const int sr = tid & 127, sh = tid >> 7;
    const bool w_valid = row0 + sr < N_end, x_valid = tok0 + sr < M_end;
    const size_t scw_base = (size_t)min(row0 + sr, N_end - 1) * p.nb;
    size_t scx_base;
    {
        const int ti = min(tok0 + sr, M_end - 1);
        scx_base = (size_t)(p.a_rowmap ? p.a_rowmap[ti] : ti) * p.nb;
    }

    auto load_stage = [&](int s) {
        const int blk0 = s * KB;
        const int koff = min(blk0 * 32 + g_chunk * 16, K - 16);  // clamped: a K tail is zeroed at store time
#pragma unroll
        for (int ps = 0; ps < 4; ps++) {
            ra[ps] = *(const uint4*)(p.xq + a_off[ps] + koff);
            if (!Q4) rb[ps] = *(const uint4*)((const int8_t*)op.wquants + b_off[ps] + koff);
        }
        if (Q4) {
            const int bq = min(blk0 + q_bi, p.nb - 1);
#pragma unroll
            for (int ps = 0; ps < 2; ps++) rb[ps] = ((const uint4*)op.wquants)[b_off[ps] + bq];
        }
        if (nb4) {
            rsw = *(const unsigned*)(op.wscales + scw_base + blk0 + 2 * sh);
            rsx = *(const uint2*)(p.xd + scx_base + blk0 + 2 * sh);
        } else {
            const int b0 = min(blk0 + 2 * sh, p.nb - 1), b1 = min(blk0 + 2 * sh + 1, p.nb - 1);
            rsw = (unsigned)op.wscales[scw_base + b0] | ((unsigned)op.wscales[scw_base + b1] << 16);
            rsx = make_uint2(__float_as_uint(p.xd[scx_base + b0]), __float_as_uint(p.xd[scx_base + b1]));
        }
    };

    auto store_stage = [&](int buf, int s) {
        char* sA = smem + buf * STAGE_BYTES;
        char* sB = sA + A_BYTES;
        float* sdw = (float*)(sB + B_BYTES);
        float* sdx = sdw + KB * 128;
        const int blk0 = s * KB;
        const bool tail = blk0 + KB > p.nb;  // uniform: only the last stage of a K that is not a stage multiple
#pragma unroll
        for (int ps = 0; ps < 4; ps++) {
            const int r = (ps * 4 + wave) * 8 + g_rowlo;
            const int off = ((g_chunk >> 1) * 4 + (r >> 5)) * FRAG + (g_chunk & 1) * HPLANE + (r & 31) * 16;
            uint4 va = ra[ps], vb = rb[ps];
            if (tail && blk0 + (g_chunk >> 1) >= p.nb) {
                va = make_uint4(0, 0, 0, 0);
                vb = va;
            }
            *(uint4*)(sA + off) = va;
            if (!Q4) *(uint4*)(sB + off) = vb;
        }
        if (Q4) {
#pragma unroll
            for (int ps = 0; ps < 2; ps++) {
                const int r = (ps * 4 + wave) * 16 + q_rowlo;
                const int off = (q_bi * 4 + (r >> 5)) * FRAG + (r & 31) * 16;
                const uint4 q = rb[ps];
                uint4 lo, hi;
                lo.x = sub8(q.x & 0x0f0f0f0fu); hi.x = sub8((q.x >> 4) & 0x0f0f0f0fu);
                lo.y = sub8(q.y & 0x0f0f0f0fu); hi.y = sub8((q.y >> 4) & 0x0f0f0f0fu);
                lo.z = sub8(q.z & 0x0f0f0f0fu); hi.z = sub8((q.z >> 4) & 0x0f0f0f0fu);
                lo.w = sub8(q.w & 0x0f0f0f0fu); hi.w = sub8((q.w >> 4) & 0x0f0f0f0fu);
                if (tail && blk0 + q_bi >= p.nb) {
                    lo = make_uint4(0, 0, 0, 0);
                    hi = lo;
                }
                *(uint4*)(sB + off) = lo;            // elements 0..15 of the block
                *(uint4*)(sB + off + HPLANE) = hi;   // elements 16..31
            }
        }
        const bool v0 = blk0 + 2 * sh < p.nb, v1 = blk0 + 2 * sh + 1 < p.nb;
        sdw[(2 * sh) * 128 + sr] = (w_valid && v0) ? h2f_((uint16_t)(rsw & 0xffff)) : 0.f;
        sdw[(2 * sh + 1) * 128 + sr] = (w_valid && v1) ? h2f_((uint16_t)(rsw >> 16)) : 0.f;
        sdx[(2 * sh) * 128 + sr] = (x_valid && v0) ? __uint_as_float(rsx.x) : 0.f;
        sdx[(2 * sh + 1) * 128 + sr] = (x_valid && v1) ? __uint_as_float(rsx.y) : 0.f;
    };

    float acc[4][16];
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[nt][i] = 0.f;
    v16i cmagic;
#pragma unroll
    for (int i = 0; i < 16; i++) cmagic[i] = MAGIC_I;

    const int frag_lane = (lane >> 5) * HPLANE + (lane & 31) * 16;
    const int half = lane >> 5, col = lane & 31;

    if (s_begin < s_end) {
        load_stage(s_begin);
        store_stage(0, s_begin);
    }
    __syncthreads();
    for (int s = s_begin; s < s_end; s++) {
        const int buf = (s - s_begin) & 1;
        if (s + 1 < s_end) load_stage(s + 1);
        const char* sA = smem + buf * STAGE_BYTES;
        const char* sB = sA + A_BYTES;
        const float* sdw = (const float*)(sB + B_BYTES);
        const float* sdx = sdw + KB * 128;
#pragma unroll 1
        for (int bi = 0; bi < KB; bi++) {
            const v4i a = *(const v4i*)(sA + (bi * 4 + wave) * FRAG + frag_lane);
            float dxr[16];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 v = *(const float4*)(sdx + bi * 128 + wave * 32 + g * 8 + half * 4);
                dxr[g * 4 + 0] = v.x; dxr[g * 4 + 1] = v.y; dxr[g * 4 + 2] = v.z; dxr[g * 4 + 3] = v.w;
            }
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                const v4i b = *(const v4i*)(sB + (bi * 4 + nt) * FRAG + frag_lane);
                const float dw = sdw[bi * 128 + nt * 32 + col];
                const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, cmagic, 0, 0, 0);
                const float ndw = -dw * MAGIC_F;  // exact: dw has an 11-bit significand
#pragma unroll
                for (int i = 0; i < 16; i++)
                    acc[nt][i] = fmaf(dxr[i], fmaf(dw, __int_as_float(d[i]), ndw), acc[nt][i]);
                if (DUMP) {
                    const int blk = s * KB + bi;
                    const int row = row0 + nt * 32 + col;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int tok = tok0 + wave * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                        if (tok < M_end && row < N_end && blk < p.nb)
                            p.dump[((size_t)tok * p.N + row) * p.nb + blk] = d[i] - MAGIC_I;
                    }
                }
            }
        }
        if (s + 1 < s_end) store_stage(buf ^ 1, s + 1);
        __syncthreads();
    }

    float* out = op.out + (size_t)blockIdx.z * p.M * p.ldo;
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const int row = row0 + nt * 32 + col;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int tok = tok0 + wave * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
            if (tok < M_end && row < N_end) out[(size_t)tok * p.ldo + col0 + nt * 32 + col] = acc[nt][i];
        }
    }
}

// y[i] = sum over slices z (ascending) of part[z][i]
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float4* __restrict__ part, float4* __restrict__ y,
                                                            size_t n4, int Z) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    float4 s = part[i];
    for (int z = 1; z < Z; z++) {
        const float4 v = part[(size_t)z * n4 + i];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    y[i] = s;
}

// Split-K factor: the reference splits only the long-K shapes (in_dim >= 12288, decode.rs:5658) to
// fill its grid; here: split when the tile grid alone leaves most of the 2-per-CU workgroup slots
// empty, into whole stages, and never so far that a slice has fewer than 8 stages.
static int pick_splitk(const smx_ctx* c, int tiles, int nstages) {
    const int slots = c->num_cu * 2;
    if (tiles * 2 > slots) return 1;
    int z = (slots + tiles - 1) / tiles;
    z = std::min(z, std::max(1, nstages / 8));
    return std::min(z, 16);
}

int launch_gemm(smx_ctx* c, const Weight& w, const int8_t* xq, const float* xd, size_t m, float* y, int32_t* dump) {
    if (w.type != kQ4_0 && w.type != kQ8_0) return fail(c, SMX_ERR_ARG, "gemm: weight type %d not supported", (int)w.type);
    if (m > (size_t(1) << 24) || w.N > (size_t(1) << 24) || w.K > (size_t(1) << 20) || m * w.K >= (size_t(1) << 31) ||
        w.N * w.K >= (size_t(1) << 31))
        return fail(c, SMX_ERR_LIMIT, "gemm: shape m=%zu N=%zu K=%zu exceeds the kernel's index range", m, w.N, w.K);
    GemmArgs p = {};
    p.op[0].wscales = w.scales;
    p.op[0].wquants = w.quants;
    p.xq = xq;
    p.xd = xd;
    p.a_rowmap = nullptr;
    p.tiles = nullptr;
    p.dump = dump;
    p.M = (int)m;
    p.N = (int)w.N;
    p.ldo = (int)w.N;
    p.nb = (int)w.nblk;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int T = p.tiles_m * p.tiles_n;
    p.xcd_remap = (T % 8 == 0) ? 1 : 0;
    const int nstages = (p.nb + KB - 1) / KB;
    int Z = (dump || (m * w.N) % 4 != 0) ? 1 : (c->tune_gemm_splitk > 0 ? std::min(c->tune_gemm_splitk, nstages) : pick_splitk(c, T, nstages));
    p.stages_per_slice = (nstages + Z - 1) / Z;
    Z = (nstages + p.stages_per_slice - 1) / p.stages_per_slice;
    p.op[0].out = y;
    if (Z > 1) {
        int rc = ensure(c, c->work, (size_t)Z * m * w.N * 4);
        if (rc != SMX_OK) return rc;
        p.op[0].out = (float*)c->work.p;
    }
    const size_t lds = 2 * STAGE_BYTES;
    const dim3 grid((unsigned)T, 1, (unsigned)Z);
    {
        ProfScope ps(c, w.type == kQ4_0 ? "gemm_i8_q4_0" : "gemm_i8_q8_0");
#define LAUNCH_GEMM(Q4, DUMP)                                                                              \
    do {                                                                                                   \
        auto k = gemm_i8_kernel<Q4, DUMP>;                                                                 \
        static size_t lds_set = 0;                                                                         \
        int rc_ = set_dyn_lds(c, k, lds, &lds_set);                                                        \
        if (rc_ != SMX_OK) return rc_;                                                                     \
        hipLaunchKernelGGL(k, grid, dim3(256), lds, c->stream, p);                                         \
    } while (0)
        if (w.type == kQ4_0) {
            if (dump) LAUNCH_GEMM(true, true); else LAUNCH_GEMM(true, false);
        } else {
            if (dump) LAUNCH_GEMM(false, true); else LAUNCH_GEMM(false, false);
        }
        SMX_HIP(c, hipGetLastError());
    }
    if (Z > 1) {
        const size_t n = m * w.N;
        ProfScope ps(c, "splitk_reduce");
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, c->stream,
                           (const float4*)c->work.p, (float4*)y, n / 4, Z);
        SMX_HIP(c, hipGetLastError());
    }
    return SMX_OK;
}

// Grouped GEMM over a tile table (MoE prefill): one launch covers every expert; grid.y selects
// one of `nops` weight/output pairs that share the activation rows (gate and up).
int launch_gemm_grouped(smx_ctx* c, const GemmArgs& args, int ntiles, int nops, const char* name) {
    if (ntiles <= 0) return SMX_OK;
    const size_t lds = 2 * STAGE_BYTES;
    ProfScope ps(c, name);
    auto k = gemm_i8_kernel<false, false>;
    static size_t lds_set = 0;
    int rc = set_dyn_lds(c, k, lds, &lds_set);
    if (rc != SMX_OK) return rc;
    hipLaunchKernelGGL(k, dim3((unsigned)ntiles, (unsigned)nops, 1), dim3(256), lds, c->stream, args);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

}  // namespace smx
