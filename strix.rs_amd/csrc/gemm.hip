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
//   * Q6_K weights (kernels.rs:1688-1735 q6_gemm_moe keeps them in their 210-byte form too): the 6-bit
//     quants are widened to signed int8 (q - 32) while being staged, and because the format scales
//     16-element sub-blocks each 32-block takes two v_mfma_i32_32x32x16_i8, one exact i32 per
//     sub-block, each rescaled by its own d * sc (four VALU operations per output per 32-block);
//   * split-K: grid.z slices of whole stages write fp32 partials that a second kernel sums in slice
//     order (deterministic, unlike the reference's atomicAdd, kernels.rs:597).
// Bound: dense int8 MFMA, 2*M*N*K operations.
#include <algorithm>

#include "mfma_dev.h"
#include "smx_internal.h"

namespace smx {

constexpr int BN = 128, KB = 4;
constexpr int GRP = 1024;                   // 8 rows x 128 B of one stage: row r at r * 128, its 16-byte chunk c at slot (c + r) % 8
constexpr int B_BYTES = 16 * GRP;           // 128 weight rows
// A workgroup of NW waves covers 32 * NW tokens x 128 weight rows (NW = 8: 256 x 128, one workgroup
// per CU; NW = 4: 128 x 128, two per CU).  The larger tile reads 25 % fewer operand bytes per
// operation through L2, which is what bounds the kernel after the epilogue FMAs.
constexpr int a_bytes(int NW) { return 4 * NW * GRP; }
constexpr int stage_bytes(int NW, bool q6 = false) { return a_bytes(NW) + B_BYTES + (q6 ? 2 : 1) * KB * 128 * 4 + KB * 32 * NW * 4; }
// four 6-bit quants (low nibbles in lo4, the two high bits in hi2) -> four signed bytes q - 32
__device__ __forceinline__ unsigned q6_bytes(unsigned lo4, unsigned hi2) {
    return (((lo4 & 0x0f0f0f0fu) | ((hi2 & 0x03030303u) << 4) | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
}

// Operand fragments of one 32-block.  SUB = 1: one K = 32 MFMA per row tile, a lane holds 16 k of
// its row; SUB = 2 (Q6_K): two K = 16 MFMAs, a lane holds 8 k of each 16-element sub-block.
template <int SUB>
struct GemmFrag {
    v4i a;           // this wave's 32 tokens x 32 k
    v4i b[4];        // 4 x (32 weight rows x 32 k)
    float4 dx[4];    // SUB = 1: activation scales of the 16 tokens this lane accumulates
    float dxv;       // SUB = 2: one scale per lane: lane n of each 16-lane row holds the scale of the token of accumulator n
    float dw[4][SUB];  // weight scale of this lane's row in each of the 4 row tiles (per sub-block)
};

constexpr int FMT_Q8 = 0, FMT_Q4 = 1, FMT_Q6 = 2;

// Optional per-workgroup timeline (development builds only: -DSMX_GEMM_TRACE; compiled out of the library): start and end of
// every workgroup of a launch on the constant 100 MHz clock, with its live tokens and the hardware unit it ran on.
#ifdef SMX_GEMM_TRACE
__device__ unsigned long long* g_gemm_trace = nullptr;   // [(grouped gate/up launch: 4096) + workgroup][4]
#define SMX_GEMM_T0 const unsigned long long smx_t0 = wall_clock64()
#define SMX_GEMM_T1(LIVE, OP)                                                                                                  \
    do {                                                                                                                        \
        if (threadIdx.x == 0 && g_gemm_trace && blockIdx.x < 4096) {                                                            \
            unsigned long long* o_ = g_gemm_trace + ((size_t)(p.nops > 1 ? 4096 : 0) + blockIdx.x) * 4;                         \
            o_[0] = smx_t0; o_[1] = wall_clock64(); o_[2] = (unsigned long long)(LIVE) | ((unsigned long long)(OP) << 32);      \
            o_[3] = (unsigned long long)__builtin_amdgcn_s_getreg(63492) | ((unsigned long long)__builtin_amdgcn_s_getreg(63508) << 32); \
        }                                                                                                                       \
    } while (0)
#else
#define SMX_GEMM_T0 do { } while (0)
#define SMX_GEMM_T1(LIVE, OP) do { } while (0)
#endif

template <int FMT, bool DUMP, int NW>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 1 : 2) void gemm_i8_kernel(GemmArgs p) {
    SMX_GEMM_T0;
    constexpr bool Q4 = FMT == FMT_Q4, Q6 = FMT == FMT_Q6;
    static_assert(!Q6 || NW == 4, "the Q6_K staging map is written for 256 threads");
    constexpr int SUB = Q6 ? 2 : 1;  // scaled sub-blocks per 32-block
    constexpr int BM = 32 * NW, A_BYTES = a_bytes(NW), STAGE_BYTES = stage_bytes(NW, Q6);
    constexpr int BG = 16 / NW;  // 8-row groups of B each wave stages
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = p.nb * 32;
    const unsigned smem_base = lds_addr(smem);

    // tile coordinates; consecutive logical tiles share a weight strip, and each XCD (blockIdx % 8)
    // gets a contiguous range of logical tiles so its L2 holds few strips
    int t = blockIdx.x;
    int tok0, row0, col0, M_end, N_end;
    int op_i = blockIdx.y;
    if (p.tiles) {  // grouped (MoE): tile table, A rows are slots of one expert, B rows that expert's rows
        // the operands (gate, up) of a tile are neighbours in the launch order, so that the table's order
        // (longest tiles first) holds for all of them
        op_i = t % p.nops;
        t /= p.nops;
        const GemmTile tl = p.tiles[t];
        tok0 = tl.tok0; M_end = tl.tok_end; row0 = tl.row0; N_end = tl.row_end; col0 = tl.col0;
    } else {
        // The first `narrow` strips of N are 96 rows high and dispatched last (see launch_gemm); each part (128-row strips,
        // 96-row strips) is walked on its own.
        const int full_strips = p.tiles_n - p.narrow;
        const int t_full = full_strips * p.tiles_m;
        const bool nar = t >= t_full;   // never without narrow strips
        if (nar) t -= t_full;
        const int ns = nar ? p.narrow : full_strips;
        const int T = ns * p.tiles_m;
        if (p.xcd_remap & (nar ? 2 : 1)) t = (t & 7) * (T >> 3) + (t >> 3);
        // logical order: token-tile group (walk_gm token tiles), weight strip, token tile inside the group
        const int per_group = p.walk_gm * ns;
        const int grp = t / per_group, in_grp = t - grp * per_group;
        const int tn = in_grp / p.walk_gm, tm = grp * p.walk_gm + (in_grp - tn * p.walk_gm);
        tok0 = tm * p.tile_m; M_end = min(p.M, tok0 + p.tile_m);
        row0 = nar ? tn * 96 : p.narrow * 96 + tn * BN;
        N_end = nar ? row0 + 96 : p.N;
        col0 = row0;
    }
    const GemmOperand op = p.op[op_i];
    // Wave roles.  A full tile gives each wave 32 tokens x 128 rows (4 row tiles).  A tile with few live
    // tokens (the tail of M, a small expert group) would leave three of the four waves idle, so its waves
    // share the token sub-tiles that are live and split the rows: <= 32 tokens: every wave takes the first
    // 32 tokens and ONE row tile; <= 64 tokens: two waves per token half, two row tiles each.
    const int live_tok = M_end - tok0;
    const int tw = NW == 4 ? (live_tok <= 32 ? 0 : live_tok <= 64 ? (wave & 1) : wave) : wave;   // token sub-tile
    const int live_rows = min(N_end - row0, BN);
    const int full_cnt = (live_rows + 31) >> 5;   // a tile at the end of N, or a 96-row strip: only the row tiles that exist
    const int nt_cnt = NW == 4 ? (live_tok <= 32 ? 1 : live_tok <= 64 ? 2 : full_cnt) : full_cnt;   // row tiles of this wave
    const int nt_base = NW == 4 ? (live_tok <= 32 ? wave : live_tok <= 64 ? (wave >> 1) * 2 : 0) : 0;

    const int nstage_total = (p.nb + KB - 1) / KB;
    const int s_begin = blockIdx.z * p.stages_per_slice;
    const int s_end = min(nstage_total, s_begin + p.stages_per_slice);

    // ---- staging.  int8 operands go global -> LDS directly, one 8-row x 128-byte group per wave
    //      instruction, lane = [row:3][slot:3]: the 8 lanes of a row fetch its whole 128-byte line
    //      (scattered 16-byte fetches run at a fraction of the L2 -> CU rate), and lane (r, slot)
    //      fetches chunk (slot - r) % 8, so that chunk c of the 8 rows of a group lies in 8 different
    //      bank groups and every MFMA fragment read below is a conflict-free 128-bit load.
    //      Rows past the tile's end and blocks past K re-read valid memory (clamped addresses) and
    //      are neutralised by zero scales.  Q4_0 weights pass through registers to be widened. ----
    const int g_rowlo = lane >> 3, g_chunk = ((lane & 7) - g_rowlo) & 7;
    const int q_bi = lane & 3, q_rowlo = lane >> 2;   // Q4_0 B: lane = [row:4][block:2], 64 contiguous bytes per row
    constexpr int QG = Q4 ? 8 / NW : 1;  // Q4_0 B: 16-byte blocks per thread per stage
    // Q6_K B: thread = [row:7][p:1]; per stage (one half of a superblock) it reads ql[16p..], ql[32 + 16p..]
    // and qh[16p..] of that half and makes the four 16-byte chunks 2j + p, j = 0..3 (ggml_quant.rs:417-426)
    const int q6_row = tid >> 1, q6_p = tid & 1;
    unsigned a_off[4], b_off[Q4 ? QG : BG];  // element offsets; the launcher keeps M*K and N*K below 2^31
#pragma unroll
    for (int ps = 0; ps < 4; ps++) {
        const int ti = min(tok0 + (ps * NW + wave) * 8 + g_rowlo, M_end - 1);
        a_off[ps] = (unsigned)(p.a_rowmap ? p.a_rowmap[ti] : ti) * (unsigned)K;
    }
    if (Q6) {
        b_off[0] = (unsigned)min(row0 + q6_row, N_end - 1) * (unsigned)(p.nb >> 3);  // first superblock of the row
    } else if (!Q4) {
#pragma unroll
        for (int ps = 0; ps < BG; ps++)
            b_off[ps] = (unsigned)min(row0 + (ps * NW + wave) * 8 + g_rowlo, N_end - 1) * (unsigned)K;
    } else {
#pragma unroll
        for (int ps = 0; ps < QG; ps++)
            b_off[ps] = (unsigned)min(row0 + (ps * NW + wave) * 16 + q_rowlo, N_end - 1) * (unsigned)p.nb;
    }
    // scales of a stage (4 blocks): threads 0..127 carry the four f16 scales of weight row tid (8
    // contiguous bytes), threads 128..128+BM-1 the four fp32 scales of token tid - 128 (16 contiguous
    // bytes): one load per thread when rows are 4-block aligned (nb % 4 == 0), four clamped loads otherwise.
    // Q6_K weight scales: thread (wr, wh) carries d and the sub-block scales 4*wh .. 4*wh+3 of row wr.
    const bool role_w = tid < 128, role_x = !role_w && tid - 128 < BM;   // wave-uniform
    const int role_r = role_w ? tid : tid - 128;
    const bool vec_sc = (p.nb & 3) == 0;
    const int wr = tid & 127, wh = tid >> 7;
    const bool w_valid = row0 + wr < N_end, x_valid = tok0 + role_r < M_end;
    const size_t scw_base = (size_t)min(row0 + wr, N_end - 1) * (Q6 ? p.nb >> 3 : p.nb);
    size_t scx_base;
    {
        const int ti = min(tok0 + role_r, M_end - 1);
        scx_base = (size_t)(p.a_rowmap ? p.a_rowmap[ti] : ti) * p.nb;
    }
    uint4 rb[Q6 ? 3 : QG];  // Q4_0 / Q6_K quants on their way through registers
    uint4 rsv = {0, 0, 0, 0};  // the thread's four raw scales: f16 pairs in .x .y (weights) or four fp32 (activations)
    uint16_t rsd = 0;   // Q6_K: d of the superblock, row wr
    unsigned rsc = 0;   // Q6_K: the four sub-block scales 4 * wh .. 4 * wh + 3 of the stage, row wr

    // issue every global read of stage s; the register-staged parts are written by finish_stage
    // all global reads of stage s (issuing them piecemeal between the blocks measures slower)
    auto issue_stage = [&](int buf, int s) {
        const unsigned sA = __builtin_amdgcn_readfirstlane(smem_base + buf * STAGE_BYTES + wave * GRP);
        const unsigned sB = sA + A_BYTES;
        const int blk0 = s * KB;
        const int koff = min(blk0 * 32 + g_chunk * 16, K - 16);
        // 8-token groups wholly past the tile's end are not fetched (nothing reads their LDS rows)
#pragma unroll
        for (int ps = 0; ps < 4; ps++)
            if ((ps * NW + wave) * 8 < live_tok) load_to_lds16(p.xq, a_off[ps] + koff, sA + ps * NW * GRP);
        if (Q6) {
            const size_t sbi = (size_t)b_off[0] + (s >> 1);
            const char* ql = (const char*)op.wquants + sbi * 128 + (s & 1) * 64 + q6_p * 16;
            rb[0] = *(const uint4*)ql;
            rb[1] = *(const uint4*)(ql + 32);
            rb[2] = *(const uint4*)((const char*)op.wqh + sbi * 64 + (s & 1) * 32 + q6_p * 16);
        } else if (!Q4) {
#pragma unroll
            for (int ps = 0; ps < BG; ps++)
                if ((ps * NW + wave) * 8 < live_rows) load_to_lds16(op.wquants, b_off[ps] + koff, sB + ps * NW * GRP);
        } else {
            const int bq = min(blk0 + q_bi, p.nb - 1);
#pragma unroll
            for (int ps = 0; ps < QG; ps++) rb[ps] = ((const uint4*)op.wquants)[b_off[ps] + bq];
        }
        // branch-free and unconverted, so that nothing here waits for a load before the MFMA work
        if (Q6) {
            rsd = op.wscales[scw_base + (s >> 1)];
            rsc = *(const unsigned*)(op.wsc + (scw_base + (s >> 1)) * 16 + (s & 1) * 8 + wh * 4);
        } else if (role_w) {
            const uint16_t* ws = op.wscales + scw_base;
            if (vec_sc) {
                const uint2 v = *(const uint2*)(ws + blk0);
                rsv.x = v.x; rsv.y = v.y;
            } else {
                const int last = p.nb - 1;
                rsv.x = (unsigned)ws[min(blk0, last)] | ((unsigned)ws[min(blk0 + 1, last)] << 16);
                rsv.y = (unsigned)ws[min(blk0 + 2, last)] | ((unsigned)ws[min(blk0 + 3, last)] << 16);
            }
        }
        if (role_x) {
            const unsigned* xs = (const unsigned*)p.xd + scx_base;
            if (vec_sc) {
                rsv = *(const uint4*)(xs + blk0);
            } else {
                const int last = p.nb - 1;
                rsv.x = xs[min(blk0, last)]; rsv.y = xs[min(blk0 + 1, last)];
                rsv.z = xs[min(blk0 + 2, last)]; rsv.w = xs[min(blk0 + 3, last)];
            }
        }
    };

    auto finish_stage = [&](int buf, int s) {
        char* sB = smem + buf * STAGE_BYTES + A_BYTES;
        float* sdw = (float*)(sB + B_BYTES);
        float* sdx = sdw + SUB * KB * 128;
        const int blk0 = s * KB;
        if (Q6) {
            const int r = q6_row;
            const int off = (r >> 3) * GRP + (r & 7) * 128;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint4 q = rb[j & 1], h = rb[2];
                const int ls = (j >> 1) * 4, hs = 2 * j;
                uint4 o;
                o.x = q6_bytes(q.x >> ls, h.x >> hs);
                o.y = q6_bytes(q.y >> ls, h.y >> hs);
                o.z = q6_bytes(q.z >> ls, h.z >> hs);
                o.w = q6_bytes(q.w >> ls, h.w >> hs);
                *(uint4*)(sB + off + ((2 * j + q6_p + r) & 7) * 16) = o;  // elements 32j + 16p .. + 15 of the stage
            }
            const float d = w_valid ? h2f_(rsd) : 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++)  // d * sc is exact in fp32 (11 x 8 significant bits)
                sdw[(wh * 4 + j) * 128 + wr] = d * (float)(int)(signed char)(rsc >> (8 * j));
        }
        if (Q4) {
#pragma unroll
            for (int ps = 0; ps < QG; ps++) {
                const int r = (ps * NW + wave) * 16 + q_rowlo;
                const int off = (r >> 3) * GRP + (r & 7) * 128;  // + slot * 16
                const uint4 q = rb[ps];
                uint4 lo, hi;
                lo.x = sub8(q.x & 0x0f0f0f0fu); hi.x = sub8((q.x >> 4) & 0x0f0f0f0fu);
                lo.y = sub8(q.y & 0x0f0f0f0fu); hi.y = sub8((q.y >> 4) & 0x0f0f0f0fu);
                lo.z = sub8(q.z & 0x0f0f0f0fu); hi.z = sub8((q.z >> 4) & 0x0f0f0f0fu);
                lo.w = sub8(q.w & 0x0f0f0f0fu); hi.w = sub8((q.w >> 4) & 0x0f0f0f0fu);
                *(uint4*)(sB + off + ((2 * q_bi + r) & 7) * 16) = lo;      // elements 0..15 of the block
                *(uint4*)(sB + off + ((2 * q_bi + 1 + r) & 7) * 16) = hi;  // elements 16..31
            }
        }
        if (!Q6 && role_w) {   // the four block scales of a row side by side: one 16-byte write here, one 16-byte read per row tile and stage
            const unsigned h[4] = {rsv.x & 0xffffu, rsv.x >> 16, rsv.y & 0xffffu, rsv.y >> 16};
            float v[KB];
#pragma unroll
            for (int j = 0; j < KB; j++) v[j] = (w_valid && blk0 + j < p.nb) ? h2f_((uint16_t)h[j]) : 0.f;
            *(float4*)(sdw + wr * 4) = make_float4(v[0], v[1], v[2], v[3]);
        }
        if (role_x) {
            const unsigned v[4] = {rsv.x, rsv.y, rsv.z, rsv.w};
#pragma unroll
            for (int j = 0; j < KB; j++) sdx[j * BM + role_r] = (x_valid && blk0 + j < p.nb) ? __uint_as_float(v[j]) : 0.f;
        }
    };

    float acc[4][16];
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[nt][i] = 0.f;
    v16i cmagic;
#pragma unroll
    for (int i = 0; i < 16; i++) cmagic[i] = MAGIC_I;
    asm volatile("" : "+v"(cmagic));  // keep the constant in vector registers: re-materialising it costs 8 moves per block

    const int half = lane >> 5, col = lane & 31;
    // fragment (tile, block bi): lane -> row lane % 32 of the tile, k-half lane / 32
    int frag_lane[KB];
#pragma unroll
    for (int bi = 0; bi < KB; bi++) frag_lane[bi] = (col >> 3) * GRP + (col & 7) * 128 + ((2 * bi + half + col) & 7) * 16;
    // Q6_K: a lane takes bytes 8 * half .. + 7 of BOTH 16-byte chunks of the block (the order of k
    // inside an MFMA does not matter as long as both operands use the same one)
    const int dx_tok = ((lane & 15) >> 2) * 8 + half * 4 + (lane & 3);  // token of accumulator lane % 16 in this lane's half
    const int frag6 = (col >> 3) * GRP + (col & 7) * 128 + half * 8;

    float4 stage_dw[4];   // Q8_0 / Q4_0: the weight scales of this lane's row in each row tile, four blocks of the stage
    auto read_stage_scales = [&](int buf) {
        if (Q6) return;
        const float* sdw = (const float*)(smem + buf * STAGE_BYTES + A_BYTES + B_BYTES);
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
            if (nt >= nt_cnt) break;
            stage_dw[nt] = *(const float4*)(sdw + ((nt_base + nt) * 32 + col) * 4);
        }
    };
    auto read_frag = [&](GemmFrag<SUB>& f, int buf, int bi) {
        const char* sA = smem + buf * STAGE_BYTES;
        const char* sB = sA + A_BYTES;
        const float* sdw = (const float*)(sB + B_BYTES);
        const float* sdx = sdw + SUB * KB * 128;
        if (Q6) {
            f.dxv = sdx[bi * BM + tw * 32 + dx_tok];
        } else {
#pragma unroll
            for (int g = 0; g < 4; g++) f.dx[g] = *(const float4*)(sdx + bi * BM + tw * 32 + g * 8 + half * 4);
        }
        const char* sBw = sB + nt_base * 4 * GRP;   // this wave's row tiles
        const float* sdww = sdw + nt_base * 32;
        if (Q6) {
            const int o0 = frag6 + ((2 * bi + col) & 7) * 16, o1 = frag6 + ((2 * bi + 1 + col) & 7) * 16;
            const int2 a0 = *(const int2*)(sA + tw * 4 * GRP + o0), a1 = *(const int2*)(sA + tw * 4 * GRP + o1);
            f.a = v4i{a0.x, a0.y, a1.x, a1.y};
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                if (nt >= nt_cnt) break;
                const int2 b0 = *(const int2*)(sBw + nt * 4 * GRP + o0), b1 = *(const int2*)(sBw + nt * 4 * GRP + o1);
                f.b[nt] = v4i{b0.x, b0.y, b1.x, b1.y};
#pragma unroll
                for (int jj = 0; jj < SUB; jj++) f.dw[nt][jj] = sdww[(2 * bi + jj) * 128 + nt * 32 + col];
            }
        } else {
            f.a = *(const v4i*)(sA + tw * 4 * GRP + frag_lane[bi]);
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                if (nt >= nt_cnt) break;
                f.b[nt] = *(const v4i*)(sBw + nt * 4 * GRP + frag_lane[bi]);
                f.dw[nt][0] = bi == 0 ? stage_dw[nt].x : (bi == 1 ? stage_dw[nt].y : (bi == 2 ? stage_dw[nt].z : stage_dw[nt].w));
            }
        }
    };

    // One block: 4 MFMAs, each followed by its 32 epilogue FMAs; MFMA nt + 1 is issued before the
    // FMAs of nt so that the matrix pipe and the vector ALU overlap within the wave.  The empty asm
    // statements pin the order: without them the FMAs of a whole stage sink below its 16 MFMAs,
    // whose results (256 registers) then spill.
    // unit u = row tile u / SUB, sub-block u % SUB
    auto mfma_unit = [&](const GemmFrag<SUB>& f, int u) -> v16i {
        if (Q6) {
            const int nt = u >> 1, jj = u & 1;
            const long a = ((long)(unsigned)f.a[2 * jj]) | ((long)f.a[2 * jj + 1] << 32);
            const long b = ((long)(unsigned)f.b[nt][2 * jj]) | ((long)f.b[nt][2 * jj + 1] << 32);
            return __builtin_amdgcn_mfma_i32_32x32x16_i8(a, b, cmagic, 0, 0, 0);
        }
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a, f.b[u], cmagic, 0, 0, 0);
    };
    auto compute = [&](const GemmFrag<SUB>& f, int blk) {
        const float dxr[16] = {f.dx[0].x, f.dx[0].y, f.dx[0].z, f.dx[0].w, f.dx[1].x, f.dx[1].y, f.dx[1].z, f.dx[1].w,
                               f.dx[2].x, f.dx[2].y, f.dx[2].z, f.dx[2].w, f.dx[3].x, f.dx[3].y, f.dx[3].z, f.dx[3].w};
        v16i d[2];
        d[0] = mfma_unit(f, 0);
#pragma unroll
        for (int u = 0; u < 4 * SUB; u++) {
            const int nt = u / SUB, jj = u % SUB;
            if (nt >= nt_cnt) break;
            if (u + 1 < 4 * SUB && (u + 1) / SUB < nt_cnt) {
                d[(u + 1) & 1] = mfma_unit(f, u + 1);
                asm volatile("" : "+v"(d[(u + 1) & 1]));
            }
            const v16i dn = d[u & 1];
            const float dw = f.dw[nt][jj];
            const float ndw = -dw * MAGIC_F;  // exact: dw has at most 18 significant bits (f16, or f16 x int8)
            if (Q6) {
                scale_accumulate(acc[nt], dn, dw, ndw, f.dxv);
            } else {
#pragma unroll
                for (int i = 0; i < 16; i++) acc[nt][i] = fmaf(dxr[i], fmaf(dw, __int_as_float(dn[i]), ndw), acc[nt][i]);
            }
            asm volatile("" : "+v"(acc[nt][0]), "+v"(acc[nt][1]), "+v"(acc[nt][2]), "+v"(acc[nt][3]), "+v"(acc[nt][4]),
                              "+v"(acc[nt][5]), "+v"(acc[nt][6]), "+v"(acc[nt][7]), "+v"(acc[nt][8]), "+v"(acc[nt][9]),
                              "+v"(acc[nt][10]), "+v"(acc[nt][11]), "+v"(acc[nt][12]), "+v"(acc[nt][13]),
                              "+v"(acc[nt][14]), "+v"(acc[nt][15]));
            if (DUMP) {
                const int row = row0 + (nt_base + nt) * 32 + col;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int tok = tok0 + tw * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                    if (tok < M_end && row < N_end && blk < p.nb)
                        p.dump[((size_t)tok * p.N + row) * (SUB * p.nb) + SUB * blk + jj] = dn[i] - MAGIC_I;
                }
            }
        }
    };

    if (s_begin < s_end) {
        issue_stage(0, s_begin);
        finish_stage(0, s_begin);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // a wave whose 32 tokens all lie past the tile's end (ragged expert groups, M tails) only helps
    // with the staging: its SIMD time goes to the other workgroup on the CU
    const bool wave_live = tw * 32 < live_tok;
    // The waves of a workgroup leave the barrier together, and 8 KB of loads per wave queue up in the
    // CU's one address unit (20 cycles per 1 KB load alone, 64 behind three other waves): even waves
    // issue the next stage's loads before block 0, odd waves after it (measured +4 %; spreading them
    // over all four blocks leaves the last ones too little time to land: +1 %).
    const int my_slot = wave & 1;
    for (int s = s_begin; s < s_end; s++) {
        const int buf = (s - s_begin) & 1;
        const bool more = s + 1 < s_end;
        if (more && (my_slot == 0 || !wave_live)) issue_stage(buf ^ 1, s + 1);
        if (wave_live) {
        GemmFrag<SUB> f0, f1;
        read_stage_scales(buf);
        read_frag(f0, buf, 0);
        read_frag(f1, buf, 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(f0, s * KB + 0);
        __builtin_amdgcn_sched_barrier(0);
        if (more && my_slot == 1) issue_stage(buf ^ 1, s + 1);
        read_frag(f0, buf, 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(f1, s * KB + 1);
        __builtin_amdgcn_sched_barrier(0);
        read_frag(f1, buf, 3);
        __builtin_amdgcn_sched_barrier(0);
        compute(f0, s * KB + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(f1, s * KB + 3);
        __builtin_amdgcn_sched_barrier(0);
        }
        if (more) finish_stage(buf ^ 1, s + 1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    float* out = op.out + (size_t)blockIdx.z * p.M * p.ldo;
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        if (nt >= nt_cnt) break;
        const int row = row0 + (nt_base + nt) * 32 + col;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int tok = tok0 + tw * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
            if (tok < M_end && row < N_end) out[(size_t)tok * p.ldo + col0 + (nt_base + nt) * 32 + col] = acc[nt][i];
        }
    }
    SMX_GEMM_T1(live_tok, op_i);
}

#ifdef SMX_GEMM_TRACE
// buf: device memory for 8192 x 4 u64 (or null to stop); the launches that follow write their workgroups' records
extern "C" int smx_debug_gemm_trace(void* buf) {
    return hipMemcpyToSymbol(HIP_SYMBOL(g_gemm_trace), &buf, sizeof(buf)) == hipSuccess ? 0 : -1;
}
#endif

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
// fill its grid; here: as many K slices as still fit the chip's workgroup slots in ONE round
// (a second, partly filled round costs more than the shorter slices save), whole stages, at least
// 6 stages per slice.  Measured on M = 64..1024 of both FFN shapes.
static int pick_splitk(int slots, int tiles, int nstages) {
    const int z = std::min(slots / std::max(tiles, 1), std::max(1, nstages / 6));
    return std::max(1, std::min(z, 16));
}

template <int FMT, bool DUMP, int NW>
static int launch_gemm_variant(smx_ctx* c, const GemmArgs& p, dim3 grid) {
    auto k = gemm_i8_kernel<FMT, DUMP, NW>;
    const size_t lds = 2 * stage_bytes(NW, FMT == FMT_Q6);
    int rc = set_dyn_lds(c, k, lds);
    if (rc != SMX_OK) return rc;
    hipLaunchKernelGGL(k, grid, dim3(64 * NW), lds, c->stream, p);
    SMX_HIP(c, hipGetLastError());
    return SMX_OK;
}

GemmOperand gemm_operand(const Weight& w, float* out) {
    GemmOperand o = {};
    o.wscales = w.scales;
    o.wquants = w.quants;
    o.out = out;
    o.wqh = w.qh;
    o.wsc = w.sc;
    return o;
}

int launch_gemm(smx_ctx* c, const Weight& w, const int8_t* xq, const float* xd, size_t m, float* y, int32_t* dump) {
    if (w.type != kQ4_0 && w.type != kQ8_0 && w.type != kQ6_K) return fail(c, SMX_ERR_ARG, "gemm: weight type %d not supported", (int)w.type);
    if (m > (size_t(1) << 24) || w.N > (size_t(1) << 24) || w.K > (size_t(1) << 20) || m * w.K >= (size_t(1) << 31) ||
        w.N * w.K >= (size_t(1) << 31))
        return fail(c, SMX_ERR_LIMIT, "gemm: shape m=%zu N=%zu K=%zu exceeds the kernel's index range", m, w.N, w.K);
    GemmArgs p = {};
    p.op[0] = gemm_operand(w, y);
    p.xq = xq;
    p.xd = xd;
    p.a_rowmap = nullptr;
    p.tiles = nullptr;
    p.dump = dump;
    p.M = (int)m;
    p.N = (int)w.N;
    p.ldo = (int)w.N;
    p.nb = (int)(w.K / 32);
    // 128 x 128 tiles, two 4-wave workgroups per CU.  Measured alternatives, all slower on every shape tried
    // (M 512..4096 of both FFN shapes, grouped MoE tiles): 256 x 128 tiles with one 8-wave workgroup per CU
    // (-7 %); three workgroups per CU with 2-block stages, every operand and scale staged LDS-direct and the
    // LDS reads software-pipelined (-5..-10 %: the third wave per SIMD raises the instruction issue rate,
    // and the clock the chip sustains drops by as much).
    const int slots = c->num_cu * 2;
    p.tiles_n = (p.N + BN - 1) / BN;
    // Tokens per tile.  65..128 tokens make one row of 128-token tiles in which half the waves of a workgroup may idle and
    // the K slices are long; as two rows of 64-token tiles (the waves pair up on two row tiles each) the launch has twice
    // the workgroups at half the work each: Q8_0 2560 x 9728 and 9728 x 2560 at 96 / 128 tokens 28.2 / 29.4 -> 25.4 /
    // 26.7 us and 25.9 / 27.3 -> 22.9 / 24.7 us, 15360 x 3840 -2..4 %, the long-K shapes and Q6_K unchanged within 2 %.
    // From 129 tokens on the gain is erratic (-10 .. +20 % with the shape and the split-K factor it meets): 128-token tiles.
    const int bm = (c->tune_gemm_tile_m == 64 || (c->tune_gemm_tile_m == 0 && p.M > 64 && p.M <= 128 && w.type != kQ6_K)) ? 64 : 128;
    p.tile_m = bm;
    p.tiles_m = (p.M + bm - 1) / bm;
    const int T = p.tiles_m * p.tiles_n;
    p.xcd_remap = (T % 8 == 0) ? 1 : 0;
    // Tile walk.  Workgroup t runs on XCD t % 8 and each XCD gets a contiguous eighth of the logical tile order, so the order
    // decides which operand bytes an XCD's 4 MB L2 must see.  Token tiles are taken in groups of walk_gm (up to 8): an XCD then
    // works on walk_gm token tiles x (tiles_n * tiles_m / walk_gm / 8) weight strips instead of all token tiles x an eighth of
    // the strips, whose activations (7.9 MB at M = 2048, K = 3840) it fetched again for every strip.  Measured L2 fills per
    // launch at M = 2048 (rocprofv3 FETCH_SIZE, Q8_0): K 3840 x N 15360 540 -> 341 MB, K 15360 x N 3840 580 -> 366 MB with groups
    // of 8; groups of 4: 360 / 363 MB; of 1 (ffn_down): 947 MB.  The launch time does not move (the kernel is bound by
    // instruction issue, and these fetches are served by the Infinity Cache).
    {
        int gm = std::min(p.tiles_m, 8);
        if (c->tune_gemm_walk > 0) gm = std::max(1, p.tiles_m / c->tune_gemm_walk);
        while (p.tiles_m % gm != 0) gm--;   // whole groups
        p.walk_gm = gm;
    }
    const int nstages = (p.nb + KB - 1) / KB;
    int Z = (dump || (m * w.N) % 4 != 0) ? 1 : (c->tune_gemm_splitk > 0 ? std::min(c->tune_gemm_splitk, nstages) : pick_splitk(slots, T, nstages));
    p.stages_per_slice = (nstages + Z - 1) / Z;
    Z = (nstages + p.stages_per_slice - 1) / p.stages_per_slice;
    // Mixed strips.  When the tiles need several rounds of the chip's workgroup slots and the last round is partly filled,
    // its idle slots cost up to a whole tile's time.  A tile of 96 weight rows runs three of the four row tiles (about 0.8
    // of the time), so with the first `narrow` strips of N cut at 96 rows and dispatched last, the last round can be made
    // of shorter tiles on more slots: 15360 rows x 2048 tokens = 1920 tiles = 3.75 rounds of 512 becomes 1536 tiles of
    // 128 rows (3 rounds) and one round of 512 tiles of 96.  Chosen by the estimated makespan; taken when it saves 3 %, for
    // Q6_K weights only: measured at that shape Q6_K 598 -> 575 us per launch, Q8_0 339.6 -> 337 and Q4_0 350.7 -> 349 (inside
    // the spread between machines, with 2.5 % more vector instructions per launch: a partly filled round runs faster
    // already, a workgroup alone on a CU has its SIMDs to itself).  The knob forces any number of strips for any format.
    if (Z == 1 && bm == 128 && !dump && c->tune_gemm_narrow != 1) {
        const auto makespan = [&](int b) -> double {   // in 128-row tile times; -1: N does not split that way
            if (96 * b > p.N) return -1.0;
            const int a = (p.N - 96 * b + BN - 1) / BN;
            const long full = (long)a * p.tiles_m, nar = (long)b * p.tiles_m;
            const double c96 = 0.80;
            const long q = full / slots, r = full % slots;
            if (nar == 0) return (double)(q + (r ? 1 : 0));
            // narrow tiles go to the slots that are free at q first, then in turn to whichever frees first
            double t_a = (double)q, t_b = (double)q + 1.0;   // slots - r slots free at t_a, r slots at t_b
            long n_a = slots - r, n_b = r, left = nar;
            double end = r ? t_b : t_a;
            while (left > 0) {
                const bool use_a = n_b == 0 || (n_a > 0 && t_a <= t_b);
                const long n = std::min(left, use_a ? n_a : n_b);
                double& tt = use_a ? t_a : t_b;
                if (n < (use_a ? n_a : n_b)) { end = std::max(end, tt + c96); break; }   // the rest of this group stays free
                tt += c96;
                end = std::max(end, tt);
                left -= n;
            }
            return end;
        };
        int best_b = 0;
        if (c->tune_gemm_narrow > 1) {
            best_b = std::min(c->tune_gemm_narrow - 1, p.N / 96);
        } else if (T > slots && w.type == kQ6_K) {
            double best = makespan(0);
            const double need = 0.97 * best;
            for (int b = 1; (long)b * p.tiles_m <= slots && 96 * b <= p.N; b++) {
                const double t = makespan(b);
                if (t > 0 && t < best && t <= need) { best = t; best_b = b; }
            }
        }
        if (best_b > 0) {
            p.narrow = best_b;
            p.tiles_n = best_b + (p.N - 96 * best_b + BN - 1) / BN;
            p.xcd_remap = (((p.tiles_n - best_b) * p.tiles_m) % 8 == 0 ? 1 : 0) | ((best_b * p.tiles_m) % 8 == 0 ? 2 : 0);
        }
    }
    const int T_launch = p.tiles_m * p.tiles_n;
    p.op[0].out = y;
    if (Z > 1) {
        int rc = ensure(c, c->work, (size_t)Z * m * w.N * 4);
        if (rc != SMX_OK) return rc;
        p.op[0].out = (float*)c->work.p;
    }
    const dim3 grid((unsigned)T_launch, 1, (unsigned)Z);
    {
        ProfScope ps(c, w.type == kQ4_0 ? "gemm_i8_q4_0" : w.type == kQ6_K ? "gemm_i8_q6_k" : "gemm_i8_q8_0");
        int rc;
        if (w.type == kQ6_K) {
            rc = dump ? launch_gemm_variant<FMT_Q6, true, 4>(c, p, grid) : launch_gemm_variant<FMT_Q6, false, 4>(c, p, grid);
        } else if (w.type == kQ4_0) {
            rc = dump ? launch_gemm_variant<FMT_Q4, true, 4>(c, p, grid) : launch_gemm_variant<FMT_Q4, false, 4>(c, p, grid);
        } else {
            rc = dump ? launch_gemm_variant<FMT_Q8, true, 4>(c, p, grid) : launch_gemm_variant<FMT_Q8, false, 4>(c, p, grid);
        }
        if (rc != SMX_OK) return rc;
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
int launch_gemm_grouped(smx_ctx* c, QType type, const GemmArgs& args, int ntiles, int nops, const char* name) {
    if (ntiles <= 0) return SMX_OK;
    ProfScope ps(c, name);
    const dim3 grid((unsigned)(ntiles * nops), 1, 1);
    GemmArgs p = args;   // one K slice: every stage
    p.nops = nops;
    p.stages_per_slice = (p.nb + KB - 1) / KB;
    if (type == kQ6_K) return launch_gemm_variant<FMT_Q6, false, 4>(c, p, grid);
    if (type == kQ8_0) return launch_gemm_variant<FMT_Q8, false, 4>(c, p, grid);
    return fail(c, SMX_ERR_ARG, "grouped gemm: weight type %d not supported", (int)type);
}

}  // namespace smx
