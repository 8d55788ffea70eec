// Small-batch matmul on the matrix cores: 5..32 activation rows against one resident Q8_0 / Q4_0 weight
// that is streamed from HBM exactly once.  Stands in for the reference's token-tile kernels
// (crates/strix-backend-rocm/src/kernels.rs:1605-1632 q8_gemm_rows, :830-857 q8_gemm_rows32, :1016-1045
// q8i_gemm_rows32; dispatch decode.rs:1742-1766): the n-gram verify step and short prefill chunks.
//
// The dot4 GEMV pays its integer dots and LDS reads once per activation row, the tiled GEMM reads
// 128-byte row pieces of mostly empty 128-token tiles; this kernel has the GEMV's memory side and the
// GEMM's arithmetic:
//   * a workgroup (8 or 16 waves) owns up to 32 consecutive weight rows and a slice of K; every wave takes a run
//     of consecutive 4-block (128 elements per row) pieces of the slice;
//   * a wave's piece (rows x 128 B) goes global -> LDS directly into the wave's own corner of LDS (no
//     registers, no workgroup barrier); LDS turns "lane = 16 bytes of one row" into the MFMA operand
//     "lane = row, k-half", chunk-rotated so the transposed reads spread over the banks (Q4_0 nibbles land
//     raw and are widened to int8 in a second step).  One piece per wave is in flight: the kernel is bound by
//     the number of vector-memory instructions a CU can take, not by bytes, and a ring of several pieces per wave
//     costs re-requested pieces at the end of every run (measured: four in flight 16.4 us, two 14.3, one 13.8 on
//     Q8_0 2560 x 9728 at 16 rows); the other waves of the CU cover a wave's wait;
//   * v_mfma_i32_32x32x32_i8 with the (up to 32) activation rows as the other operand gives the exact
//     i32 block dots of 32 tokens x 32 rows; per block acc += dx * (dw * I) as in the prefill GEMM
//     (magic-constant conversion, activation scale through a DPP row broadcast);
//   * the waves' partial tiles meet in LDS and are added in wave order (deterministic).  With two K
//     slices per row group the two workgroups add onto an output the quantiser launch has zeroed:
//     0 + a + b does not depend on which arrives first.
// HBM-bound by bytes: weight bytes once + m * K activation bytes per workgroup from L2.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "smx_internal.h"

namespace smx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int kMagicI = 0x4B400000;       // float 12582912 = 1.5 * 2^23: adding an i32 |I| < 2^22 to its bits adds I to its value
constexpr float kMagicF = 12582912.f;
constexpr int kPiece = 32 * 128;          // LDS bytes of one piece: 32 rows x 4 blocks of int8
// LDS bytes per wave: the landing area of its piece (Q8_0: 4 KB, already in operand order; Q4_0: 2 KB of raw
// nibbles and the 4 KB area the widened piece is built in)
// and, when the activation fragments travel through LDS too (ALDS, up to 16 token slots), 2 KB for those of a piece
// Q6_K: 2 KB of ql + 1 KB of qh as they are, and the 4 KB widened area.
constexpr int FMT_Q8 = 0, FMT_Q4 = 1, FMT_Q6 = 2;
constexpr int weight_lds(int fmt) { return fmt == FMT_Q4 ? 2048 + kPiece : (fmt == FMT_Q6 ? 3072 + kPiece : kPiece); }
constexpr int wave_lds(int fmt, bool alds) { return weight_lds(fmt) + (alds ? 2048 : 0); }

struct SkinnyArgs {
    const uint16_t* wscales;  // f16 [N][nb]; Q6_K: d [N][K / 256]
    const void* wquants;      // Q8_0: i8 [N][K]; Q4_0: 16 B [N][nb]; Q6_K: ql, 128 B per superblock
    const void* wqh;          // Q6_K: 64 B per superblock
    const int8_t* wsc;        // Q6_K: 16 sub-block scales per superblock
    const int8_t* xq;         // fragment order: [nb][2 k-halves][tslots tokens][16 B] (see skinny_quant_kernel)
    const float* xd;          // [pieces][tslots][4]: the four block scales of a piece side by side per token slot
    float* y;                 // [m][N]
    int* dump;                // optional [m][N][nb] i32 block dots (Q6_K: [m][N][2 nb] sub-block dots)
    size_t xq_tile, xd_tile;  // two token tiles (33..64 rows): bytes from tile 0's quants to tile 1's, floats between their scales
    int m, N, nb;
    int tslots;               // token slots of the fragment-ordered activations: 8, 16 or 32 (per token tile)
    int ksplit;               // K slices per row group (1 or 2)
    int pieces_per_slice;     // 4-block pieces in a slice
    int rows_per_group;       // weight rows a workgroup owns (<= 32): chosen so that the workgroups fill whole rounds of CUs
};

__device__ __forceinline__ float h2f_s(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ unsigned sub8s(unsigned x) { return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u; }

#define SMX_SK_FMAC(I)                                                                      \
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #I " row_mask:0xf bank_mask:0xf" : "+v"(av[I]) : "v"(dxv), "v"(t[I]))

// 64 lanes x 16 bytes from global memory straight into LDS (no register round trip): lane i's bytes land at
// LDS byte address lds_base + 16 * i; lds_base is wave-uniform (M0).  Completion is counted by vmcnt.
__device__ __forceinline__ void load_to_lds16(const void* g, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(g)
                 : "memory", "m0");
}
// Four 6-bit quants -> four signed bytes q - 32.  ql: the dword whose nibbles (low: LS = 0, high: LS = 4) are the low four
// bits; qh: the dword whose bit pairs HS, HS + 1 of every byte are the high two.  q + 96 stays below 256 in every byte, and
// flipping bit 7 then subtracts 128 where it is set and adds 128 (= -128 mod 256) where it is not: two operations after
// the merge, five or six per dword in all.
template <int LS, int HS>
__device__ __forceinline__ unsigned q6_bytes_s(unsigned ql, unsigned qh) {
    const unsigned hi = (HS <= 4 ? qh << (4 - HS) : qh >> (HS - 4)) & 0x30303030u;
    const unsigned q = ((ql >> LS) & 0x0f0f0f0fu) | hi;
    return (q + 0x60606060u) ^ 0x80808080u;
}

__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)p;
}

// What travels in registers for one piece: the activation fragments of its four blocks and the raw scales.
// (Named members, no arrays: the struct travels by value and must stay in registers.)  The weight bytes
// go global -> LDS directly and are counted by vmcnt only.
struct PieceRegs {
    v4i a0, a1, a2, a3;    // activation fragment of each block: lane = (token lane % 32, k-half lane / 32)
    uint2 dw;              // four f16 scales of this lane's weight row; Q6_K: the eight int8 sub-block scales of the piece
    uint16_t d6;           // Q6_K: d of the row's superblock
    uint4 dx;              // four f32 scales (one per block) of the token whose accumulators this lane feeds by row broadcast
    v4i c0, c1, c2, c3;    // second token tile (33..64 rows): its fragments ...
    uint4 dx1;             // ... and scales
};
// vector-memory loads per piece: 6 that return into registers, then up to 4 (Q8_0: 8 rows x 128 B each)
// or 2 (Q4_0: 16 rows x 64 B of nibbles each) LDS-direct ones

// NW waves per workgroup: 16 when the launch has at most one workgroup per CU (otherwise a CU would hold 8 waves
// with one piece in flight each), 8 when two workgroups share a CU.
// ALDS (8 or 16 token slots): the activation fragments of a piece, tslots * 128 contiguous bytes, go global -> LDS
// directly in one or two instructions and every lane reads its own from there, instead of four register loads in
// which most lanes fetch a copy (the kernel is bound by the number of vector-memory instructions).
// Q6_K (always with ALDS, so up to 16 rows): a piece is half a superblock; its ql and qh bytes land as they are (3 LDS-direct
// instructions), the wave widens them to signed int8 in operand order (thread = [row:5][p:1] makes the 16-byte chunks 2j + p,
// ggml_quant.rs:417-426), and a 32-block is two v_mfma_i32_32x32x16_i8, one per 16-element sub-block with its own d * sc.
// NACC: accumulators per lane that hold live tokens (accumulator i of lane half h is token (i / 4) * 8 + 4 h + i % 4: 4 for up
// to 8 token slots, 8 for 16); only those are rescaled -- with all 16 the Q6_K variant would be bound by its vector ALU work,
// and Q4_0 9728 x 2560 takes 1.3 us longer at 5..16 rows.
// TT = 2 (33..64 rows of a Q8_0 / Q4_0 weight): two 32-token tiles share every weight piece -- two MFMAs per block on the same
// weight fragment, 32 accumulators per lane -- so the weight is still read once (the tiled GEMM takes 22 us where 32 rows
// take 14: 128-row strips leave it 20 tiles to split over K, and a reduction launch behind them).
template <int FMT, bool DUMP, int NW, bool ALDS, int NACC = 16, int TT = 1>
__global__ __launch_bounds__(64 * NW) void skinny_kernel(const SkinnyArgs p) {
    constexpr bool Q4 = FMT == FMT_Q4, Q6 = FMT == FMT_Q6;
    static_assert(!Q6 || ALDS, "the Q6_K variant reads its activation fragments from LDS");
    static_assert(TT == 1 || (!ALDS && !Q6 && NACC == 16), "two token tiles: fragments through registers, all accumulators live");
    constexpr int kWaves = NW;
    constexpr int kWaveLds = wave_lds(FMT, ALDS);
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int K = p.nb * 32;
    const int rg = blockIdx.x / p.ksplit, slice = blockIdx.x - rg * p.ksplit;
    const int R = p.rows_per_group;
    const int r0 = rg * R;
    const int r_last = min(r0 + R, p.N) - 1;   // rows of the tile past the group re-read its last row (and are not stored)
    const int piece0 = slice * p.pieces_per_slice;
    const int npieces_total = (p.nb + 3) >> 2;
    const int piece_end = min(piece0 + p.pieces_per_slice, npieces_total);
    char* mine = smem + wave * kWaveLds;
    const unsigned mine_lds = __builtin_amdgcn_readfirstlane(lds_addr(mine));
    const char* mine_a = mine + weight_lds(FMT);   // ALDS: the piece's activation fragments

    // loop-invariant lane roles
    const int wrow = min(r0 + col, r_last);                         // this lane's weight row (MFMA operand and scales)
    const int m0 = TT == 2 ? 32 : p.m, m1 = p.m - 32;                // rows of the first / second token tile
    const int atok = min(col, m0 - 1);                              // this lane's token as the other MFMA operand
    const int atok1 = min(col, max(m1, 1) - 1);
    const int nrows = r_last - r0 + 1;                              // rows of this group: load instructions past them are not issued
    const int dx_slot = ((lane & 15) >> 2) * 8 + half * 4 + (lane & 3);
    const int dx_tok = min(dx_slot, m0 - 1);   // token of accumulator lane % 16 in this lane half
    const int dx_tok1 = min(dx_slot, max(m1, 1) - 1);
    const bool vec_sc = (p.nb & 3) == 0;
    // Q8_0 landing: lane = [row:3][slot:3] of an 8-row group; the lane fetches chunk (slot - row) % 8 of its row, so
    // chunk c of row r sits in slot (c + r) % 8 and the transposed fragment reads spread over the banks
    const int g_rowlo = lane >> 3, g_chunk = ((lane & 7) - g_rowlo) & 7;

    // Every load of a piece: the register loads, then the LDS-direct ones.
    auto request = [&](int piece) -> PieceRegs {
        PieceRegs r;
        const int blk0 = piece * 4;
        if (ALDS) {   // chunk (b * 2 + half) * tslots + token of the whole row set; chunks past the last block re-read it
            const unsigned last = (unsigned)p.nb * 2 * p.tslots - 1;
            for (int j = 0; j * 8 < p.tslots; j++)   // wave-uniform
                load_to_lds16(p.xq + (size_t)min((unsigned)(piece * 8 * p.tslots + j * 64 + lane), last) * 16,
                              mine_lds + weight_lds(FMT) + j * 1024);
            r.a0 = r.a1 = r.a2 = r.a3 = v4i{0, 0, 0, 0};
        } else {   // with 32 token slots a wave's fragment load is one contiguous kilobyte
            auto la = [&](int bi) {
                return *(const v4i*)(p.xq + ((size_t)(min(blk0 + bi, p.nb - 1) * 2 + half) * p.tslots + atok) * 16);
            };
            r.a0 = la(0); r.a1 = la(1); r.a2 = la(2); r.a3 = la(3);
            if constexpr (TT == 2) {
                auto lc = [&](int bi) {
                    return *(const v4i*)(p.xq + p.xq_tile + ((size_t)(min(blk0 + bi, p.nb - 1) * 2 + half) * p.tslots + atok1) * 16);
                };
                r.c0 = lc(0); r.c1 = lc(1); r.c2 = lc(2); r.c3 = lc(3);
            }
        }
        const uint16_t* ws = p.wscales + (size_t)wrow * p.nb;
        r.dx = *(const uint4*)(p.xd + ((size_t)piece * p.tslots + dx_tok) * 4);   // 16 contiguous bytes per token slot
        if constexpr (TT == 2) r.dx1 = *(const uint4*)(p.xd + p.xd_tile + ((size_t)piece * p.tslots + dx_tok1) * 4);
        r.d6 = 0;
        if (Q6) {
            const size_t sb = (size_t)wrow * (p.nb >> 3) + (piece >> 1);
            r.d6 = p.wscales[sb];
            r.dw = *(const uint2*)(p.wsc + sb * 16 + (piece & 1) * 8);
        } else if (vec_sc) {
            r.dw = *(const uint2*)(ws + blk0);
        } else {   // (the scalar form costs more loads; the waits below are then over-conservative, never too lax)
            const int last = p.nb - 1;
            r.dw.x = (unsigned)ws[min(blk0, last)] | ((unsigned)ws[min(blk0 + 1, last)] << 16);
            r.dw.y = (unsigned)ws[min(blk0 + 2, last)] | ((unsigned)ws[min(blk0 + 3, last)] << 16);
        }
        if (Q6) {   // ql: lane = [row:4][chunk:2], 64 bytes per row and half superblock; qh: lane = [row:5][chunk:1], 32 bytes
            const int nsb = p.nb >> 3, sbi = piece >> 1, hs = piece & 1;
#pragma unroll
            for (int j = 0; j < 2; j++)
                if (j * 16 < nrows)   // wave-uniform
                    load_to_lds16((const char*)p.wquants + ((size_t)min(r0 + j * 16 + (lane >> 2), r_last) * nsb + sbi) * 128 + hs * 64 + (lane & 3) * 16,
                                  mine_lds + j * 1024);
            load_to_lds16((const char*)p.wqh + ((size_t)min(r0 + (lane >> 1), r_last) * nsb + sbi) * 64 + hs * 32 + (lane & 1) * 16,
                          mine_lds + 2048);
        } else if (Q4) {   // lane = [row:4][block:2]: 64 contiguous bytes of nibbles per row, landing as they are
            const int b = min(blk0 + (lane & 3), p.nb - 1);
#pragma unroll
            for (int j = 0; j < 2; j++)
                if (j * 16 < nrows)   // wave-uniform
                    load_to_lds16((const uint4*)p.wquants + (size_t)min(r0 + j * 16 + (lane >> 2), r_last) * p.nb + b,
                                  mine_lds + j * 1024);
        } else {
            const int koff = min(blk0 * 32 + g_chunk * 16, K - 16);
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (j * 8 < nrows)   // wave-uniform
                    load_to_lds16((const int8_t*)p.wquants + (size_t)min(r0 + j * 8 + g_rowlo, r_last) * K + koff,
                                  mine_lds + j * 1024);
        }
        return r;
    };

    float acc[16], acc1[TT == 2 ? 16 : 1];
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < (TT == 2 ? 16 : 1); i++) acc1[i] = 0.f;
    v16i cmagic;
#pragma unroll
    for (int i = 0; i < 16; i++) cmagic[i] = kMagicI;

    auto consume = [&](const PieceRegs r, int piece) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the piece's LDS-direct loads (the compiler does not see them)
        const char* buf;
        if (Q6) {   // thread (row, p): ql[16p ..], ql[32 + 16p ..], qh[16p ..] of the row's half superblock -> chunks 2j + p
            char* wide = mine + 3072;
            const int r = lane >> 1, pp = lane & 1;
            const uint4 qa = *(const uint4*)(mine + r * 64 + pp * 16), qb = *(const uint4*)(mine + r * 64 + 32 + pp * 16);
            const uint4 h = *(const uint4*)(mine + 2048 + r * 32 + pp * 16);
            auto chunk = [&](auto jc) {   // chunk 2j + p: ql nibble j / 2 of ql half j % 2, bit pair 2j of qh
                constexpr int j = decltype(jc)::value;
                const uint4 q = (j & 1) ? qb : qa;
                uint4 o;
                o.x = q6_bytes_s<(j >> 1) * 4, 2 * j>(q.x, h.x);
                o.y = q6_bytes_s<(j >> 1) * 4, 2 * j>(q.y, h.y);
                o.z = q6_bytes_s<(j >> 1) * 4, 2 * j>(q.z, h.z);
                o.w = q6_bytes_s<(j >> 1) * 4, 2 * j>(q.w, h.w);
                *(uint4*)(wide + r * 128 + ((2 * j + pp + r) & 7) * 16) = o;   // elements 32 j + 16 p .. + 15 of the piece
            };
            chunk(std::integral_constant<int, 0>()); chunk(std::integral_constant<int, 1>());
            chunk(std::integral_constant<int, 2>()); chunk(std::integral_constant<int, 3>());
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            buf = wide;
        } else if (Q4) {   // widen the raw nibbles (lane = [row:4][block:2]) into the operand-order area
            char* wide = mine + 2048;
            const char* raw = mine;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int row = j * 16 + (lane >> 2), bi = lane & 3;
                const uint4 q = *(const uint4*)(raw + j * 1024 + lane * 16);
                uint4 lo, hi;
                lo.x = sub8s(q.x & 0x0f0f0f0fu); hi.x = sub8s((q.x >> 4) & 0x0f0f0f0fu);
                lo.y = sub8s(q.y & 0x0f0f0f0fu); hi.y = sub8s((q.y >> 4) & 0x0f0f0f0fu);
                lo.z = sub8s(q.z & 0x0f0f0f0fu); hi.z = sub8s((q.z >> 4) & 0x0f0f0f0fu);
                lo.w = sub8s(q.w & 0x0f0f0f0fu); hi.w = sub8s((q.w >> 4) & 0x0f0f0f0fu);
                *(uint4*)(wide + row * 128 + ((2 * bi + row) & 7) * 16) = lo;       // elements 0..15 of the block
                *(uint4*)(wide + row * 128 + ((2 * bi + 1 + row) & 7) * 16) = hi;   // elements 16..31
            }
            // the wave's own LDS writes above are read back by other lanes of the same wave below
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            buf = wide;
        } else {
            buf = mine;
        }
        const int blk0 = piece * 4;
        const unsigned dwh[4] = {r.dw.x & 0xffffu, r.dw.x >> 16, r.dw.y & 0xffffu, r.dw.y >> 16};
        const unsigned dxs[4] = {r.dx.x, r.dx.y, r.dx.z, r.dx.w};
        // acc[i] += dx(token of accumulator i) * fl(dw * I) for the live accumulators, I the exact i32 of MFMA result d
        auto rescale = [&](float (&av)[16], const v16i& d, float dw, float dxv) {
            const float ndw = -dw * kMagicF;   // exact: dw has at most 18 significant bits (f16, or f16 x int8)
            float t[16];
#pragma unroll
            for (int i = 0; i < NACC; i++) t[i] = fmaf(dw, __int_as_float(d[i]), ndw);
            SMX_SK_FMAC(0); SMX_SK_FMAC(1); SMX_SK_FMAC(2); SMX_SK_FMAC(3);
            if constexpr (NACC > 4) { SMX_SK_FMAC(4); SMX_SK_FMAC(5); SMX_SK_FMAC(6); SMX_SK_FMAC(7); }
            if constexpr (NACC > 8) {
                SMX_SK_FMAC(8); SMX_SK_FMAC(9); SMX_SK_FMAC(10); SMX_SK_FMAC(11); SMX_SK_FMAC(12); SMX_SK_FMAC(13); SMX_SK_FMAC(14); SMX_SK_FMAC(15);
            }
        };
#pragma unroll
        for (int bi = 0; bi < 4; bi++) {
            const bool live = blk0 + bi < p.nb;                       // blocks past K: clamped loads, zero weight scale
            // The activation scale is used as it was loaded: the quantiser launch writes zeros into the scale slots past K, and a
            // select here would be a vector write of the register the hand-written DPP multiply-adds below read through DPP
            // (two wait states the compiler's hazard recogniser does not insert for inline assembly).
            const float dxv = __uint_as_float(dxs[bi]);
            if constexpr (Q6) {
                const float d6 = h2f_s(r.d6), d6m128 = -128.f * d6;
#pragma unroll
                for (int jj = 0; jj < 2; jj++) {   // sub-block jj: chunk 2 bi + jj; a lane holds bytes 8 half .. + 7 of it on both sides
                    const long bw = *(const long*)(buf + col * 128 + ((2 * bi + jj + col) & 7) * 16 + half * 8);
                    const long aw = *(const long*)(mine_a + ((bi * 2 + jj) * p.tslots + min(col, p.tslots - 1)) * 16 + half * 8);
                    const v16i d = __builtin_amdgcn_mfma_i32_32x32x16_i8(aw, bw, cmagic, 0, 0, 0);
                    // d * sc, exact in fp32 (11 x 8 significant bits): sc + 128 as an unsigned byte -> float, then one FMA
                    const unsigned scw = ((2 * bi + jj) < 4 ? r.dw.x : r.dw.y) ^ 0x80808080u;
                    const float dw = fmaf((float)((scw >> (8 * ((2 * bi + jj) & 3))) & 0xffu), d6, d6m128);
                    rescale(acc, d, dw, dxv);
                    if (DUMP) {
                        const int row = r0 + col;
#pragma unroll
                        for (int i = 0; i < NACC; i++) {
                            const int tok = (i >> 2) * 8 + half * 4 + (i & 3);
                            if (tok < p.m && row <= r_last) p.dump[((size_t)tok * p.N + row) * (2 * p.nb) + 2 * (blk0 + bi) + jj] = d[i] - kMagicI;
                        }
                    }
                }
            } else {
                const v4i bfrag = *(const v4i*)(buf + col * 128 + ((2 * bi + half + col) & 7) * 16);
                const v4i afrag = ALDS ? *(const v4i*)(mine_a + ((bi * 2 + half) * p.tslots + min(col, p.tslots - 1)) * 16)
                                       : (bi == 0 ? r.a0 : (bi == 1 ? r.a1 : (bi == 2 ? r.a2 : r.a3)));
                const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag, bfrag, cmagic, 0, 0, 0);
                const float dw = live ? h2f_s((uint16_t)dwh[bi]) : 0.f;
                rescale(acc, d, dw, dxv);
                if (DUMP) {
                    const int row = r0 + col;
#pragma unroll
                    for (int i = 0; i < NACC; i++) {
                        const int tok = (i >> 2) * 8 + half * 4 + (i & 3);
                        if (live && tok < p.m && row <= r_last) p.dump[((size_t)tok * p.N + row) * p.nb + blk0 + bi] = d[i] - kMagicI;
                    }
                }
                if constexpr (TT == 2) {   // the second token tile on the same weight fragment
                    const v4i cfrag = bi == 0 ? r.c0 : (bi == 1 ? r.c1 : (bi == 2 ? r.c2 : r.c3));
                    const v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(cfrag, bfrag, cmagic, 0, 0, 0);
                    const unsigned dxs1[4] = {r.dx1.x, r.dx1.y, r.dx1.z, r.dx1.w};
                    rescale(acc1, d1, dw, __uint_as_float(dxs1[bi]));
                    if (DUMP) {
                        const int row = r0 + col;
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const int tok = 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                            if (live && tok < p.m && row <= r_last) p.dump[((size_t)tok * p.N + row) * p.nb + blk0 + bi] = d1[i] - kMagicI;
                        }
                    }
                }
            }
        }
        // the landing area is requested into again right after: every lane's reads of it are done (their
        // results were used above), and no LDS-direct write may overtake them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // This wave's pieces: a run of consecutive ones (a wave's scale loads and its 128-byte weight lines then
    // follow each other in memory), split evenly: the first `rem` waves take one piece more.
    {
        const int np = piece_end - piece0, base = np / kWaves, rem = np - base * kWaves;
        const int pc0 = piece0 + wave * base + min(wave, rem);
        const int my_end = pc0 + base + (wave < rem ? 1 : 0);
        for (int pc = pc0; pc < my_end; pc++) consume(request(pc), pc);
    }

    // the waves' partial tiles, added in wave order (one token tile after the other through the same LDS)
    float* red = (float*)smem;   // [wave][16][64]
#pragma unroll
    for (int tile = 0; tile < TT; tile++) {
        __syncthreads();
        const float* av = (TT == 2 && tile == 1) ? acc1 : acc;
#pragma unroll
        for (int i = 0; i < NACC; i++) red[(wave * 16 + i) * 64 + lane] = av[i];
        __syncthreads();
#pragma unroll
        for (int i = wave; i < NACC; i += kWaves) {   // accumulator index; lane as above
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; w++) s += red[(w * 16 + i) * 64 + lane];
            const int tok = tile * 32 + (i >> 2) * 8 + half * 4 + (i & 3), row = r0 + col;
            if (tok < p.m && row <= r_last) {
                float* o = p.y + (size_t)tok * p.N + row;
                if (p.ksplit == 1) *o = s;
                else atomicAdd(o, s);   // two addends onto a zeroed output: the sum does not depend on their order
            }
        }
    }
}
#undef SMX_SK_FMAC

// The activation quantiser of this path (arithmetic of actquant_kernel: d = amax / 127, q = rint(x / d),
// crates/strix-backend-rocm/src/kernels.rs:75-96, 1000-1013) writing the quants in MFMA fragment order:
// for block b, k-half h, token slot t the 16 bytes xq[t][32 b + 16 h ..] form chunk (b * 2 + h) * tslots + t,
// so a wave's operand load for a block is one contiguous piece, and so is every wave's store here: one
// thread per chunk (16 values), its block partner tslots lanes away.  Slots past m are zero.  The block
// scales go out as [piece = b / 4][token slot][b % 4].  The same launch zeroes the output when two K slices are going to add into it.
__global__ __launch_bounds__(256) void skinny_quant_kernel(const float* __restrict__ x, int m, int nb, int tslots,
                                                           uint4* __restrict__ xq, float* __restrict__ xd,
                                                           float4* __restrict__ zero, size_t zero_n4, size_t xq_tile16,
                                                           size_t xd_tile) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int tile = blockIdx.y;   // token tile: rows 32 * tile .. (its quants xq_tile16 chunks, its scales xd_tile floats further on)
    if (tile == 0 && gid < zero_n4) zero[gid] = make_float4(0.f, 0.f, 0.f, 0.f);
    xq += tile * xq_tile16;
    xd += tile * xd_tile;
    const size_t nchunks = (size_t)nb * 2 * tslots;
    const int t = (int)(gid % tslots), h = (int)((gid / tslots) & 1);
    const size_t b = gid / (2 * (size_t)tslots);
    const int row = tile * 32 + t;
    const bool live = gid < nchunks && row < m;
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = 0.f;
    if (live) {
        const float4* src = (const float4*)(x + ((size_t)row * nb + b) * 32 + h * 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float4 f = src[i];
            v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
        }
    }
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) a = fmaxf(a, fabsf(v[i]));
    a = fmaxf(a, __shfl_xor(a, tslots));   // the other half of the block (tslots = 8, 16 or 32: inside the wave)
    const float d = a / 127.f;
    const float inv = d > 0.f ? 1.f / d : 0.f;
    unsigned w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        unsigned pk = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) pk |= (unsigned)(max(-127, min(127, (int)rintf(v[4 * i + k] * inv))) & 0xff) << (8 * k);
        w[i] = pk;
    }
    if (gid < nchunks) xq[gid] = make_uint4(w[0], w[1], w[2], w[3]);
    if (live && h == 0) {
        xd[((b >> 2) * tslots + t) * 4 + (b & 3)] = d;
        if (b == (size_t)nb - 1)   // the scale slots of the last piece past K: zero, not what an earlier call left there
            for (size_t bb = b + 1; bb < (((size_t)nb + 3) & ~(size_t)3); bb++) xd[((bb >> 2) * tslots + t) * 4 + (bb & 3)] = 0.f;
    }
}

}  // namespace

// Measured on MI355X (Q8_0 2560 x 9728 / Q4_0 9728 x 2560 / Q8_0 9728 x 2560, quantiser launch included): 10.4 / 9.6 /
// 10.1 us at 5 rows, 12.0 / 10.7 / 11.6 us at 16 rows and 14.3 / 12.6 / 13.7 us at 32 rows; the dot4 GEMV takes 13.3 /
// 11.8 / 13.0 us at 5 rows and 13.9 / 12.3 / 13.0 us at 8, 10.9 / 9.0 / 10.7 us at 4 (where it stays), and the tiled
// GEMM with split-K 22 - 27 us.
bool skinny_serves(const Weight& w, size_t m) {
    // 17..32 rows of a very tall weight: the tiled GEMM is ahead (Q8_0 65536 x 3840 at 32 rows 61.6 against 70.7 us; at 16 rows
    // 58.3 / 61.8, at 8 rows the dot4 GEMV 68.2 / 57.6 us; 262144 x 2560: 174.5 / 169.6, 159.2 / 155.5, 171.6 / 139.0 us)
    if (m < SMX_SKINNY_MIN_M || m > SMX_SKINNY_MAX_M || w.K < 128) return false;
    if (w.type == kQ6_K) return m <= 16;   // its activation fragments travel through LDS: up to 16 token slots
    // 33..64 rows: two token tiles per weight piece
    return (w.type == kQ8_0 || w.type == kQ4_0) && (m <= 16 || w.N <= 32768);
}

static size_t skinny_slots(size_t m) { return m <= 8 ? 8 : (m <= 16 ? 16 : (m <= 32 ? 32 : 64)); }   // 64: two tiles of 32
size_t skinny_xq_bytes(size_t m, size_t K) { return (K / 32) * 2 * skinny_slots(m) * 16; }
size_t skinny_xd_bytes(size_t m, size_t K) { return ((K / 32 + 3) / 4) * skinny_slots(m) * 16; }

// y[m][N] for m <= 32 fp32 rows x[m][K]: quantiser launch (fragment-ordered quants into sc.xq, skinny_xq_bytes(m, K)
// bytes; scales into sc.xd) and the matmul launch.  dump (optional): out[m][N][K/32].
int launch_skinny(smx_ctx* c, const Weight& w, const float* x, size_t m, float* y, int32_t* dump, const ActScratch& sc) {
    if (!skinny_serves(w, m)) return fail(c, SMX_ERR_ARG, "small-batch matmul: weight type %d, %zu rows", (int)w.type, m);
    if (w.N > (size_t(1) << 24) || w.K > (size_t(1) << 20) || w.N * w.K >= (size_t(1) << 40))
        return fail(c, SMX_ERR_LIMIT, "small-batch matmul: shape N=%zu K=%zu exceeds the kernel's index range", w.N, w.K);
    SkinnyArgs p = {};
    p.wscales = w.scales;
    p.wquants = w.quants;
    p.wqh = w.qh;
    p.wsc = w.sc;
    p.xq = sc.xq;
    p.xd = sc.xd;
    p.y = y;
    p.dump = dump;
    p.m = (int)m;
    p.N = (int)w.N;
    p.nb = (int)(w.K / 32);   // 32-blocks per row in every format
    p.tslots = m <= 8 ? 8 : (m <= 16 ? 16 : 32);
    const int npieces = (p.nb + 3) / 4;
    const int ntiles = m > 32 ? 2 : 1;   // token tiles
    p.xq_tile = (size_t)p.nb * 2 * 32 * 16;
    p.xd_tile = (size_t)npieces * 32 * 4;
    // Rows per workgroup and K slices: one workgroup per CU, so the launch takes ceil(workgroups / CUs) rounds.  Two K
    // slices when a single round of 32-row groups would leave CUs without work (and every wave still gets a piece);
    // then as few rows per group as keep the number of rounds (a last round of a few 32-row workgroups costs
    // as much as a full one, and 19-row groups in two full rounds are 40 % less work per CU than 32-row groups in 1.2).
    int nrg = (int)((w.N + 31) / 32);
    int ksplit = c->tune_gemm_splitk > 0 ? std::min(c->tune_gemm_splitk, 2) : ((nrg <= c->num_cu && npieces >= 16) ? 2 : 1);
    if (dump || ((uintptr_t)y & 15) != 0 || (m * w.N) % 4 != 0) ksplit = 1;
    {
        const int rounds = (nrg * ksplit + c->num_cu - 1) / c->num_cu;
        const int groups = rounds * c->num_cu / ksplit;            // row groups that fit these rounds
        const int R = std::max(8, std::min(32, (int)((w.N + groups - 1) / groups)));   // (below 8 rows a group is all padding)
        p.rows_per_group = R;
        nrg = (int)((w.N + p.rows_per_group - 1) / p.rows_per_group);
    }
    p.ksplit = ksplit;
    p.pieces_per_slice = (npieces + ksplit - 1) / ksplit;
    {
        const size_t threads = (size_t)p.nb * 2 * p.tslots, zero_n4 = ksplit > 1 ? m * w.N / 4 : 0;
        const size_t grid = (std::max(threads, zero_n4) + 255) / 256;
        ProfScope ps(c, "skinny_quant");
        hipLaunchKernelGGL(skinny_quant_kernel, dim3((unsigned)grid, (unsigned)ntiles), dim3(256), 0, c->stream, x, (int)m, p.nb, p.tslots,
                           (uint4*)sc.xq, sc.xd, (float4*)y, zero_n4, p.xq_tile / 16, p.xd_tile);
        SMX_HIP(c, hipGetLastError());
    }
    const int fmt = w.type == kQ4_0 ? FMT_Q4 : (w.type == kQ6_K ? FMT_Q6 : FMT_Q8);
    const int nwg = nrg * ksplit;
    const int nw = (nwg <= c->num_cu && ntiles == 1) ? 16 : 8;   // waves per workgroup (see the kernel; two token tiles: 32 more accumulators per lane)
    const bool alds = p.tslots <= 16;
    const size_t lds = (size_t)nw * wave_lds(fmt, alds);   // the reduction reuses the first nw * 4 KB
    const dim3 grid((unsigned)nwg);
    ProfScope ps(c, fmt == FMT_Q4 ? "skinny_q4_0" : (fmt == FMT_Q6 ? "skinny_q6_k" : "skinny_q8_0"));
    auto go = [&](auto kern) -> int {
        int rc = set_dyn_lds(c, kern, lds);
        if (rc != SMX_OK) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(64 * nw), lds, c->stream, p);
        SMX_HIP(c, hipGetLastError());
        return SMX_OK;
    };
#define SMX_SK_GO(F_, NW_, AL_, NA_) (dump ? go(skinny_kernel<F_, true, NW_, AL_, NA_>) : go(skinny_kernel<F_, false, NW_, AL_, NA_>))
    if (fmt == FMT_Q6) {
        if (nw == 16) return p.tslots == 8 ? SMX_SK_GO(FMT_Q6, 16, true, 4) : SMX_SK_GO(FMT_Q6, 16, true, 8);
        return p.tslots == 8 ? SMX_SK_GO(FMT_Q6, 8, true, 4) : SMX_SK_GO(FMT_Q6, 8, true, 8);
    }
    // live accumulators per lane: 4 with up to 8 token slots, 8 with 16, all 16 with 32
#define SMX_SK_ROWS(F_, NW_)                                                                      \
    (p.tslots == 8 ? SMX_SK_GO(F_, NW_, true, 4) : (p.tslots == 16 ? SMX_SK_GO(F_, NW_, true, 8) : SMX_SK_GO(F_, NW_, false, 16)))
    if (ntiles == 2) {
        if (fmt == FMT_Q4) return dump ? go(skinny_kernel<FMT_Q4, true, 8, false, 16, 2>) : go(skinny_kernel<FMT_Q4, false, 8, false, 16, 2>);
        return dump ? go(skinny_kernel<FMT_Q8, true, 8, false, 16, 2>) : go(skinny_kernel<FMT_Q8, false, 8, false, 16, 2>);
    }
    if (nw == 16) return fmt == FMT_Q4 ? SMX_SK_ROWS(FMT_Q4, 16) : SMX_SK_ROWS(FMT_Q8, 16);
    return fmt == FMT_Q4 ? SMX_SK_ROWS(FMT_Q4, 8) : SMX_SK_ROWS(FMT_Q8, 8);
#undef SMX_SK_ROWS
#undef SMX_SK_GO
}

}  // namespace smx
