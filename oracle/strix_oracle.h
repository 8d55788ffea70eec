/*
 * strix_oracle.h — CPU restatement of the Strix.rs quantized-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product library links, loads or
 * calls this code; only the tests, the smoke check and the CPU-baseline leg
 * of the benchmark do, and there only as the checker / the timed baseline.
 *
 * Two oracles live here:
 *
 *  f32 oracle  — what strix-backend-cpu computes: dequantise a weight row to
 *                f32, dot it with the f32 activation.
 *                  block decode   crates/strix-models/src/ggml_quant.rs:239-262, 401-430
 *                  sequential sum crates/strix-backend-cpu/src/gemma.rs:318-329
 *                  8-lane sum     crates/strix-backend-cpu/src/mellum.rs:278-293
 *                Pinned by: the literal-value block tests of
 *                ggml_quant.rs:443-469, 497-514, 562-565, and the reference's
 *                own seeded GEMV test data (crates/strix-backend-rocm/src/lib.rs:135-180).
 *
 *  Q8 oracle   — the integer path the reference runs only on the device:
 *                activations quantised per 32-block (kernels.rs:75-96), exact
 *                i32 block dots (kernels.rs:228-255, 894-912), fp32 combine
 *                acc += (dw*dx)*float(isum) in ascending block order
 *                (kernels.rs:517-522).
 *                PARITY UNPINNED BY THE REFERENCE: no reference test or CPU
 *                code computes these integer dots (its tightest check of the
 *                path is rel < 2e-2 against f32,
 *                crates/strix-backend-vulkan/src/qgemv.rs:2660-2666).  It is
 *                pinned instead by what the mathematics fixes: brute-force
 *                int64 dots over dequantised integers, the identity
 *                sum((q-8)x) = sum(qx) - 8 sum(x), quantiser invariants, and
 *                agreement with the f32 oracle to activation-rounding error.
 *                The Q6_K x Q8 arithmetic is new (the reference's Q6_K kernels
 *                take f32 activations, kernels.rs:607-640): parity unpinned,
 *                pinned by the same brute-force checks.
 *
 *  Requantisation sources — Q4_1, Q5_0, Q5_1, Q4_K, Q5_K decode
 *                (ggml_quant.rs:265-400), host-side only.  Q4_K and Q5_K are
 *                pinned by the literal blocks of ggml_quant.rs:472-494, 525-541;
 *                Q4_1, Q5_0, Q5_1 have no reference test: PARITY UNPINNED BY THE
 *                REFERENCE, pinned bit for bit against a vectorised numpy decoder
 *                written from the published block layouts.
 *
 *  Activation producers (rmsnorm, SwiGLU, GeGLU in front of a GEMV) and the
 *  MoE chain follow crates/strix-backend-cpu/src/ops.rs:15-27, 74-87, 110-121
 *  and mellum.rs:1623-1669.  Pinned by the reference's literal checks
 *  (ops.rs:204-232, 260-276, 287-294) and float64 formulas.  Two deliberate
 *  departures, both far inside the reference's own tolerances (1e-5 / 1e-3):
 *  exp/tanh are fixed sequences of fp32 operations instead of libm calls, and
 *  rmsnorm forms the mean of squares in double and rounds the scale once
 *  (the reference sums in fp32 on the CPU and uses rsqrtf on the device), so
 *  that the quantised int8 activations are reproducible bit for bit.
 */
#ifndef STRIX_ORACLE_H
#define STRIX_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_Q4_0 = 2, ORC_Q8_0 = 8, ORC_Q6_K = 14, /* GGML type ids, ggml_quant.rs:43-58 */
       ORC_Q4_1 = 3, ORC_Q5_0 = 6, ORC_Q5_1 = 7, ORC_Q4_K = 12, ORC_Q5_K = 13 }; /* dequantised only (requantisation sources) */

/* ---- half precision (exact conversions; `half` crate semantics) ---- */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f); /* round to nearest even */

/* ---- block geometry, ggml_quant.rs:83-124 ---- */
int orc_block_elems(int type);
int orc_block_bytes(int type);

/* ggml_quant.rs:139-183.  Returns 0, or -1 when n is not a block multiple or
 * nbytes is too small (the reference's two error cases). */
int orc_dequantize(int type, const uint8_t* bytes, size_t nbytes, float* out, size_t n);

/* ggml_quant.rs:193-207 and :212-237 (CPU-side GGUF quantisers). */
void orc_quantize_q8_0(const float* x, size_t n, uint8_t* out);
void orc_quantize_q4_0(const float* x, size_t n, uint8_t* out);

/* ---- f32 oracle ---- */
/* y[t*N + o] = dot(dequant(row o), x[t*K ..]).  order 0: strictly sequential
 * (gemma.rs:323-326); order 1: dot_f32 8-lane + fixed tree (mellum.rs:278-293).
 * Rows are split over `nthreads` OpenMP threads (rayon analogue; results do
 * not depend on it). */
int orc_matmul_f32(int type, const uint8_t* w, int K, int N, const float* x, int m,
                   float* y, int order, int nthreads);

/* ---- Q8 oracle ---- */
/* Device activation quantiser, kernels.rs:75-96 / :1000-1013:
 *   d = amax/127 (f32), inv = d>0 ? 1/d : 0, q = clamp(rint(x*inv), -127, 127).
 * xq[m][K], xd[m][K/32], xs16[m][K/16] (sum of q over each 16 elements; the
 * reference keeps one sum per 32, kernels.rs:93 — a 32-sum is two of these). */
void orc_actquant(const float* x, int m, int K, int8_t* xq, float* xd, int16_t* xs16);

/* Exact integer dots of one quantised activation row against every weight row.
 * Q4_0 / Q8_0: out[N][K/32] = sum over the block of (q_w [-8]) * q_x.
 * Q6_K:        out[N][K/16] = sum over the 16-element sub-block of (q-32) * q_x. */
int orc_block_dots(int type, const uint8_t* w, int K, int N, const int8_t* xq, int32_t* out);

/* y[t*N + o] for m quantised rows.  Q4_0/Q8_0: acc += (dw*dx[b]) * float(isum_b),
 * b ascending.  Q6_K: per 32-block j of the superblock,
 * t = sc[2j]*isum16[2j] + sc[2j+1]*isum16[2j+1] (exact in i32),
 * acc += (d*dx[j]) * float(t).  Row-parallel over nthreads. */
int orc_matmul_q8(int type, const uint8_t* w, int K, int N, const int8_t* xq, const float* xd,
                  int m, float* y, int nthreads);

/* ---- MoE (Q8_0 experts) ---- */
/* exp() used by silu on both the device and here: a fixed sequence of IEEE
 * fp32 operations, so both sides produce the same bits from the same input. */
float orc_expf(float x);
float orc_silu(float x); /* x / (1 + exp(-x)), ops.rs:73-76 */
float orc_tanhf(float z);
float orc_gelu_tanh(float x); /* ops.rs:110-113 */
enum { ORC_ACT_NONE = 0, ORC_ACT_RMSNORM = 1, ORC_ACT_SILU_MUL = 2, ORC_ACT_GEGLU = 3 };
/* activation producers in front of a GEMV (kernels.rs:101-226): rmsnorm(a)*b, silu(a)*b, gelu_tanh(a)*b */
int orc_act_produce(int act, const float* a, const float* b, int n, float eps, float* out);

/* One token through k routed experts, crates/strix-backend-cpu/src/mellum.rs:1623-1669
 * with the integer arithmetic of kernels.rs:942-996, 1875-1882:
 *   xq = quant(x); g,u = Q8 matmul; a = silu(g)*u; aq = quant(a); dy = Q8 matmul;
 *   y = sum_k wexp[k]*dy_k in routed order.
 * gate/up: [ne][eff rows][hidden/32 blocks] raw Q8_0; down: [ne][hidden rows][eff/32].
 * Optional stage outputs (may be NULL): gu[k][2][eff], aq[k][eff], ad[k][eff/32].
 * If aq_in/ad_in are non-NULL the down stage uses them instead of its own. */
int orc_moe_ffn_q8(const uint8_t* gate, const uint8_t* up, const uint8_t* down, int hidden, int eff,
                   int ne, const int32_t* ids, const float* wexp, int k, const float* x, float* y,
                   float* gu, int8_t* aq, float* ad, const int8_t* aq_in, const float* ad_in);
/* The same with the expert tensors in `type` = ORC_Q8_0 or ORC_Q6_K (decode.rs:2793-2852: Q6_K expert
 * layers; hidden and eff multiples of 256, 210-byte superblocks). */
int orc_moe_ffn(int type, const uint8_t* gate, const uint8_t* up, const uint8_t* down, int hidden, int eff,
                int ne, const int32_t* ids, const float* wexp, int k, const float* x, float* y,
                float* gu, int8_t* aq, float* ad, const int8_t* aq_in, const float* ad_in);

/* Top-k routing, mellum.rs:1178-1192: softmax over all experts, k largest
 * (ties -> lowest index, kernels.rs:1843-1845), renormalise. */
void orc_route_topk(const float* logits, int ne, int k, int32_t* ids, float* w);

/* ---- seeded generator shared by the reference's device tests ---- */
/* seed = seed*6364136223846793005 + 1; out = (u32)(seed >> 33)
 * (crates/strix-backend-rocm/src/lib.rs:141-144). */
void orc_lcg_fill(uint64_t* seed, uint32_t* out, size_t n);

#ifdef __cplusplus
}
#endif
#endif
