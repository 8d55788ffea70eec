/*
 * strix_mi355.h — C ABI of the MI355X (gfx950) quantized-matmul backend.
 *
 * This is the boundary a Strix.rs `WeightAccel` implementation binds to
 * (trait: crates/strix-core/src/accel.rs:147).  Each entry point names the
 * trait method / reference function it stands in for.  Plain pointers and
 * sizes only.
 *
 * Return convention (all int-returning calls):
 *     1   done
 *     0   declined exactly where the reference declines with `false`/`None`
 *         because the key/layer is not resident (accel.rs:142-146)
 *    <0   error (SMX_ERR_*); text via smx_last_error().  There is no CPU
 *         fallback inside the library.
 *
 * One context = one device + one HIP stream.  Calls on one context must be
 * serialised by the caller (the reference is driven the same way,
 * crates/strix-backend-rocm/src/decode.rs:559-562); distinct contexts are
 * independent.  Host-pointer entry points copy in, run, copy out and
 * synchronise; `_dev` entry points take device pointers, enqueue on the
 * context's stream and return without synchronising.
 */
#ifndef STRIX_MI355_H
#define STRIX_MI355_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct smx_ctx smx_ctx;

enum {
    SMX_OK = 1,
    SMX_NOT_RESIDENT = 0,
    SMX_ERR_ARG = -1,    /* null pointer, bad size, shape mismatch */
    SMX_ERR_HIP = -2,    /* a HIP runtime call failed */
    SMX_ERR_LIMIT = -3,  /* a documented limit exceeded */
    SMX_ERR_NOMEM = -4   /* device or host allocation failed */
};

/* ---- context: replaces HipGpu::new + kernel compilation,
 *      crates/strix-backend-rocm/src/hip.rs:135-160, decode.rs:563-830 ---- */
int smx_create(int device, smx_ctx** out);
void smx_destroy(smx_ctx* ctx); /* frees every device buffer the context owns */
/* Last error text of this context (of the calling thread's last failed
 * smx_create when ctx is NULL).  Valid until the next call on the context. */
const char* smx_last_error(const smx_ctx* ctx);
const char* smx_name(const smx_ctx* ctx);          /* WeightAccel::name, accel.rs:405 */
size_t smx_resident_count(const smx_ctx* ctx);     /* WeightAccel::resident_count, accel.rs:402 */
size_t smx_resident_bytes(const smx_ctx* ctx);     /* device bytes held by resident weights */

/* ---- weight upload: raw GGUF block bytes, [out_dim rows][in_dim/QK blocks].
 *      The bytes are copied; the caller may drop them afterwards.
 *      Re-uploading a key replaces the previous weight. ---- */
/* WeightAccel::upload_q4_0, accel.rs:150; decode.rs:2491-2521 */
int smx_upload_q4_0(smx_ctx* ctx, const char* key, const void* bytes, size_t nbytes,
                    size_t in_dim, size_t out_dim);
/* WeightAccel::upload_q8_0, accel.rs:163; decode.rs:2683-2714 */
int smx_upload_q8_0(smx_ctx* ctx, const char* key, const void* bytes, size_t nbytes,
                    size_t in_dim, size_t out_dim);
/* WeightAccel::upload_q6_k, accel.rs:159; decode.rs:2629-2681 */
int smx_upload_q6_k(smx_ctx* ctx, const char* key, const void* bytes, size_t nbytes,
                    size_t in_dim, size_t out_dim);
/* WeightAccel::upload_moe_q8, accel.rs:170-181; decode.rs:2717-2791.
 * gate/up: ne experts x [eff rows][hidden/32 blocks]; down: ne x [hidden rows][eff/32]. */
int smx_upload_moe_q8(smx_ctx* ctx, size_t layer, const void* gate, size_t gate_nbytes,
                      const void* up, size_t up_nbytes, const void* down, size_t down_nbytes,
                      size_t hidden, size_t eff, size_t ne);
/* WeightAccel::upload_moe_q6, accel.rs:185-196; decode.rs:2793-2831: the same tensors as Q6_K
 * superblocks (hidden and eff multiples of 256).  Served by smx_moe_ffn (one token) and by
 * smx_moe_layer[_dev] (grouped prefill; stands in for q6_gemm_moe, kernels.rs:1688-1735, and
 * moe_layer_ffn, decode.rs:3552-3629). */
int smx_upload_moe_q6(smx_ctx* ctx, size_t layer, const void* gate, size_t gate_nbytes,
                      const void* up, size_t up_nbytes, const void* down, size_t down_nbytes,
                      size_t hidden, size_t eff, size_t ne);
/* Drop one resident weight (the reference never frees, decode.rs:458-460).  While a captured graph of
 * the context is alive the device memory is kept until smx_destroy (a replay may still read it); the
 * same holds for the old allocation when a key or an expert layer is uploaded again. */
int smx_evict(smx_ctx* ctx, const char* key);
/* Shape of a resident weight as given at upload (what the trait's gemv sizes its result with,
 * decode.rs:3830-3832): 1 and the dimensions, 0 when the key is not resident.  Either out pointer may be NULL. */
int smx_weight_dims(const smx_ctx* ctx, const char* key, size_t* in_dim, size_t* out_dim);

/* ---- decode GEMV ---- */
/* WeightAccel::gemv, accel.rs:391; decode.rs:3827-3898.  y = W.x with x
 * quantised per 32-block on the device (kernels.rs:75-96) and integer block
 * dots (kernels.rs:259-287, 894-912).  in_len must equal in_dim, out_cap >= out_dim. */
int smx_gemv(smx_ctx* ctx, const char* key, const float* x, size_t in_len, float* y,
             size_t out_cap);
/* The same product with fp32 activations: no quantiser, every weight widened to fp32 and multiplied with x,
 * the arithmetic of the kernels the reference launches for WeightAccel::gemv (kernels.rs:41-69 q4_gemv,
 * :646-668 q8_0_gemv, :607-640 q6_gemv) and of strix-backend-cpu, whose result it matches to fp32 rounding
 * (the reference's own device test asks for rel < 1e-3, strix-backend-rocm/src/lib.rs:231).  smx_gemv above
 * differs from the CPU result by the activation rounding of the decode path (about 1e-2 relative).
 * in_dim <= SMX_GEMV_F32_MAX_IN_DIM (the fp32 row is staged in LDS). */
#define SMX_GEMV_F32_MAX_IN_DIM 32768
int smx_gemv_f32(smx_ctx* ctx, const char* key, const float* x, size_t in_len, float* y, size_t out_cap);
int smx_gemv_f32_dev(smx_ctx* ctx, const char* key, const float* x_dev, float* y_dev);
/* Small batches, m <= SMX_GEMV_ROWS_MAX rows against one weight read once (kernels.rs:1605-1632 q8_gemm_rows,
 * :830-857 q8_gemm_rows32, :1016-1045 q8i_gemm_rows32; the n-gram verify step and short prefill chunks):
 * xs[m][in_dim] -> y[m][out_dim].  Up to 4 rows run in the dot4 GEMV; 5..32 rows of a Q8_0 / Q4_0 weight (17..32 rows:
 * weights of up to 32768 rows) and 5..16 rows of a Q6_K weight in the small-batch kernel on the matrix cores; every other
 * case in the tiled GEMM.  The integer block dots do not depend on which, the fp32 sums agree within 1e-5. */
#define SMX_GEMV_MAX_M 8
#define SMX_GEMV_ROWS_MAX 32
int smx_gemv_rows(smx_ctx* ctx, const char* key, const float* xs, size_t m, size_t in_dim,
                  float* y, size_t y_cap);
/* WeightAccel::gemv_batch, accel.rs:397; decode.rs:3227-3255.  n (key, x)
 * pairs, one device job, one sync.  status[i] receives the per-item code. */
int smx_gemv_batch(smx_ctx* ctx, size_t n, const char* const* keys, const float* const* xs,
                   const size_t* in_lens, float* const* ys, const size_t* out_caps, int* status);
/* The same batch in the arithmetic of smx_gemv_f32 (what the reference's gemv_batch launches,
 * decode.rs:3227-3255 over the fp32-activation kernels): one launch per item, back to back, one sync. */
int smx_gemv_f32_batch(smx_ctx* ctx, size_t n, const char* const* keys, const float* const* xs,
                       const size_t* in_lens, float* const* ys, const size_t* out_caps, int* status);

/* ---- prefill GEMM ---- */
/* WeightAccel::prefill_q8_gemm, accel.rs:213; decode.rs:3257-3297 (and the
 * Q4_0 GEMMs kernels.rs:481-601, the Q6_K GEMM :1688-1735).  xs[m][in_dim] -> y[m][out_dim], any
 * resident Q4_0/Q8_0/Q6_K weight, any m; split-K is chosen internally. */
int smx_gemm(smx_ctx* ctx, const char* key, const float* xs, size_t m, size_t in_dim, float* y,
             size_t y_cap);
/* WeightAccel::lm_head_argmax_rows, accel.rs:217; decode.rs:3631-3690.
 * out[t] = argmax_r (W.xs[t])[r], lowest index on ties. */
int smx_lm_head_argmax_rows(smx_ctx* ctx, const char* key, const float* xs, size_t m,
                            size_t in_dim, uint32_t* out);

/* ---- MoE ---- */
/* WeightAccel::moe_ffn, accel.rs:201-210; decode.rs:2833-2870, 1923-2128.
 * y[hidden] = sum_k wexp[k] * down_k( silu(gate_k x) * (up_k x) ), k routed
 * experts accumulated in routed order.  sgate != 0 adds sgate * shared_expert(x), the dense FFN
 * blk.<layer>.ffn_{gate,up,down}_shexp.weight (decode.rs:1820-1855 queue_shexp); as in the
 * reference the call declines (0) when those three weights are not resident. */
int smx_moe_ffn(smx_ctx* ctx, size_t layer, const int32_t* ids, const float* wexp, size_t k,
                const float* x, size_t x_len, float sgate, float* y, size_t y_cap);
/* WeightAccel::moe_layer_q8_dev, accel.rs:311-321; decode.rs:1608-1739.
 * xs[m][hidden]; plan[nplan][3] = (expert, slot_off, count); slot_tok[slots],
 * wslot[slots]; y[m][hidden] = sum over the token's slots (ascending slot
 * index) of wslot * expert_ffn(xs[token]). */
/* WeightAccel::moe_layer_ffn, accel.rs:238-246; decode.rs:3552-3629 (and the per-expert forms
 * moe_expert_ffn / moe_expert_queue + flush, accel.rs:220-262, which are this call with one group).
 * xs[rows][hidden] holds the rows of every expert group back to back (gathered by the caller),
 * plan[nplan][2] = (expert, rows of the group); dy[rows][hidden] = the unweighted expert outputs,
 * for the caller's weighted scatter.  Q8_0 and Q6_K expert layers. */
int smx_moe_layer_ffn(smx_ctx* ctx, size_t layer, const int32_t* plan, size_t nplan, const float* xs,
                      size_t rows, float* dy, size_t dy_cap);
int smx_moe_expert_ffn(smx_ctx* ctx, size_t layer, size_t expert, const float* xs, size_t m, float* y,
                       size_t y_cap);
int smx_moe_layer(smx_ctx* ctx, size_t layer, const float* xs, size_t m, const size_t* plan,
                  size_t nplan, const int32_t* slot_tok, const float* wslot, size_t slots,
                  float* y, size_t y_cap);

/* ---- device-resident variants (async on the context's stream) ---- */
int smx_dev_alloc(smx_ctx* ctx, size_t nbytes, void** dptr);
int smx_dev_free(smx_ctx* ctx, void* dptr);
int smx_h2d(smx_ctx* ctx, void* dst_dev, const void* src_host, size_t nbytes);
int smx_d2h(smx_ctx* ctx, void* dst_host, const void* src_dev, size_t nbytes); /* syncs */
int smx_sync(smx_ctx* ctx);
/* Plain device-to-device copy kernel (nbytes a multiple of 16, 16-byte aligned pointers), async.
 * Also the known-size reference kernel against which hardware traffic counters are scaled. */
int smx_dev_copy(smx_ctx* ctx, void* dst_dev, const void* src_dev, size_t nbytes);
int smx_gemv_dev(smx_ctx* ctx, const char* key, const float* xs_dev, size_t m, float* y_dev);
/* smx_gemv_dev for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same kernels and results
 * as smx_gemv_dev; the rows quantised for m >= 2 live in a static device array of the library (160 KB per
 * GPU, held until the process ends) instead of the context's growable scratch, so the call never
 * allocates or frees device or host memory.  Limits: m <= SMX_NOALLOC_MAX_ROWS, and for m >= 2 in_dim <= SMX_NOALLOC_MAX_IN_DIM
 * (SMX_ERR_LIMIT beyond; a single row is quantised inside the GEMV and does not use the array).  All contexts of one GPU share the array: calls that overlap on one GPU race. */
#define SMX_NOALLOC_MAX_IN_DIM 16384
#define SMX_NOALLOC_MAX_ROWS 8
int smx_gemv_noalloc_dev(smx_ctx* ctx, const char* key, const float* xs_dev, size_t m, float* y_dev);
/* Up to 8 single-row GEMVs of one format and in_dim in ONE launch (gate+up, q/k/v, a batch of
 * weights against their activations); 0 if any key is not resident. */
int smx_gemv_batch_dev(smx_ctx* ctx, size_t n, const char* const* keys, const float* const* xs_dev,
                       float* const* ys_dev);
int smx_gemm_dev(smx_ctx* ctx, const char* key, const float* xs_dev, size_t m, float* y_dev);

/* ---- the step BEFORE a decode GEMV fused into it: the reference's rmsnorm_xquant / silu_xquant /
 *      geglu_xquant (crates/strix-backend-rocm/src/kernels.rs:101-147, 191-226, 151-187) write the
 *      quantised activation for the GEMVs that follow; here the producer runs inside the GEMV's own
 *      activation staging, so norm + quantiser + up to 16 GEMVs of one format and in_dim (q/k/v,
 *      gate+up, down) are ONE launch and no fp32 or int8 activation goes through HBM.
 *      RMSNORM : x = (a * 1/sqrt(mean(a^2) + eps)) * b   (b = norm weight, may be NULL; ops.rs:15-27.
 *                The mean is formed in double and rounded once, where the reference uses rsqrtf.)
 *      SILU_MUL: x = silu(a) * b        (ops.rs:74-87)     GEGLU: x = gelu_tanh(a) * b  (ops.rs:110-121)
 *      a, b: fp32 [in_dim].  1 done, 0 if any key is not resident, <0 error. ---- */
#define SMX_ACT_NONE 0
#define SMX_ACT_RMSNORM 1
#define SMX_ACT_SILU_MUL 2
#define SMX_ACT_GEGLU 3
int smx_gemv_fused_dev(smx_ctx* ctx, size_t n, const char* const* keys, int act, const float* a_dev,
                       const float* b_dev, float eps, float* const* ys_dev);
int smx_gemv_fused(smx_ctx* ctx, const char* key, int act, const float* a, const float* b, size_t in_len,
                   float eps, float* y, size_t out_cap);

/* The gate and up projections of a dense FFN decode step in ONE launch with the SwiGLU / GeGLU product in the kernel's
 * tail: h[i] = act(gate_i . x') * (up_i . x') with x' = x or (norm = 1) rmsnorm(x, eps) * norm_w (norm_w may be NULL);
 * act = SMX_ACT_SILU_MUL or SMX_ACT_GEGLU.  The reference runs q4_gemv_dp2 (kernels.rs:324-339) and then silu_xquant /
 * geglu_xquant (:151-226) over the two outputs; here a workgroup walks the same rows of both weights and holds both dots
 * of a row, so h leaves the first launch and the down projection (smx_gemv_dev on h) quantises it in its own staging:
 * two launches per FFN instead of three.  Each dot is formed exactly as smx_gemv_fused_dev forms it (same bits).
 * gate and up: same format and shape.  SMX_NOT_RESIDENT when either key is unknown. */
int smx_ffn_gate_up_dev(smx_ctx* ctx, const char* gate_key, const char* up_key, int act, const float* x_dev, int norm,
                        const float* norm_w_dev, float eps, float* h_dev);
/* The prefill form (kernels.rs:1174-1187 silu_quant_rows, :1000-1013 xquant8_rows behind a norm): m rows
 * a_dev[m][in_dim] go through the producer inside the quantiser launch that feeds the int8 GEMM, so the
 * normalised / gated fp32 rows are never written.  b_dev: the norm weight [in_dim] (or NULL) for RMSNORM,
 * the second operand [m][in_dim] for SILU_MUL / GEGLU.  y_dev[m][out_dim]. */
int smx_gemm_fused_dev(smx_ctx* ctx, const char* key, int act, const float* a_dev, const float* b_dev, size_t m,
                       float eps, float* y_dev);

/* y_dev += sgate * shared_expert(x_dev) for layer `layer` (the second half of moe_ffn with a shared
 * expert, decode.rs:1820-1855), to follow smx_moe_ffn_dev on device-resident activations. */
int smx_moe_shexp_dev(smx_ctx* ctx, size_t layer, float sgate, const float* x_dev, float* y_dev);
int smx_moe_ffn_dev(smx_ctx* ctx, size_t layer, const int32_t* ids, const float* wexp, size_t k,
                    const float* x_dev, float* y_dev);
/* The router on the device (kernels.rs:1846-1872 topk_router; mellum.rs:1178-1192): softmax over the ne
 * logits, the k largest probabilities in descending order (equal ones: lowest index first), weights
 * renormalised over the chosen k.  ids_dev[k] i32, w_dev[k] f32; ne <= 1024, k <= 64.  smx_moe_route is the
 * same with host buffers (one sync). */
int smx_moe_route_dev(smx_ctx* ctx, const float* logits_dev, size_t ne, size_t k, int32_t* ids_dev, float* w_dev);
int smx_moe_route(smx_ctx* ctx, const float* logits, size_t ne, size_t k, int32_t* ids, float* w);
/* Router logits and routing in one call: logits = W_router . x for the resident router weight `key` (out_dim = number of
 * experts; the reference launches f32_gemv on its router weight and then topk_router, decode.rs:1136-1166), then the routing
 * of smx_moe_route_dev on them (two launches; capturable).  The logits have the bits of smx_gemv_dev, the routing those of
 * smx_moe_route_dev on them.  logits_dev (optional, [out_dim]) also receives the logits. */
int smx_moe_router_dev(smx_ctx* ctx, const char* key, const float* x_dev, size_t k, int32_t* ids_dev, float* w_dev,
                       float* logits_dev);
/* smx_moe_ffn_dev with the routing read from device memory when the kernels run (what smx_moe_route_dev
 * wrote): router + expert FFN of a decode token can be captured once and replayed with every token's own
 * routing (decode.rs:1923-2128 reads the router's device output the same way).  Ids outside 0 .. ne - 1
 * are clamped. */
int smx_moe_ffn_routed_dev(smx_ctx* ctx, size_t layer, const int32_t* ids_dev, const float* w_dev, size_t k,
                           const float* x_dev, float* y_dev);
/* The routed expert FFN of a decode token straight from the router logits (topk_router followed by moe_launches,
 * decode.rs:1154-1180, as ONE call): y_dev = sum_k w_k * expert_{id_k}(x_dev) with (ids, w) = the routing of
 * smx_moe_route_dev on logits_dev[ne], ne = the layer's expert count.  For up to 64 experts and k <= 8 the routing runs in the
 * prologue of the experts' gate/up launch (every workgroup repeats the 64-logit top-k; no routing launch: two launches per
 * token instead of three); other shapes run the routing launch first.  ids_dev[k] / w_dev[k] receive the routing (the down
 * launch reads them).  Same bits as smx_moe_route_dev + smx_moe_ffn_routed_dev.  Capturable. */
int smx_moe_ffn_logits_dev(smx_ctx* ctx, size_t layer, const float* logits_dev, size_t k, const float* x_dev, float* y_dev,
                           int32_t* ids_dev, float* w_dev);
/* smx_moe_layer with the activations and the result on the device (y_dev: m x hidden floats); the
 * routing tables still come from the host at every call, so it cannot be captured in a graph. */
int smx_moe_layer_dev(smx_ctx* ctx, size_t layer, const float* xs_dev, size_t m, const size_t* plan,
                      size_t nplan, const int32_t* slot_tok, const float* wslot, size_t slots,
                      float* y_dev);

/* ---- HIP graph capture of a sequence of `_dev` calls: the role of the reference's captured decode
 *      token (decode.rs:3053-3203), so a launch-bound chain of small GEMVs replays without per-launch
 *      host cost.  Between begin and end only `_dev` entry points may be called, with shapes already
 *      seen once outside capture (no scratch growth while capturing); per-kernel timing is off.
 *      A graph stays valid when later calls grow the context's scratch (the buffers it captured are
 *      kept until the context closes); it does NOT survive smx_evict of a weight it uses, nor the
 *      caller freeing the activation buffers it was captured with. ---- */
typedef struct smx_graph smx_graph;
int smx_graph_begin(smx_ctx* ctx);
int smx_graph_end(smx_ctx* ctx, smx_graph** out);
int smx_graph_launch(smx_ctx* ctx, smx_graph* g);   /* enqueue one replay on the context's stream */
void smx_graph_destroy(smx_ctx* ctx, smx_graph* g);

/* Measurement hook, not part of the operator surface (no counterpart in the reference; a binding has no reason to
 * call it): launch-geometry overrides for sweeps; value 0 restores the built-in choice.  They shape
 * a kernel's launch, never which kernel a shape is served by.
 * Knobs: "gemm_splitk" (K slices of the GEMM), "gemm_tile_m" (tokens per GEMM tile: 64 or 128), "gemm_walk" (token-tile
 * groups of the GEMM's tile walk), "gemm_narrow" (1: every weight strip of the GEMM 128 rows; 1 + n: the first n strips 96 rows); for shapes served by the row-per-wavefront GEMV (rows that
 * are not a whole number of 16-byte unit groups, or longer than 16384 elements): "gemv_rpw" (rows per
 * wavefront: 1, 2, 4), "gemv_ks" (wavefronts sharing a row: 1, 2, 4), "gemv_lpr" (lanes per row: 16, 32,
 * 64), "gemv_wpc" (workgroups per CU); "host_io" (host-pointer GEMV calls: 0 = the kernels read and write the context's
 * pinned staging buffers themselves where that is the rule, 1 = a copy command each way, 2 = a copy command in, the result
 * written by the kernel).  Results do not depend on them beyond fp32 summation order. */
int smx_tune(smx_ctx* ctx, const char* knob, int value);

/* ---- GGUF file -> resident weights: the loader side of the path, crates/strix-models/src/gguf.rs:104-238
 *      (memory-mapped GGUF v2/v3: header, metadata, tensor index) and the upload loops of the models'
 *      attach_accel (crates/strix-backend-cpu/src/mellum.rs:460-535, gemma.rs:415-470).  Host code;
 *      smx_gguf_open / the accessors need no GPU.  Errors of smx_gguf_open go to err (may be NULL). ---- */
typedef struct smx_gguf smx_gguf;
int smx_gguf_open(const char* path, smx_gguf** out, char* err, size_t err_cap);
void smx_gguf_close(smx_gguf* g);
size_t smx_gguf_tensor_count(const smx_gguf* g);
/* Tensor `index` in file order: name, ggml type number, dims in GGUF order (fastest first; at most
 * dims_cap written), pointer to its bytes inside the mapping and their count (gguf.rs:217-238).
 * Any out pointer may be NULL. */
int smx_gguf_tensor(const smx_gguf* g, size_t index, const char** name, int* ggml_type, size_t* n_dims,
                    size_t* dims, size_t dims_cap, const void** data, size_t* nbytes);
int smx_gguf_find(const smx_gguf* g, const char* name, size_t* index);          /* 0: no such tensor */
/* Metadata with the reference's widening rules (MetaValue::as_u64 / as_f32 / as_str, gguf.rs:43-72):
 * 1 found, 0 no such key, <0 the value has another kind. */
int smx_gguf_meta_u64(const smx_gguf* g, const char* key, uint64_t* value);
int smx_gguf_meta_f32(const smx_gguf* g, const char* key, float* value);
int smx_gguf_meta_str(const smx_gguf* g, const char* key, const char** value);
/* attach_accel: every "*.weight" matrix (>= 2 dims; in_dim = dims[0], out_dim = the product of the
 * rest) stored as Q4_0, Q8_0 or Q6_K is uploaded under its GGUF name; every layer whose
 * blk.<il>.ffn_{gate,up,down}_exps.weight triple is Q8_0 or Q6_K becomes expert layer <il>.  Tensors in
 * other encodings are left to the caller (see the host quantisers below).  Counts may be NULL. */
int smx_gguf_attach(smx_ctx* ctx, const smx_gguf* g, size_t* n_weights, size_t* n_expert_layers);
/* One matrix re-encoded on the host as Q8_0 (target_type 8) or Q4_0 (2) and uploaded under `key`
 * (NULL: its own name): the reference's repacks of tensors in an encoding the device path does not
 * serve (gemma3n.rs:455-470, a Q4_K token_embd becomes the Q8_0 lm_head) or that should be lighter
 * (qwen35.rs:741-760, Q8_0 -> Q4_0).  0: no such tensor. */
int smx_gguf_upload_as(smx_ctx* ctx, const smx_gguf* g, const char* tensor, const char* key, int target_type);
/* Host quantisers the reference uses to bring a tensor into a served format before upload
 * (crates/strix-models/src/ggml_quant.rs:193-207 quantize_q8_0, :212-237 quantize_q4_0) and the
 * dequantisers that feed them (:128-430; ggml types 0 F32, 1 F16, 2 Q4_0, 3 Q4_1, 6 Q5_0, 7 Q5_1,
 * 8 Q8_0, 12 Q4_K, 13 Q5_K, 14 Q6_K; others return SMX_ERR_LIMIT, as the reference's dequantize errs).
 * n elements, a multiple of the block size; out: n/32*34, n/32*18 bytes, n floats. */
int smx_host_quantize_q8_0(const float* x, size_t n, void* out);
int smx_host_quantize_q4_0(const float* x, size_t n, void* out);
int smx_host_dequantize(int ggml_type, const void* bytes, size_t n, float* out);

/* ---- per-kernel timing: the role of STRIX_PROF, decode.rs:25-69, 2190-2203,
 *      done with HIP events on the context's stream instead of host syncs ---- */
int smx_prof_enable(smx_ctx* ctx, int on);   /* on: bracket each matmul kernel with an event pair */
int smx_prof_reset(smx_ctx* ctx);
/* Total milliseconds and launch count recorded for kernels whose name starts
 * with `prefix` (syncs the stream).  Names: smx_prof_names(). */
int smx_prof_read(smx_ctx* ctx, const char* prefix, double* total_ms, size_t* launches);
const char* smx_prof_names(smx_ctx* ctx);    /* comma-separated kernel names seen so far */
/* Stream-level stopwatch: events around whatever is enqueued in between. */
int smx_timer_begin(smx_ctx* ctx);
int smx_timer_end(smx_ctx* ctx, float* ms);  /* syncs */

/* ---- parity instrumentation: the kernel the same call would run without the dump (same launch
 *      geometry, same device code), with the integers it forms also written out ---- */
/* Device activation quantiser: xq[m][k] i8, xd[m][k/32] f32, xs16[m][k/16] i16. */
int smx_quantize(smx_ctx* ctx, const float* x, size_t m, size_t k, int8_t* xq, float* xd,
                 int16_t* xs16);
/* Per-block i32 dots formed by the GEMV kernel: out[out_dim][in_dim/32]
 * (Q6_K: [out_dim][in_dim/16]). */
int smx_gemv_block_dots(smx_ctx* ctx, const char* key, const float* x, size_t in_len,
                        int32_t* out, size_t out_cap);
/* Per-block i32 accumulators formed by the MFMA GEMM: out[m][out_dim][in_dim/32]. */
int smx_gemm_block_dots(smx_ctx* ctx, const char* key, const float* xs, size_t m, size_t in_dim,
                        int32_t* out, size_t out_cap);
/* smx_moe_ffn with its intermediate stages: gu[k][2][eff] (gate, up outputs),
 * aq[k][eff] / ad[k][eff/32] (quantised silu(g)*u).  Any of them may be NULL. */
int smx_moe_ffn_stages(smx_ctx* ctx, size_t layer, const int32_t* ids, const float* wexp, size_t k,
                       const float* x, size_t x_len, float* y, float* gu, int8_t* aq, float* ad);
/* smx_moe_layer (decode.rs:1608-1739) with the stages of its grouped path copied out per slot:
 * gu[slots][2][eff] (gate, up outputs of the slot's expert: after gather_xq8 + the two GEMMs),
 * aq[slots][eff] / ad[slots][eff/32] (silu_quant_rows), dy[slots][hidden] (the down GEMM, before
 * scatter_add_w).  Any of them may be NULL. */
int smx_moe_layer_stages(smx_ctx* ctx, size_t layer, const float* xs, size_t m, const size_t* plan,
                         size_t nplan, const int32_t* slot_tok, const float* wslot, size_t slots,
                         float* y, size_t y_cap, float* gu, int8_t* aq, float* ad, float* dy);

#ifdef __cplusplus
}
#endif
#endif
