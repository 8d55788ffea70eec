// Internal declarations shared by the library's translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <new>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/strix_mi355.h"

namespace smx {

enum QType { kQ4_0 = 2, kQ8_0 = 8, kQ6_K = 14 };

// A resident weight: one device allocation, planes at 256-byte aligned offsets,
// at on-disk density (no f32 scale expansion).
//   Q4_0: scales f16[N*nb]            | quants  16 B/block [N*nb]   (nibble bytes as stored)
//   Q8_0: scales f16[N*nb]            | quants  i8[N*nb*32]
//   Q6_K: ql 128 B/sb | qh 64 B/sb | sc i8 16/sb | d f16 /sb       (sb = 256-wide superblock)
struct Weight {
    QType type;
    size_t K = 0, N = 0;   // in_dim, out_dim
    size_t nblk = 0;       // blocks (Q4_0/Q8_0) or superblocks (Q6_K) per row
    char* base = nullptr;  // device allocation
    size_t bytes = 0;
    // plane pointers into base
    const uint16_t* scales = nullptr;  // Q4_0/Q8_0 f16 block scales; Q6_K: per-superblock d
    const void* quants = nullptr;      // Q4_0/Q8_0 quants; Q6_K: ql
    const void* qh = nullptr;          // Q6_K
    const int8_t* sc = nullptr;        // Q6_K sub-scales
};

// A resident MoE layer (Q8_0 or Q6_K experts): three planar tensors whose rows are
// the experts' rows back to back (expert e, row r -> row e*rows + r).
struct MoeLayer {
    QType type = kQ8_0;
    size_t hidden = 0, eff = 0, ne = 0;
    Weight gate, up, down;  // gate/up: N = ne*eff, K = hidden; down: N = ne*hidden, K = eff
};

struct DevBuf {
    char* p = nullptr;
    size_t cap = 0;
};

struct ProfRec {
    std::string name;
    hipEvent_t e0, e1;
};

}  // namespace smx

struct smx_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string name;
    std::string err;
    std::unordered_map<std::string, smx::Weight> weights;
    std::unordered_map<size_t, smx::MoeLayer> moe;
    int num_cu = 256;

    // scratch, grown on demand (never shrinks)
    smx::DevBuf xf32;   // staged fp32 activations
    smx::DevBuf xq;     // int8 activations
    smx::DevBuf xd;     // f32 block scales
    smx::DevBuf xs;     // packed i16 pairs: sums of each 16-element half block
    smx::DevBuf yf32;   // staged outputs
    smx::DevBuf work;   // split-K partials, MoE intermediates, dumps
    smx::DevBuf work2;
    smx::DevBuf tab;    // small tables (ids, weights, tile tables)
    smx::DevBuf raw;    // upload staging: the raw GGUF blocks of the tensor being repacked (kept up to kRawKeepBytes between uploads)
    smx::DevBuf hx, hy; // pinned HOST staging of the host-pointer calls' activations and results
    smx::DevBuf htab;   // pinned HOST staging of the small tables of enqueue-only calls
    hipEvent_t htab_done = nullptr;  // recorded after the last copy out of htab (null: htab is free)

    // tuning overrides (0 = automatic)
    int tune_gemv_rpw = 0, tune_gemv_ks = 0, tune_gemv_wpc = 0, tune_gemv_lpr = 0, tune_gemm_splitk = 0, tune_gemm_tile_m = 0, tune_gemm_walk = 0, tune_host_io = 0, tune_gemm_narrow = 0;

    // dynamic-LDS limit already raised on this context's device, per kernel (see set_dyn_lds): a fixed
    // open-addressing table, so that a launch never allocates host memory
    static constexpr int kLdsSlots = 512;
    const void* lds_kern[kLdsSlots] = {};
    size_t lds_size[kLdsSlots] = {};

    // device address of the library's static scratch array on this context's device (see noalloc.hip)
    void* static_scratch = nullptr;

    bool capturing = false;  // between smx_graph_begin and smx_graph_end
    // A captured graph holds the addresses of the scratch buffers its kernels used.  While any graph
    // of this context is alive, a scratch buffer that has to grow is retired (kept until the context
    // closes) instead of freed, so that replays keep reading and writing valid memory.
    int live_graphs = 0;
    std::vector<char*> retired;

    // profiling
    bool prof_on = false;
    std::vector<smx::ProfRec> prof;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> ev_pool;
    std::string prof_names;
    hipEvent_t t0 = nullptr, t1 = nullptr;
};

namespace smx {

int fail(smx_ctx* c, int code, const char* fmt, ...);
int hip_fail(smx_ctx* c, hipError_t e, const char* what);
#define SMX_GEMV_GROUP_MAX 16  // single-row GEMVs that may share one launch

#define SMX_HIP(c, call)                                                   \
    do {                                                                   \
        hipError_t e_ = (call);                                            \
        if (e_ != hipSuccess) return ::smx::hip_fail((c), e_, #call);      \
    } while (0)

// No C++ exception may cross the C ABI: entry points that use standard containers run their body
// through this and report allocation failure as SMX_ERR_NOMEM.
template <class F>
int guarded(smx_ctx* c, const char* who, F&& body) {
    try {
        return body();
    } catch (const std::bad_alloc&) {
        return fail(c, SMX_ERR_NOMEM, "%s: out of host memory", who);
    } catch (const std::exception& e) {
        return fail(c, SMX_ERR_ARG, "%s: %s", who, e.what());
    }
}

int ensure(smx_ctx* c, DevBuf& b, size_t bytes);
// Frees a device allocation that kernels of the context may name, or, while a captured graph of the
// context is alive, keeps it until the context closes (a replay may still read it).
void release_device(smx_ctx* c, char* p);
// the same for a pinned host buffer (hipHostMalloc)
int ensure_host(smx_ctx* c, DevBuf& b, size_t bytes);

// Raises a kernel's dynamic-LDS limit when it asks for more than the 48 KB default (remembered per
// context and kernel so that replays and captured launches do not repeat the call).
template <typename Kern>
int set_dyn_lds(smx_ctx* c, Kern kern, size_t lds) {
    if (lds <= 48 * 1024) return SMX_OK;
    const void* key = (const void*)kern;
    unsigned slot = (unsigned)(((uintptr_t)key >> 4) * 2654435761u) % smx_ctx::kLdsSlots;
    int probes = 0;
    while (c->lds_kern[slot] && c->lds_kern[slot] != key && probes < smx_ctx::kLdsSlots) {
        slot = (slot + 1) % smx_ctx::kLdsSlots;
        probes++;
    }
    const bool have_slot = probes < smx_ctx::kLdsSlots;   // a full table only costs the repeated attribute call
    if (have_slot && c->lds_kern[slot] == key && lds <= c->lds_size[slot]) return SMX_OK;
    hipError_t e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return hip_fail(c, e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    if (have_slot) {
        c->lds_kern[slot] = key;
        c->lds_size[slot] = lds;
    }
    return SMX_OK;
}

// Brackets one kernel launch with an event pair when profiling is on.
struct ProfScope {
    smx_ctx* c;
    int idx = -1;
    ProfScope(smx_ctx* c, const char* name);
    ~ProfScope();
};

// One weight/output pair of a GEMM launch.
struct GemmOperand {
    const uint16_t* wscales;  // f16 [rows][nb]; Q6_K: the superblock scale d, [rows][nb / 8]
    const void* wquants;      // Q8_0: i8 [rows][K];  Q4_0: 16 B [rows][nb];  Q6_K: ql, 128 B [rows][nb / 8]
    float* out;               // [M][ldo] (split-K: Z such planes)
    const void* wqh;          // Q6_K: qh, 64 B [rows][nb / 8]
    const int8_t* wsc;        // Q6_K: sub-block scales, 16 per superblock
};
// One 128 x 128 output tile of a grouped GEMM.
struct GemmTile {
    int tok0, tok_end;  // activation rows [tok0, tok_end) (through a_rowmap if set)
    int row0, row_end;  // weight rows, limit = end of this expert's rows
    int col0;           // output column of row0
};
struct GemmArgs {
    GemmOperand op[2];
    const int8_t* xq;       // [*][K]
    const float* xd;        // [*][nb]
    const int* a_rowmap;    // optional: activation row index per logical row (MoE gather)
    const GemmTile* tiles;  // optional tile table; dense tiling when null
    int* dump;              // optional [M][N][nb] (Q6_K: [M][N][2 * nb], one per 16-element sub-block)
    int M, N, nb, ldo;
    int tiles_m, tiles_n;
    int tile_m;             // dense tiling: tokens per tile, 128 or 64 (a 64-token tile's waves pair up on two row tiles each)
    int stages_per_slice;   // stages (of 4 blocks) each grid.z slice covers
    int xcd_remap;
    int walk_gm;            // dense tiling: token tiles per group of the tile walk (see launch_gemm)
    int nops;               // grouped launches: operands per tile (workgroup x serves tile x / nops, operand x % nops)
    int narrow;             // dense tiling: the first `narrow` weight strips have 96 rows and are dispatched last (see launch_gemm)
};

// ---- launchers (all enqueue on c->stream; return SMX_OK or an error) ----
// Activation quantiser: x[m][K] f32 -> xq[m][K], xd[m][K/32], xs[m][K/32] (two i16 sums per block).
int launch_actquant(smx_ctx* c, const float* x, size_t m, size_t K, int8_t* xq, float* xd, int32_t* xs);
// n rows act(as[j]) * bs[j] (SMX_ACT_SILU_MUL or SMX_ACT_GEGLU), quantised: row j at xq + j*K, xd/xs + j*K/32.
int launch_actprod_quant(smx_ctx* c, int kind, const float* const* as, const float* const* bs, int n, size_t K,
                         int8_t* xq, float* xd, int32_t* xs);
// m rows [m][K] through a producer (SMX_ACT_RMSNORM with weight b[K] or null; SMX_ACT_SILU_MUL / SMX_ACT_GEGLU with
// b[m][K]) and the quantiser: xq[m][K], xd/xs[m][K/32].
int launch_rows_prod_quant(smx_ctx* c, int kind, const float* a, const float* b, size_t m, size_t K, float eps, int8_t* xq,
                           float* xd, int32_t* xs);
// Room for m quantised activation rows of length K: xq[m][K], xd[m][K/32], xs[m][K/32].
struct ActScratch {
    int8_t* xq;
    float* xd;
    int32_t* xs;
};
// GEMV with the activation quantiser fused into its LDS staging: x fp32 [m][K] -> y[m][N],
// m <= SMX_GEMV_MAX_M.  dump (optional): per-block i32 dots of row 0.  Several rows are quantised once
// into `sc`, or into the context's own scratch (grown on demand) when sc is null.
int launch_gemv(smx_ctx* c, const Weight& w, const float* x, size_t m, float* y, int32_t* dump,
                const ActScratch* sc = nullptr);
// y[N] = dequant(W) . x with fp32 activations (no quantiser): the arithmetic of the reference's per-weight gemv.
int launch_gemv_f32(smx_ctx* c, const Weight& w, const float* x, float* y);
// Quantise m device rows and run the kernel that serves this (weight, m): the dot4 GEMV, the small-batch MFMA
// kernel or the tiled GEMM (force_gemm: never the GEMV).  sc: caller-provided room for the quantised rows.
int run_matmul_dev(smx_ctx* c, const Weight& w, const float* xs_dev, size_t m, float* y_dev, bool force_gemm, int32_t* dump,
                   const ActScratch* sc);
// Looks the library's static scratch array up on the context's device (called once by smx_create).
int noalloc_init(smx_ctx* c);
// n <= 8 single-row GEMVs of one format and row length in one launch (device pointers).
// prod (optional): activation producer applied to every job's x before the fused quantiser.
struct ActProd {
    int kind;        // SMX_ACT_*
    const float* b;  // rmsnorm weight (or null) / the `up` operand of silu_mul, geglu
    float eps;
};
// Jobs whose weight is one expert of a stacked expert tensor chosen on the device: job j reads expert
// ids[slot[j]] (clamped to 0 .. ne - 1); its Weight is the view of expert 0, blocks_per_expert the
// number of blocks (Q6_K: superblocks) from one expert's rows to the next.
struct GemvIndirect {
    const int* ids;
    int ne;
    size_t blocks_per_expert;
    int slot[SMX_GEMV_GROUP_MAX];
    // paired launches only: route inside the launch from the ne <= 64 router logits (top route_k); ids_out / w_out
    // receive the routing for the launches behind it (ids may then be null)
    const float* logits = nullptr;
    int route_k = 0;
    int* ids_out = nullptr;
    float* w_out = nullptr;
};
// x2s (optional, with prod): a second operand per job instead of prod->b.
int launch_gemv_group(smx_ctx* c, const Weight* const* ws, const float* const* xs, float* const* ys, int n,
                      const char* name = nullptr, const ActProd* prod = nullptr, const float* const* x2s = nullptr,
                      const GemvIndirect* ind = nullptr);
// npairs (gate, up) pairs in one launch with the activation product in the kernel's tail: hs[p][r] = act2(gate . x) * (up . x);
// yg / yu (optional) also receive the dots.  *served = false and nothing launched when the shape does not take the flat form.
int launch_gemv_dual(smx_ctx* c, const Weight* const* wg, const Weight* const* wu, const float* const* xs, float* const* yg,
                     float* const* yu, float* const* hs, int npairs, int act2, const ActProd* prod, const char* name, bool* served,
                     const GemvIndirect* ind = nullptr);
// GEMM: y[m][N] on int8 MFMA.  dump (optional): out[m][N][K/32] i32.
int launch_gemm(smx_ctx* c, const Weight& w, const int8_t* xq, const float* xd, size_t m, float* y,
                int32_t* dump);

// Small-batch matmul on the matrix cores (skinny.hip): m <= SMX_SKINNY_MAX_M fp32 rows against a Q8_0 / Q4_0
// weight read once (its own quantiser launch + the matmul launch).  dump (optional): out[m][N][K/32] i32.
#define SMX_SKINNY_MAX_M 64
#define SMX_SKINNY_MIN_M 5
bool skinny_serves(const Weight& w, size_t m);
// bytes of sc.xq the call needs (quants in MFMA fragment order, 8, 16 or 32 token slots)
size_t skinny_xq_bytes(size_t m, size_t K);
size_t skinny_xd_bytes(size_t m, size_t K);   // of sc.xd (block scales, piece-major)
int launch_skinny(smx_ctx* c, const Weight& w, const float* x, size_t m, float* y, int32_t* dump, const ActScratch& sc);

int launch_gemm_grouped(smx_ctx* c, QType type, const GemmArgs& args, int ntiles, int nops, const char* name);
// the weight planes of w as a GEMM operand writing to out
GemmOperand gemm_operand(const Weight& w, float* out);

}  // namespace smx
