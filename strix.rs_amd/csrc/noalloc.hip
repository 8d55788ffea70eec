// The one entry point of the library that allocates nothing: smx_gemv_noalloc_dev, for callers that
// cannot call hipMalloc (code under HIP graph capture, tight serving loops, harnesses that forbid it).
//
// It is smx_gemv_dev (1..8 activation rows against one resident weight, the small-batch verify step)
// with the scratch of that call -- the rows quantised once for all workgroups: int8 quants, f32 block
// scales, packed 16-element sums -- taken from a file-scope device array instead of the context's
// growable buffers.  The array exists once per GPU the library runs on and is held until the process
// ends.  Its name is a host-side stand-in, not a device address: the address on a device comes from
// hipGetSymbolAddress with that device current (noalloc_init, called by smx_create), and only that
// pointer is ever handed to kernels.
//
// Every call on a GPU shares that GPU's array, whatever context it comes through; the array keeps
// the last call's contents.  Nothing in it has to start at zero: the quantiser launch writes every
// byte the GEMV launch behind it reads.  Calls that overlap on one GPU (two contexts, i.e. two
// streams, on the same device) race on the array; calls on one context are ordered by its stream.
#include "smx_internal.h"

namespace smx {

// 8 rows of at most 16384 elements: quants 8 x 16384, scales and sums 8 x 512 dwords each
constexpr size_t kNoallocMaxRows = SMX_NOALLOC_MAX_ROWS;
constexpr size_t kNoallocMaxK = SMX_NOALLOC_MAX_IN_DIM;
constexpr size_t kScratchQ = kNoallocMaxRows * kNoallocMaxK;
constexpr size_t kScratchD = kNoallocMaxRows * (kNoallocMaxK / 32) * 4;
constexpr size_t kScratchBytes = kScratchQ + 2 * kScratchD;   // 163840

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

static void* g_scratch_of_device[64] = {};   // address of `scratch` on each device, once looked up

int noalloc_init(smx_ctx* c) {
    if (c->device >= 0 && c->device < 64 && g_scratch_of_device[c->device]) {
        c->static_scratch = g_scratch_of_device[c->device];
        return SMX_OK;
    }
    SMX_HIP(c, hipSetDevice(c->device));
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return hip_fail(c, e, "hipGetSymbolAddress(scratch)");
    c->static_scratch = ptr;
    if (c->device >= 0 && c->device < 64) g_scratch_of_device[c->device] = ptr;
    return SMX_OK;
}

}  // namespace smx

using namespace smx;

extern "C" int smx_gemv_noalloc_dev(smx_ctx* c, const char* key, const float* xs_dev, size_t m, float* y_dev) {
    if (!c) return SMX_ERR_ARG;
    if (!key || !xs_dev || !y_dev) return fail(c, SMX_ERR_ARG, "gemv_noalloc_dev: null argument");
    const Weight* w = nullptr;
    for (const auto& kv : c->weights)   // compared in place: no temporary std::string, no host allocation
        if (kv.first == key) {
            w = &kv.second;
            break;
        }
    if (!w) return SMX_NOT_RESIDENT;
    if (m == 0 || m > kNoallocMaxRows)
        return fail(c, SMX_ERR_LIMIT, "gemv_noalloc_dev: %zu rows (1..%zu supported)", m, kNoallocMaxRows);
    // one row is quantised inside the GEMV's staging and never touches the scratch: rows of any length the GEMV serves
    if (m >= 2 && w->K > kNoallocMaxK)
        return fail(c, SMX_ERR_LIMIT, "gemv_noalloc_dev: in_dim %zu exceeds the static scratch (%zu rows of at most %zu elements)",
                    w->K, m, kNoallocMaxK);
    if (!c->static_scratch) return fail(c, SMX_ERR_HIP, "gemv_noalloc_dev: the static scratch was not located on device %d", c->device);
    unsigned char* base = (unsigned char*)c->static_scratch;   // the device pointer, never the array's name
    const ActScratch sc = {(int8_t*)base, (float*)(base + kScratchQ), (int32_t*)(base + kScratchQ + kScratchD)};
    const bool prof = c->prof_on;   // per-kernel timing creates events on first use: off for this call
    c->prof_on = false;
    const int rc = run_matmul_dev(c, *w, xs_dev, m, y_dev, false, nullptr, &sc);   // the kernels smx_gemv_dev runs for this call
    c->prof_on = prof;
    return rc;
}
