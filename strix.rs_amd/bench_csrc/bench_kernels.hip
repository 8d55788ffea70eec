// Measurement-only kernels (libstrix_bench.so): what the machine allows at the sizes of the matmul
// path, timed the same way as the path itself (HIP events around back-to-back launches on one stream).
// Nothing here is part of the product library and the product never loads it.
//
//   sbk_empty_launch   back-to-back launches of a kernel that does nothing: the fixed cost of a launch (and, as
//                      sbk_empty_launch_graph, of a launch inside a replayed graph)
//                      of a given grid (what a 14 MB GEMV pays before its first byte moves)
//   sbk_read_floor     a kernel that only reads a buffer cache-cold (rotating buffers larger than the
//                      Infinity Cache), one xor and one store per wave: the floor of a GEMV of that size
//   sbk_copy           plain copy, the streaming rate of the box
//   sbk_mfma_valu      the int8 GEMM's compute phase alone (MFMA 32x32x32 i8 + the two FMAs per output
//                      of exact per-block rescaling), with and without its LDS reads: the kernel's ceiling
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#define SBK_OK 1
#define SBK_ERR (-1)

namespace {

struct Timer {
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok = false;
    Timer() {
        ok = hipStreamCreate(&s) == hipSuccess && hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
    }
    ~Timer() {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (s) (void)hipStreamDestroy(s);
    }
    void begin() { (void)hipEventRecord(e0, s); }
    // microseconds between begin() and now (synchronises)
    double end_us() {
        (void)hipEventRecord(e1, s);
        if (hipEventSynchronize(e1) != hipSuccess) return -1.0;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.0;
        return (double)ms * 1e3;
    }
};

__global__ __launch_bounds__(1024) void empty_kernel(int* p) {
    if (p && threadIdx.x == 0xffffff) *p = 1;   // never true: the kernel has a body the compiler keeps
}

// The skeleton of a dependent GEMV launch: every workgroup fetches the K-float activation that the launch in front of it
// wrote, meets at a barrier and stores `rows` outputs, which the next launch reads as its activation.
__global__ __launch_bounds__(1024) void skeleton_kernel(const float* __restrict__ x, float* __restrict__ y, int K, int rows) {
    __shared__ float red[1024];
    float s = 0.f;
    for (int i = threadIdx.x; i < K / 4; i += 1024) {
        const float4 v = ((const float4*)x)[i];
        s += v.x + v.y + v.z + v.w;
    }
    red[threadIdx.x] = s;
    __syncthreads();
    s = red[(threadIdx.x * 7) & 1023];
    if ((int)threadIdx.x < rows) y[blockIdx.x * rows + threadIdx.x] = s * 0.f + 1.f;
}

// Workgroup b reads units [b * per_wg, (b + 1) * per_wg) of 16 bytes; wave w takes 64-unit loads
// w, w + nw, ... of that slab, UNR loads requested before the first is used.  Lanes past the end re-read
// the slab's last unit (no conditional loads).
template <int UNR>
__global__ __launch_bounds__(1024) void read_kernel(const uint4* __restrict__ buf, unsigned n16, unsigned per_wg,
                                                    unsigned* __restrict__ sink) {
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const unsigned u0 = blockIdx.x * per_wg;
    const unsigned u1 = min(u0 + per_wg, n16);
    if (u0 >= u1) return;
    const unsigned nloads = (u1 - u0 + 63) >> 6;
    unsigned x = 0;
    for (unsigned t = wave; t < nloads; t += nw * UNR) {
        uint4 v[UNR];
#pragma unroll
        for (int k = 0; k < UNR; k++) {
            const unsigned u = min(u0 + (t + k * nw) * 64 + lane, u1 - 1);
            v[k] = buf[u];
        }
#pragma unroll
        for (int k = 0; k < UNR; k++) x ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
    }
    for (int off = 32; off > 0; off >>= 1) x ^= __shfl_xor(x, off);
    if (lane == 0) sink[blockIdx.x * nw + wave] = x;
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// The compute phase of the int8 GEMM for a 32-token x 128-row wave tile: per 32-block, four MFMAs
// (one per 32-row tile), each result rescaled into its fp32 accumulators with two FMAs per output:
// t = fma(dw, float_bits(I + magic), -dw * magic); acc += dx * t.  The scales change every block (read
// from LDS, as in the GEMM), MFMA u + 1 is issued before the FMAs of u.
//   MODE 0: MFMAs only            MODE 1: FMAs only (the MFMA result registers are reused unchanged)
//   MODE 2: MFMAs + FMAs, operand fragments kept in registers
//   MODE 3: MFMAs + FMAs + the five 16-byte fragment reads per block from LDS (double-buffered in registers)
//   MODE 4: MFMAs + FMAs, B fragments from LDS, A fragment straight from global memory (fragment-ordered
//           activations: one coalesced 1 KB load per wave and block), the 16 activation scales of a block
//           as ONE dword per lane read through a DPP row broadcast in the second FMA
//   MODE 5: as 4 with the activation scales as four 16-byte LDS reads (16 registers)
constexpr int kMagicI = 0x4B400000;
constexpr float kMagicF = 12582912.f;

#define SBK_FMAC_BC(I)                                                                     \
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #I " row_mask:0xf bank_mask:0xf" : "+v"(accv[I]) : "v"(dxv), "v"(t[I]))
__device__ __forceinline__ void scale_accumulate_dpp(float (&accv)[16], const v16i& dn, float dw, float ndw, float dxv) {
    float t[16];
#pragma unroll
    for (int i = 0; i < 16; i++) t[i] = fmaf(dw, __int_as_float(dn[i]), ndw);
    SBK_FMAC_BC(0); SBK_FMAC_BC(1); SBK_FMAC_BC(2); SBK_FMAC_BC(3); SBK_FMAC_BC(4); SBK_FMAC_BC(5); SBK_FMAC_BC(6); SBK_FMAC_BC(7);
    SBK_FMAC_BC(8); SBK_FMAC_BC(9); SBK_FMAC_BC(10); SBK_FMAC_BC(11); SBK_FMAC_BC(12); SBK_FMAC_BC(13); SBK_FMAC_BC(14); SBK_FMAC_BC(15);
}

template <int MODE, int NT, int OCC>
__global__ __launch_bounds__(256, OCC) void mfma_valu_kernel(const float* __restrict__ scales, int nblocks, float* __restrict__ out,
                                                           unsigned long long* __restrict__ cycles, const v4i* __restrict__ aglob) {
    extern __shared__ __align__(16) char smem[];
    // LDS: 32 KB of operand bytes (what one stage of the GEMM holds) + 64 blocks of scales
    // LDS: 32 KB of operand bytes (what one stage of the GEMM holds) + 16 blocks of scales
    float* sdx = (float*)(smem + 32768);            // [16][128 tokens]
    float* sdw = sdx + 16 * 128;                    // [16][128 rows]
    for (int i = threadIdx.x; i < 32768 / 4; i += 256) ((int*)smem)[i] = (i * 2654435761u) >> 7;
    for (int i = threadIdx.x; i < 16 * 128; i += 256) sdx[i] = scales[i & 1023];
    for (int i = threadIdx.x; i < 16 * 128; i += 256) sdw[i] = (float)__half2float(__float2half(scales[(i * 7) & 1023]));
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = lane >> 5, col = lane & 31;
    float acc[NT][16];
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[nt][i] = 0.f;
    v16i cmagic;
#pragma unroll
    for (int i = 0; i < 16; i++) cmagic[i] = kMagicI;
    asm volatile("" : "+v"(cmagic));
    v4i fa = *(const v4i*)(smem + wave * 4096 + lane * 16);
    v4i fb[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) fb[nt] = *(const v4i*)(smem + 16384 + nt * 4096 + lane * 16);
    v16i d[2];
#pragma unroll
    for (int i = 0; i < 16; i++) d[0][i] = d[1][i] = kMagicI + lane + i;
    const unsigned long long t0 = clock64();
    // MODE 4: lane n of each 16-lane row holds the scale of accumulator n of that row's lane half
    const int dx_tok = ((lane & 15) >> 2) * 8 + half * 4 + (lane & 3);
    const v4i* ag = aglob + ((size_t)(blockIdx.x * 4 + wave) * 64) * 64 + lane;   // 64 blocks of 1 KB per wave, reused
    v4i fa_next = fa;
    if (MODE == 4 || MODE == 5) fa_next = ag[0];
    for (int b = 0; b < nblocks; b++) {
        const int bs = b & 15;
        float dxr[16], dw[NT];
        float dxv = 0.f;
        if (MODE != 0 && MODE != 6) {
            if (MODE == 4) {
                dxv = sdx[bs * 128 + wave * 32 + dx_tok];
            } else {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 v = *(const float4*)(sdx + bs * 128 + wave * 32 + g * 8 + half * 4);
                    dxr[4 * g] = v.x; dxr[4 * g + 1] = v.y; dxr[4 * g + 2] = v.z; dxr[4 * g + 3] = v.w;
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; nt++) dw[nt] = sdw[bs * 128 + nt * 32 + col];
        }
        if constexpr (MODE == 6) {
            // Q6_K arithmetic: the format scales 16-element sub-blocks, so a 32-block of a row tile is two K = 16 MFMAs, each
            // rescaled by its own weight scale: four vector operations per output per 32-block (the activation scale through a
            // DPP row broadcast, as the Q6_K GEMM reads it)
            dxv = sdx[bs * 128 + wave * 32 + dx_tok];
            float dw2[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                dw[nt] = sdw[bs * 128 + nt * 32 + col];
                dw2[nt] = sdw[((bs + 1) & 15) * 128 + nt * 32 + col];
            }
            auto unit = [&](int v) -> v16i {
                const int nt = v >> 1, jj = v & 1;
                const long a = ((long)(unsigned)fa[2 * jj]) | ((long)fa[2 * jj + 1] << 32);
                const long bq = ((long)(unsigned)fb[nt][2 * jj]) | ((long)fb[nt][2 * jj + 1] << 32);
                return __builtin_amdgcn_mfma_i32_32x32x16_i8(a, bq, cmagic, 0, 0, 0);
            };
            d[0] = unit(0);
#pragma unroll
            for (int v = 0; v < 2 * NT; v++) {
                if (v + 1 < 2 * NT) {
                    d[(v + 1) & 1] = unit(v + 1);
                    asm volatile("" : "+v"(d[(v + 1) & 1]));
                }
                const int u = v >> 1;
                const float dwv = (v & 1) ? dw2[u] : dw[u];
                scale_accumulate_dpp(acc[u], d[v & 1], dwv, -dwv * kMagicF, dxv);
                asm volatile("" : "+v"(acc[u][0]), "+v"(acc[u][1]), "+v"(acc[u][2]), "+v"(acc[u][3]), "+v"(acc[u][4]),
                                  "+v"(acc[u][5]), "+v"(acc[u][6]), "+v"(acc[u][7]), "+v"(acc[u][8]), "+v"(acc[u][9]),
                                  "+v"(acc[u][10]), "+v"(acc[u][11]), "+v"(acc[u][12]), "+v"(acc[u][13]),
                                  "+v"(acc[u][14]), "+v"(acc[u][15]));
            }
            continue;
        }
        if (MODE >= 4) {
            fa = fa_next;
            fa_next = ag[(size_t)((b + 1) & 63) * 64];
            const int rot = ((b & 3) * 2 + half + col) & 7;
#pragma unroll
            for (int nt = 0; nt < NT; nt++) fb[nt] = *(const v4i*)(smem + 16384 + nt * 4096 + (col >> 3) * 1024 + (col & 7) * 128 + rot * 16);
        }
        if (MODE == 3) {   // the next block's fragments (the GEMM rotates its reads over the 8 chunks of a 128-byte row)
            const int rot = ((b & 3) * 2 + half + col) & 7;
            fa = *(const v4i*)(smem + wave * 4096 + (col >> 3) * 1024 + (col & 7) * 128 + rot * 16);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) fb[nt] = *(const v4i*)(smem + 16384 + nt * 4096 + (col >> 3) * 1024 + (col & 7) * 128 + rot * 16);
        }
        if (MODE != 1) {
            d[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb[0], cmagic, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < NT; u++) {
            if (MODE != 1 && u + 1 < NT) {
                d[(u + 1) & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb[u + 1], cmagic, 0, 0, 0);
                asm volatile("" : "+v"(d[(u + 1) & 1]));
            }
            if (MODE != 0) {
                const v16i dn = d[u & 1];
                const float ndw = -dw[u] * kMagicF;
                if (MODE == 4) {
                    scale_accumulate_dpp(acc[u], dn, dw[u], ndw, dxv);
                } else {
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[u][i] = fmaf(dxr[i], fmaf(dw[u], __int_as_float(dn[i]), ndw), acc[u][i]);
                }
                asm volatile("" : "+v"(acc[u][0]), "+v"(acc[u][1]), "+v"(acc[u][2]), "+v"(acc[u][3]), "+v"(acc[u][4]),
                                  "+v"(acc[u][5]), "+v"(acc[u][6]), "+v"(acc[u][7]), "+v"(acc[u][8]), "+v"(acc[u][9]),
                                  "+v"(acc[u][10]), "+v"(acc[u][11]), "+v"(acc[u][12]), "+v"(acc[u][13]),
                                  "+v"(acc[u][14]), "+v"(acc[u][15]));
            } else {
                asm volatile("" : "+v"(d[u & 1]));
            }
        }
    }
    const unsigned long long t1 = clock64();
    float s = 0.f;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) s += acc[nt][i];
    if (MODE == 0) s += (float)(d[0][0] + d[1][5]);
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
    if (lane == 0) cycles[(size_t)blockIdx.x * 4 + wave] = t1 - t0;
}

int num_cus() {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    return prop.multiProcessorCount;
}

}  // namespace

extern "C" {

// Average microseconds per launch of an empty kernel with the given grid and workgroup size.
int sbk_empty_launch(unsigned grid, unsigned block, int launches, double* us_per_launch) {
    if (!us_per_launch || grid == 0 || block == 0 || block > 1024 || launches <= 0) return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    for (int i = 0; i < 20; i++) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, t.s, (int*)nullptr);
    (void)hipStreamSynchronize(t.s);
    t.begin();
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, t.s, (int*)nullptr);
    const double us = t.end_us();
    if (us < 0 || hipGetLastError() != hipSuccess) return SBK_ERR;
    *us_per_launch = us / launches;
    return SBK_OK;
}

// The same launches captured as ONE graph and replayed: what a dependent launch costs the device when no host call sits
// between two launches (the stream figure above is bound by how fast the host submits).
int sbk_empty_launch_graph(unsigned grid, unsigned block, int launches, double* us_per_launch) {
    if (!us_per_launch || grid == 0 || block == 0 || block > 1024 || launches <= 0) return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    for (int i = 0; i < 20; i++) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, t.s, (int*)nullptr);
    (void)hipStreamSynchronize(t.s);
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    if (hipStreamBeginCapture(t.s, hipStreamCaptureModeThreadLocal) != hipSuccess) return SBK_ERR;
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, t.s, (int*)nullptr);
    if (hipStreamEndCapture(t.s, &g) != hipSuccess || !g) return SBK_ERR;
    int rc = SBK_ERR;
    if (hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) == hipSuccess && ge) {
        if (hipGraphLaunch(ge, t.s) == hipSuccess && hipStreamSynchronize(t.s) == hipSuccess) {   // first replay untimed
            t.begin();
            const bool ok = hipGraphLaunch(ge, t.s) == hipSuccess;
            const double us = t.end_us();
            if (ok && us >= 0) {
                *us_per_launch = us / launches;
                rc = SBK_OK;
            }
        }
        (void)hipGraphExecDestroy(ge);
    }
    (void)hipGraphDestroy(g);
    return rc;
}

// `launches` skeleton launches (grid workgroups x 1024 threads, K-float activation, rows outputs per workgroup; grid * rows
// >= K), each reading what the one in front wrote, as one replayed graph: microseconds per launch.
int sbk_skeleton_graph(int K, int rows, unsigned grid, int launches, double* us_per_launch) {
    if (!us_per_launch || K <= 0 || K % 4 != 0 || rows <= 0 || rows > 1024 || grid == 0 || (size_t)grid * rows < (size_t)K || launches <= 0)
        return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    float *a = nullptr, *b = nullptr;
    const size_t bytes = (size_t)grid * rows * 4;
    if (hipMalloc(&a, bytes) != hipSuccess || hipMalloc(&b, bytes) != hipSuccess || hipMemset(a, 0, bytes) != hipSuccess ||
        hipMemset(b, 0, bytes) != hipSuccess) {
        if (a) (void)hipFree(a);
        if (b) (void)hipFree(b);
        return SBK_ERR;
    }
    auto launch = [&](int i) { hipLaunchKernelGGL(skeleton_kernel, dim3(grid), dim3(1024), 0, t.s, (i & 1) ? b : a, (i & 1) ? a : b, K, rows); };
    for (int i = 0; i < 20; i++) launch(i);
    (void)hipStreamSynchronize(t.s);
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    int rc = SBK_ERR;
    if (hipStreamBeginCapture(t.s, hipStreamCaptureModeThreadLocal) == hipSuccess) {
        for (int i = 0; i < launches; i++) launch(i);
        if (hipStreamEndCapture(t.s, &g) == hipSuccess && g && hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) == hipSuccess && ge) {
            if (hipGraphLaunch(ge, t.s) == hipSuccess && hipStreamSynchronize(t.s) == hipSuccess) {
                t.begin();
                const bool ok = hipGraphLaunch(ge, t.s) == hipSuccess;
                const double us = t.end_us();
                if (ok && us >= 0) {
                    *us_per_launch = us / launches;
                    rc = SBK_OK;
                }
            }
            (void)hipGraphExecDestroy(ge);
        }
        if (g) (void)hipGraphDestroy(g);
    }
    (void)hipFree(a);
    (void)hipFree(b);
    return rc;
}

// Reads `bytes` (a multiple of 16) per launch from one of `nbuf` distinct buffers in rotation (choose
// nbuf * bytes above the 256 MB Infinity Cache for a cache-cold figure; nbuf = 1 reads the same buffer
// hot).  grid x block threads, `unr` (1, 2, 4, 8 or 16) 16-byte loads in flight per thread.
int sbk_read_floor(size_t bytes, int nbuf, unsigned grid, unsigned block, int unr, int launches, double* us_per_launch) {
    if (!us_per_launch || bytes == 0 || bytes % 16 != 0 || bytes / 16 > 0x7fffffffu || nbuf <= 0 || grid == 0 || block == 0 ||
        block > 1024 || block % 64 != 0 || launches <= 0)
        return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    std::vector<uint4*> bufs((size_t)nbuf, nullptr);
    unsigned* sink = nullptr;
    int rc = SBK_OK;
    const unsigned n16 = (unsigned)(bytes / 16), per_wg = (n16 + grid - 1) / grid;
    auto launch = [&](int i) {
        const uint4* b = bufs[(size_t)(i % nbuf)];
        switch (unr) {
            case 1: hipLaunchKernelGGL(read_kernel<1>, dim3(grid), dim3(block), 0, t.s, b, n16, per_wg, sink); break;
            case 2: hipLaunchKernelGGL(read_kernel<2>, dim3(grid), dim3(block), 0, t.s, b, n16, per_wg, sink); break;
            case 4: hipLaunchKernelGGL(read_kernel<4>, dim3(grid), dim3(block), 0, t.s, b, n16, per_wg, sink); break;
            case 8: hipLaunchKernelGGL(read_kernel<8>, dim3(grid), dim3(block), 0, t.s, b, n16, per_wg, sink); break;
            default: hipLaunchKernelGGL(read_kernel<16>, dim3(grid), dim3(block), 0, t.s, b, n16, per_wg, sink); break;
        }
    };
    if (unr != 1 && unr != 2 && unr != 4 && unr != 8 && unr != 16) rc = SBK_ERR;
    if (rc == SBK_OK && hipMalloc((void**)&sink, (size_t)grid * 16 * 4) != hipSuccess) rc = SBK_ERR;
    for (int i = 0; i < nbuf && rc == SBK_OK; i++) {
        if (hipMalloc((void**)&bufs[(size_t)i], bytes) != hipSuccess) rc = SBK_ERR;
        else if (hipMemsetAsync(bufs[(size_t)i], i + 1, bytes, t.s) != hipSuccess) rc = SBK_ERR;
    }
    if (rc == SBK_OK) {
        for (int i = 0; i < nbuf + 8; i++) launch(i);
        (void)hipStreamSynchronize(t.s);
        t.begin();
        for (int i = 0; i < launches; i++) launch(i);
        const double us = t.end_us();
        if (us < 0 || hipGetLastError() != hipSuccess) rc = SBK_ERR;
        else *us_per_launch = us / launches;
    }
    (void)hipStreamSynchronize(t.s);
    for (uint4* b : bufs)
        if (b) (void)hipFree(b);
    if (sink) (void)hipFree(sink);
    return rc;
}

// Plain copy of `bytes`: microseconds per launch.
int sbk_copy(size_t bytes, int launches, double* us_per_launch) {
    if (!us_per_launch || bytes == 0 || bytes % 16 != 0 || launches <= 0) return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    uint4 *src = nullptr, *dst = nullptr;
    int rc = SBK_OK;
    if (hipMalloc((void**)&src, bytes) != hipSuccess || hipMalloc((void**)&dst, bytes) != hipSuccess) rc = SBK_ERR;
    if (rc == SBK_OK) {
        (void)hipMemsetAsync(src, 1, bytes, t.s);
        const unsigned grid = (unsigned)num_cus() * 32;
        for (int i = 0; i < 3; i++) hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, t.s, src, dst, bytes / 16);
        (void)hipStreamSynchronize(t.s);
        t.begin();
        for (int i = 0; i < launches; i++) hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, t.s, src, dst, bytes / 16);
        const double us = t.end_us();
        if (us < 0 || hipGetLastError() != hipSuccess) rc = SBK_ERR;
        else *us_per_launch = us / launches;
    }
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    return rc;
}

// The GEMM's compute phase alone on the whole chip: `wgs_per_cu` workgroups of 4 waves per CU (1 or 2
// waves per SIMD), `nblocks` 32-blocks per wave (4 MFMA units each).  Returns the launch time, the int8
// operation rate it corresponds to (2 * 32 * 32 * 32 per MFMA) and the average shader-clock cycles one wave
// spent per MFMA unit.
// `row_tiles` (4 or 2): 32-row tiles per wave, i.e. a 32 x 128 or 32 x 64 wave tile; wgs_per_cu 1..4 (4-wave workgroups,
// so also waves per SIMD; 32 x 128 tiles fit at most 3 per SIMD in registers).
// `warm_launches` untimed launches come first: under matrix load the chip takes some 20 ms to settle at the clock it
// then sustains (the first launches after idle run 15 % slower), and a prefill is hundreds of such launches.
int sbk_mfma_valu(int mode, int row_tiles, int wgs_per_cu, int nblocks, int warm_launches, double* us, double* tops, double* cycles_per_unit) {
    if (!us || !tops || !cycles_per_unit || mode < 0 || mode > 6 || wgs_per_cu < 1 || wgs_per_cu > 4 || nblocks <= 0 || warm_launches < 1) return SBK_ERR;
    if ((row_tiles != 4 && row_tiles != 2) || (row_tiles == 4 && wgs_per_cu > 3)) return SBK_ERR;
    Timer t;
    if (!t.ok) return SBK_ERR;
    const unsigned grid = (unsigned)(num_cus() * wgs_per_cu);
    const size_t lds = 32768 + 2 * 16 * 128 * 4;
    float *scales = nullptr, *out = nullptr;
    unsigned long long* cyc = nullptr;
    v4i* aglob = nullptr;
    int rc = SBK_OK;
    const size_t abytes = (size_t)grid * 4 * 64 * 1024;   // 64 fragment blocks of 1 KB per wave
    if (hipMalloc((void**)&aglob, abytes) != hipSuccess || hipMemset(aglob, 3, abytes) != hipSuccess) rc = SBK_ERR;
    if (rc == SBK_OK && (hipMalloc((void**)&scales, 1024 * 4) != hipSuccess || hipMalloc((void**)&out, (size_t)grid * 256 * 4) != hipSuccess ||
        hipMalloc((void**)&cyc, (size_t)grid * 4 * 8) != hipSuccess))
        rc = SBK_ERR;
    if (rc == SBK_OK) {
        std::vector<float> h(1024);
        for (int i = 0; i < 1024; i++) h[(size_t)i] = 0.001f + 0.00001f * (float)((i * 37) % 1024);
        (void)hipMemcpy(scales, h.data(), 1024 * 4, hipMemcpyHostToDevice);
        typedef void (*kern_t)(const float*, int, float*, unsigned long long*, const v4i*);
        // [mode][tile 4/2][occupancy class: waves per SIMD the register budget is set for]
        static const kern_t k4lo[7] = {mfma_valu_kernel<0, 4, 2>, mfma_valu_kernel<1, 4, 2>, mfma_valu_kernel<2, 4, 2>, mfma_valu_kernel<3, 4, 2>,
                                       mfma_valu_kernel<4, 4, 2>, mfma_valu_kernel<5, 4, 2>, mfma_valu_kernel<6, 4, 2>};
        static const kern_t k4hi[7] = {mfma_valu_kernel<0, 4, 3>, mfma_valu_kernel<1, 4, 3>, mfma_valu_kernel<2, 4, 3>, mfma_valu_kernel<3, 4, 3>,
                                       mfma_valu_kernel<4, 4, 3>, mfma_valu_kernel<5, 4, 3>, mfma_valu_kernel<6, 4, 3>};
        static const kern_t k2[7] = {mfma_valu_kernel<0, 2, 4>, mfma_valu_kernel<1, 2, 4>, mfma_valu_kernel<2, 2, 4>, mfma_valu_kernel<3, 2, 4>,
                                     mfma_valu_kernel<4, 2, 4>, mfma_valu_kernel<5, 2, 4>, mfma_valu_kernel<6, 2, 4>};
        const kern_t kern = row_tiles == 2 ? k2[mode] : (wgs_per_cu <= 2 ? k4lo[mode] : k4hi[mode]);
        auto launch = [&]() { hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, t.s, (const float*)scales, nblocks, out, cyc, (const v4i*)aglob); };
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) rc = SBK_ERR;
        if (rc == SBK_OK) {
            for (int i = 0; i < warm_launches; i++) launch();
            (void)hipStreamSynchronize(t.s);
            const int reps = 5;
            t.begin();
            for (int i = 0; i < reps; i++) launch();
            const double total = t.end_us();
            if (total < 0 || hipGetLastError() != hipSuccess) {
                rc = SBK_ERR;
            } else {
                *us = total / reps;
                const double units = (double)grid * 4.0 * (double)nblocks * (double)row_tiles;
                *tops = units * 65536.0 / (*us * 1e-6) / 1e12;
                std::vector<unsigned long long> hc((size_t)grid * 4);
                (void)hipMemcpy(hc.data(), cyc, hc.size() * 8, hipMemcpyDeviceToHost);
                double sum = 0;
                for (unsigned long long v : hc) sum += (double)v;
                *cycles_per_unit = sum / (double)hc.size() / ((double)nblocks * (double)row_tiles);
            }
        }
    }
    if (scales) (void)hipFree(scales);
    if (out) (void)hipFree(out);
    if (cyc) (void)hipFree(cyc);
    if (aglob) (void)hipFree(aglob);
    return rc;
}

}  // extern "C"
