// Drives the C++ mirror of the accelerator seam the way a Strix.rs model forward would:
// adopt weights, run per-weight GEMVs and a prefill GEMM, and fall through on keys that were never
// adopted.  Without a GPU it only checks that creating the backend fails with a clear error.
//   g++ -std=c++17 selftest.cpp -o selftest -L.. -lstrix_mi355 -Wl,-rpath,'$ORIGIN/..'
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>

#include "weight_accel.hpp"

static uint32_t lcg(uint64_t& s) {  // generator of the reference's device tests (strix-backend-rocm/src/lib.rs:141-144)
    s = s * 6364136223846793005ULL + 1ULL;
    return (uint32_t)(s >> 33);
}

int main() {
    std::unique_ptr<strix::Mi355WeightAccel> acc;
    try {
        acc.reset(new strix::Mi355WeightAccel(0));
    } catch (const strix::BackendError& e) {
        std::printf("no device: %s\n", e.what());
        return 77;
    }
    const size_t K = 256, N = 64, nb = K / 32;
    uint64_t seed = 0xA5A51234ULL;
    std::vector<uint8_t> raw(N * nb * 34);
    for (size_t b = 0; b < N * nb; b++) {
        raw[b * 34] = 0x00;
        raw[b * 34 + 1] = 0x24;  // f16 0.015625
        for (int i = 0; i < 32; i++) raw[b * 34 + 2 + i] = (uint8_t)(int8_t)((int)(lcg(seed) % 255) - 127);
    }
    // uploaded the way the trait does it (upload_q8_0, accel.rs:163), not through a convenience wrapper
    if (!acc->upload_q8_0("blk.0.attn_q.weight", raw.data(), raw.size(), K, N)) return 1;
    std::vector<float> x(K);
    for (size_t i = 0; i < K; i++) x[i] = 0.5f * std::sin(0.017f * (float)i);
    auto y = acc->gemv("blk.0.attn_q.weight", x);
    if (!y || y->size() != N) return 2;
    // dequantised f32 dot for comparison (activation rounding only)
    double maxref = 0, maxerr = 0;
    for (size_t r = 0; r < N; r++) {
        double s = 0;
        for (size_t i = 0; i < K; i++) s += 0.015625 * (double)(int8_t)raw[(r * nb + i / 32) * 34 + 2 + i % 32] * x[i];
        maxref = std::fmax(maxref, std::fabs(s));
        maxerr = std::fmax(maxerr, std::fabs(s - (*y)[r]));
    }
    std::printf("%s: gemv rel err vs f32 %.3e, resident %zu\n", acc->name().c_str(), maxerr / maxref, acc->resident_count());
    if (maxerr / maxref > 2e-2) return 3;
    if (acc->gemv("never.adopted", x)) return 4;  // declined -> caller keeps its own path
    std::vector<float> xs(5 * K);
    for (size_t i = 0; i < xs.size(); i++) xs[i] = 0.5f * std::sin(0.011f * (float)i);
    auto g = acc->prefill_q8_gemm("blk.0.attn_q.weight", xs, 5);
    if (!g || g->size() != 5 * N) return 5;
    try {
        std::vector<float> bad(K - 32);
        acc->gemv("blk.0.attn_q.weight", bad);
        return 6;
    } catch (const strix::BackendError&) {
    }
    {   // rmsnorm fused into the GEMV == GEMV of the normalised row computed here
        double ss = 0;
        for (size_t i = 0; i < K; i++) ss += (double)x[i] * (double)x[i];
        const float scale = (float)(1.0 / std::sqrt(ss / (double)K + 1e-6));
        std::vector<float> xn(K);
        for (size_t i = 0; i < K; i++) xn[i] = x[i] * scale;
        auto yf = acc->gemv_fused("blk.0.attn_q.weight", SMX_ACT_RMSNORM, x, nullptr, 1e-6f);
        auto yn = acc->gemv("blk.0.attn_q.weight", xn);
        if (!yf || !yn) return 7;
        for (size_t r = 0; r < N; r++)
            if (std::fabs((*yf)[r] - (*yn)[r]) > 1e-5 * maxref * scale) return 8;
        if (acc->gemv_fused("never.adopted", SMX_ACT_RMSNORM, x, nullptr, 1e-6f)) return 9;
    }
    {   // a weight that arrives through a GGUF file (attach_gguf) is served the same way
        const char* path = "/tmp/strix_selftest.gguf";
        std::FILE* f = std::fopen(path, "wb");
        if (!f) return 10;
        auto put = [&](const void* p, size_t n) { std::fwrite(p, 1, n, f); };
        auto put_u32 = [&](uint32_t v) { put(&v, 4); };
        auto put_u64 = [&](uint64_t v) { put(&v, 8); };
        const std::string tname = "blk.1.attn_q.weight";
        put_u32(0x46554747u); put_u32(3); put_u64(1); put_u64(0);          // magic, version, 1 tensor, 0 metadata
        put_u64(tname.size()); put(tname.data(), tname.size());
        put_u32(2); put_u64(K); put_u64(N); put_u32(8); put_u64(0);       // 2 dims (in_dim first), Q8_0, offset 0
        long pos = std::ftell(f);
        for (; pos % 32 != 0; pos++) std::fputc(0, f);                     // data section is 32-byte aligned
        put(raw.data(), raw.size());
        std::fclose(f);
        if (acc->attach_gguf(path) != 1) return 11;
        std::remove(path);
        auto yg = acc->gemv(tname, x);
        if (!yg || yg->size() != N) return 12;
        for (size_t r = 0; r < N; r++)
            if ((*yg)[r] != (*y)[r]) return 13;                            // same bytes, same kernel, same result
        std::vector<std::pair<std::string, const std::vector<float>*>> calls = {{tname, &x}, {"never.adopted", &x}};
        auto yb = acc->gemv_batch(calls);
        if (!yb[0] || yb[0]->size() != N || yb[1]) return 14;
    }
    std::printf("selftest ok\n");
    return 0;
}
