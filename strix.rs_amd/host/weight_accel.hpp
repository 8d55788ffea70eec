// Host-side mirror of the reference's accelerator seam, in C++ over the C ABI.
//
// `strix::WeightAccel` restates the quantized-matmul part of the Rust trait
// `WeightAccel` (crates/strix-core/src/accel.rs:147-405): same method names, argument meaning and
// decline behaviour (`false` / empty optional when a key or layer is not resident).
// `strix::Mi355WeightAccel` implements it on libstrix_mi355.so, the role
// `RocmWeightAccel` plays in the reference (crates/strix-backend-rocm/src/decode.rs:2490-3900).
// Failures the reference folds into a decline (bad shapes, HIP errors) throw `strix::BackendError`,
// the counterpart of StrixError::Backend (crates/strix-core/src/error.rs:14-43): this backend has no
// CPU path to decline to.
#pragma once
#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "../../include/strix_mi355.h"

namespace strix {

struct BackendError : std::runtime_error {
    int code;
    BackendError(int c, const std::string& m) : std::runtime_error("strix-mi355: " + m), code(c) {}
};

class WeightAccel {
  public:
    virtual ~WeightAccel() = default;
    // accel.rs:150-165 — adopt a weight [out_dim, in_dim] given as raw GGUF block bytes
    virtual bool upload_q4_0(const std::string& key, const uint8_t* bytes, size_t nbytes, size_t in_dim, size_t out_dim) = 0;
    virtual bool upload_q6_k(const std::string& key, const uint8_t* bytes, size_t nbytes, size_t in_dim, size_t out_dim) = 0;
    virtual bool upload_q8_0(const std::string& key, const uint8_t* bytes, size_t nbytes, size_t in_dim, size_t out_dim) = 0;
    // accel.rs:170-181
    virtual bool upload_moe_q8(size_t layer, const uint8_t* gate, size_t gate_n, const uint8_t* up, size_t up_n,
                               const uint8_t* down, size_t down_n, size_t hidden, size_t eff, size_t ne) = 0;
    // accel.rs:391
    virtual std::optional<std::vector<float>> gemv(const std::string& key, const std::vector<float>& x) = 0;
    // accel.rs:397
    virtual std::vector<std::optional<std::vector<float>>> gemv_batch(
        const std::vector<std::pair<std::string, const std::vector<float>*>>& calls) = 0;
    // accel.rs:213 — y[m][out] token-major
    virtual std::optional<std::vector<float>> prefill_q8_gemm(const std::string& key, const std::vector<float>& xs, size_t m) = 0;
    // accel.rs:217
    virtual std::optional<std::vector<uint32_t>> lm_head_argmax_rows(const std::string& key, const std::vector<float>& xs, size_t m) = 0;
    // accel.rs:201-210
    virtual std::optional<std::vector<float>> moe_ffn(size_t layer, const std::vector<int32_t>& ids,
                                                      const std::vector<float>& wexp, const std::vector<float>& x, float sgate) = 0;
    // accel.rs:311-321 — plan = (expert, slot_off, count)
    virtual std::optional<std::vector<float>> moe_layer_q8_dev(size_t layer, const std::vector<float>& xs, size_t m,
                                                               const std::vector<std::tuple<size_t, size_t, size_t>>& plan,
                                                               const std::vector<int32_t>& slot_tok,
                                                               const std::vector<float>& wslot) = 0;
    virtual size_t resident_count() const = 0;  // accel.rs:402
    virtual std::string name() const = 0;       // accel.rs:405
};

class Mi355WeightAccel final : public WeightAccel {
  public:
    explicit Mi355WeightAccel(int device = 0) {
        const int rc = smx_create(device, &ctx_);
        if (rc != SMX_OK) throw BackendError(rc, smx_last_error(nullptr));
    }
    ~Mi355WeightAccel() override { smx_destroy(ctx_); }
    Mi355WeightAccel(const Mi355WeightAccel&) = delete;
    Mi355WeightAccel& operator=(const Mi355WeightAccel&) = delete;

    bool upload_q4_0(const std::string& key, const uint8_t* b, size_t n, size_t in_dim, size_t out_dim) override {
        return ok(smx_upload_q4_0(ctx_, key.c_str(), b, n, in_dim, out_dim));
    }
    bool upload_q6_k(const std::string& key, const uint8_t* b, size_t n, size_t in_dim, size_t out_dim) override {
        return ok(smx_upload_q6_k(ctx_, key.c_str(), b, n, in_dim, out_dim));
    }
    bool upload_q8_0(const std::string& key, const uint8_t* b, size_t n, size_t in_dim, size_t out_dim) override {
        return ok(smx_upload_q8_0(ctx_, key.c_str(), b, n, in_dim, out_dim));
    }
    // The upload loop of the models' attach_accel (mellum.rs:460-535) over a GGUF file: returns the
    // number of adopted matrices plus expert layers.
    size_t attach_gguf(const std::string& path) {
        smx_gguf* g = nullptr;
        char err[256] = {0};
        const int rc = smx_gguf_open(path.c_str(), &g, err, sizeof err);
        if (rc != SMX_OK) throw BackendError(rc, err);
        size_t nw = 0, nl = 0;
        const int ra = smx_gguf_attach(ctx_, g, &nw, &nl);
        smx_gguf_close(g);
        if (ra != SMX_OK) throw BackendError(ra, smx_last_error(ctx_));
        return nw + nl;
    }
    // One matrix of a GGUF file re-encoded on the host as Q8_0 (8) or Q4_0 (2) and uploaded under
    // `key`: the repacks of gemma3n.rs:455-470 (Q4_K token_embd -> Q8_0 lm_head) and qwen35.rs:741-760.
    bool upload_as(const std::string& path, const std::string& tensor, const std::string& key, int target_type) {
        smx_gguf* g = nullptr;
        char err[256] = {0};
        const int rc = smx_gguf_open(path.c_str(), &g, err, sizeof err);
        if (rc != SMX_OK) throw BackendError(rc, err);
        const int ru = smx_gguf_upload_as(ctx_, g, tensor.c_str(), key.c_str(), target_type);
        smx_gguf_close(g);
        return ok(ru);
    }
    // accel.rs:238-246 moe_layer_ffn: plan = (expert, rows) pairs over expert-major rows; returns dy[rows][hidden]
    std::optional<std::vector<float>> moe_layer_ffn(size_t layer, const std::vector<std::pair<int32_t, int32_t>>& plan,
                                                    const std::vector<float>& xs, size_t rows) {
        if (rows == 0 || xs.size() % rows != 0) return std::nullopt;
        std::vector<int32_t> flat;
        for (const auto& p : plan) { flat.push_back(p.first); flat.push_back(p.second); }
        std::vector<float> dy(xs.size());
        if (!ok(smx_moe_layer_ffn(ctx_, layer, flat.data(), plan.size(), xs.data(), rows, dy.data(), dy.size()))) return std::nullopt;
        return dy;
    }
    // accel.rs:185-196
    bool upload_moe_q6(size_t layer, const uint8_t* gate, size_t gate_n, const uint8_t* up, size_t up_n, const uint8_t* down,
                       size_t down_n, size_t hidden, size_t eff, size_t ne) {
        return ok(smx_upload_moe_q6(ctx_, layer, gate, gate_n, up, up_n, down, down_n, hidden, eff, ne));
    }
    bool upload_moe_q8(size_t layer, const uint8_t* gate, size_t gate_n, const uint8_t* up, size_t up_n, const uint8_t* down,
                       size_t down_n, size_t hidden, size_t eff, size_t ne) override {
        return ok(smx_upload_moe_q8(ctx_, layer, gate, gate_n, up, up_n, down, down_n, hidden, eff, ne));
    }
    // The C ABI writes into caller-provided buffers: results are sized with what the library holds for
    // the key (smx_weight_dims), however the weight got there (upload_*, attach_gguf, upload_as).

    std::optional<std::vector<float>> gemv(const std::string& key, const std::vector<float>& x) override {
        std::vector<float> y(out_of(key));
        if (!ok(smx_gemv(ctx_, key.c_str(), x.data(), x.size(), y.empty() ? &dummy_ : y.data(), y.size()))) return std::nullopt;
        return y;
    }
    std::vector<std::optional<std::vector<float>>> gemv_batch(
        const std::vector<std::pair<std::string, const std::vector<float>*>>& calls) override {
        const size_t n = calls.size();
        std::vector<std::vector<float>> ys(n);
        std::vector<const char*> keys(n);
        std::vector<const float*> xs(n);
        std::vector<float*> yp(n);
        std::vector<size_t> il(n), oc(n);
        std::vector<int> st(n);
        for (size_t i = 0; i < n; i++) {
            ys[i].resize(out_of(calls[i].first));
            keys[i] = calls[i].first.c_str();
            xs[i] = calls[i].second->data();
            il[i] = calls[i].second->size();
            yp[i] = ys[i].empty() ? &dummy_ : ys[i].data();
            oc[i] = ys[i].size();
        }
        ok(smx_gemv_batch(ctx_, n, keys.data(), xs.data(), il.data(), yp.data(), oc.data(), st.data()));
        std::vector<std::optional<std::vector<float>>> out(n);
        for (size_t i = 0; i < n; i++) {
            if (st[i] < 0) throw BackendError(st[i], smx_last_error(ctx_));
            if (st[i] == SMX_OK) out[i] = std::move(ys[i]);
        }
        return out;
    }
    // Beyond the trait: the producer of the step before the GEMV (rmsnorm / SwiGLU / GeGLU, the
    // reference's rmsnorm_xquant, silu_xquant, geglu_xquant, kernels.rs:101-226) fused into it.
    // b: norm weight (may be null) or the `up` operand.
    std::optional<std::vector<float>> gemv_fused(const std::string& key, int act, const std::vector<float>& a,
                                                 const std::vector<float>* b, float eps) {
        if (b && b->size() != a.size()) throw BackendError(SMX_ERR_ARG, "gemv_fused: operand lengths differ");
        std::vector<float> y(out_of(key));
        if (!ok(smx_gemv_fused(ctx_, key.c_str(), act, a.data(), b ? b->data() : nullptr, a.size(), eps,
                               y.empty() ? &dummy_ : y.data(), y.size())))
            return std::nullopt;
        return y;
    }
    std::optional<std::vector<float>> prefill_q8_gemm(const std::string& key, const std::vector<float>& xs, size_t m) override {
        if (m == 0) throw BackendError(SMX_ERR_ARG, "prefill_q8_gemm: m == 0");
        std::vector<float> y(m * out_of(key));
        if (!ok(smx_gemm(ctx_, key.c_str(), xs.data(), m, xs.size() / m, y.empty() ? &dummy_ : y.data(), y.size()))) return std::nullopt;
        return y;
    }
    std::optional<std::vector<uint32_t>> lm_head_argmax_rows(const std::string& key, const std::vector<float>& xs, size_t m) override {
        if (m == 0) throw BackendError(SMX_ERR_ARG, "lm_head_argmax_rows: m == 0");
        std::vector<uint32_t> out(m);
        if (!ok(smx_lm_head_argmax_rows(ctx_, key.c_str(), xs.data(), m, xs.size() / m, out.data()))) return std::nullopt;
        return out;
    }
    std::optional<std::vector<float>> moe_ffn(size_t layer, const std::vector<int32_t>& ids, const std::vector<float>& wexp,
                                              const std::vector<float>& x, float sgate) override {
        if (ids.size() != wexp.size()) throw BackendError(SMX_ERR_ARG, "moe_ffn: ids / wexp length mismatch");  // decode.rs:2854
        std::vector<float> y(x.size());
        if (!ok(smx_moe_ffn(ctx_, layer, ids.data(), wexp.data(), ids.size(), x.data(), x.size(), sgate, y.data(), y.size())))
            return std::nullopt;
        return y;
    }
    std::optional<std::vector<float>> moe_layer_q8_dev(size_t layer, const std::vector<float>& xs, size_t m,
                                                       const std::vector<std::tuple<size_t, size_t, size_t>>& plan,
                                                       const std::vector<int32_t>& slot_tok,
                                                       const std::vector<float>& wslot) override {
        if (slot_tok.size() != wslot.size()) throw BackendError(SMX_ERR_ARG, "moe_layer_q8_dev: slot_tok / wslot length mismatch");
        std::vector<size_t> flat;
        flat.reserve(plan.size() * 3);
        for (auto& p : plan) {
            flat.push_back(std::get<0>(p));
            flat.push_back(std::get<1>(p));
            flat.push_back(std::get<2>(p));
        }
        std::vector<float> y(xs.size());
        if (!ok(smx_moe_layer(ctx_, layer, xs.data(), m, flat.data(), plan.size(), slot_tok.data(), wslot.data(),
                              slot_tok.size(), y.data(), y.size())))
            return std::nullopt;
        return y;
    }
    size_t resident_count() const override { return smx_resident_count(ctx_); }
    std::string name() const override { return smx_name(ctx_); }
    smx_ctx* raw() { return ctx_; }

    // convenience: upload by GGML type number
    bool adopt(int ggml_type, const std::string& key, const std::vector<uint8_t>& bytes, size_t in_dim, size_t out_dim) {
        if (ggml_type == 2) return upload_q4_0(key, bytes.data(), bytes.size(), in_dim, out_dim);
        if (ggml_type == 8) return upload_q8_0(key, bytes.data(), bytes.size(), in_dim, out_dim);
        if (ggml_type == 14) return upload_q6_k(key, bytes.data(), bytes.size(), in_dim, out_dim);
        return false;
    }

  private:
    bool ok(int rc) const {
        if (rc < 0) throw BackendError(rc, smx_last_error(ctx_));
        return rc == SMX_OK;
    }
    // out_dim of a resident weight; 0 for an unknown key (the library then answers "not resident")
    size_t out_of(const std::string& key) const {
        size_t out_dim = 0;
        return smx_weight_dims(ctx_, key.c_str(), nullptr, &out_dim) == SMX_OK ? out_dim : 0;
    }
    smx_ctx* ctx_ = nullptr;
    float dummy_ = 0.f;
};

}  // namespace strix
