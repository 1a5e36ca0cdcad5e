// C++ host-side mirror of the reference's quantized projection interface over
// the C ABI of libizwi_qmm (include/izwi_qmm.h).  Header-only; link with
// -lizwi_qmm.
//
// Names and error behaviour follow the reference (izwi-core,
// crates/izwi-core/src/models/architectures/qwen3/core.rs, and the Candle types
// it calls):
//   QTensor                       candle_core::quantized::QTensor (core.rs:710-715, 853-895)
//   QMatMul                       candle_core::quantized::QMatMul::{from_arc, from_qtensor, forward}
//   packed_qmatmul_from_qtensors  core.rs:846-889
//   quantized_storage_bytes       core.rs:891-909
//   Qwen3Projection               core.rs:671-674, 710-718, 791-831 (quantized arm)
//   GgufLoader, is_gguf_file      crates/izwi-core/src/models/shared/weights/gguf.rs:36-203, 366-377
//   Error                         crates/izwi-core/src/error.rs:69-73 (InferenceError /
//                                 ModelLoadError / InvalidInput)
// There is no CPU fallback: without a gfx950 device every operation throws.
#pragma once

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "izwi_decode_ops.h"
#include "izwi_gguf.h"
#include "izwi_qmm.h"

namespace izwi {

enum class GgmlDType : int { Q8_0 = IZWI_QMM_Q8_0, Q4K = IZWI_QMM_Q4_K, Q6K = IZWI_QMM_Q6_K };
inline int block_size(GgmlDType t) { return t == GgmlDType::Q8_0 ? 32 : 256; }
inline int type_size(GgmlDType t) { return t == GgmlDType::Q8_0 ? 34 : (t == GgmlDType::Q6K ? 210 : 144); }

enum class MemSpace : int { Device = IZWI_QMM_DEVICE, Host = IZWI_QMM_HOST };

// The reference maps Candle errors to InferenceError, load-time ones to ModelLoadError.
class Error : public std::runtime_error {
public:
    enum class Kind { InvalidInput, ModelLoadError, InferenceError };
    Error(Kind kind, int status, const std::string& msg) : std::runtime_error(msg), kind_(kind), status_(status) {}
    Kind kind() const { return kind_; }
    int status() const { return status_; }

private:
    Kind kind_;
    int status_;
};

inline void check(int rc) {
    if (rc == IZWI_QMM_OK) return;
    const std::string msg = izwi_qmm_last_error();
    switch (rc) {
        case IZWI_QMM_ERR_INVALID: throw Error(Error::Kind::InvalidInput, rc, msg);
        case IZWI_QMM_ERR_UNSUPPORTED:
        case IZWI_QMM_ERR_NO_DEVICE: throw Error(Error::Kind::ModelLoadError, rc, msg);
        default: throw Error(Error::Kind::InferenceError, rc, msg);
    }
}

// `quantized_storage_bytes(rows, cols, dtype)`, core.rs:891-909.
inline uint64_t quantized_storage_bytes(int64_t rows, int64_t cols, GgmlDType dtype) {
    uint64_t out = 0;
    check(izwi_qmm_storage_bytes((int)dtype, rows, cols, &out));
    return out;
}

// A quantized [n, k] weight (or a stack [e, n, k] of expert weights) on the GPU.
class QTensor {
public:
    // `ggml_file::qtensor_from_ggml(dtype, raw, dims, device)`: raw GGUF block bytes -> tensor.
    static std::shared_ptr<QTensor> from_blocks(GgmlDType dtype, const void* blocks, uint64_t nbytes,
                                                int64_t n, int64_t k, MemSpace space = MemSpace::Host) {
        izwi_qmm_weight* h = nullptr;
        check(izwi_qmm_weight_create((int)dtype, n, k, blocks, nbytes, (int)space, &h));
        return std::shared_ptr<QTensor>(new QTensor(h));
    }
    static std::shared_ptr<QTensor> from_expert_blocks(GgmlDType dtype, const void* blocks, uint64_t nbytes,
                                                       int32_t n_experts, int64_t n, int64_t k,
                                                       MemSpace space = MemSpace::Host) {
        izwi_qmm_weight* h = nullptr;
        check(izwi_qmm_weight_create_stacked((int)dtype, n_experts, n, k, blocks, nbytes, (int)space, &h));
        return std::shared_ptr<QTensor>(new QTensor(h));
    }
    // `QTensor::quantize(&tensor, dtype)` (candle-core quantized/mod.rs; the reference's use: qwen3/core.rs:3112):
    // an f32 [n, k] matrix in host memory -> Q8_0 / Q4_K tensor, blocks as the reference's CPU quantizer writes them.
    static std::shared_ptr<QTensor> quantize(const std::vector<float>& w, int64_t n, int64_t k, GgmlDType dtype) {
        if ((int64_t)w.size() != n * k)
            throw Error(Error::Kind::InvalidInput, IZWI_QMM_ERR_INVALID, "quantize: the tensor does not hold n * k values");
        std::vector<uint8_t> blocks(quantized_storage_bytes(n, k, dtype));
        check(izwi_qmm_quantize_weights_f32((int)dtype, w.data(), n, k, blocks.data(), IZWI_QMM_HOST, nullptr));
        return from_blocks(dtype, blocks.data(), blocks.size(), n, k);
    }
    // takes ownership of a handle made by the C ABI
    static std::shared_ptr<QTensor> adopt(izwi_qmm_weight* h) { return std::shared_ptr<QTensor>(new QTensor(h)); }
    ~QTensor() { izwi_qmm_weight_destroy(h_); }
    QTensor(const QTensor&) = delete;
    QTensor& operator=(const QTensor&) = delete;

    GgmlDType dtype() const { return (GgmlDType)info_.ggml_dtype; }
    int64_t rows() const { return info_.n; }
    int64_t cols() const { return info_.k; }
    int32_t n_stacked() const { return info_.n_stacked; }
    // `shape().dims2()`: an expert stack is rank 3
    std::pair<int64_t, int64_t> dims2() const {
        if (info_.n_stacked != 1)
            throw Error(Error::Kind::InvalidInput, IZWI_QMM_ERR_INVALID, "unexpected rank, expected: 2, got: 3");
        return {info_.n, info_.k};
    }
    uint64_t storage_size_in_bytes() const { return info_.nbytes; }
    // `QTensor::data()`: the GGUF block bytes the tensor was built from.
    std::vector<uint8_t> data() const {
        std::vector<uint8_t> out(info_.nbytes);
        check(izwi_qmm_weight_data(h_, out.data(), out.size(), IZWI_QMM_HOST, nullptr));
        return out;
    }
    // `QTensor::dequantize(device)`: f32 [n_stacked * n, k].
    std::vector<float> dequantize() const {
        std::vector<float> out((size_t)info_.n_stacked * info_.n * info_.k);
        check(izwi_qmm_dequantize_f32(h_, out.data(), IZWI_QMM_HOST, nullptr));
        return out;
    }
    // `Embedding::forward(input_ids)` on the dequantized table (qwen3/core.rs:2000-2007, 2083-2085):
    // f32 [ids.size(), k], the rows of `dequantize()` with those ids; an id outside [0, n) is an error.
    std::vector<float> dequantize_rows(const std::vector<int32_t>& ids) const {
        std::vector<float> out(ids.size() * (size_t)info_.k);
        check(izwi_qmm_dequantize_rows(h_, ids.data(), (int64_t)ids.size(), IZWI_QMM_HOST, out.data(), IZWI_QMM_OUT_F32,
                                       IZWI_QMM_HOST, nullptr));
        return out;
    }
    izwi_qmm_weight* handle() const { return h_; }

private:
    explicit QTensor(izwi_qmm_weight* h) : h_(h) {
        const int rc = izwi_qmm_weight_get_info(h, &info_);
        if (rc != IZWI_QMM_OK) {
            izwi_qmm_weight_destroy(h);
            check(rc);
        }
    }
    izwi_qmm_weight* h_;
    izwi_qmm_weight_info info_{};
};

// `QMatMul`: y[.., n] = x[.., k] * W^T.
class QMatMul {
public:
    static QMatMul from_arc(std::shared_ptr<QTensor> q) {
        q->dims2(); // a projection is rank 2
        return QMatMul(std::move(q));
    }
    static QMatMul from_qtensor(std::shared_ptr<QTensor> q) { return from_arc(std::move(q)); }

    // `Module::forward` for f32 activations: x is [m, k] contiguous, y [m, n]; both in `space`.
    // Device pointers: asynchronous on `stream`.  Host pointers: returns when y is written.
    void forward(const float* x, int64_t m, float* y, MemSpace space, void* stream = nullptr) const {
        check(izwi_qmm_forward_f32(q_->handle(), x, m, y, (int)space, stream));
    }
    // host convenience form: x.size() must be a multiple of k
    std::vector<float> forward(const std::vector<float>& x) const {
        const int64_t k = q_->cols();
        if (k == 0 || x.size() % (size_t)k)
            throw Error(Error::Kind::InvalidInput, IZWI_QMM_ERR_INVALID,
                        "input has " + std::to_string(x.size()) + " elements, not a multiple of k = " + std::to_string(k));
        const int64_t m = (int64_t)(x.size() / (size_t)k);
        std::vector<float> y((size_t)m * q_->rows());
        forward(x.data(), m, y.data(), MemSpace::Host);
        return y;
    }
    // prefill form: bf16 activations, y bf16 (out_bf16) or f32
    void forward_bf16(const uint16_t* x, int64_t m, void* y, bool out_bf16, MemSpace space,
                      void* stream = nullptr) const {
        check(izwi_qmm_forward_bf16(q_->handle(), x, m, y, out_bf16 ? IZWI_QMM_OUT_BF16 : IZWI_QMM_OUT_F32,
                                    (int)space, stream));
    }
    // The whole `Quantized` arm of `Qwen3Projection::forward` (core.rs:795-829) plus the residual add
    // that follows o_proj / down_proj (core.rs:1875, 1879) in one call: x is f32 or bf16 (`x_bf16`),
    // y = x W^T + residual stored as f32 or bf16 (`y_bf16`); residual has y's type, may be y, may be null.
    void forward_fused(const void* x, bool x_bf16, int64_t m, const void* residual, void* y, bool y_bf16,
                       MemSpace space, void* stream = nullptr) const {
        check(izwi_qmm_forward_fused(q_->handle(), x, x_bf16 ? IZWI_QMM_OUT_BF16 : IZWI_QMM_OUT_F32, m, residual, y,
                                     y_bf16 ? IZWI_QMM_OUT_BF16 : IZWI_QMM_OUT_F32, (int)space, stream));
    }
    // RMSNorm (weight `norm_weight` [k], `eps`) of x and the projection of the result, as one call
    // (the final norm + lm_head, core.rs:1690-1702).
    void forward_normed(const float* x, int64_t m, const float* norm_weight, float eps, float* y, MemSpace space,
                        void* stream = nullptr) const {
        check(izwi_qmm_forward_normed_f32(q_->handle(), x, m, norm_weight, eps, y, (int)space, stream));
    }
    const std::shared_ptr<QTensor>& qtensor() const { return q_; }
    int64_t out_features() const { return q_->rows(); }
    int64_t in_features() const { return q_->cols(); }

private:
    explicit QMatMul(std::shared_ptr<QTensor> q) : q_(std::move(q)) {}
    std::shared_ptr<QTensor> q_;
};

// `packed_qmatmul_from_qtensors` (core.rs:846-889): one [sum(rows), k] projection from
// several tensors of equal k and dtype (fused QKV, fused gate/up).
inline QMatMul packed_qmatmul_from_qtensors(const std::vector<std::shared_ptr<QTensor>>& parts) {
    if (parts.empty())
        throw Error(Error::Kind::ModelLoadError, IZWI_QMM_ERR_INVALID, "Packed quantized projection group was empty");
    std::vector<std::vector<uint8_t>> datas;
    std::vector<int64_t> rows;
    std::vector<const void*> ptrs;
    std::vector<uint64_t> lens;
    for (const auto& p : parts) {
        p->dims2();
        datas.push_back(p->data());
        rows.push_back(p->rows());
    }
    for (const auto& d : datas) {
        ptrs.push_back(d.data());
        lens.push_back(d.size());
    }
    izwi_qmm_weight* h = nullptr;
    check(izwi_qmm_weight_create_packed((int)parts[0]->dtype(), (int32_t)parts.size(), rows.data(),
                                        parts[0]->cols(), ptrs.data(), lens.data(), IZWI_QMM_HOST, &h));
    return QMatMul::from_arc(QTensor::adopt(h)); // the new handle owns its own copy of the bytes
}

// The `Separate` arms of `Qwen3QkvProjection::forward` / `Qwen3GateUpProjection::forward`
// (core.rs:1119-1127, 1274-1282): several projections on the same activations in one call;
// ys[i] is [m, projections[i].out_features()].
inline void forward_group(const std::vector<const QMatMul*>& projections, const float* x, int64_t m,
                          const std::vector<float*>& ys, MemSpace space, void* stream = nullptr) {
    std::vector<const izwi_qmm_weight*> handles;
    for (const QMatMul* p : projections) handles.push_back(p->qtensor()->handle());
    check(izwi_qmm_forward_group_f32(handles.data(), (int32_t)handles.size(), x, m, ys.data(), (int)space, stream));
}

// The same with the RMSNorm that precedes the group folded in (input_layernorm + q / k / v,
// core.rs:1866, 1455-1462): x is the un-normed hidden state.
inline void forward_group_normed(const std::vector<const QMatMul*>& projections, const float* x, int64_t m,
                                 const float* norm_weight, float eps, const std::vector<float*>& ys, MemSpace space,
                                 void* stream = nullptr) {
    std::vector<const izwi_qmm_weight*> handles;
    for (const QMatMul* p : projections) handles.push_back(p->qtensor()->handle());
    check(izwi_qmm_forward_group_normed_f32(handles.data(), (int32_t)handles.size(), x, m, norm_weight, eps, ys.data(),
                                            (int)space, stream));
}

// `Qwen3GateUpProjection::forward_silu_mul` (core.rs:1250-1300), `Separate` arm: h = silu(x Wg^T) * (x Wu^T),
// [m, intermediate]; with `norm_weight` the post-attention RMSNorm of x is folded in (core.rs:1877).
inline void forward_gate_up_silu(const QMatMul& gate, const QMatMul& up, const float* x, int64_t m, float* h,
                                 MemSpace space, void* stream = nullptr, const float* norm_weight = nullptr,
                                 float eps = 1e-6f) {
    if (norm_weight)
        check(izwi_qmm_forward_gate_up_silu_normed_f32(gate.qtensor()->handle(), up.qtensor()->handle(), x, m,
                                                       norm_weight, eps, h, (int)space, stream));
    else
        check(izwi_qmm_forward_gate_up_silu_f32(gate.qtensor()->handle(), up.qtensor()->handle(), x, m, h, (int)space,
                                                stream));
}

// `Qwen3Mlp::forward` (core.rs:1786-1798), `Separate` gate / up pair: y = down(silu(x Wg^T) * (x Wu^T)),
// [m, hidden], the results of forward_gate_up_silu followed by down.forward bit for bit.
inline void mlp_forward(const QMatMul& gate, const QMatMul& up, const QMatMul& down, const float* x, int64_t m,
                        float* y, MemSpace space, void* stream = nullptr) {
    check(izwi_qmm_mlp_forward_f32(gate.qtensor()->handle(), up.qtensor()->handle(), down.qtensor()->handle(), x, m, y,
                                   (int)space, stream));
}

// The fused-kernel hooks of crates/izwi-core/src/kernels/mod.rs:109-225, f32 arm.  The reference's
// hooks return None where no kernel applies; these throw izwi::Error where the library refuses.
namespace kernels {
inline void rms_norm(const float* x, const float* weight, int64_t rows, int64_t hidden, float eps, float* y,
                     MemSpace space, void* stream = nullptr) {
    check(izwi_rms_norm_f32(x, weight, rows, hidden, eps, y, (int)space, stream));
}
inline void qk_rms_norm(const float* q, const float* k, const float* qk_weight, int64_t q_rows, int64_t k_rows,
                        int64_t head_dim, float eps, float* q_out, float* k_out, MemSpace space,
                        void* stream = nullptr) {
    check(izwi_qk_rms_norm_f32(q, k, qk_weight, q_rows, k_rows, head_dim, eps, q_out, k_out, (int)space, stream));
}
inline void rope_pair_bshd(const float* q, const float* k, const float* cos_sin, int64_t batch, int64_t seq,
                           int64_t q_heads, int64_t k_heads, int64_t head_dim, float* q_out, float* k_out,
                           MemSpace space, void* stream = nullptr) {
    check(izwi_rope_pair_bshd_f32(q, k, cos_sin, batch, seq, q_heads, k_heads, head_dim, q_out, k_out, (int)space,
                                  stream));
}
inline void decode_gqa_attention(const float* q, const float* k, const float* v, int64_t num_heads,
                                 int64_t num_kv_heads, int64_t head_dim, int64_t kv_len, int64_t kv_capacity,
                                 float scale, float* out, MemSpace space, void* stream = nullptr) {
    check(izwi_decode_gqa_attention_f32(q, k, v, num_heads, num_kv_heads, head_dim, kv_len, kv_capacity, scale, out,
                                        (int)space, stream));
}
// One token of `Qwen3Attention::forward` between the projections and o_proj (core.rs:1464-1575): q/k
// norm, rotary embedding, cache append and the attention over positions 0 .. pos, device pointers.
inline void decode_attention_step(const float* q, const float* k, const float* v, const float* qk_weight,
                                  const float* cos_sin, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                  float eps, float* k_cache, float* v_cache, int64_t kv_capacity, int64_t pos,
                                  float scale, float* out, void* stream = nullptr) {
    check(izwi_decode_attention_step_f32(q, k, v, qk_weight, cos_sin, num_heads, num_kv_heads, head_dim, eps, k_cache,
                                         v_cache, kv_capacity, pos, scale, out, stream));
}
// The same without the attention: q to q_out, the new key / value into position `pos` of the caches.
inline void qk_norm_rope_append(const float* q, const float* k, const float* v, const float* qk_weight,
                                const float* cos_sin, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                float eps, float* q_out, float* k_cache, float* v_cache, int64_t kv_capacity,
                                int64_t pos, void* stream = nullptr) {
    check(izwi_qk_norm_rope_append_f32(q, k, v, qk_weight, cos_sin, num_heads, num_kv_heads, head_dim, eps, q_out,
                                       k_cache, v_cache, kv_capacity, pos, stream));
}
inline void argmax(const float* logits, int64_t rows, int64_t n, uint32_t* out, MemSpace space,
                   void* stream = nullptr) {
    check(izwi_argmax_f32(logits, rows, n, out, (int)space, stream));
}
} // namespace kernels

// `Qwen3Projection` (quantized arm): the op always receives f32 activations and
// returns f32 (core.rs:772-831); callers with other activation dtypes cast around it.
class Qwen3Projection {
public:
    static Qwen3Projection quantized(std::shared_ptr<QTensor> q) { return Qwen3Projection(QMatMul::from_arc(std::move(q))); }
    static Qwen3Projection packed_quantized(const std::vector<std::shared_ptr<QTensor>>& parts) {
        return Qwen3Projection(packed_qmatmul_from_qtensors(parts));
    }
    void forward(const float* x, int64_t m, float* y, MemSpace space, void* stream = nullptr) const {
        mm_.forward(x, m, y, space, stream);
    }
    std::vector<float> forward(const std::vector<float>& x) const { return mm_.forward(x); }
    const QMatMul& qmatmul() const { return mm_; }

    // `Qwen3Projection::logits_for_tokens` (core.rs:745-758): (token id, logit) pairs of one hidden
    // state for the given ids; only the weight rows of those ids are read.
    std::vector<std::pair<uint32_t, float>> logits_for_tokens(const std::vector<float>& hidden,
                                                              const std::vector<uint32_t>& token_ids) const {
        std::vector<std::pair<uint32_t, float>> out;
        if (token_ids.empty()) return out;
        if ((int64_t)hidden.size() != mm_.qtensor()->cols())
            throw Error(Error::Kind::InferenceError, IZWI_QMM_ERR_INVALID,
                        "Qwen3 selected-token logits expected [1,vocab] or [1,1,vocab]");
        std::vector<float> values(token_ids.size());
        check(izwi_qmm_forward_rows_f32(mm_.qtensor()->handle(), token_ids.data(), (int64_t)token_ids.size(), hidden.data(),
                                        1, values.data(), IZWI_QMM_HOST, nullptr));
        for (size_t i = 0; i < token_ids.size(); i++) out.emplace_back(token_ids[i], values[i]);
        return out;
    }

private:
    explicit Qwen3Projection(QMatMul mm) : mm_(std::move(mm)) {}
    QMatMul mm_;
};

// `is_gguf_file` (gguf.rs:366-377).
inline bool is_gguf_file(const std::string& path) { return izwi_gguf_is_gguf_file(path.c_str()) != 0; }

// `GgufMmapMode` / `GgufReaderKind` (backends/model_io.rs:13-45, 85-89).
enum class GgufMmapMode : int { Auto = IZWI_GGUF_MMAP_AUTO, On = IZWI_GGUF_MMAP_ON, Off = IZWI_GGUF_MMAP_OFF };
enum class GgufReaderKind : int { Buffered = IZWI_GGUF_READER_BUFFERED, Mapped = IZWI_GGUF_READER_MAPPED };
// `GgufMmapMode::parse`: false for the empty string and unknown words.
inline bool parse_gguf_mmap_mode(const std::string& raw, GgufMmapMode* out) {
    const int m = izwi_gguf_parse_mmap_mode(raw.c_str());
    if (m < 0) return false;
    *out = (GgufMmapMode)m;
    return true;
}

// `GgufLoader` (gguf.rs:36-203): one GGUF file, mapped or (mode off, or a mapping that fails) read
// with buffered I/O as `open_gguf_reader_with_mode` does (model_io.rs:127-160); tensors go from there
// straight into weight handles on the current HIP device.  Parsing and lookups need no GPU.
class GgufLoader {
public:
    static std::shared_ptr<GgufLoader> from_path(const std::string& path, const GgufMmapMode* configured = nullptr) {
        izwi_gguf* g = nullptr;
        const int rc = izwi_gguf_open_with_mode(path.c_str(), configured ? (int)*configured : -1, &g);
        if (rc != IZWI_QMM_OK) // `Error::ModelLoadError("Failed to open / parse GGUF file: ...")`
            throw Error(Error::Kind::ModelLoadError, rc, izwi_qmm_last_error());
        return std::shared_ptr<GgufLoader>(new GgufLoader(g));
    }
    ~GgufLoader() { izwi_gguf_close(g_); }
    GgufLoader(const GgufLoader&) = delete;
    GgufLoader& operator=(const GgufLoader&) = delete;

    GgufReaderKind reader_kind() const { return (GgufReaderKind)izwi_gguf_reader_kind(g_); }
    size_t tensor_count() const { return (size_t)izwi_gguf_tensor_count(g_); }
    std::vector<std::string> tensor_names() const {
        std::vector<std::string> out;
        for (int64_t i = 0; i < izwi_gguf_tensor_count(g_); i++) {
            const char* name = nullptr;
            check(izwi_gguf_tensor_name(g_, i, &name));
            out.emplace_back(name);
        }
        return out;
    }
    bool has_tensor(const std::string& name) const {
        izwi_gguf_tensor_info info;
        return izwi_gguf_tensor_info_get(g_, name.c_str(), &info) == IZWI_QMM_OK;
    }
    // `tensor_shape`: empty optional upstream, here an empty vector with `found` false
    std::vector<int64_t> tensor_shape(const std::string& name, bool* found = nullptr) const {
        izwi_gguf_tensor_info info;
        const bool ok = izwi_gguf_tensor_info_get(g_, name.c_str(), &info) == IZWI_QMM_OK;
        if (found) *found = ok;
        return ok ? std::vector<int64_t>(info.dims, info.dims + info.n_dims) : std::vector<int64_t>();
    }
    // `get_metadata_string` / `get_metadata_u64`: false if the key is absent or of another type
    bool get_metadata_string(const std::string& key, std::string* out) const {
        const char* p = nullptr;
        uint64_t n = 0;
        if (izwi_gguf_metadata_string(g_, key.c_str(), &p, &n) != IZWI_QMM_OK) return false;
        out->assign(p, n);
        return true;
    }
    bool get_metadata_u64(const std::string& key, uint64_t* out) const {
        return izwi_gguf_metadata_u64(g_, key.c_str(), out) == IZWI_QMM_OK;
    }
    // `load_qtensor(name, device)`
    std::shared_ptr<QTensor> load_qtensor(const std::string& name) const {
        izwi_qmm_weight* h = nullptr;
        const int rc = izwi_gguf_load_weight(g_, name.c_str(), &h);
        if (rc != IZWI_QMM_OK) throw Error(Error::Kind::ModelLoadError, rc, izwi_qmm_last_error());
        return QTensor::adopt(h);
    }
    // `packed_quantized_qmatmul(loader, device, names)` (core.rs:834-845)
    QMatMul load_packed_qmatmul(const std::vector<std::string>& names) const {
        std::vector<const char*> ptrs;
        for (const std::string& n : names) ptrs.push_back(n.c_str());
        izwi_qmm_weight* h = nullptr;
        check(izwi_gguf_load_packed(g_, ptrs.data(), (int32_t)ptrs.size(), &h));
        return QMatMul::from_qtensor(QTensor::adopt(h));
    }
    // `load_tensor(name, DType::F32, device)` into host memory
    std::vector<float> load_tensor(const std::string& name) const {
        izwi_gguf_tensor_info info;
        const int rc = izwi_gguf_tensor_info_get(g_, name.c_str(), &info);
        if (rc != IZWI_QMM_OK) throw Error(Error::Kind::ModelLoadError, rc, izwi_qmm_last_error());
        uint64_t count = 1;
        for (int i = 0; i < info.n_dims; i++) count *= (uint64_t)info.dims[i];
        std::vector<float> out(count);
        const int rc2 = izwi_gguf_load_tensor_f32(g_, name.c_str(), out.data(), count, IZWI_QMM_HOST, nullptr);
        if (rc2 != IZWI_QMM_OK) throw Error(Error::Kind::ModelLoadError, rc2, izwi_qmm_last_error());
        return out;
    }
    const izwi_gguf* handle() const { return g_; }

private:
    explicit GgufLoader(izwi_gguf* g) : g_(g) {}
    izwi_gguf* g_;
};

} // namespace izwi
