/*
 * izwi_decode_ops — the decode-step neighbours of the quantized projections: RMSNorm, the
 * q/k head norm, rotary embedding and single-token grouped-query attention, f32 and f16.
 *
 * Each entry point is the device side of one of the reference's fused-kernel hooks
 * (crates/izwi-core/src/kernels/mod.rs:109-225), which today dispatch to Metal only
 * (crates/izwi-core/src/kernels/metal.rs) and return None elsewhere, so that the caller falls
 * back to Candle's eager operators.  Arithmetic follows the reference's shaders
 * (metal.rs:59-381) in f32; only the order of the sums differs (the reference's tests allow
 * 1e-5 against the eager operators, metal.rs:2956).
 *
 * Conventions are those of izwi_qmm.h: return IZWI_QMM_OK or a negative izwi_qmm_status, message
 * through izwi_qmm_last_error(); `mem_space` says whether the pointers are device or host
 * memory (host buffers are staged, synchronous); `stream` is a hipStream_t or NULL.  All tensors
 * are contiguous row-major, f32 unless the entry point's name says f16.  Outputs may alias the corresponding inputs (in-place).
 */
#ifndef IZWI_DECODE_OPS_H
#define IZWI_DECODE_OPS_H

#include <stdint.h>

#include "izwi_qmm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* `try_fused_rms_norm(input, weight, eps)` (kernels/mod.rs:141-155, metal.rs:1979-2024, shader
 * metal.rs:147-186): y[r, i] = x[r, i] * rsqrt(mean_i(x[r, :]^2) + eps) * weight[i] for `rows` rows
 * of `hidden` values.  The reference refuses rows == 0 and hidden == 0 (returns None): here rows ==
 * 0 is a no-op and hidden == 0 is IZWI_QMM_ERR_INVALID. */
int izwi_rms_norm_f32(const float* x, const float* weight, int64_t rows, int64_t hidden, float eps,
                      float* y, int mem_space, void* stream);

/* `try_fused_qk_rms_norm(q, k, qk_weight, eps)` (kernels/mod.rs:109-123, metal.rs:1906-1975,
 * shader metal.rs:59-101): the per-head norms of Qwen3 attention (qwen3/core.rs:1470) in one
 * launch.  q is `[q_rows, head_dim]` (q_rows = batch * heads for one token), k is
 * `[k_rows, head_dim]`, qk_weight is `[2 * head_dim]`: q's weights, then k's.  The reference's
 * shader is limited to head_dim <= 256 and one token; this kernel takes any row counts and
 * head_dim <= 8192. */
int izwi_qk_rms_norm_f32(const float* q, const float* k, const float* qk_weight, int64_t q_rows,
                         int64_t k_rows, int64_t head_dim, float eps, float* q_out, float* k_out,
                         int mem_space, void* stream);

/* `try_fused_rope_pair_bshd(q, k, cos_sin)` (kernels/mod.rs:157-171, metal.rs:2026-2094, shader
 * metal.rs:227-265): q is `[batch, seq, q_heads, head_dim]`, k is `[batch, seq, k_heads,
 * head_dim]`, cos_sin is `[seq, head_dim]` with the cosines in the first half of a row and the
 * sines in the second; head_dim even.  The two halves of a head rotate against each other:
 * out[d] = x[d] cos[d] - x[half + d] sin[d], out[half + d] = x[d] sin[d] + x[half + d] cos[d]. */
int izwi_rope_pair_bshd_f32(const float* q, const float* k, const float* cos_sin, int64_t batch,
                            int64_t seq, int64_t q_heads, int64_t k_heads, int64_t head_dim,
                            float* q_out, float* k_out, int mem_space, void* stream);

/* The hooks' `DType::F16` arm (the reference's `*_f16` shaders, metal.rs:103-144, 187-225, 267-305,
 * 383-457): the same four operations on IEEE half tensors (raw bits as uint16_t), every tensor of a
 * call f16 as the reference's wrappers require; values are widened on load, all arithmetic is f32
 * and each result is rounded to f16 once.  The reference's tests allow 5e-3 for this arm
 * (metal.rs:2956).  Shapes, limits and error behaviour are those of the f32 entry points. */
int izwi_rms_norm_f16(const uint16_t* x, const uint16_t* weight, int64_t rows, int64_t hidden, float eps,
                      uint16_t* y, int mem_space, void* stream);

/* izwi_rms_norm_f32 whose result goes, quantized, straight into the activation records of the batched
 * decode kernels (izwi_qmm.h, "activation records"): the layer norm in front of q|k|v and gate|up
 * (qwen3/core.rs:1866, 1877) and the quantization inside the following `QMatMul::forward` as one
 * launch.  The records equal izwi_qmm_quantize_records_f32(izwi_rms_norm_f32(x)) bit for bit.  f32,
 * device pointers, hidden a multiple of 256 up to 16384, 16-byte aligned buffers. */
int izwi_rms_norm_quantize_records_f32(int ggml_weight_dtype, const float* x, const float* weight, int64_t rows,
                                       int64_t hidden, float eps, void* records, void* stream);
int izwi_qk_rms_norm_f16(const uint16_t* q, const uint16_t* k, const uint16_t* qk_weight, int64_t q_rows,
                         int64_t k_rows, int64_t head_dim, float eps, uint16_t* q_out, uint16_t* k_out,
                         int mem_space, void* stream);
int izwi_rope_pair_bshd_f16(const uint16_t* q, const uint16_t* k, const uint16_t* cos_sin, int64_t batch,
                            int64_t seq, int64_t q_heads, int64_t k_heads, int64_t head_dim,
                            uint16_t* q_out, uint16_t* k_out, int mem_space, void* stream);
int izwi_decode_gqa_attention_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t kv_len,
                                  int64_t kv_capacity, float scale, uint16_t* out, int mem_space,
                                  void* stream);

/* The single-token sequence of `Qwen3Attention::forward` between the q/k/v projections and the
 * attention itself as ONE launch: `apply_qk_norm_pair` (qwen3/core.rs:1464-1478), `apply_rope_pair`
 * (core.rs:1480-1575) and the append of the new key / value rows to the cache.  q is `[num_heads,
 * head_dim]`, k and v are `[num_kv_heads, head_dim]` (the projections' outputs), qk_weight is
 * `[2 * head_dim]` (q's norm weights, then k's), cos_sin is `[head_dim]` for this position
 * (cos | sin).  Writes the normed, rotated q to q_out (may be q), the normed, rotated k and the
 * unchanged v to position `pos` of the head-major caches `[num_kv_heads, kv_capacity, head_dim]`.
 * Values are those of izwi_qk_rms_norm_f32 followed by izwi_rope_pair_bshd_f32 up to the order
 * of the norm's sum.  Device pointers only (the caches live on the device).  It has no single counterpart among the
 * reference's hooks: it is their composition for one token. */
int izwi_qk_norm_rope_append_f32(const float* q, const float* k, const float* v, const float* qk_weight,
                                 const float* cos_sin, int64_t num_heads, int64_t num_kv_heads,
                                 int64_t head_dim, float eps, float* q_out, float* k_cache, float* v_cache,
                                 int64_t kv_capacity, int64_t pos, void* stream);

/* The same sequence AND the attention behind it as one launch (two when the positions are split):
 * the attention kernel norms and rotates its query heads and the new key itself, takes the new
 * (key, value) as position `pos` and appends them to the caches on its way.  Arguments as
 * izwi_qk_norm_rope_append_f32 (without q_out) and izwi_decode_gqa_attention_f32 with
 * kv_len = pos + 1; out is `[num_heads, head_dim]`.  Results are those of the two calls bit for bit
 * (the same arithmetic in the same order).  Device pointers only; head_dim 64, 128 or 256. */
int izwi_decode_attention_step_f32(const float* q, const float* k, const float* v, const float* qk_weight,
                                   const float* cos_sin, int64_t num_heads, int64_t num_kv_heads,
                                   int64_t head_dim, float eps, float* k_cache, float* v_cache,
                                   int64_t kv_capacity, int64_t pos, float scale, float* out, void* stream);

/* `try_fused_decode_gqa_attention_with_kv_len(q, k, v, num_heads, num_kv_heads, head_dim, kv_len,
 * scale)` (kernels/mod.rs:199-225, metal.rs:2121-2193, shader metal.rs:307-381): attention of one
 * query token.  q is `[1, num_heads, 1, head_dim]`, k and v are `[1, num_kv_heads, kv_capacity,
 * head_dim]` (head-major cache) of which the first kv_len positions count; head h reads kv head
 * h / (num_heads / num_kv_heads); out is `[1, num_heads, 1, head_dim]`,
 * softmax_p((q . k_p) * scale) . v.  The reference's shader refuses kv_len > 2048; here the
 * positions are split over workgroups and merged (any kv_len).  head_dim must be 64, 128 or 256
 * (IZWI_QMM_ERR_UNSUPPORTED otherwise).  Uses the library's per-stream scratch when the positions
 * are split. */
int izwi_decode_gqa_attention_f32(const float* q, const float* k, const float* v, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t kv_len,
                                  int64_t kv_capacity, float scale, float* out, int mem_space,
                                  void* stream);

/* Greedy next token: `argmax(&logits)` after the LM head (qwen3/chat.rs:574-597,
 * qwen3/asr/mod.rs:2762-2789, i.e. `logits.argmax(D::Minus1)` as u32), on the device, so that four
 * bytes per row come back instead of the logits.  logits is `[rows, n]`, out `[rows]`: the first
 * index of the row's maximum (ties go to the smaller index, as a left-to-right scan keeps the
 * first; a NaN is never the maximum; a row of NaNs gives 0). */
int izwi_argmax_f32(const float* logits, int64_t rows, int64_t n, uint32_t* out, int mem_space, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* IZWI_DECODE_OPS_H */
