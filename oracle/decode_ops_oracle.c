/*
 * CPU oracle for the decode-step neighbours of the quantized projections (TEST
 * INFRASTRUCTURE ONLY; nothing in the product library may link, import or call this file).
 *
 * Plain-C restatement of the f32 arithmetic of the reference's fused kernels, i.e. of the
 * Metal shader source it ships in crates/izwi-core/src/kernels/metal.rs (the hooks
 * `try_fused_rms_norm`, `try_fused_qk_rms_norm`, `try_fused_rope_pair_bshd`,
 * `try_fused_decode_gqa_attention_with_kv_len`, kernels/mod.rs:109-225).  The shaders reduce
 * with a tree over a threadgroup; here the sums run left to right in f32, which the
 * reference's own tests allow for (they compare the shaders with Candle's eager operators
 * within 1e-5, metal.rs:2917-3290).
 *
 * Pin status: each function is checked in tests/test_oracle_decode_ops.py against the input
 * vectors of the reference's tests (metal.rs:2921-2937, 2970-2999, 3079-3110, 3153-3181,
 * 3203-3226) with expected values from the closed-form definitions evaluated in f64, and
 * against an independent numpy restatement on random inputs.
 *
 * Compile with -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

/* metal.rs:147-186 (`izwi_rms_norm_f32`): y = x * rsqrt(mean(x^2) + eps) * weight, evaluated as
 * (x * scale) * weight. */
void oracle_rms_norm(const float* x, const float* weight, int64_t rows, int64_t hidden, float eps, float* y) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        float sum = 0.0f;
        for (int64_t i = 0; i < hidden; i++) sum += xr[i] * xr[i];
        const float scale = 1.0f / sqrtf(sum / (float)hidden + eps);
        for (int64_t i = 0; i < hidden; i++) y[r * hidden + i] = xr[i] * scale * weight[i];
    }
}

/* metal.rs:59-101 (`izwi_qk_rms_norm_f32`): rows of q, then rows of k, each normalized over
 * head_dim; q rows use weights[0 .. head_dim), k rows weights[head_dim .. 2 head_dim).  The
 * shader writes one [q_rows + k_rows, head_dim] buffer that the wrapper splits
 * (metal.rs:1959-1969). */
void oracle_qk_rms_norm(const float* q, const float* k, const float* qk_weight, int64_t q_rows, int64_t k_rows,
                        int64_t head_dim, float eps, float* q_out, float* k_out) {
    oracle_rms_norm(q, qk_weight, q_rows, head_dim, eps, q_out);
    oracle_rms_norm(k, qk_weight + head_dim, k_rows, head_dim, eps, k_out);
}

/* metal.rs:227-265 (`izwi_rope_pair_bshd_f32`): q is [batch, seq, q_heads, head_dim], k is
 * [batch, seq, k_heads, head_dim], cos_sin is [seq, head_dim] with the cosines in the first half
 * of a row and the sines in the second.  Row r of a tensor has position (r / heads) % seq; the
 * two halves of a row rotate against each other:
 *   out[d]        = x[d] * cos[d] - x[half + d] * sin[d]
 *   out[half + d] = x[d] * sin[d] + x[half + d] * cos[d] */
static void rope_rows(const float* x, const float* cos_sin, int64_t rows, int64_t seq, int64_t heads,
                      int64_t head_dim, float* out) {
    const int64_t half = head_dim / 2;
    for (int64_t r = 0; r < rows; r++) {
        const int64_t pos = (r / heads) % seq;
        const float* cs = cos_sin + pos * head_dim;
        const float* xr = x + r * head_dim;
        for (int64_t d = 0; d < half; d++) {
            const float x1 = xr[d], x2 = xr[half + d];
            out[r * head_dim + d] = x1 * cs[d] - x2 * cs[half + d];
            out[r * head_dim + half + d] = x1 * cs[half + d] + x2 * cs[d];
        }
    }
}

void oracle_rope_pair_bshd(const float* q, const float* k, const float* cos_sin, int64_t batch, int64_t seq,
                           int64_t q_heads, int64_t k_heads, int64_t head_dim, float* q_out, float* k_out) {
    rope_rows(q, cos_sin, batch * seq * q_heads, seq, q_heads, head_dim, q_out);
    rope_rows(k, cos_sin, batch * seq * k_heads, seq, k_heads, head_dim, k_out);
}

/* metal.rs:307-381 (`izwi_decode_gqa_attention_f32`): one query token; q is [heads, head_dim],
 * k and v are [kv_heads, kv_capacity, head_dim] of which the first kv_len positions count.
 * Head h reads kv head h / (heads / kv_heads); score = (q . k) * scale, softmax over the
 * positions with the maximum subtracted, out = sum_p (e_p * (1 / sum e)) * v_p.  (The shader
 * refuses kv_len > 2048, a limit of its threadgroup memory; the arithmetic has no such limit.) */
int oracle_decode_gqa_attention(const float* q, const float* k, const float* v, int64_t heads, int64_t kv_heads,
                                int64_t head_dim, int64_t kv_len, int64_t kv_capacity, float scale, float* out) {
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || kv_len <= 0 || kv_len > kv_capacity) return -1;
    const int64_t group = heads / kv_heads;
    float* scores = (float*)malloc((size_t)kv_len * sizeof(float));
    for (int64_t h = 0; h < heads; h++) {
        const int64_t kvh = h / group;
        float max_score = -INFINITY;
        for (int64_t p = 0; p < kv_len; p++) {
            const float* kr = k + (kvh * kv_capacity + p) * head_dim;
            float dot = 0.0f;
            for (int64_t d = 0; d < head_dim; d++) dot += q[h * head_dim + d] * kr[d];
            scores[p] = dot * scale;
            if (scores[p] > max_score) max_score = scores[p];
        }
        float sum = 0.0f;
        for (int64_t p = 0; p < kv_len; p++) {
            scores[p] = expf(scores[p] - max_score);
            sum += scores[p];
        }
        const float inv_sum = 1.0f / sum;
        for (int64_t d = 0; d < head_dim; d++) {
            float acc = 0.0f;
            for (int64_t p = 0; p < kv_len; p++) acc += (scores[p] * inv_sum) * v[(kvh * kv_capacity + p) * head_dim + d];
            out[h * head_dim + d] = acc;
        }
    }
    free(scores);
    return 0;
}

/* `logits.argmax(D::Minus1)` of the reference's greedy samplers (qwen3/chat.rs:592,
 * qwen3/asr/mod.rs:2780; the reduction itself is candle-core's, not shipped): a left-to-right scan
 * that replaces the running maximum only by a strictly larger value, i.e. the first index of the
 * maximum.  Pinned by numpy.argmax (same definition); "parity unpinned" against the crate's own
 * tie and NaN behaviour, which no test of the reference exercises. */
void oracle_argmax(const float* x, int64_t rows, int64_t n, uint32_t* out) {
    for (int64_t r = 0; r < rows; r++) {
        const float* row = x + r * n;
        int64_t best = -1;
        for (int64_t i = 0; i < n; i++) {
            if (row[i] != row[i]) continue;
            if (best < 0 || row[i] > row[best]) best = i;
        }
        out[r] = best < 0 ? 0u : (uint32_t)best;
    }
}
