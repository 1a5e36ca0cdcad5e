/*
 * izwi_qmm — C ABI of the MI355X (gfx950) quantized linear-layer library.
 *
 * This is the drop-in boundary for the Candle `QMatMul` forward that
 * izwi-core's Qwen3-family decoders call for every projection and the LM head
 * (reference: crates/izwi-core/src/models/architectures/qwen3/core.rs:791-831).
 * Every entry point is plain C: pointers, sizes and integer codes; no C++ or
 * framework types cross it.  A Rust FFI crate (or cgo / ctypes) binds exactly
 * these symbols.
 *
 * Conventions
 *   - every function returns IZWI_QMM_OK (0) or a negative izwi_qmm_status;
 *     the message of the last failure on the calling thread is returned by
 *     izwi_qmm_last_error().  Shape and dtype mismatches are errors, never
 *     aborts (the reference maps them to Error::InferenceError,
 *     crates/izwi-core/src/error.rs:69-73).
 *   - weights are `[n, k]` row-major in GGUF block layout (blocks along k),
 *     ggml dtype ids as in GGUF: Q8_0 = 8, Q4_K = 12, Q6_K = 14.
 *   - `mem_space` says where the caller's buffers live: IZWI_QMM_DEVICE (HIP
 *     device pointers, the fast path, asynchronous on `stream`) or
 *     IZWI_QMM_HOST (ordinary host memory; the library stages it through
 *     pooled pinned buffers that it keeps for the life of the process, and
 *     the call is synchronous).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - all entry points may be called from several host threads at once; a
 *     weight handle is immutable after creation and may be shared by
 *     concurrent callers (the reference calls forward from several threads,
 *     engine/executor/dispatch.rs:150-204, backends/policy.rs:28-30).  Calls
 *     that need device scratch (m >= 3, split-k prefill, MoE, split attention)
 *     take their stream's scratch buffer for the duration of the call: two
 *     threads calling on the SAME stream (NULL included) are serialised while
 *     one of them queues its launches, and the stream then runs the two calls
 *     one after the other; calls on different streams neither wait nor share.
 *     The scratch of a stream only grows; an outgrown buffer stays allocated
 *     until the process ends (queued work and captured graphs may still
 *     address it).  It cannot grow while its stream is being captured into a
 *     HIP graph: such a call fails with IZWI_QMM_ERR_HIP; reserve beforehand
 *     (izwi_qmm_scratch_reserve, or one eager call of the same size).
 *   - there is no CPU fallback: without a usable HIP device every call fails
 *     with IZWI_QMM_ERR_NO_DEVICE.
 */
#ifndef IZWI_QMM_H
#define IZWI_QMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IZWI_QMM_ABI_VERSION 1

typedef enum izwi_qmm_status {
    IZWI_QMM_OK = 0,
    IZWI_QMM_ERR_INVALID = -1,     /* bad shape, size, dtype or NULL pointer */
    IZWI_QMM_ERR_UNSUPPORTED = -2, /* valid request this build cannot run */
    IZWI_QMM_ERR_HIP = -3,         /* a HIP runtime call failed */
    IZWI_QMM_ERR_NO_DEVICE = -4    /* no gfx950 device available */
} izwi_qmm_status;

/* ggml / GGUF tensor type ids (candle-core GgmlDType) */
#define IZWI_QMM_Q8_0 8
#define IZWI_QMM_Q4_K 12
#define IZWI_QMM_Q6_K 14

typedef enum izwi_qmm_mem_space { IZWI_QMM_DEVICE = 0, IZWI_QMM_HOST = 1 } izwi_qmm_mem_space;

/* element type of y in izwi_qmm_forward_bf16, of x and y in izwi_qmm_forward_fused */
typedef enum izwi_qmm_out_dtype { IZWI_QMM_OUT_F32 = 0, IZWI_QMM_OUT_BF16 = 1 } izwi_qmm_out_dtype;

typedef struct izwi_qmm_weight izwi_qmm_weight; /* opaque: QTensor + QMatMul */

typedef struct izwi_qmm_weight_info {
    int32_t ggml_dtype;
    int32_t n_stacked; /* 1 for a plain matrix, E for an expert stack */
    int64_t n;         /* output features (rows) */
    int64_t k;         /* input features (cols) */
    uint64_t nbytes;   /* GGUF block bytes of the whole handle */
    int32_t device;    /* HIP device ordinal the weights live on */
    int32_t reserved;
} izwi_qmm_weight_info;

/* Mirrors Qwen3RuntimeProfileSnapshot (qwen3/core.rs:571-582): the counters
 * `izwi bench` reads (crates/izwi-cli/src/commands/bench.rs:266-289).  Times
 * are host wall time around the call, synchronised on the stream when
 * profiling is enabled. */
typedef struct izwi_qmm_profile_snapshot {
    uint64_t qmatmul_calls;
    uint64_t qmatmul_ns;
    uint64_t qmatmul_input_casts;
    uint64_t qmatmul_input_cast_ns;
    uint64_t qmatmul_output_casts;
    uint64_t qmatmul_output_cast_ns;
    uint64_t lm_head_calls;
    uint64_t lm_head_ns;
    uint64_t silu_mul_fused_calls;
    uint64_t silu_mul_fallback_calls;
} izwi_qmm_profile_snapshot;

/* --- library ------------------------------------------------------------ */

int izwi_qmm_abi_version(void);

/* Selects and checks the HIP device (must be gfx950).  Optional: the first
 * weight_create calls it with the current device. */
int izwi_qmm_init(int device);

/* Thread-local message of the last failing call ("" if none). */
const char* izwi_qmm_last_error(void);

/* --- weights: QTensor / QMatMul construction ---------------------------- */

/* `quantized_storage_bytes(rows, cols, dtype)` (qwen3/core.rs:891-909):
 * rows*cols must divide by the block size; bytes = blocks * type_size. */
int izwi_qmm_storage_bytes(int ggml_dtype, int64_t rows, int64_t cols, uint64_t* out_bytes);

/* `QMatMul::from_arc(Arc<QTensor>)` as used by `Qwen3Projection::quantized`
 * (qwen3/core.rs:710-715): takes the tensor's raw GGUF block bytes
 * (`QTensor::data()`), validates `nbytes` with the rule above, copies them to
 * the device and re-tiles them for the kernels.  `k` must divide by the block
 * size (`QTensor::quantize` requirement). */
int izwi_qmm_weight_create(int ggml_dtype, int64_t n, int64_t k, const void* blocks,
                           uint64_t nbytes, int mem_space, izwi_qmm_weight** out);

/* `packed_qmatmul_from_qtensors` (qwen3/core.rs:846-889): row-concatenates
 * `n_parts` tensors of equal `k` and dtype into one `[sum(rows), k]` weight
 * (fused QKV / gate-up, qwen3/core.rs:992-1044,1179-1221).  Errors mirror the
 * reference: empty group, input (k) mismatch, byte-count mismatch. */
int izwi_qmm_weight_create_packed(int ggml_dtype, int32_t n_parts, const int64_t* part_rows,
                                  int64_t k, const void* const* part_blocks,
                                  const uint64_t* part_nbytes, int mem_space,
                                  izwi_qmm_weight** out);

/* Expert stack for the grouped MoE form: `n_experts` consecutive `[n, k]`
 * matrices in one buffer.  No counterpart in the reference (it has no MoE
 * code); the stacking matches how GGUF stores `ffn_*_exps` tensors. */
int izwi_qmm_weight_create_stacked(int ggml_dtype, int32_t n_experts, int64_t n, int64_t k,
                                   const void* blocks, uint64_t nbytes, int mem_space,
                                   izwi_qmm_weight** out);

/* `QTensor::quantize(&tensor, dtype)` (candle-core quantized/mod.rs; the reference's own use:
 * qwen3/core.rs:3112, where its packed-projection test builds Q8_0 tensors from f32 ones): the
 * GGUF block bytes of an f32 `[n, k]` matrix, rows contiguous, blocks along k — BlockQ8_0::from_float
 * (34 bytes per 32 values) or BlockQ4K::from_float (144 bytes per 256 values: the
 * `make_qkx1_quants(15, 5, ..)` search per sub-block, 6-bit scales and mins, nibble pairs), value
 * for value what the reference's CPU quantizer writes.  `out_blocks` receives
 * izwi_qmm_storage_bytes(dtype, n, k) bytes and is what izwi_qmm_weight_create takes.  Other
 * target types: IZWI_QMM_ERR_UNSUPPORTED. */
int izwi_qmm_quantize_weights_f32(int ggml_dtype, const float* w, int64_t n, int64_t k, void* out_blocks,
                                  int mem_space, void* stream);

/* Drop of the Arc<QTensor>. NULL is ignored. */
void izwi_qmm_weight_destroy(izwi_qmm_weight* w);

/* `QTensor::{dtype, shape}`. */
int izwi_qmm_weight_get_info(const izwi_qmm_weight* w, izwi_qmm_weight_info* out);

/* Arithmetic of the f32 / fused forward calls beyond 64 activation rows, process-wide (see
 * izwi_qmm_forward_f32).  No counterpart in the reference, whose CPU path has one arithmetic. */
typedef enum izwi_qmm_large_m { IZWI_QMM_LARGE_M_BF16 = 0, IZWI_QMM_LARGE_M_INT8 = 1 } izwi_qmm_large_m;
int izwi_qmm_set_large_m_arithmetic(int mode);
int izwi_qmm_get_large_m_arithmetic(void);

/* Form of the bf16 prefill product (more than 128 activation rows, Q4_K / Q8_0 weights, k a multiple
 * of 64), process-wide.  IZWI_QMM_PREFILL_LDS: the weights are dequantized to bf16 inside the matmul
 * kernel, tile by tile, on their way into LDS.  IZWI_QMM_PREFILL_PLANE: one pass per call dequantizes
 * the weight into a bf16 plane in the stream's scratch memory (2 bytes per weight element, see
 * izwi_qmm_scratch_reserve), and the matmul kernel streams both operands into LDS without touching
 * them.  IZWI_QMM_PREFILL_AUTO (the default): chosen by size - today the in-LDS form everywhere, which
 * is the faster one up to 4096 rows on the Qwen3-8B shapes.  IZWI_QMM_PREFILL_FORM=lds / plane at
 * start-up forces one.  Same bf16 operands and f32 accumulation in both; the sums may
 * differ in their last bits (order of the k steps inside a matrix instruction is the same, the split
 * of k over workgroups is not).  No counterpart in the reference. */
typedef enum izwi_qmm_prefill_form { IZWI_QMM_PREFILL_AUTO = -1, IZWI_QMM_PREFILL_LDS = 0, IZWI_QMM_PREFILL_PLANE = 1 } izwi_qmm_prefill_form;
int izwi_qmm_set_prefill_form(int form);
int izwi_qmm_get_prefill_form(void);

/* Form of the MoE expert MLP at many pairs per expert (16-row tiles on the matrix cores): 1 = the
 * expert form (a workgroup per expert and part of its rows keeps up to four activation tiles in LDS,
 * every wave walks weight panels on its own), 0 = the one-shot form (a workgroup per group of row
 * tiles, all panels requested at once), negative = chosen per call (the default: the expert form
 * wherever two activation tiles of an expert over all of k fit in LDS).  IZWI_QMM_MOE_EXPERT_FORM=1 / 0
 * at start-up forces one.  The integer block dots are the same; the two forms add the k panels of
 * a row in a different order, so results can differ in the last bits of the f32 sums.
 * In the expert form every activation row is quantized once, on its own (the token rows inside the
 * routing kernel), and a workgroup puts its tiles together from the rows' records; 2 = the expert
 * form on records quantized tile by tile through the sort's tables, as the one-shot form reads them
 * (kept for comparison: the same bits as 1, one more launch and an index chain per tile).
 * No counterpart in the reference (it has no MoE code). */
int izwi_qmm_set_moe_expert_form(int enabled);

/* Grows the scratch buffer of (current device, stream) to at least `bytes` now, so that later
 * calls on that stream allocate nothing (needed before the stream is captured into a HIP graph).
 * No counterpart in the reference. */
int izwi_qmm_scratch_reserve(uint64_t bytes, void* stream);

/* `QTensor::data()` (qwen3/core.rs:855,870): the original GGUF block bytes,
 * byte-identical to what weight_create was given. */
int izwi_qmm_weight_data(const izwi_qmm_weight* w, void* out_blocks, uint64_t nbytes,
                         int mem_space, void* stream);

/* `QTensor::dequantize` (shared/weights/gguf.rs:127-143): f32 `[n_stacked*n, k]`,
 * bit-identical to candle-core's `to_float`. */
int izwi_qmm_dequantize_f32(const izwi_qmm_weight* w, float* out, int mem_space, void* stream);

/* The embedding lookup: `Qwen3Model::embeddings` = `Embedding::forward(input_ids)` (qwen3/core.rs:2083-2085)
 * on the table that `GgufLoader::load_tensor` dequantizes and casts to the model dtype
 * (qwen3/core.rs:2000-2007, shared/weights/gguf.rs:127-143): out[i, :] = row row_ids[i] of
 * izwi_qmm_dequantize_f32's matrix (first matrix of the handle), value for value, as f32 or rounded to
 * bf16 (izwi_qmm_out_dtype) - without the dense [vocab, hidden] table in memory.  `row_ids` may be host
 * or device memory (the id the device argmax left); host ids outside [0, n) are refused as the
 * reference's index_select refuses them, device ids are not read by the host: such a row comes back
 * as zeros.  out is `[n_rows, k]`. */
int izwi_qmm_dequantize_rows(const izwi_qmm_weight* w, const int32_t* row_ids, int64_t n_rows, int ids_mem_space,
                             void* out, int out_dtype, int out_mem_space, void* stream);

/* --- forward: QMatMul::forward ------------------------------------------ */

/* `QMatMul::forward(x)` for f32 activations (qwen3/core.rs:812; the reference
 * always hands f32 to the op on accelerators, qwen3/core.rs:772-789).
 * x is `[m, k]` row-major contiguous, y is `[m, n]`.  Any m >= 0.
 * m <= 64: activations are quantized on chip to the weight type's dot type
 * exactly as candle-core does (Q8_0 -> Q8_0 blocks, Q4_K and Q6_K -> Q8_K
 * blocks) and multiplied as integers, so results agree with the reference's
 * CPU path up to f32 summation order (about 1e-6 of max|y|).
 * m > 64 (prefill sizes) is ANOTHER arithmetic by default: x is rounded to
 * bf16, the weights are dequantized to bf16, products run on the bf16 matrix
 * cores with f32 accumulation; the result differs from the reference's by up
 * to about 5e-3 of max|y| (the reference's own int8 activation rounding is
 * of that size; the stated bound is 1e-2).  A caller that wants the
 * reference's arithmetic at every m selects it with
 * izwi_qmm_set_large_m_arithmetic(IZWI_QMM_LARGE_M_INT8) or the environment
 * variable IZWI_QMM_LARGE_M=int8: rows then run 64 at a time through the
 * integer kernel (slower at prefill sizes: the weights are streamed once per
 * 64 rows).  izwi_qmm_forward_group_f32, izwi_qmm_forward_gate_up_silu_f32,
 * izwi_qmm_forward_fused and the *_normed_* calls follow the same rule. */
int izwi_qmm_forward_f32(const izwi_qmm_weight* w, const float* x, int64_t m, float* y,
                         int mem_space, void* stream);

/* `Qwen3Projection::logits_for_tokens` / `Qwen3Model::logits_from_hidden_for_tokens`, quantized
 * arm (qwen3/core.rs:745-758, 2125-2131, 2155-2171): the reference computes the full LM head and
 * then `index_select`s the wanted token ids.  Weight rows are independent, so this call reads only
 * the 16-row tiles that hold a selected row (36 KB per token id at k = 4096 Q4_K instead of the
 * 350 MB of a 151936-row head):
 *     y[i, j] = forward_f32(x)[i, row_ids[j]]        y is [m, n_rows], row-major
 * bit for bit (the same kernel with the same split along k, over a list of row-tiles).  The
 * reference accepts one hidden state ([1, vocab] or [1, 1, vocab] logits); m = 1 or 2 here,
 * IZWI_QMM_ERR_UNSUPPORTED beyond.  row_ids may repeat and need not be sorted; with host pointers
 * an id >= n is IZWI_QMM_ERR_INVALID (as `index_select` refuses it), with device pointers (no host
 * round trip) its outputs are NaN. */
int izwi_qmm_forward_rows_f32(const izwi_qmm_weight* w, const uint32_t* row_ids, int64_t n_rows, const float* x,
                              int64_t m, float* y, int mem_space, void* stream);

/* --- activation records: quantized activations handed over by their producer ---------- */

/* For 3 <= m <= 64 rows (5 <= m <= 64 where k <= 3072: three and four rows of a short k stay on the
 * single-launch kernel, four rows per pass) izwi_qmm_forward_f32 is two launches: the activation quantizer (candle-core's
 * `BlockQ8_0::from_float` / `BlockQ8K::from_float` per row, qwen3 call site core.rs:812) writes
 * "records" into scratch, the matrix-core kernel multiplies them.  The kernel that PRODUCES the
 * activations can write the records itself and save that launch on the token's critical path:
 *   izwi_rms_norm_quantize_records_f32 (izwi_decode_ops.h)   input / post-attention RMSNorm -> q|k|v, gate|up
 *   izwi_qmm_silu_mul_quantize_records_f32                    silu(gate) * up              -> down
 *   izwi_qmm_quantize_records_f32                             any other f32 activations    (the plain quantizer)
 * and izwi_qmm_forward_group_records_f32 is izwi_qmm_forward_group_f32 on such records: results
 * are bit-identical to the calls on the f32 activations at the row counts named above (for fewer rows
 * the call on f32 activations runs the single-launch kernel: the same integer block dots, the f32
 * sums in another order).  Records are opaque device memory of
 * izwi_qmm_records_bytes(weight dtype, m, k) bytes, 16-byte aligned, valid for weights whose dot
 * type matches (Q8_0 weights: Q8_0 records; Q4_K and Q6_K weights: the same Q8_K records).
 * Device pointers only.  No counterpart in the reference, whose CPU matmul quantizes inside the op. */
uint64_t izwi_qmm_records_bytes(int ggml_weight_dtype, int64_t m, int64_t k);
int izwi_qmm_quantize_records_f32(int ggml_weight_dtype, const float* x, int64_t m, int64_t k, void* records,
                                  void* stream);
/* records of silu(gate[i]) * up[i] (`Qwen3Mlp::forward`, qwen3/core.rs:1786-1796), gate and up [m, k] */
int izwi_qmm_silu_mul_quantize_records_f32(int ggml_weight_dtype, const float* gate, const float* up, int64_t m,
                                           int64_t k, void* records, void* stream);
int izwi_qmm_forward_group_records_f32(const izwi_qmm_weight* const* weights, int32_t n_weights, const void* records,
                                       int64_t m, float* const* ys, void* stream);

/* --- chained decode: the projections of one token as one launch ----------- */

/* EXPERIMENTAL, and SLOWER than the separate calls it replaces (1.44 against 1.01 ms per Qwen3-8B token,
 * see the end of this comment): kept as the measured alternative for callers whose constraint is the
 * number of launches, not time.  The interface may change or go.  Restrictions that follow from its
 * design (one resident workgroup per compute unit, steps handed over through counters in memory):
 *  - single stream, not re-entrant: a chain owns one set of counters and one error word; running the
 *    same chain on two streams, or twice at the same time, corrupts both runs and nothing detects it;
 *  - nothing else may run on the GPU beside it (it needs every compute unit for the whole launch);
 *  - once a wait inside a run has given up, the error word stays set: every later run or graph replay
 *    leaves all its waits at once and writes invalid results until izwi_qmm_chain_status has been
 *    called (it reports the failure and clears the word).  Call it after every token you care about.
 *
 * One token's projections in the order `Qwen3Layer::forward` issues them (qwen3/core.rs:1863-1881:
 * q|k|v, o, gate|up, down, layer after layer; `Qwen3Model::logits_from_hidden`, core.rs:2114-2125,
 * at the end) depend on each other: each reads activations that an earlier one (or the attention /
 * activation kernel between them) wrote.  As separate calls every one of them pays the gap
 * between two dependent launches and its own ramp-up and drain.  A chain is that list of calls
 * prepared once and run as ONE kernel launch per token; step i does not read its x before step
 * i - 1 has completed (exactly the order a stream gives the separate calls), and the weights of
 * the next step are requested while the current step finishes.
 *
 * A step is izwi_qmm_forward_group_f32 at m = 1: 1..4 weights of equal k, one x [k], one y [n_i]
 * per weight; results are bit-identical to that call.  All buffers are device memory and must
 * stay valid, at the same addresses, for the life of the chain; the weights of a chain share one
 * block type and the current device; k <= 12288 (12 panels of 1024) and n < 256 * (compute units)
 * (an LM head runs as a call of its own behind the chain).  The launch occupies every
 * compute unit with one resident workgroup: run nothing else beside it.  Waits inside the kernel
 * are bounded: if one gives up (another kernel held the GPU for about a second), the results of that
 * run are invalid, every workgroup still exits, and izwi_qmm_chain_status returns IZWI_QMM_ERR_HIP
 * (and makes the chain usable again).  izwi_qmm_chain_run is asynchronous on `stream`, allocates
 * nothing and may be captured into a HIP graph; one chain must not run twice at the same time.
 * Measured on MI355X (Qwen3-8B, Q4_K, 144 steps): 1.44 ms per token against 1.01 ms for the same
 * steps as separate calls in a HIP graph: a grid-wide hand-over through memory (write-through
 * stores, counters, device-scope loads) costs about 7 us per dependent step where a kernel
 * boundary costs about 3.5, and the overlap of the next step's weight stream does not make up for
 * it.  The separate calls stay the fast path; the chain is kept as the measured alternative.
 * No counterpart in the reference, which issues one Candle op per projection. */
typedef struct izwi_qmm_chain izwi_qmm_chain;
typedef struct izwi_qmm_chain_step {
    const izwi_qmm_weight* weights[4];
    int32_t n_weights;
    int32_t reserved;
    const float* x; /* device, [k] */
    float* ys[4];   /* device, [n_i] */
} izwi_qmm_chain_step;
int izwi_qmm_chain_create(const izwi_qmm_chain_step* steps, int32_t n_steps, izwi_qmm_chain** out);
void izwi_qmm_chain_destroy(izwi_qmm_chain* chain);
int izwi_qmm_chain_run(izwi_qmm_chain* chain, void* stream);
/* Waits for `stream`, then reports whether a wait inside any run since the last status call gave up. */
int izwi_qmm_chain_status(izwi_qmm_chain* chain, void* stream);
/* Polls (about 0.5 us each) after which a wait gives up; default 2^21, also IZWI_QMM_CHAIN_SPIN_LIMIT.
 * 0 makes every wait that is not already satisfied give up at once (for tests of the error path). */
int izwi_qmm_chain_set_spin_limit(izwi_qmm_chain* chain, uint32_t polls);

/* izwi_qmm_forward_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same kernels and the same results, bit for bit, as izwi_qmm_forward_f32 with
 * IZWI_QMM_DEVICE pointers; the quantized activation records of the batched kernels (from three rows on,
 * from five where k <= 3072)
 * live in a static device array of IZWI_QMM_NOALLOC_SCRATCH_BYTES inside the library's image
 * (each GPU the library runs on holds its own copy until the process ends) instead of the
 * per-stream scratch buffer, and the call performs no hipMalloc / hipFree whatever its size.
 * Limits: x and y are device pointers; the weight's device must be the current device; m <= 64;
 * ceil(m / 16) * (k / 256) records of 4416 (Q4_K, Q6_K) or 4608 (Q8_0) bytes must fit the array
 * (k = 12288 at m = 64 does: 884,736 bytes), otherwise IZWI_QMM_ERR_UNSUPPORTED.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (other
 * streams, other threads) race on it; calls on one stream are ordered and safe.  The array keeps
 * the previous call's contents; each call rewrites every record it reads. */
#define IZWI_QMM_NOALLOC_SCRATCH_BYTES 1048576
int izwi_qmm_forward_f32_noalloc(const izwi_qmm_weight* w, const float* x, int64_t m, float* y, void* stream);

/* `Qwen3QkvProjection::forward` and `Qwen3GateUpProjection::forward`, `Separate` arms
 * (qwen3/core.rs:1119-1127, 1274-1282): several projections applied to the same
 * activations, y_i = QMatMul_i.forward(x), bit-identical to n_weights calls of
 * izwi_qmm_forward_f32 up to 128 rows (beyond, in the bf16 matrix-core arithmetic, equal up to the
 * f32 summation order: the shared launch may split k differently).  The weights must share k; with equal block types the decode
 * sizes run as one kernel launch (m <= 2; m <= 4 where k <= 3072) or as one activation quantization and one
 * matmul launch (m <= 64), prefill sizes (m > 128, bf16 matrix-core arithmetic) share one conversion of x
 * and one launch; members of several block types (attn_q / attn_k in Q4_K beside attn_v in
 * Q6_K, as Q4_K_M files have them) are grouped by type, one such launch per type.
 * n_weights <= 4. */
int izwi_qmm_forward_group_f32(const izwi_qmm_weight* const* weights, int32_t n_weights,
                               const float* x, int64_t m, float* const* ys, int mem_space,
                               void* stream);

/* izwi_qmm_forward_group_f32 for bf16 activations (prefill): y_i = izwi_qmm_forward_bf16(weights[i], x)
 * for 1..4 weights of equal k on the same x, `out_dtype` f32 or bf16 for every y_i.  With equal block
 * types, device pointers and m > 128 the members run as ONE launch of the bf16 matrix-core kernel
 * (its grid is the members' column tiles one after the other, planned as one matrix): k / v
 * (n = 1024) no longer run alone on a quarter of the chip.  Results are those of the separate calls
 * up to f32 summation order (the tile plan may split k differently). */
int izwi_qmm_forward_group_bf16(const izwi_qmm_weight* const* weights, int32_t n_weights, const uint16_t* x_bf16,
                                int64_t m, void* const* ys, int out_dtype, int mem_space, void* stream);

/* The gate / up pair of `Qwen3Mlp::forward` (qwen3/core.rs:1786-1798) with its activation:
 *     h[m, n] = silu(gate.forward(x)) * up.forward(x)
 * i.e. `gate_up_proj.forward(x)` followed by `try_fused_silu_mul` (kernels/mod.rs:94-108) or
 * `ops::silu(&gate)?.broadcast_mul(&up)` in one call.  `gate` and `up` are [n, k] weights of the
 * same shape and type.  The two sums are those of izwi_qmm_forward_f32 bit for bit; silu(v) =
 * v / (1 + exp(-v)) in f32.  For m <= 2 the product is applied inside the decode kernel (one
 * launch, h is the only output written); for larger m the two projections run as a projection
 * group into scratch and one elementwise kernel follows.  Counted in
 * `silu_mul_fused_calls` of the profile snapshot. */
int izwi_qmm_forward_gate_up_silu_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                                      const float* x, int64_t m, float* h, int mem_space,
                                      void* stream);

/* `Qwen3Mlp::forward` (qwen3/core.rs:1786-1798) as one call:
 *     y[m, hidden] = down.forward( silu(gate.forward(x)) * up.forward(x) )
 * `gate` and `up` are [intermediate, hidden] weights of the same shape, `down` is
 * [hidden, intermediate]; any of the built block types.  The results are those of
 * izwi_qmm_forward_gate_up_silu_f32 followed by izwi_qmm_forward_f32, bit for bit.  What the call
 * adds is the route between the three projections: for 3 <= m <= 64 (5 <= m where hidden or
 * intermediate is at most 3072; gate and up of one block type) x is quantized once, gate | up run as one launch on its records, silu(g) * u is quantized
 * straight into the records that `down` multiplies (four launches; the separate calls take five
 * and write and read the intermediate as an f32 matrix); other sizes run the two calls with the
 * intermediate in the stream's scratch. */
int izwi_qmm_mlp_forward_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up, const izwi_qmm_weight* down,
                             const float* x, int64_t m, float* y, int mem_space, void* stream);

/* Prefill form: bf16 activations `[m, k]`, weights dequantized to bf16 in LDS,
 * MFMA with f32 accumulation; y is f32 or bf16 per `out_dtype`.  Replaces the
 * to_dtype(F32) -> QMatMul -> to_dtype(activation dtype) sequence of
 * qwen3/core.rs:798-828 with one kernel. */
int izwi_qmm_forward_bf16(const izwi_qmm_weight* w, const uint16_t* x_bf16, int64_t m, void* y,
                          int out_dtype, int mem_space, void* stream);

/* `Qwen3Projection::forward`, `Quantized` arm (qwen3/core.rs:795-829), with the residual add of
 * `Qwen3Layer::forward` (qwen3/core.rs:1875, 1879) folded in: the cast of the activations to f32,
 * the product, the cast of the result back to the activation type and `x.broadcast_add(&out)` as
 * ONE call whose kernels read x in its own type and store y once.
 *   x: `[m, k]` of x_dtype; y: `[m, n]` of y_dtype (izwi_qmm_out_dtype values: f32 = 0, bf16 = 1);
 *   residual: `[m, n]` of y_dtype or NULL; it may be y itself (each element is read before it is
 *   written by the same thread).
 * The sums are those of izwi_qmm_forward_f32 on the widened activations, bit for bit, for m <= 64
 * (bf16 -> f32 is exact), those of izwi_qmm_forward_bf16 beyond; y = sum + residual is rounded
 * once (the reference rounds the product to the activation type first and the sum again).  The
 * profile snapshot counts the folded casts (`qmatmul_input_casts` for bf16 x, `qmatmul_output_casts`
 * for bf16 y); their time is inside `qmatmul_ns`, the `_cast_ns` fields stay 0. */
int izwi_qmm_forward_fused(const izwi_qmm_weight* w, const void* x, int x_dtype, int64_t m,
                           const void* residual, void* y, int y_dtype, int mem_space, void* stream);

/* The RMSNorm that precedes a projection folded into the projection's call:
 * `Qwen3Layer::forward`'s `input_layernorm.forward(x)` before the q/k/v projections and
 * `post_attention_layernorm.forward(&x)` before gate/up (qwen3/core.rs:1872, 1877), and the final
 * norm before the LM head.  y_i = QMatMul_i.forward(rms_norm(x, norm_weight, eps)) with
 * rms_norm(x) = x * rsqrt(mean(x^2) + eps) * norm_weight (the reference's `try_fused_rms_norm`),
 * norm_weight `[k]` f32.  For m <= 2 on device buffers this is ONE launch: the decode kernel, whose
 * workgroups read all of x anyway, quantizes x * norm_weight, sums the squares on the side and
 * multiplies the finished sums by the row's rsqrt (the activation quantizers are invariant under
 * a positive scale of their input: the quants stay, the block scale moves).  Against the two
 * separate calls the results differ by f32 rounding for Q4_K / Q6_K weights (a quant on a rounding
 * tie may move by one); for Q8_0 weights, whose activation blocks carry an f16 scale, that scale is
 * rounded before the row's factor is applied instead of after: up to 2^-11 per block, the size of
 * the rounding the format has anyway.  Other sizes and memory spaces run the norm into scratch and
 * the plain call after it. */
int izwi_qmm_forward_normed_f32(const izwi_qmm_weight* w, const float* x, int64_t m, const float* norm_weight,
                                float eps, float* y, int mem_space, void* stream);
int izwi_qmm_forward_group_normed_f32(const izwi_qmm_weight* const* weights, int32_t n_weights, const float* x,
                                      int64_t m, const float* norm_weight, float eps, float* const* ys,
                                      int mem_space, void* stream);
int izwi_qmm_forward_gate_up_silu_normed_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                                             const float* x, int64_t m, const float* norm_weight, float eps,
                                             float* h, int mem_space, void* stream);

/* `T::VecDotType::from_float` per row (candle-core k_quants.rs `matmul`):
 * the activation blocks the decode kernel builds on chip, written out in the
 * reference's block layout (BlockQ8_0, 34 B per 32 values, for Q8_0 weights;
 * BlockQ8K, 292 B per 256 values, for Q4_K weights).  Exported so that the
 * on-chip quantizer can be checked bit for bit. */
int izwi_qmm_quantize_activations(int ggml_weight_dtype, const float* x, int64_t m, int64_t k,
                                  void* out_blocks, int mem_space, void* stream);

/* --- expert-grouped MoE form (no counterpart in the reference) ----------- */

/* Router: per token the top_k largest logits (ties: lower expert index), slots
 * in descending-logit order; weights = softmax restricted to the selected
 * slots (== renormalised softmax).  logits `[t, n_experts]`, ids/weights
 * `[t, top_k]`.  ids are bit-exact by construction. */
int izwi_moe_route(const float* logits, int64_t t, int32_t n_experts, int32_t top_k,
                   int32_t* ids, float* weights, int mem_space, void* stream);

/* Stable counting sort of the t*top_k (token, slot) pairs by expert id:
 * perm `[t*top_k]` lists pair indices grouped by expert (ascending pair index
 * inside a group), offsets `[n_experts+1]` is the exclusive prefix sum of the
 * per-expert counts. */
int izwi_moe_sort(const int32_t* ids, int64_t t, int32_t top_k, int32_t n_experts, int32_t* perm,
                  int32_t* offsets, int mem_space, void* stream);

/* Grouped expert MLP: for every pair p = (token, slot) with expert e:
 *   h = silu(W_gate[e] x_token) * (W_up[e] x_token),  y_p = W_down[e] h
 * (each matmul with QMatMul semantics), then out[token] = sum_slot w * y_p in
 * slot order.  gate/up are stacks of `[inter, hidden]`, down of
 * `[hidden, inter]`; x `[t, hidden]`, out `[t, hidden]`, all f32. */
int izwi_moe_forward_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                         const izwi_qmm_weight* down, const float* x, int64_t t,
                         const int32_t* ids, const float* weights, int32_t top_k,
                         const int32_t* perm, const int32_t* offsets, float* out, int mem_space,
                         void* stream);

/* One MoE layer in one call: izwi_moe_route, izwi_moe_sort and izwi_moe_forward_f32 composed
 * (same results bit for bit).  logits `[t, n_experts]`, x and out `[t, hidden]`; ids_out /
 * weights_out `[t, top_k]` receive the routing if not NULL.  Up to 1024 (token, slot) pairs and
 * 256 experts, routing, sort and the kernel's segment tables are one launch (the layer is then 4
 * launches instead of 8); up to 64 pairs (8 tokens at top-8) with an expert intermediate size up to
 * 1024 the layer is TWO launches: every workgroup of the gate / up launch routes its own token, the
 * down launch adds the slots in order (IZWI_QMM_MOE_SMALL_MAX_PAIRS changes the bound, 0 = never). */
int izwi_moe_layer_f32(const izwi_qmm_weight* gate, const izwi_qmm_weight* up,
                       const izwi_qmm_weight* down, const float* logits, const float* x, int64_t t,
                       int32_t top_k, float* out, int32_t* ids_out, float* weights_out,
                       int mem_space, void* stream);

/* --- profiling counters (IZWI_QWEN3_PROFILE, qwen3/core.rs:624-657) ------ */

/* Enabled by izwi_qmm_profile_enable(1) or the IZWI_QWEN3_PROFILE env toggle.
 * `is_lm_head` calls are additionally counted in lm_head_* when the caller
 * marks the handle with izwi_qmm_weight_set_lm_head. */
int izwi_qmm_profile_enable(int enabled);
int izwi_qmm_profile_enabled(void); /* `qwen3_runtime_profiling_enabled` (qwen3/core.rs:624-640): 1 or 0 */
int izwi_qmm_profile_snapshot_get(izwi_qmm_profile_snapshot* out);
int izwi_qmm_profile_reset(void);
/* `argmax_calls` / `argmax_ms` of the ASR profile diagnostics `izwi bench` prints
 * (qwen3/asr/mod.rs:116-131, crates/izwi-cli/src/commands/bench.rs:281-295): calls of
 * izwi_argmax_f32 and their wall time in ns while profiling is enabled. */
int izwi_qmm_profile_argmax_get(uint64_t* calls, uint64_t* ns);
int izwi_qmm_weight_set_lm_head(izwi_qmm_weight* w, int is_lm_head);

#ifdef __cplusplus
}
#endif
#endif /* IZWI_QMM_H */
