// Internal interfaces between the C ABI (qmm_api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <exception>
#include <new>

#include "qmm_layout.h"

// ---- device helpers --------------------------------------------------------
#if defined(__HIPCC__)

__device__ __forceinline__ float qmm_f16_bits_to_f32(uint16_t bits) {
    union {
        uint16_t u;
        _Float16 h;
    } c;
    c.u = bits;
    return (float)c.h; // exact
}

__device__ __forceinline__ uint16_t qmm_f32_to_f16_bits(float f) {
    union {
        uint16_t u;
        _Float16 h;
    } c;
    c.h = (_Float16)f; // round to nearest even, as half::f16::from_f32
    return c.u;
}

// The 12 scale bytes of a Q4_K block (three little-endian dwords) -> packed
// 6-bit scales and mins: byte j of sc_lo/sc_hi is scale j / j+4, same for mins.
__device__ __forceinline__ void qmm_unpack_q4k_scales(uint32_t u0, uint32_t u1, uint32_t u2,
                                                      uint32_t& sc_lo, uint32_t& sc_hi,
                                                      uint32_t& mn_lo, uint32_t& mn_hi) {
    sc_lo = u0 & 0x3f3f3f3fu;
    mn_lo = u1 & 0x3f3f3f3fu;
    sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
}

__device__ __forceinline__ uint32_t qmm_byte_of(uint32_t lo, uint32_t hi, int j) {
    return ((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xffu;
}

// The activation quantizers' `round` (Rust f32::round / C roundf: halves away from zero) and clamp
// as three instructions: the truncation of v + copysign(0.5 - 2^-25, v), the float just below a
// half.  For every float of magnitude below 2^22 that is roundf(v) exactly (tests/test_round_identity.py
// checks every float up to 512: where v + 0.5 would round a value just below a half up to the next
// integer, this sum stays below it, and an exact half still reaches the integer because the sum's
// tie rounds to even); beyond the clamp nothing changes.  NaN gives 0.
__device__ __forceinline__ int qmm_round_clamp_i8(float v) {
    const float half_below = __uint_as_float(0x3effffffu | (__float_as_uint(v) & 0x80000000u));
    const int q = (int)__fadd_rn(v, half_below);
    return min(max(q, -128), 127);
}
// The low bytes of four ints as one dword (a, b, c, d from the lowest byte up).
__device__ __forceinline__ uint32_t qmm_pack_i8x4(int a, int b, int c, int d) {
    const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

__device__ __forceinline__ float qmm_bf16_bits_to_f32(uint16_t b) {
    return __uint_as_float((uint32_t)b << 16);
}

// round to nearest even, NaN kept quiet
__device__ __forceinline__ uint16_t qmm_f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

#endif // __HIPCC__

// What a projection call folds into its kernels besides the product: the activations may be
// bf16 (widened to f32 exactly on load), the result may get a residual of the output's type
// added and may be stored as bf16 (one rounding, of sum + residual).  residual may alias y.
struct QmmIo {
    int x_bf16;
    const void* residual;
    int y_bf16;
};
struct QmmEpilogue {
    const void* residual;
    int y_bf16;
};
// RMSNorm folded into a decode kernel (m <= 2): the kernel reads x, multiplies by weight[k] and
// applies rsqrt(mean(x^2) + eps) to the finished sums (the activation quantizers are invariant
// under a positive scale of their input).
struct QmmNorm {
    const float* weight;
    float eps;
};

#if defined(__HIPCC__)
__device__ __forceinline__ void qmm_store(void* y, const QmmEpilogue& ep, int64_t idx, float v) {
    if (ep.y_bf16) {
        if (ep.residual) v += qmm_bf16_bits_to_f32(static_cast<const uint16_t*>(ep.residual)[idx]);
        static_cast<uint16_t*>(y)[idx] = qmm_f32_to_bf16_bits(v);
    } else {
        if (ep.residual) v += static_cast<const float*>(ep.residual)[idx];
        static_cast<float*>(y)[idx] = v;
    }
}
#endif

#define QMM_ERR_HIP_CODE (-3) /* IZWI_QMM_ERR_HIP (checked by a static_assert in qmm_api.hip) */
// Records the calling thread's error message (read with izwi_qmm_last_error) and returns `code`.
int qmm_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// No C++ exception may cross the C boundary (the entry points use std::vector, std::unordered_map,
// std::string and new): every exported function with a status result runs its body through this.
// The status is IZWI_QMM_ERR_HIP ("the call could not be carried out"), the message names the call.
template <class F>
int qmm_guarded(const char* what, F&& f) {
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return qmm_fail(QMM_ERR_HIP_CODE, "%s: out of host memory", what);
    } catch (const std::exception& e) {
        return qmm_fail(QMM_ERR_HIP_CODE, "%s: %s", what, e.what());
    } catch (...) {
        return qmm_fail(QMM_ERR_HIP_CODE, "%s: unknown failure", what);
    }
}

// The current HIP device, validated (IZWI_QMM_ERR_NO_DEVICE without one), and its CU count.
int qmm_current_device(int* device, int* n_cus);
// The library's scratch buffer of (device, stream): at least `bytes`, reused by the next call on
// the same stream (work on a stream is ordered).  The calling thread holds the buffer exclusively
// from this request until its outermost QmmCallScope ends; other host threads that call on the
// same stream wait for that.  Grows with hipMalloc (an outgrown buffer is kept until the process
// ends, never freed); hipErrorStreamCaptureUnsupported if it would have to grow during a capture.
hipError_t qmm_get_scratch(int device, hipStream_t stream, size_t bytes, void** out);
// Profiling (IZWI_QWEN3_PROFILE / izwi_qmm_profile_enable) for the library's other source files:
// whether it is on, whether a stream is being captured (no waits then), one device argmax call.
bool qmm_profiling();
bool qmm_stream_is_capturing(hipStream_t stream);
void qmm_profile_count_argmax(uint64_t ns);
// Whether the expert-grouped matrix-core kernel takes its expert form (a tuning switch, off by default).
int qmm_moe_expert_form(); // 1 / 0: forced on / off, -1: chosen by the number of pairs per expert
// A weight handle's layout, device matrix and device ordinal, for the library's other source files.
struct izwi_qmm_weight;
const QmmLayout* qmm_weight_layout(const izwi_qmm_weight* w);
const void* qmm_weight_tiled(const izwi_qmm_weight* w);
int qmm_weight_device(const izwi_qmm_weight* w);
// One library call on this thread: every exported entry point that may reach qmm_get_scratch
// opens one first.  Scopes nest (entry points call each other); the outermost one releases the
// scratch buffers its call took.
struct QmmCallScope {
    QmmCallScope();
    ~QmmCallScope();
    QmmCallScope(const QmmCallScope&) = delete;
    QmmCallScope& operator=(const QmmCallScope&) = delete;
};

// ---- launchers -------------------------------------------------------------
hipError_t qmm_launch_repack(const QmmLayout& L, const void* native, void* tiled,
                             hipStream_t stream);
hipError_t qmm_launch_unpack(const QmmLayout& L, const void* tiled, void* native,
                             hipStream_t stream);
hipError_t qmm_launch_dequant(const QmmLayout& L, const void* tiled, float* out,
                              hipStream_t stream);
// out[i, :] = row rows[i] (device ints) of the first matrix, dequantized as above, f32 or rounded to bf16;
// a row id outside [0, n) gives zeros.
// BlockQ4K::from_float over `n_blocks` blocks of 256 consecutive f32 values: 144 bytes each into `out`
hipError_t qmm_launch_quantize_q4k_weights(const float* x, int64_t n_blocks, void* out, hipStream_t stream);
hipError_t qmm_launch_dequant_rows(const QmmLayout& L, const void* tiled, const int32_t* rows, int64_t n_rows,
                                   void* out, int out_bf16, hipStream_t stream);

// Decode kernel: y[m, n] = QMatMul(x[m, k]) for one matrix of the handle.
// `n_cus` sizes the grid.  Returns hipErrorInvalidValue for shapes it cannot run.
// With `io`: x and y are of the types it names (bf16 activations: m <= 2 only,
// hipErrorNotSupported beyond).
hipError_t qmm_launch_gemv(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                           float* y, int n_cus, hipStream_t stream, const QmmIo* io = nullptr,
                           const QmmNorm* norm = nullptr);

// Selected output rows (m <= 2, hipErrorNotSupported beyond): out[mi, i] = row token_ids[i] of
// the product, bit-identical to qmm_launch_gemv followed by a gather; only the 16-row tiles that
// hold a selected row are read.  `workspace`: qmm_gemv_rows_workspace_bytes(m, count) bytes.
size_t qmm_gemv_rows_workspace_bytes(int64_t m, int64_t count);
hipError_t qmm_launch_gemv_rows(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                                const uint32_t* token_ids, int64_t count, float* out, void* workspace, int n_cus,
                                hipStream_t stream);

// Decode kernel for the gate / up pair of an MLP: y[m, n] = silu(W_gate x) * (W_up x), both
// matrices of layout L, m <= 2 (hipErrorNotSupported beyond).  The sums are those of
// qmm_launch_gemv; the product is applied where the waves that split k are combined.
hipError_t qmm_launch_gemv_gated(const QmmLayout& L, const void* tiled_gate, const void* tiled_up,
                                 const float* x, int64_t m, float* y, int n_cus, hipStream_t stream,
                                 const QmmNorm* norm = nullptr);
// out[i] = silu(gate[i]) * up[i]
hipError_t qmm_launch_silu_mul(const float* gate, const float* up, float* out, int64_t count,
                               hipStream_t stream);

// Batched decode kernel (int8 MFMA) for 3 <= m <= 64.  `workspace` must hold
// qmm_gemv_mfma_workspace_bytes(L, m) bytes and stay untouched until the work
// queued on `stream` has run.
// `quantize` false: the workspace already holds the quantized activations of x for this k
// and type (a previous call on the same x), only the matmul is launched.
size_t qmm_gemv_mfma_workspace_bytes(const QmmLayout& L, int64_t m);
// With `io`: x and y are of the types it names; hipErrorNotSupported (nothing launched) if the
// epilogue cannot be folded into the form this shape takes.
hipError_t qmm_launch_gemv_mfma(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                                float* y, void* workspace, int n_cus, hipStream_t stream,
                                bool quantize = true, const QmmIo* io = nullptr);

// Activation quantizer written out in the reference's block layout.
hipError_t qmm_launch_quantize_activations(int weight_dtype, const float* x, int64_t m, int64_t k,
                                           void* out_blocks, hipStream_t stream);

// Prefill kernel: bf16 activations, bf16 MFMA, f32 accumulate.  Products with few output
// tiles are split along k and need `workspace` (qmm_gemm_workspace_bytes, 0 if not split).
size_t qmm_gemm_workspace_bytes(const QmmLayout& L, int64_t m, int n_cus);
// `residual` (of y's type, may alias y, may be NULL) is added to the sums before the store.
hipError_t qmm_launch_gemm_bf16(const QmmLayout& L, const void* tiled, const uint16_t* x_bf16,
                                int64_t m, void* y, int out_bf16, void* workspace, int n_cus,
                                hipStream_t stream, const void* residual = nullptr);
// Several weights of equal k and type on the same bf16 activations in ONE launch of the pipelined
// tiles (m > 128): the grid is the members' column tiles one after the other, planned as one
// matrix with all the columns.  Per-member results are those of qmm_launch_gemm_bf16 up to the
// tile plan (which may split k differently).  hipErrorNotSupported: no single-launch form
// (m <= 128), call the members one by one.
size_t qmm_gemm_group_workspace_bytes(const QmmLayout* const* layouts, int n_weights, int64_t m, int n_cus);
hipError_t qmm_launch_gemm_bf16_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                      const uint16_t* x_bf16, int64_t m, void* const* ys, int out_bf16,
                                      void* workspace, int n_cus, hipStream_t stream);
// Plane form of the prefill product (Q4_K / Q8_0, k a multiple of 64, more than 128 rows): the
// weights are dequantized once per call into a bf16 plane in `planes` (qmm_gemm_plane_bytes per
// member, members one after the other) and multiplied by a plain bf16 matrix-core loop fed with
// LDS-direct loads.  qmm_gemm_plane_applies: whether a call of m rows takes this form
// (qmm_set_prefill_form: 0 in-LDS form always, 1 plane form wherever it can run, -1 by size).
bool qmm_gemm_plane_applies(const QmmLayout& L, int64_t m);
size_t qmm_gemm_plane_bytes(const QmmLayout& L);
void qmm_set_prefill_form(int form);
int qmm_get_prefill_form();
hipError_t qmm_launch_gemm_plane(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                 const uint16_t* x_bf16, int64_t m, void* const* ys, int out_bf16, void* planes,
                                 int n_cus, hipStream_t stream, const void* residual = nullptr);
// y[i] = t[i] (+ residual[i]) as f32 or bf16: the epilogue as a kernel of its own, for the forms
// that cannot fold it
hipError_t qmm_launch_epilogue(const float* t, const void* residual, void* y, int y_bf16, int64_t count,
                               hipStream_t stream);
// bf16 -> f32, exact
hipError_t qmm_launch_bf16_to_f32(const uint16_t* x, float* out, int64_t count, hipStream_t stream);
// f32 activations for m > 64: converted to bf16 into `x_bf16_ws` (m*k elements) first.
hipError_t qmm_launch_f32_to_bf16(const float* x, uint16_t* out, int64_t count,
                                  hipStream_t stream);

// Several weights of equal k and type applied to the same activations (m <= 2) in one launch
// of the decode kernel; y_i = x W_i^T exactly as separate launches would give.
// hipErrorNotSupported: the shapes have no single-launch form, launch them one by one.
#define QMM_MAX_GROUP 4
hipError_t qmm_launch_gemv_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                 const float* x, int64_t m, float* const* ys, int n_cus,
                                 hipStream_t stream, const QmmNorm* norm = nullptr);

// The same for 3 <= m <= 16 on the matrix cores: `workspace` holds the activations already
// quantized (qmm_launch_quantize_ws), all weights read the same records in one launch.
hipError_t qmm_launch_quantize_ws(int dtype, const float* x, int64_t m, int64_t k, void* workspace,
                                  hipStream_t stream, bool x_bf16 = false);
// silu(gate) * up quantized straight into the records; bytes of the records of m rows of k values
hipError_t qmm_launch_quantize_silu_mul_ws(int dtype, const float* gate, const float* up, int64_t m, int64_t k,
                                           void* workspace, hipStream_t stream);
size_t qmm_records_bytes(int dtype, int64_t m, int64_t k);
hipError_t qmm_launch_gemv_mfma_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                      int64_t m, float* const* ys, const void* workspace, int n_cus,
                                      hipStream_t stream);

// ---- MoE ---------------------------------------------------------------------
// Sorted pairs are processed in segments of this many rows that share one expert.
#define QMM_MOE_SEG_ROWS 4

hipError_t qmm_launch_moe_route(const float* logits, int64_t t, int n_experts, int top_k,
                                int32_t* ids, float* weights, hipStream_t stream,
                                const float* x = nullptr, int64_t k = 0, int dot_dtype = 0, void* x_blocks = nullptr);
// (x, k, dot_dtype, x_blocks: the wave that routes a token also quantizes the token's row of x [t, k]
// for weights of block type `dot_dtype` into its x blocks)

// Stable counting sort of `pairs` expert ids.  `seg_offsets` (n_experts + 1 ints,
// may be NULL) receives the exclusive prefix sum of ceil(count / seg_rows): the table of the
// 4-row segments or of the 16-row tiles, whichever the expert MLP behind the sort runs on, and
// `seg_expert` (may be NULL; up to max_segments entries) the expert of every such segment.
// `scratch` must hold qmm_moe_sort_scratch_ints(pairs, n_experts) ints.
// `expert_order` (8 ints per expert, may be NULL; only where qmm_moe_sort_ranks_experts says so): the
// experts by falling segment count, ties by index - the order in which the expert form of the
// grouped matrix-core kernel numbers its work items (it ranks the experts itself without it).
// Entry r: the expert of rank r, its first segment, its segment count, its first and last + 1 sorted pair.
hipError_t qmm_launch_moe_sort(const int32_t* ids, int64_t pairs, int n_experts, int32_t* perm,
                               int32_t* offsets, int32_t* seg_offsets, int32_t* scratch,
                               hipStream_t stream, int seg_rows = QMM_MOE_SEG_ROWS, int32_t* seg_expert = nullptr,
                               int64_t max_segments = 0, int32_t* expert_order = nullptr);
bool qmm_moe_sort_ranks_experts(int64_t pairs, int n_experts);
int64_t qmm_moe_sort_scratch_ints(int64_t pairs, int n_experts);

// Expert-grouped decode kernel over sorted pairs.  Row i of the sorted list is
// pair p = perm[i]; its activation row is x[p / x_div], its output row y[p].
// With `tiled2` the result is silu(W x) * (W2 x).
hipError_t qmm_launch_gemv_grouped(const QmmLayout& L, const void* tiled, const void* tiled2,
                                   const float* x, int x_div, float* y, const int32_t* perm,
                                   const int32_t* offsets, const int32_t* seg_offsets,
                                   const int32_t* seg_expert, int n_experts, int64_t max_segments,
                                   int n_cus, hipStream_t stream, const void* x_blocks = nullptr, int64_t x_rows = 0);
// `x_blocks`: the x_rows activation rows quantized ahead of the launch (qmm_x_blocks_bytes bytes, written
// by the routing kernels below when they are given x); then the workgroups copy instead of quantizing.
size_t qmm_x_blocks_bytes(int64_t rows, int64_t k);

// seg_offsets[e] = exclusive prefix sum of ceil(count(e) / seg_rows) from caller-provided
// offsets; seg_expert (may be NULL; max_segments ints) = the expert of every segment, -1
// past the last one.  `expert_order` (may be NULL; only where qmm_moe_segments_rank_experts says so): the
// table of the ranked experts that qmm_launch_moe_sort describes.
hipError_t qmm_launch_moe_segments(const int32_t* offsets, int n_experts, int seg_rows,
                                   int32_t* seg_offsets, int32_t* seg_expert, int64_t max_segments,
                                   hipStream_t stream, int32_t* expert_order = nullptr);
bool qmm_moe_segments_rank_experts(int n_experts);

// Expert-grouped batched decode on the int8 matrix cores (many pairs per expert).
// Sorted pairs are cut into tiles of QMM_MOE_TILE_ROWS rows that share one expert;
// `tile_offsets` is qmm_launch_moe_segments(.., QMM_MOE_TILE_ROWS, ..).
// Step 1 quantizes the activation rows of all tiles into `records`
// (qmm_moe_records_bytes): row i of the sorted list is pair p = perm[i], its
// activations are x[p / x_div] or, with x2, silu(x[p / x_div]) * x2[p / x_div].
// Step 2 multiplies: output row y[p].
#define QMM_MOE_TILE_ROWS 16
size_t qmm_moe_records_bytes(int dtype, int64_t max_tiles, int64_t k);
hipError_t qmm_launch_quantize_grouped(int dtype, const float* x, const float* x2, int x_div,
                                       int64_t k, const int32_t* perm, const int32_t* offsets,
                                       const int32_t* tile_offsets, int n_experts,
                                       int64_t max_tiles, void* records, hipStream_t stream,
                                       const int32_t* tile_expert = nullptr);
// false if the matrix shape has no grouped matrix-core form (too many panels per row-tile)
bool qmm_gemv_mfma_grouped_supported(const QmmLayout& L);
// With tiled2 / y2 a second stack of the same shape is multiplied by the same records
// in the same launch (the expert MLP's gate and up projections).
// row_div > 0: `records` are row records (below) and sorted pair p reads source row perm[p] / row_div.
hipError_t qmm_launch_gemv_mfma_grouped(const QmmLayout& L, const void* tiled, const void* tiled2,
                                        const void* records, float* y, float* y2, const int32_t* perm,
                                        const int32_t* offsets, const int32_t* tile_offsets,
                                        int n_experts, int64_t pairs, hipStream_t stream, int n_cus,
                                        int row_div = 0, const int32_t* expert_order = nullptr);
// Row records: every source row is quantized once, on its own (no tile tables), and the expert form
// of the grouped kernel puts its tiles together from the rows' records while it copies them to LDS.
// Whether a stack of layout L with `rows` source rows, read as perm[p] / row_div, runs that way:
bool qmm_moe_row_records_apply(const QmmLayout& L, int n_cus, int64_t pairs, int64_t rows, int row_div);
size_t qmm_row_records_bytes(int64_t rows, int64_t k);
// rows of x, or of silu(x) * x2
hipError_t qmm_launch_quantize_rows(int dtype, const float* x, const float* x2, int64_t rows, int64_t k,
                                    void* row_records, hipStream_t stream);
// qmm_launch_moe_route that also writes the row records of the tokens' activation rows x [t, k]
hipError_t qmm_launch_moe_route_rows(const float* logits, int64_t t, int n_experts, int top_k, int32_t* ids,
                                     float* weights, hipStream_t stream, const float* x, int64_t k, int dtype,
                                     void* row_records);

// Small batches: routing, sort and the segment tables (seg_rows rows per segment) of the grouped
// decode kernel in one launch; same results as route + sort + segments.
bool qmm_moe_plan_small_supported(int64_t t, int n_experts, int top_k);
hipError_t qmm_launch_moe_plan_small(const float* logits, int64_t t, int n_experts, int top_k, int seg_rows,
                                     int64_t max_segments, int32_t* ids, float* weights, int32_t* perm,
                                     int32_t* offsets, int32_t* seg_offsets, int32_t* seg_expert,
                                     hipStream_t stream);

// The whole expert MLP of a small batch (t * top_k <= 64 pairs, inter <= 1024) in TWO launches:
// routing inside the gate / up launch (every workgroup routes its own token), the weighted
// combine inside the down launch (a wave per slot, slots added in order).  Same results as
// route + sort + grouped kernels + combine.  `h` [pairs, inter], `ids` / `weights` [pairs] are
// scratch; ids_out / weights_out may be NULL.  hipErrorNotSupported: use the general path.
bool qmm_moe_small_supported(const QmmLayout& G, const QmmLayout& D, int64_t t, int n_experts, int top_k);
hipError_t qmm_launch_moe_small(const QmmLayout& G, const void* gate, const void* up, const QmmLayout& D, const void* down,
                                const float* logits, const float* x, int64_t t, int n_experts, int top_k, float* h,
                                int32_t* ids, float* weights, int32_t* ids_out, float* weights_out, float* out,
                                int64_t max_segments, int n_cus, hipStream_t stream);

// out[t, :] = sum over slots s (in order) of weights[t, s] * y[t * top_k + s, :]
hipError_t qmm_launch_moe_combine(const float* y, const float* weights, int64_t t, int top_k,
                                  int64_t hidden, float* out, hipStream_t stream);
