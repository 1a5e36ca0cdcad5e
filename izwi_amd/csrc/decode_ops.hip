// Decode-step neighbours of the quantized projections: RMSNorm, q/k head norm, rotary
// embedding, single-token grouped-query attention (f32).  All four are bounded by HBM traffic or,
// at one token, by launch latency; none is GEMM-shaped.
//
//  * norms: one workgroup per row, 16-byte loads when the row allows it, the row stays in
//    registers between the reduction and the scaling (read once, written once);
//  * rotary: one thread per (row, pair);
//  * attention: the KV cache of a kv head is read ONCE for all query heads that share it.
//    Positions are split over workgroups (enough of them to fill the chip at any cache length),
//    each keeps running (max, sum, weighted value sum) per head and the splits are merged by a
//    second small kernel.  Inside a workgroup 8 lanes share a cache row as 8 x 16 B pieces of
//    every 128-byte segment (coalesced), 32 rows are in flight per workgroup.
#include <hip/hip_runtime.h>

#include <chrono>

#include <type_traits>

#include <math.h>
#include <stdlib.h>

#include "../../include/izwi_decode_ops.h"
#include "qmm_internal.h"
#include "qmm_records.h"

namespace {

#define OPS_TRY(expr)                                                                     \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess) {                                                           \
            (void)hipGetLastError();                                                      \
            return qmm_fail(IZWI_QMM_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_));    \
        }                                                                                 \
    } while (0)

// Device view of a caller buffer: the pointer itself, or a staged copy of host memory.
struct Buf {
    void* dev = nullptr;
    void* host = nullptr;
    size_t bytes = 0;
    bool owned = false, copy_back = false;
    ~Buf() {
        if (owned && dev) (void)hipFree(dev);
    }
    hipError_t in(const void* p, size_t n, int mem_space) {
        bytes = n;
        if (mem_space == IZWI_QMM_DEVICE || n == 0) {
            dev = const_cast<void*>(p);
            return hipSuccess;
        }
        owned = true;
        hipError_t e = hipMalloc(&dev, n);
        return e != hipSuccess ? e : hipMemcpy(dev, p, n, hipMemcpyHostToDevice);
    }
    hipError_t out(void* p, size_t n, int mem_space) {
        bytes = n;
        if (mem_space == IZWI_QMM_DEVICE || n == 0) {
            dev = p;
            return hipSuccess;
        }
        owned = copy_back = true;
        host = p;
        return hipMalloc(&dev, n);
    }
    hipError_t finish(hipStream_t stream) {
        if (!copy_back) return hipSuccess;
        hipError_t e = hipStreamSynchronize(stream);
        return e != hipSuccess ? e : hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost);
    }
};

int check_space(int mem_space) {
    if (mem_space != IZWI_QMM_DEVICE && mem_space != IZWI_QMM_HOST)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "bad mem_space %d", mem_space);
    return IZWI_QMM_OK;
}

// The hooks' two element types: f32, and f16 widened on load and rounded once on store (all
// arithmetic is f32, as in the reference's *_f16 shaders, metal.rs:103-144, 187-225, 267-305,
// 383-457).  A 16-byte piece holds kEC<T> consecutive elements.
typedef _Float16 f16_t;
template <typename T>
constexpr int kEC = 16 / (int)sizeof(T);
template <typename T>
__device__ __forceinline__ float ld1(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void st1(T* p, float v) { *p = (T)v; }
template <typename T>
__device__ __forceinline__ void ld16(const T* p, float (&v)[kEC<T>]) {
    if constexpr (sizeof(T) == 4) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
    } else {
        typedef f16_t h8 __attribute__((ext_vector_type(8)));
        const h8 t = *reinterpret_cast<const h8*>(p);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)t[i];
    }
}
template <typename T>
__device__ __forceinline__ void st16(T* p, const float (&v)[kEC<T>]) {
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        typedef f16_t h8 __attribute__((ext_vector_type(8)));
        h8 t;
#pragma unroll
        for (int i = 0; i < 8; i++) t[i] = (f16_t)v[i];
        *reinterpret_cast<h8*>(p) = t;
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ---- norms ---------------------------------------------------------------------------
// Row r < rows_a comes from a / goes to out_a with weight_a, the others from b (the q/k pair);
// a plain RMSNorm has rows_b == 0.  VEC: hidden is a multiple of 4 and all rows are 16-byte
// aligned.  A thread keeps up to PER values of its row in registers; longer rows are re-read.
template <typename T>
struct NormParams {
    const T* a;
    const T* b;
    const T* weight_a;
    const T* weight_b;
    T* out_a;
    T* out_b;
    int64_t rows_a, rows_b;
    int hidden;
    float eps;
    // REC variants: instead of out_a the normalized rows go, quantized, into the activation records
    // of the batched decode kernels (row r of tile r / 16); rows rows_a .. rec_rows - 1 are zero rows
    uint8_t* records;
    int64_t rec_rows;
};

template <bool VEC, typename T, int REC = 0>
__global__ void rms_norm_kernel(NormParams<T> P) {
    constexpr int PER = 4, EC = kEC<T>; // 16-byte pieces (VEC) or single values kept per thread
    __shared__ float partial[16];
    extern __shared__ __attribute__((aligned(16))) float normed_row[]; // REC: the normalized row, [hidden]
    const int64_t row = blockIdx.x;
    if constexpr (REC != 0) {
        if (row >= P.rows_a) { // a padding row of the last 16-row tile: zeros
            const float zero[16] = {};
            for (int t = threadIdx.x; t < P.hidden / 16; t += blockDim.x)
                quantize_into_record<REC>(zero, t & 15, (int)(row & 15),
                                          P.records + ((row >> 4) * (P.hidden / 256) + (t >> 4)) * Unit<REC>::kBytes);
            return;
        }
    }
    const bool first = row < P.rows_a;
    const T* x = first ? P.a + row * P.hidden : P.b + (row - P.rows_a) * P.hidden;
    const T* w = first ? P.weight_a : P.weight_b;
    T* y = first ? P.out_a + row * P.hidden : P.out_b + (row - P.rows_a) * P.hidden;
    const int tid = threadIdx.x, nt = blockDim.x;
    float sum = 0.0f;
    float keepv[PER][EC];
    float keep1[PER];
    const int nv = P.hidden / EC;
    if (VEC) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * nt;
            if (idx < nv) ld16<T>(x + (int64_t)idx * EC, keepv[i]);
#pragma unroll
            for (int c = 0; c < EC; c++) {
                if (idx >= nv) keepv[i][c] = 0.0f;
                sum += keepv[i][c] * keepv[i][c];
            }
        }
        for (int idx = tid + PER * nt; idx < nv; idx += nt) {
            float v[EC];
            ld16<T>(x + (int64_t)idx * EC, v);
#pragma unroll
            for (int c = 0; c < EC; c++) sum += v[c] * v[c];
        }
    } else {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * nt;
            keep1[i] = idx < P.hidden ? ld1(x + idx) : 0.0f;
            sum += keep1[i] * keep1[i];
        }
        for (int idx = tid + PER * nt; idx < P.hidden; idx += nt) sum += ld1(x + idx) * ld1(x + idx);
    }
    sum = wave_sum(sum);
    if ((tid & 63) == 0) partial[tid >> 6] = sum;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < (nt + 63) / 64; i++) total += partial[i];
    const float scale = 1.0f / sqrtf(total / (float)P.hidden + P.eps);
    if (VEC) {
        auto finish = [&](int idx, const float (&v)[EC]) {
            float ww[EC], o[EC];
            ld16<T>(w + (int64_t)idx * EC, ww);
#pragma unroll
            for (int c = 0; c < EC; c++) o[c] = v[c] * scale * ww[c];
            if constexpr (REC != 0) {
#pragma unroll
                for (int c = 0; c < EC; c++) normed_row[idx * EC + c] = o[c];
            } else {
                st16<T>(y + (int64_t)idx * EC, o);
            }
        };
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * nt;
            if (idx < nv) finish(idx, keepv[i]);
        }
        for (int idx = tid + PER * nt; idx < nv; idx += nt) {
            float v[EC];
            ld16<T>(x + (int64_t)idx * EC, v);
            finish(idx, v);
        }
    } else {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * nt;
            if (idx < P.hidden) st1(y + idx, keep1[i] * scale * ld1(w + idx));
        }
        for (int idx = tid + PER * nt; idx < P.hidden; idx += nt) st1(y + idx, ld1(x + idx) * scale * ld1(w + idx));
    }
    if constexpr (REC != 0) {
        // the row as the record quantizer wants it: 16 consecutive values per lane, 16 lanes per unit
        __syncthreads();
        for (int t = tid; t < P.hidden / 16; t += nt) {
            float v[16];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float4 f = *reinterpret_cast<const float4*>(normed_row + 16 * t + 4 * i);
                v[4 * i] = f.x, v[4 * i + 1] = f.y, v[4 * i + 2] = f.z, v[4 * i + 3] = f.w;
            }
            quantize_into_record<REC>(v, t & 15, (int)(row & 15),
                                      P.records + ((row >> 4) * (P.hidden / 256) + (t >> 4)) * Unit<REC>::kBytes);
        }
    }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
hipError_t launch_norm(const NormParams<T>& P, hipStream_t stream) {
    const int64_t rows = P.rows_a + P.rows_b;
    if (rows == 0) return hipSuccess;
    if (rows > 0x7fffffff) return hipErrorInvalidValue;
    const bool vec = P.hidden % kEC<T> == 0 && aligned16(P.a) && aligned16(P.out_a) && aligned16(P.weight_a) &&
                     (P.rows_b == 0 || (aligned16(P.b) && aligned16(P.out_b) && aligned16(P.weight_b)));
    // one 16-byte piece (or value) per thread up to four per thread; at most 1024 threads
    const int items = vec ? P.hidden / kEC<T> : P.hidden;
    int threads = 64;
    while (threads < 1024 && threads < items) threads *= 2;
    if (vec) rms_norm_kernel<true, T><<<(unsigned)rows, threads, 0, stream>>>(P);
    else rms_norm_kernel<false, T><<<(unsigned)rows, threads, 0, stream>>>(P);
    return hipGetLastError();
}

// RMSNorm straight into activation records (f32 rows, hidden a multiple of 256, 16-byte aligned):
// the sums and products are those of rms_norm_kernel<true, float> with the same thread count, so
// the records equal those of the norm followed by the record quantizer bit for bit.
hipError_t launch_norm_records(NormParams<float> P, int weight_dtype, hipStream_t stream) {
    if (P.rec_rows > 0x7fffffff) return hipErrorInvalidValue;
    int threads = 64;
    while (threads < 1024 && threads < P.hidden / 4) threads *= 2;
    const size_t lds = (size_t)P.hidden * sizeof(float);
    if (lds > 64 * 1024) return hipErrorNotSupported;
    if (weight_dtype == IZWI_QMM_Q8_0) {
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&rms_norm_kernel<true, float, QMM_Q8_0>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            if (e != hipSuccess) return e;
        }
        rms_norm_kernel<true, float, QMM_Q8_0><<<(unsigned)P.rec_rows, threads, lds, stream>>>(P);
    } else { // Q4_K and Q6_K weights both dot against Q8_K activations: one record format
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&rms_norm_kernel<true, float, QMM_Q4_K>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            if (e != hipSuccess) return e;
        }
        rms_norm_kernel<true, float, QMM_Q4_K><<<(unsigned)P.rec_rows, threads, lds, stream>>>(P);
    }
    return hipGetLastError();
}

// ---- rotary embedding ----------------------------------------------------------------------
template <typename T>
__global__ void rope_pair_kernel(const T* __restrict__ cos_sin, const T* q, const T* k, T* q_out, T* k_out,
                                 int64_t q_rows, int64_t k_rows, int seq, int q_heads, int k_heads, int head_dim) {
    const int half = head_dim >> 1;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (q_rows + k_rows) * half) return;
    const int64_t row = idx / half;
    const int d = (int)(idx - row * half);
    const bool is_q = row < q_rows;
    const int64_t local = is_q ? row : row - q_rows;
    const int pos = (int)((local / (is_q ? q_heads : k_heads)) % seq);
    const T* x = (is_q ? q : k) + local * head_dim;
    T* y = (is_q ? q_out : k_out) + local * head_dim;
    const float c = ld1(cos_sin + (int64_t)pos * head_dim + d), s = ld1(cos_sin + (int64_t)pos * head_dim + half + d);
    const float x1 = ld1(x + d), x2 = ld1(x + half + d);
    st1(y + d, x1 * c - x2 * s);
    st1(y + half + d, x1 * s + x2 * c);
}

// ---- greedy sampling: first index of the row maximum ------------------------------------------
// One workgroup per row; a thread keeps (value, index) of its strided share, ties to the smaller
// index, NaN never wins; wave reduction by shuffles, then the waves' results through LDS.
__device__ __forceinline__ void argmax_merge(float& v, unsigned& i, float ov, unsigned oi) {
    if (ov > v || (ov == v && oi < i)) v = ov, i = oi;
}
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ x, int64_t n, uint32_t* __restrict__ out) {
    __shared__ float vals[16];
    __shared__ unsigned idxs[16];
    const float* row = x + (int64_t)blockIdx.x * n;
    float v = -INFINITY;
    unsigned idx = 0xffffffffu;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float t = row[i];
        if (t > v || idx == 0xffffffffu) { // strided visit in rising order: a later equal value never replaces
            if (t > v || (idx == 0xffffffffu && !(t != t))) v = t, idx = (unsigned)i;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(v, idx, __shfl_xor(v, o), (unsigned)__shfl_xor((int)idx, o));
    if ((threadIdx.x & 63) == 0) vals[threadIdx.x >> 6] = v, idxs[threadIdx.x >> 6] = idx;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) argmax_merge(v, idx, vals[w], idxs[w]);
        out[blockIdx.x] = idx == 0xffffffffu ? 0u : idx; // a row of NaNs: index 0
    }
}

// Long rows of few: blockIdx.y scans a chunk of the row into a (value, index) candidate, a second
// launch merges the candidates (same rule, so the result is the one-launch kernel's).
__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ x, int64_t n, int64_t chunk,
                                                          float* __restrict__ pv, uint32_t* __restrict__ pi) {
    __shared__ float vals[4];
    __shared__ unsigned idxs[4];
    const float* row = x + (int64_t)blockIdx.x * n;
    const int64_t begin = (int64_t)blockIdx.y * chunk, end = begin + chunk < n ? begin + chunk : n;
    float v = -INFINITY;
    unsigned idx = 0xffffffffu;
    for (int64_t i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const float t = row[i];
        if (t > v || (idx == 0xffffffffu && !(t != t))) v = t, idx = (unsigned)i;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(v, idx, __shfl_xor(v, o), (unsigned)__shfl_xor((int)idx, o));
    if ((threadIdx.x & 63) == 0) vals[threadIdx.x >> 6] = v, idxs[threadIdx.x >> 6] = idx;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) argmax_merge(v, idx, vals[w], idxs[w]);
        pv[(int64_t)blockIdx.x * gridDim.y + blockIdx.y] = v;
        pi[(int64_t)blockIdx.x * gridDim.y + blockIdx.y] = idx;
    }
}
__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const uint32_t* __restrict__ pi,
                                                          int parts, uint32_t* __restrict__ out) {
    float v = -INFINITY;
    unsigned idx = 0xffffffffu;
    for (int p = threadIdx.x; p < parts; p += 64)
        argmax_merge(v, idx, pv[(int64_t)blockIdx.x * parts + p], pi[(int64_t)blockIdx.x * parts + p]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(v, idx, __shfl_xor(v, o), (unsigned)__shfl_xor((int)idx, o));
    if (threadIdx.x == 0) out[blockIdx.x] = idx == 0xffffffffu ? 0u : idx;
}

// ---- q/k norm + rotary + cache append, one token ---------------------------------------------
// One wave per head: rows 0 .. heads-1 are q, then kv_heads rows of k, then kv_heads rows of v.
// Lane l holds the pairs (p, p + half) for p = l, l + 64, ..: the norm's sum runs over the wave,
// the rotation stays inside the lane.  q goes to q_out, k and v to position `pos` of the caches.
struct QkvPrepParams {
    const float* q;
    const float* k;
    const float* v;
    const float* qk_weight; // [2 * head_dim]
    const float* cos_sin;   // [head_dim]: cos | sin of this position
    float* q_out;
    float* k_cache;
    float* v_cache; // [kv_heads, capacity, head_dim]
    int heads, kv_heads, head_dim;
    int64_t capacity, pos;
    float eps;
};

__global__ __launch_bounds__(256) void qkv_prep_kernel(QkvPrepParams P) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int total = P.heads + 2 * P.kv_heads;
    if (row >= total) return;
    const int hd = P.head_dim, half = hd >> 1;
    if (row >= P.heads + P.kv_heads) { // v: a plain copy into the cache
        const int h = row - P.heads - P.kv_heads;
        const float* src = P.v + (int64_t)h * hd;
        float* dst = P.v_cache + ((int64_t)h * P.capacity + P.pos) * hd;
        for (int i = lane; i < hd; i += 64) dst[i] = src[i];
        return;
    }
    const bool is_q = row < P.heads;
    const int h = is_q ? row : row - P.heads;
    const float* src = (is_q ? P.q : P.k) + (int64_t)h * hd;
    const float* w = P.qk_weight + (is_q ? 0 : hd);
    float* dst = is_q ? P.q_out + (int64_t)h * hd : P.k_cache + ((int64_t)h * P.capacity + P.pos) * hd;
    constexpr int MAXP = 2; // pairs kept per lane: head_dim <= 256; longer heads are re-read
    float x1[MAXP], x2[MAXP];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        const int p = lane + 64 * i;
        x1[i] = p < half ? src[p] : 0.0f;
        x2[i] = p < half ? src[half + p] : 0.0f;
        sum += x1[i] * x1[i] + x2[i] * x2[i];
    }
    for (int p = lane + 64 * MAXP; p < half; p += 64) sum += src[p] * src[p] + src[half + p] * src[half + p];
    sum = wave_sum(sum);
    const float scale = 1.0f / sqrtf(sum / (float)hd + P.eps);
    auto rotate = [&](int p, float a, float b) {
        // the norm as the norm kernel writes it (x * scale * weight), then the rotation of the pair
        const float n1 = a * scale * w[p], n2 = b * scale * w[half + p];
        const float c = P.cos_sin[p], s = P.cos_sin[half + p];
        dst[p] = n1 * c - n2 * s;
        dst[half + p] = n1 * s + n2 * c;
    };
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        const int p = lane + 64 * i;
        if (p < half) rotate(p, x1[i], x2[i]);
    }
    for (int p = lane + 64 * MAXP; p < half; p += 64) rotate(p, src[p], src[half + p]);
}

// ---- single-token GQA attention ------------------------------------------------------------
template <typename T>
struct AttnParams {
    const T* q;
    const T* k;
    const T* v;
    T* out;
    float* part; // [heads][splits][head_dim + 2]: weighted value sums, running max, sum of weights
    int heads, kv_heads, group;
    int kv_len, chunk, splits; // split s covers positions [s * chunk, min(kv_len, (s + 1) * chunk))
    int64_t kv_capacity;
    float scale;
    // PREP form (f32, the step of one new token): q, k_new and v_new are the projections' outputs;
    // the kernel norms and rotates q and k_new itself (the arithmetic of qkv_prep_kernel), takes
    // (k_new, v_new) as position kv_len - 1 and appends them to the caches
    const float* k_new;
    const float* v_new;
    const float* qk_weight; // [2 * head_dim]
    const float* cos_sin;   // [head_dim]: cos | sin of position kv_len - 1
    float* k_append;
    float* v_append;
    float eps;
};

// e^x for x <= 0 on the hardware's exp2 (relative error about 2^-22; e^-inf = 0)
__device__ __forceinline__ float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// weight of a partial result with running maximum m when merged under the maximum mn
__device__ __forceinline__ float merge_weight(float m, float mn) { return m == -INFINITY ? 0.0f : exp_neg(m - mn); }

// sum over the 8 lanes of a row group, in every lane of the group (two quad permutes and a
// mirror of the half row: no LDS traffic)
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float sum8(float v) {
    v += dpp_f<0xB1>(v);  // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);  // quad_perm [2,3,0,1]
    v += dpp_f<0x141>(v); // row_half_mirror
    return v;
}

// HD = head_dim; G query heads of one kv head per workgroup.  Lane j of an 8-lane row group
// holds, of a cache row and of the query heads, the 16-byte pieces j, j + 8, ..: elements
// 8 EC i + EC j + c (i < NI, c < EC; EC = 4 for f32, 8 for f16).
template <typename T, int HD, int G, bool PREP = false>
__global__ __launch_bounds__(256) void attn_partial_kernel(AttnParams<T> P) {
    static_assert(!PREP || std::is_same<T, float>::value, "the one-token step is built for f32");
    constexpr int EC = kEC<T>, NI = HD / (8 * EC), E = EC * NI;
    __shared__ __attribute__((aligned(16))) float red[16][G][HD + 4]; // [.. HD): sums, [HD]: maximum, [HD + 1]: weight sum
    __shared__ __attribute__((aligned(16))) float prep[PREP ? G + 1 : 1][PREP ? HD : 4]; // normed, rotated q heads, then k_new
    const int kvh = blockIdx.x, sp = blockIdx.y, h0 = kvh * P.group + blockIdx.z * G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 7, slot = wave * 8 + (lane >> 3);
    const int p0 = sp * P.chunk, p1 = min(P.kv_len, p0 + P.chunk);
    const int pos = P.kv_len - 1;
    const int p1c = PREP ? min(p1, pos) : p1; // PREP: the new position is not in the cache yet
    const T* kb = P.k + (int64_t)kvh * P.kv_capacity * HD + EC * j;
    const T* vb = P.v + (int64_t)kvh * P.kv_capacity * HD + EC * j;
    auto load_row = [&](int p, float (&kr)[E], float (&vr)[E]) {
#pragma unroll
        for (int i = 0; i < NI; i++) {
            float t[EC];
            ld16<T>(kb + (int64_t)p * HD + 8 * EC * i, t);
#pragma unroll
            for (int c = 0; c < EC; c++) kr[EC * i + c] = t[c];
        }
#pragma unroll
        for (int i = 0; i < NI; i++) {
            float t[EC];
            ld16<T>(vb + (int64_t)p * HD + 8 * EC * i, t);
#pragma unroll
            for (int c = 0; c < EC; c++) vr[EC * i + c] = t[c];
        }
    };
    // PREP: the first cache row is requested before the query is prepared, so that its latency
    // runs beside the norm's
    float kr0[PREP ? E : 1], vr0[PREP ? E : 1];
    const bool first = PREP && p0 + slot < p1c;
    if constexpr (PREP) {
        if (first) load_row(p0 + slot, kr0, vr0);
    }

    if constexpr (PREP) {
        // a wave per row (the group's q heads, then the kv head's new k), as qkv_prep_kernel does it
        constexpr int half = HD / 2, NP = (half + 63) / 64;
        for (int r = wave; r <= G; r += 4) {
            const float* src = r < G ? reinterpret_cast<const float*>(P.q) + (int64_t)(h0 + r) * HD : P.k_new + (int64_t)kvh * HD;
            const float* w = P.qk_weight + (r < G ? 0 : HD);
            float x1[NP], x2[NP];
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < NP; i++) {
                const int p = lane + 64 * i;
                x1[i] = p < half ? src[p] : 0.0f;
                x2[i] = p < half ? src[half + p] : 0.0f;
                sum += x1[i] * x1[i] + x2[i] * x2[i];
            }
            sum = wave_sum(sum);
            const float scale = 1.0f / sqrtf(sum / (float)HD + P.eps);
#pragma unroll
            for (int i = 0; i < NP; i++) {
                const int p = lane + 64 * i;
                if (p < half) {
                    const float n1 = x1[i] * scale * w[p], n2 = x2[i] * scale * w[half + p];
                    const float c = P.cos_sin[p], sn = P.cos_sin[half + p];
                    prep[r][p] = n1 * c - n2 * sn;
                    prep[r][half + p] = n1 * sn + n2 * c;
                }
            }
        }
        __syncthreads();
        // the workgroup whose positions end with the new one appends it to the caches; nobody reads
        // that cache row in this launch
        if (pos >= p0 && pos < p1 && blockIdx.z == 0) {
            for (int t = threadIdx.x; t < HD; t += 256) {
                P.k_append[((int64_t)kvh * P.kv_capacity + pos) * HD + t] = prep[G][t];
                P.v_append[((int64_t)kvh * P.kv_capacity + pos) * HD + t] = P.v_new[(int64_t)kvh * HD + t];
            }
        }
    }

    float qr[G][E];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int i = 0; i < NI; i++) {
            float t[EC];
            if constexpr (PREP) {
#pragma unroll
                for (int c = 0; c < EC; c++) t[c] = prep[g][8 * EC * i + EC * j + c];
            } else {
                ld16<T>(P.q + (int64_t)(h0 + g) * HD + 8 * EC * i + EC * j, t);
            }
#pragma unroll
            for (int c = 0; c < EC; c++) qr[g][EC * i + c] = t[c];
        }
    float m[G], l[G], acc[G][E];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = -INFINITY;
        l[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < E; e++) acc[g][e] = 0.0f;
    }
    // one position into the running softmax of every query head of the group
    auto accumulate = [&](const float (&kr)[E], const float (&vr)[E]) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < E; e++) dot += qr[g][e] * kr[e];
            const float s = sum8(dot) * P.scale;
            if (s > m[g]) { // a new maximum (rare after the first positions): rescale what was summed
                const float alpha = merge_weight(m[g], s);
                l[g] *= alpha;
#pragma unroll
                for (int e = 0; e < E; e++) acc[g][e] *= alpha;
                m[g] = s;
            }
            const float pe = exp_neg(s - m[g]);
            l[g] += pe;
#pragma unroll
            for (int e = 0; e < E; e++) acc[g][e] += pe * vr[e];
        }
    };
    if constexpr (PREP) {
        if (first) accumulate(kr0, vr0);
    }
    {
        // the next row of the group is requested before the current one is used (two register sets,
        // taken in turns), rows in rising order as before
        float ka[E], va[E], kb2[E], vb2[E];
        int pa = p0 + slot + (PREP ? 32 : 0);
        bool have_a = pa < p1c;
        if (have_a) load_row(pa, ka, va);
        while (have_a) {
            const int pb = pa + 32;
            const bool have_b = pb < p1c;
            if (have_b) load_row(pb, kb2, vb2);
            accumulate(ka, va);
            if (!have_b) break;
            pa = pb + 32;
            have_a = pa < p1c;
            if (have_a) load_row(pa, ka, va);
            accumulate(kb2, vb2);
        }
    }
    if constexpr (PREP) {
        // the new position, last of its row group as it would be from the cache
        if (pos >= p0 && pos < p1 && ((pos - p0) & 31) == slot) {
            float kr[E], vr[E];
#pragma unroll
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int c = 0; c < EC; c++) {
                    kr[EC * i + c] = prep[G][8 * EC * i + EC * j + c];
                    vr[EC * i + c] = P.v_new[(int64_t)kvh * HD + 8 * EC * i + EC * j + c];
                }
            accumulate(kr, vr);
        }
    }
    // Merge the 32 row groups of the workgroup: neighbours 8 lanes apart inside a 16-lane row by a
    // row rotation (no LDS), the remaining 16 partial results through LDS, where every output
    // element then sums its 16 terms.  (Shuffling all partial sums across the wave three times was
    // an LDS-latency chain of ~200 dependent permutes: 6 us of a 9 us kernel.)
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float mo = dpp_f<0x128>(m[g]), lo = dpp_f<0x128>(l[g]); // row_ror:8 = lane ^ 8
        const float mn = fmaxf(m[g], mo);
        const float wa = merge_weight(m[g], mn), wb = merge_weight(mo, mn);
        l[g] = l[g] * wa + lo * wb;
#pragma unroll
        for (int e = 0; e < E; e++) acc[g][e] = acc[g][e] * wa + dpp_f<0x128>(acc[g][e]) * wb;
        m[g] = mn;
    }
    if ((lane & 8) == 0) {
        const int entry = wave * 4 + (lane >> 4);
#pragma unroll
        for (int g = 0; g < G; g++) {
#pragma unroll
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int c = 0; c < EC; c += 4)
                    *reinterpret_cast<float4*>(&red[entry][g][8 * EC * i + EC * j + c]) =
                        make_float4(acc[g][EC * i + c], acc[g][EC * i + c + 1], acc[g][EC * i + c + 2], acc[g][EC * i + c + 3]);
            if (j == 0) red[entry][g][HD] = m[g], red[entry][g][HD + 1] = l[g];
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < G * HD; t += 256) {
        const int g = t / HD, d = t - g * HD;
        float mn = -INFINITY;
#pragma unroll
        for (int w = 0; w < 16; w++) mn = fmaxf(mn, red[w][g][HD]);
        float a = 0.0f, lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < 16; w++) {
            const float ww = merge_weight(red[w][g][HD], mn);
            a += red[w][g][d] * ww;
            lsum += red[w][g][HD + 1] * ww;
        }
        const int h = h0 + g;
        if (P.splits == 1) {
            st1(P.out + (int64_t)h * HD + d, a * (1.0f / lsum));
        } else {
            float* dst = P.part + ((int64_t)h * P.splits + sp) * (HD + 2);
            dst[d] = a;
            if (d == 0) dst[HD] = mn, dst[HD + 1] = lsum;
        }
    }
}

// out[h] = merge of the splits' partial results.  One workgroup per head: the splits' maxima and
// weights are worked out once, in parallel over the splits, and kept in LDS; the weighted sums
// then run over the splits with their loads independent of each other (unrolled), not one memory
// round trip per split.
constexpr int kMaxSplits = 1024;
template <typename T>
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ part, T* __restrict__ out,
                                                         int splits, int head_dim) {
    __shared__ float weight[kMaxSplits];
    __shared__ float red[8];
    const int h = blockIdx.x, tid = threadIdx.x;
    const float* base = part + (int64_t)h * splits * (head_dim + 2);
    float mloc = -INFINITY;
    for (int s = tid; s < splits; s += 256) {
        weight[s] = base[(int64_t)s * (head_dim + 2) + head_dim];
        mloc = fmaxf(mloc, weight[s]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, o));
    if ((tid & 63) == 0) red[tid >> 6] = mloc;
    __syncthreads();
    const float mn = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float lloc = 0.0f;
    for (int s = tid; s < splits; s += 256) {
        const float w = merge_weight(weight[s], mn);
        weight[s] = w;
        lloc += base[(int64_t)s * (head_dim + 2) + head_dim + 1] * w;
    }
    lloc = wave_sum(lloc);
    if ((tid & 63) == 0) red[4 + (tid >> 6)] = lloc;
    __syncthreads();
    const float inv = 1.0f / (red[4] + red[5] + red[6] + red[7]);
    for (int d = tid; d < head_dim; d += 256) {
        float a = 0.0f;
#pragma unroll 8
        for (int s = 0; s < splits; s++) a += base[(int64_t)s * (head_dim + 2) + d] * weight[s];
        st1(out + (int64_t)h * head_dim + d, a * inv);
    }
}

template <typename T, int HD, bool PREP>
hipError_t launch_attn_partial_form(const AttnParams<T>& P, int g, dim3 grid, hipStream_t stream) {
    if (g == 4) {
        if constexpr (HD <= 128) attn_partial_kernel<T, HD, 4, PREP><<<grid, 256, 0, stream>>>(P);
        else return hipErrorInvalidValue;
    } else if (g == 2) {
        attn_partial_kernel<T, HD, 2, PREP><<<grid, 256, 0, stream>>>(P);
    } else {
        attn_partial_kernel<T, HD, 1, PREP><<<grid, 256, 0, stream>>>(P);
    }
    return hipGetLastError();
}
template <typename T, int HD>
hipError_t launch_attn_partial(const AttnParams<T>& P, int g, dim3 grid, hipStream_t stream) {
    if constexpr (std::is_same<T, float>::value) {
        if (P.k_new) return launch_attn_partial_form<T, HD, true>(P, g, grid, stream);
    }
    return launch_attn_partial_form<T, HD, false>(P, g, grid, stream);
}

// The extra inputs of the one-token step (see AttnParams)
struct AttnPrep {
    const float* k_new;
    const float* v_new;
    const float* qk_weight;
    const float* cos_sin;
    float eps;
};


template <typename T>
int rms_norm_impl(const T* x, const T* weight, int64_t rows, int64_t hidden, float eps, T* y,
                      int mem_space, void* stream_) {
    if (int rc = check_space(mem_space)) return rc;
    if (rows < 0 || hidden <= 0 || hidden > 0x3fffffff)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "rms_norm: bad shape [%lld, %lld]", (long long)rows, (long long)hidden);
    if (rows == 0) return IZWI_QMM_OK;
    if (!x || !weight || !y) return qmm_fail(IZWI_QMM_ERR_INVALID, "rms_norm: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Buf xi, wi, yo;
    OPS_TRY(xi.in(x, (size_t)rows * hidden * sizeof(T), mem_space));
    OPS_TRY(wi.in(weight, (size_t)hidden * sizeof(T), mem_space));
    OPS_TRY(yo.out(y, (size_t)rows * hidden * sizeof(T), mem_space));
    NormParams<T> P{(const T*)xi.dev, nullptr, (const T*)wi.dev, nullptr, (T*)yo.dev, nullptr, rows, 0,
                 (int)hidden, eps, nullptr, 0};
    OPS_TRY(launch_norm(P, stream));
    OPS_TRY(yo.finish(stream));
    return IZWI_QMM_OK;
}

template <typename T>
int qk_rms_norm_impl(const T* q, const T* k, const T* qk_weight, int64_t q_rows, int64_t k_rows,
                         int64_t head_dim, float eps, T* q_out, T* k_out, int mem_space, void* stream_) {
    if (int rc = check_space(mem_space)) return rc;
    if (q_rows < 0 || k_rows < 0 || head_dim <= 0 || head_dim > 8192)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "qk_rms_norm: bad shape q [%lld, %lld], k [%lld, %lld]", (long long)q_rows,
                        (long long)head_dim, (long long)k_rows, (long long)head_dim);
    if (q_rows + k_rows == 0) return IZWI_QMM_OK;
    if (!qk_weight || (q_rows && (!q || !q_out)) || (k_rows && (!k || !k_out)))
        return qmm_fail(IZWI_QMM_ERR_INVALID, "qk_rms_norm: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Buf qi, ki, wi, qo, ko;
    OPS_TRY(qi.in(q, (size_t)q_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(ki.in(k, (size_t)k_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(wi.in(qk_weight, (size_t)2 * head_dim * sizeof(T), mem_space));
    OPS_TRY(qo.out(q_out, (size_t)q_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(ko.out(k_out, (size_t)k_rows * head_dim * sizeof(T), mem_space));
    // (with no q rows the first operand of the kernel is the k tensor)
    NormParams<T> P;
    if (q_rows)
        P = NormParams<T>{(const T*)qi.dev, (const T*)ki.dev, (const T*)wi.dev, (const T*)wi.dev + head_dim,
                       (T*)qo.dev, (T*)ko.dev, q_rows, k_rows, (int)head_dim, eps, nullptr, 0};
    else
        P = NormParams<T>{(const T*)ki.dev, nullptr, (const T*)wi.dev + head_dim, nullptr, (T*)ko.dev, nullptr,
                       k_rows, 0, (int)head_dim, eps, nullptr, 0};
    if (P.rows_b == 0) P.b = nullptr, P.weight_b = nullptr, P.out_b = nullptr;
    OPS_TRY(launch_norm(P, stream));
    OPS_TRY(qo.finish(stream));
    OPS_TRY(ko.finish(stream));
    return IZWI_QMM_OK;
}

template <typename T>
int rope_pair_impl(const T* q, const T* k, const T* cos_sin, int64_t batch, int64_t seq,
                            int64_t q_heads, int64_t k_heads, int64_t head_dim, T* q_out, T* k_out,
                            int mem_space, void* stream_) {
    if (int rc = check_space(mem_space)) return rc;
    if (batch < 0 || seq < 0 || q_heads < 0 || k_heads < 0 || head_dim <= 0 || head_dim % 2 || head_dim > 0x3fffffff ||
        seq > 0x3fffffff || q_heads > 0x3fffffff || k_heads > 0x3fffffff)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "rope_pair_bshd: bad shape [%lld, %lld, %lld | %lld, %lld] (head_dim must be even)",
                        (long long)batch, (long long)seq, (long long)q_heads, (long long)k_heads, (long long)head_dim);
    const int64_t q_rows = batch * seq * q_heads, k_rows = batch * seq * k_heads;
    if (q_rows + k_rows == 0) return IZWI_QMM_OK;
    if (!cos_sin || (q_rows && (!q || !q_out)) || (k_rows && (!k || !k_out)))
        return qmm_fail(IZWI_QMM_ERR_INVALID, "rope_pair_bshd: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Buf qi, ki, ci, qo, ko;
    OPS_TRY(qi.in(q, (size_t)q_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(ki.in(k, (size_t)k_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(ci.in(cos_sin, (size_t)seq * head_dim * sizeof(T), mem_space));
    OPS_TRY(qo.out(q_out, (size_t)q_rows * head_dim * sizeof(T), mem_space));
    OPS_TRY(ko.out(k_out, (size_t)k_rows * head_dim * sizeof(T), mem_space));
    const int64_t pairs = (q_rows + k_rows) * (head_dim / 2);
    const int64_t grid = (pairs + 255) / 256;
    if (grid > 0x7fffffff) return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "rope_pair_bshd: too many elements");
    rope_pair_kernel<T><<<(unsigned)grid, 256, 0, stream>>>((const T*)ci.dev, (const T*)qi.dev, (const T*)ki.dev,
                                                         (T*)qo.dev, (T*)ko.dev, q_rows, k_rows, (int)seq,
                                                         (int)(q_heads ? q_heads : 1), (int)(k_heads ? k_heads : 1),
                                                         (int)head_dim);
    OPS_TRY(hipGetLastError());
    OPS_TRY(qo.finish(stream));
    OPS_TRY(ko.finish(stream));
    return IZWI_QMM_OK;
}

template <typename T>
int decode_attention_impl(const T* q, const T* k, const T* v, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t kv_len, int64_t kv_capacity,
                                  float scale, T* out, int mem_space, void* stream_, const AttnPrep* prep = nullptr) {
    if (int rc = check_space(mem_space)) return rc;
    if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || num_heads > 65535 || kv_len <= 0 ||
        kv_len > kv_capacity || kv_capacity > 0x3fffffff || head_dim <= 0)
        return qmm_fail(IZWI_QMM_ERR_INVALID,
                        "decode_gqa_attention: bad shape (heads %lld, kv heads %lld, head_dim %lld, kv_len %lld of %lld)",
                        (long long)num_heads, (long long)num_kv_heads, (long long)head_dim, (long long)kv_len,
                        (long long)kv_capacity);
    if (head_dim != 64 && head_dim != 128 && head_dim != 256)
        return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "decode_gqa_attention: head_dim %lld (64, 128 and 256 are built)",
                        (long long)head_dim);
    if (!q || !k || !v || !out) return qmm_fail(IZWI_QMM_ERR_INVALID, "decode_gqa_attention: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    const size_t qbytes = (size_t)num_heads * head_dim * sizeof(T);
    const size_t cbytes = (size_t)num_kv_heads * kv_capacity * head_dim * sizeof(T);
    Buf qi, ki, vi, oo;
    OPS_TRY(qi.in(q, qbytes, mem_space));
    OPS_TRY(ki.in(k, cbytes, mem_space));
    OPS_TRY(vi.in(v, cbytes, mem_space));
    OPS_TRY(oo.out(out, qbytes, mem_space));
    const int group = (int)(num_heads / num_kv_heads);
    // query heads per workgroup: as many of the group as the register file takes
    int g = group % 4 == 0 && head_dim <= 128 ? 4 : (group % 2 == 0 ? 2 : 1);
    const int z = group / g;
    // Enough workgroups for one per CU (IZWI_ATTN_WGS_PER_CU, tuning knob), at least 32 positions
    // each (IZWI_ATTN_MIN_CHUNK: one per row group of a workgroup, a single round of loads; 64 was
    // 4 % slower on a whole decode step at 256 positions, 16 no faster): more splits only add
    // merge work (measured: 2 per CU is 5-10 % slower between 4k and 16k positions, 4 per CU 30 %).
    static const int wgs_per_cu = [] { const char* e = getenv("IZWI_ATTN_WGS_PER_CU"); int v = e ? atoi(e) : 1; return v > 0 ? v : 1; }();
    static const int min_chunk = [] { const char* e = getenv("IZWI_ATTN_MIN_CHUNK"); int v = e ? atoi(e) : 32; return v > 0 ? v : 32; }();
    const int64_t base_wgs = num_kv_heads * z;
    int64_t splits = (wgs_per_cu * (int64_t)n_cus + base_wgs - 1) / base_wgs;
    const int64_t max_splits = (kv_len + min_chunk - 1) / min_chunk;
    if (splits > max_splits) splits = max_splits;
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits < 1) splits = 1;
    const int chunk = (int)((kv_len + splits - 1) / splits);
    splits = (kv_len + chunk - 1) / chunk; // every split holds at least one position
    AttnParams<T> P;
    P.q = (const T*)qi.dev;
    P.k = (const T*)ki.dev;
    P.v = (const T*)vi.dev;
    P.out = (T*)oo.dev;
    P.part = nullptr;
    P.heads = (int)num_heads;
    P.kv_heads = (int)num_kv_heads;
    P.group = group;
    P.kv_len = (int)kv_len;
    P.chunk = chunk;
    P.splits = (int)splits;
    P.kv_capacity = kv_capacity;
    P.scale = scale;
    P.k_new = P.v_new = P.qk_weight = P.cos_sin = nullptr;
    P.k_append = P.v_append = nullptr;
    P.eps = 0.0f;
    if (prep) { // device pointers only (checked by the caller): the caches are written in place
        P.k_new = prep->k_new, P.v_new = prep->v_new, P.qk_weight = prep->qk_weight, P.cos_sin = prep->cos_sin;
        P.k_append = (float*)ki.dev, P.v_append = (float*)vi.dev;
        P.eps = prep->eps;
    }
    QmmCallScope call; // the split partials stay this call's until the merge is queued
    if (splits > 1) {
        void* scratch = nullptr;
        OPS_TRY(qmm_get_scratch(device, stream, (size_t)num_heads * splits * (head_dim + 2) * sizeof(float), &scratch));
        P.part = (float*)scratch;
    }
    const dim3 grid((unsigned)num_kv_heads, (unsigned)splits, (unsigned)z);
    hipError_t e = head_dim == 64    ? launch_attn_partial<T, 64>(P, g, grid, stream)
                   : head_dim == 128 ? launch_attn_partial<T, 128>(P, g, grid, stream)
                                     : launch_attn_partial<T, 256>(P, g, grid, stream);
    OPS_TRY(e);
    if (splits > 1) {
        attn_merge_kernel<T><<<(unsigned)num_heads, 256, 0, stream>>>(P.part, P.out, (int)splits, (int)head_dim);
        OPS_TRY(hipGetLastError());
    }
    OPS_TRY(oo.finish(stream));
    return IZWI_QMM_OK;
}


} // namespace

extern "C" {

int izwi_rms_norm_f32(const float* x, const float* weight, int64_t rows, int64_t hidden, float eps, float* y,
                      int mem_space, void* stream) {
    return qmm_guarded("izwi_rms_norm_f32", [&]() -> int {
    return rms_norm_impl<float>(x, weight, rows, hidden, eps, y, mem_space, stream);
    });
}
int izwi_rms_norm_quantize_records_f32(int ggml_weight_dtype, const float* x, const float* weight, int64_t rows,
                                       int64_t hidden, float eps, void* records, void* stream) {
    return qmm_guarded("izwi_rms_norm_quantize_records_f32", [&]() -> int {
    if (ggml_weight_dtype != IZWI_QMM_Q8_0 && ggml_weight_dtype != IZWI_QMM_Q4_K && ggml_weight_dtype != IZWI_QMM_Q6_K)
        return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "ggml dtype %d is not supported", ggml_weight_dtype);
    if (rows < 0 || hidden <= 0) return qmm_fail(IZWI_QMM_ERR_INVALID, "rms_norm: bad shape [%lld, %lld]", (long long)rows, (long long)hidden);
    if (hidden % 256 || hidden > 16384)
        return qmm_fail(IZWI_QMM_ERR_UNSUPPORTED, "rms_norm into records: hidden = %lld is not a multiple of 256 up to 16384",
                        (long long)hidden);
    if (rows == 0) return IZWI_QMM_OK;
    if (!x || !weight || !records) return qmm_fail(IZWI_QMM_ERR_INVALID, "rms_norm: NULL buffer");
    if (!aligned16(x) || !aligned16(weight) || !aligned16(records))
        return qmm_fail(IZWI_QMM_ERR_INVALID, "rms_norm into records: buffers must be 16-byte aligned");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    NormParams<float> P{x, nullptr, weight, nullptr, nullptr, nullptr, rows, 0, (int)hidden, eps,
                        static_cast<uint8_t*>(records), (rows + 15) / 16 * 16};
    OPS_TRY(launch_norm_records(P, ggml_weight_dtype, (hipStream_t)stream));
    return IZWI_QMM_OK;
    });
}
int izwi_rms_norm_f16(const uint16_t* x, const uint16_t* weight, int64_t rows, int64_t hidden, float eps, uint16_t* y,
                      int mem_space, void* stream) {
    return qmm_guarded("izwi_rms_norm_f16", [&]() -> int {
    return rms_norm_impl<f16_t>((const f16_t*)x, (const f16_t*)weight, rows, hidden, eps, (f16_t*)y, mem_space, stream);
    });
}

int izwi_qk_rms_norm_f32(const float* q, const float* k, const float* qk_weight, int64_t q_rows, int64_t k_rows,
                         int64_t head_dim, float eps, float* q_out, float* k_out, int mem_space, void* stream) {
    return qmm_guarded("izwi_qk_rms_norm_f32", [&]() -> int {
    return qk_rms_norm_impl<float>(q, k, qk_weight, q_rows, k_rows, head_dim, eps, q_out, k_out, mem_space, stream);
    });
}
int izwi_qk_rms_norm_f16(const uint16_t* q, const uint16_t* k, const uint16_t* qk_weight, int64_t q_rows, int64_t k_rows,
                         int64_t head_dim, float eps, uint16_t* q_out, uint16_t* k_out, int mem_space, void* stream) {
    return qmm_guarded("izwi_qk_rms_norm_f16", [&]() -> int {
    return qk_rms_norm_impl<f16_t>((const f16_t*)q, (const f16_t*)k, (const f16_t*)qk_weight, q_rows, k_rows, head_dim, eps,
                                   (f16_t*)q_out, (f16_t*)k_out, mem_space, stream);
    });
}

int izwi_rope_pair_bshd_f32(const float* q, const float* k, const float* cos_sin, int64_t batch, int64_t seq,
                            int64_t q_heads, int64_t k_heads, int64_t head_dim, float* q_out, float* k_out,
                            int mem_space, void* stream) {
    return qmm_guarded("izwi_rope_pair_bshd_f32", [&]() -> int {
    return rope_pair_impl<float>(q, k, cos_sin, batch, seq, q_heads, k_heads, head_dim, q_out, k_out, mem_space, stream);
    });
}
int izwi_rope_pair_bshd_f16(const uint16_t* q, const uint16_t* k, const uint16_t* cos_sin, int64_t batch, int64_t seq,
                            int64_t q_heads, int64_t k_heads, int64_t head_dim, uint16_t* q_out, uint16_t* k_out,
                            int mem_space, void* stream) {
    return qmm_guarded("izwi_rope_pair_bshd_f16", [&]() -> int {
    return rope_pair_impl<f16_t>((const f16_t*)q, (const f16_t*)k, (const f16_t*)cos_sin, batch, seq, q_heads, k_heads,
                                 head_dim, (f16_t*)q_out, (f16_t*)k_out, mem_space, stream);
    });
}

namespace {
// `argmax_calls` / `argmax_ms` of the reference's ASR profile (asr/mod.rs:116-131): counted and,
// outside a capture, timed to completion when profiling is on.
struct ArgmaxProfile {
    bool on;
    hipStream_t stream;
    std::chrono::steady_clock::time_point t0;
    explicit ArgmaxProfile(hipStream_t s) : on(qmm_profiling()), stream(s) {
        if (on) t0 = std::chrono::steady_clock::now();
    }
    ~ArgmaxProfile() {
        if (!on) return;
        if (!qmm_stream_is_capturing(stream)) (void)hipStreamSynchronize(stream);
        qmm_profile_count_argmax((uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
                                     std::chrono::steady_clock::now() - t0).count());
    }
};
} // namespace

int izwi_argmax_f32(const float* logits, int64_t rows, int64_t n, uint32_t* out, int mem_space, void* stream_) {
    return qmm_guarded("izwi_argmax_f32", [&]() -> int {
    QmmCallScope call;
    ArgmaxProfile prof((hipStream_t)stream_);
    if (int rc = check_space(mem_space)) return rc;
    if (rows < 0 || n <= 0 || n > 0xfffffffeLL || rows > 0x7fffffff)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "argmax: bad shape [%lld, %lld]", (long long)rows, (long long)n);
    if (rows == 0) return IZWI_QMM_OK;
    if (!logits || !out) return qmm_fail(IZWI_QMM_ERR_INVALID, "argmax: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    hipStream_t stream = (hipStream_t)stream_;
    Buf li, oo;
    OPS_TRY(li.in(logits, (size_t)rows * n * sizeof(float), mem_space));
    OPS_TRY(oo.out(out, (size_t)rows * sizeof(uint32_t), mem_space));
    if (n > 16384 && rows < 2 * (int64_t)n_cus) {
        // too few rows to fill the GPU with one workgroup each: chunks of the row, then a merge
        const int64_t chunk = 2048;
        const int64_t parts = (n + chunk - 1) / chunk;
        void* scratch = nullptr;
        OPS_TRY(qmm_get_scratch(device, stream, (size_t)rows * parts * 8, &scratch));
        float* pv = (float*)scratch;
        uint32_t* pi = (uint32_t*)scratch + rows * parts;
        argmax_part_kernel<<<dim3((unsigned)rows, (unsigned)parts), 256, 0, stream>>>((const float*)li.dev, n, chunk, pv, pi);
        OPS_TRY(hipGetLastError());
        argmax_final_kernel<<<(unsigned)rows, 64, 0, stream>>>(pv, pi, (int)parts, (uint32_t*)oo.dev);
        OPS_TRY(hipGetLastError());
    } else {
        int threads = 64;
        while (threads < 1024 && threads * 4 < n) threads *= 2;
        argmax_kernel<<<(unsigned)rows, threads, 0, stream>>>((const float*)li.dev, n, (uint32_t*)oo.dev);
        OPS_TRY(hipGetLastError());
    }
    OPS_TRY(oo.finish(stream));
    return IZWI_QMM_OK;
    });
}

int izwi_qk_norm_rope_append_f32(const float* q, const float* k, const float* v, const float* qk_weight,
                                 const float* cos_sin, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                 float eps, float* q_out, float* k_cache, float* v_cache, int64_t kv_capacity,
                                 int64_t pos, void* stream_) {
    return qmm_guarded("izwi_qk_norm_rope_append_f32", [&]() -> int {
    if (num_heads <= 0 || num_kv_heads <= 0 || num_heads + 2 * num_kv_heads > 0x3fffffff || head_dim <= 0 ||
        head_dim % 2 || head_dim > 8192 || pos < 0 || pos >= kv_capacity)
        return qmm_fail(IZWI_QMM_ERR_INVALID,
                        "qk_norm_rope_append: bad shape (heads %lld, kv heads %lld, head_dim %lld, position %lld of %lld)",
                        (long long)num_heads, (long long)num_kv_heads, (long long)head_dim, (long long)pos,
                        (long long)kv_capacity);
    if (!q || !k || !v || !qk_weight || !cos_sin || !q_out || !k_cache || !v_cache)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "qk_norm_rope_append: NULL buffer");
    int device = 0, n_cus = 0;
    if (int rc = qmm_current_device(&device, &n_cus)) return rc;
    QkvPrepParams P{q, k, v, qk_weight, cos_sin, q_out, k_cache, v_cache, (int)num_heads, (int)num_kv_heads,
                    (int)head_dim, kv_capacity, pos, eps};
    const int64_t rows = num_heads + 2 * num_kv_heads;
    qkv_prep_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, (hipStream_t)stream_>>>(P);
    OPS_TRY(hipGetLastError());
    return IZWI_QMM_OK;
    });
}

int izwi_decode_attention_step_f32(const float* q, const float* k, const float* v, const float* qk_weight,
                                   const float* cos_sin, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                   float eps, float* k_cache, float* v_cache, int64_t kv_capacity, int64_t pos,
                                   float scale, float* out, void* stream) {
    return qmm_guarded("izwi_decode_attention_step_f32", [&]() -> int {
    if (pos < 0 || pos >= kv_capacity)
        return qmm_fail(IZWI_QMM_ERR_INVALID, "decode_attention_step: position %lld of %lld", (long long)pos,
                        (long long)kv_capacity);
    if (!k || !v || !qk_weight || !cos_sin) return qmm_fail(IZWI_QMM_ERR_INVALID, "decode_attention_step: NULL buffer");
    const AttnPrep prep{k, v, qk_weight, cos_sin, eps};
    return decode_attention_impl<float>(q, k_cache, v_cache, num_heads, num_kv_heads, head_dim, pos + 1, kv_capacity,
                                        scale, out, IZWI_QMM_DEVICE, stream, &prep);
    });
}

int izwi_decode_gqa_attention_f32(const float* q, const float* k, const float* v, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t kv_len, int64_t kv_capacity,
                                  float scale, float* out, int mem_space, void* stream) {
    return qmm_guarded("izwi_decode_gqa_attention_f32", [&]() -> int {
    return decode_attention_impl<float>(q, k, v, num_heads, num_kv_heads, head_dim, kv_len, kv_capacity, scale, out,
                                        mem_space, stream);
    });
}
int izwi_decode_gqa_attention_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t kv_len, int64_t kv_capacity,
                                  float scale, uint16_t* out, int mem_space, void* stream) {
    return qmm_guarded("izwi_decode_gqa_attention_f16", [&]() -> int {
    return decode_attention_impl<f16_t>((const f16_t*)q, (const f16_t*)k, (const f16_t*)v, num_heads, num_kv_heads,
                                        head_dim, kv_len, kv_capacity, scale, (f16_t*)out, mem_space, stream);
    });
}

} // extern "C"
