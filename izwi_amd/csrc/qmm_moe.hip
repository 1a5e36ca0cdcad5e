// MoE routing, expert sort and weighted combine.  All index work is integer
// arithmetic with a fixed order, so ids / perm / offsets do not depend on
// scheduling: same input, same bits.
#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

constexpr int kSortChunk = 256; // pairs per chunk of the sort

// One wavefront per token.  Lane l holds logits l, l+64, ...; top_k rounds of
// a wave-wide arg-max (larger logit first, lower expert index on ties).
template <int PER_LANE>
__global__ void route_kernel(const float* __restrict__ logits, int64_t t, int n_experts, int top_k,
                             int32_t* __restrict__ ids, float* __restrict__ weights) {
    const int lane = threadIdx.x & 63;
    const int64_t tok = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (tok >= t) return; // whole waves leave together
    const float* row = logits + tok * n_experts;
    float v[PER_LANE];
    bool taken[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; i++) {
        int e = lane + 64 * i;
        v[i] = e < n_experts ? row[e] : 0.0f;
        taken[i] = e >= n_experts;
    }
    float my_logit = 0.0f; // lane s keeps the logit of slot s
    int my_id = 0;
    float lmax = 0.0f;
    for (int s = 0; s < top_k; s++) {
        // local candidate: first (lowest index) maximum among the lane's untaken values
        int best = -1;
        float bv = 0.0f;
#pragma unroll
        for (int i = 0; i < PER_LANE; i++) {
            if (!taken[i] && (best < 0 || v[i] > bv)) {
                best = lane + 64 * i;
                bv = v[i];
            }
        }
        int be = best < 0 ? 0x7fffffff : best;
        // NaN never wins a `>` comparison; treat it as the smallest value so that
        // the selection stays a total order
        bool bnan = bv != bv;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            float ov = __shfl_xor(bv, off);
            int oe = __shfl_xor(be, off);
            int onan = __shfl_xor((int)bnan, off);
            bool other_valid = oe != 0x7fffffff, self_valid = be != 0x7fffffff;
            bool take_other;
            if (!other_valid) take_other = false;
            else if (!self_valid) take_other = true;
            else if (onan != (int)bnan) take_other = bnan; // the non-NaN one wins
            else if (ov > bv) take_other = true;
            else if (ov < bv) take_other = false;
            else take_other = oe < be;
            if (take_other) {
                bv = ov;
                be = oe;
                bnan = onan != 0;
            }
        }
        if (s == 0) lmax = bv;
        if (lane == s) {
            my_logit = bv;
            my_id = be;
        }
        if ((be & 63) == lane) {
#pragma unroll
            for (int i = 0; i < PER_LANE; i++)
                if (i == (be >> 6)) taken[i] = true;
        }
    }
    // weights: exp(l - lmax) over the selected slots, summed in slot order
    float p = lane < top_k ? expf(my_logit - lmax) : 0.0f;
    float denom = 0.0f;
    for (int s = 0; s < top_k; s++) denom += __shfl(p, s);
    if (lane < top_k) {
        ids[tok * top_k + lane] = my_id;
        weights[tok * top_k + lane] = p / denom;
    }
}

// ---- sort ----------------------------------------------------------------
// hist[c][e] = number of pairs of chunk c routed to expert e
__global__ void sort_hist_kernel(const int32_t* __restrict__ ids, int64_t pairs, int n_experts,
                                 int32_t* __restrict__ hist) {
    extern __shared__ int32_t sh[];
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) sh[e] = 0;
    __syncthreads();
    int64_t p = (int64_t)blockIdx.x * kSortChunk + threadIdx.x;
    if (threadIdx.x < kSortChunk && p < pairs) {
        int32_t e = ids[p];
        if ((uint32_t)e < (uint32_t)n_experts) atomicAdd(&sh[e], 1); // integer adds: order-free
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x)
        hist[(int64_t)blockIdx.x * n_experts + e] = sh[e];
}

// One block: offsets = exclusive scan of the per-expert totals; hist[c][e] is
// replaced by the position where chunk c starts writing expert e.
__global__ void sort_scan_kernel(int32_t* __restrict__ hist, int64_t chunks, int n_experts,
                                 int32_t* __restrict__ offsets, int32_t* __restrict__ seg_offsets) {
    extern __shared__ int32_t sh[]; // totals[n_experts]
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        int32_t tot = 0;
        for (int64_t c = 0; c < chunks; c++) tot += hist[c * n_experts + e];
        sh[e] = tot;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int32_t run = 0, seg = 0;
        for (int e = 0; e < n_experts; e++) {
            int32_t c = sh[e];
            offsets[e] = run;
            if (seg_offsets) seg_offsets[e] = seg;
            sh[e] = run;
            run += c;
            seg += (c + QMM_MOE_SEG_ROWS - 1) / QMM_MOE_SEG_ROWS;
        }
        offsets[n_experts] = run;
        if (seg_offsets) seg_offsets[n_experts] = seg;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        int32_t run = sh[e];
        for (int64_t c = 0; c < chunks; c++) {
            int32_t h = hist[c * n_experts + e];
            hist[c * n_experts + e] = run;
            run += h;
        }
    }
}

// Thread e walks the chunk's ids in order and emits the pairs of expert e:
// ascending pair index inside every expert group (stable).
__global__ void sort_scatter_kernel(const int32_t* __restrict__ ids, int64_t pairs, int n_experts,
                                    const int32_t* __restrict__ start, int32_t* __restrict__ perm) {
    __shared__ int32_t chunk_ids[kSortChunk];
    const int64_t base = (int64_t)blockIdx.x * kSortChunk;
    const int count = (int)min((int64_t)kSortChunk, pairs - base);
    for (int i = threadIdx.x; i < count; i += blockDim.x) chunk_ids[i] = ids[base + i];
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        int32_t pos = start[(int64_t)blockIdx.x * n_experts + e];
        for (int i = 0; i < count; i++)
            if (chunk_ids[i] == e) perm[pos++] = (int32_t)(base + i);
    }
}

// seg_offsets[e] = sum over e' < e of ceil(count(e') / seg_rows).  One block:
// every thread sums a contiguous run of experts, the runs are scanned in LDS.
// With seg_expert: seg_expert[s] = expert of segment s, -1 for s past the last
// segment (up to max_segments entries).
__global__ void segments_kernel(const int32_t* __restrict__ offsets, int n_experts, int seg_rows,
                                int32_t* __restrict__ seg_offsets, int32_t* __restrict__ seg_expert,
                                int max_segments) {
    __shared__ int32_t part[256];
    const int per = (n_experts + 255) / 256;
    const int e0 = min(n_experts, (int)threadIdx.x * per), e1 = min(n_experts, e0 + per);
    int32_t sum = 0;
    for (int e = e0; e < e1; e++) sum += (offsets[e + 1] - offsets[e] + seg_rows - 1) / seg_rows;
    part[threadIdx.x] = sum;
    __syncthreads();
    // inclusive scan over the 256 partial sums (integers: any order gives the same result)
    for (int d = 1; d < 256; d <<= 1) {
        const int32_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += add;
        __syncthreads();
    }
    int32_t run = part[threadIdx.x] - sum;
    for (int e = e0; e < e1; e++) {
        seg_offsets[e] = run;
        const int32_t n = (offsets[e + 1] - offsets[e] + seg_rows - 1) / seg_rows;
        if (seg_expert)
            for (int32_t i = 0; i < n && run + i < max_segments; i++) seg_expert[run + i] = e;
        run += n;
    }
    const int32_t total = part[255];
    if (threadIdx.x == 255) seg_offsets[n_experts] = total;
    if (seg_expert)
        for (int s = total + threadIdx.x; s < max_segments; s += 256) seg_expert[s] = -1;
}

__global__ void combine_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                               int64_t t, int top_k, int64_t hidden, float* __restrict__ out) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= t * hidden) return;
    int64_t tok = idx / hidden, c = idx - tok * hidden;
    float acc = 0.0f;
    for (int s = 0; s < top_k; s++)
        acc += weights[tok * top_k + s] * y[(tok * top_k + s) * hidden + c];
    out[idx] = acc;
}

} // namespace

hipError_t qmm_launch_moe_route(const float* logits, int64_t t, int n_experts, int top_k,
                                int32_t* ids, float* weights, hipStream_t stream) {
    if (t <= 0) return hipSuccess;
    if (n_experts < 1 || n_experts > 1024 || top_k < 1 || top_k > 64 || top_k > n_experts)
        return hipErrorInvalidValue;
    const int waves_per_block = 4;
    unsigned grid = (unsigned)((t + waves_per_block - 1) / waves_per_block);
    int per_lane = (n_experts + 63) / 64;
    if (per_lane <= 2)
        route_kernel<2><<<grid, 256, 0, stream>>>(logits, t, n_experts, top_k, ids, weights);
    else if (per_lane <= 4)
        route_kernel<4><<<grid, 256, 0, stream>>>(logits, t, n_experts, top_k, ids, weights);
    else
        route_kernel<16><<<grid, 256, 0, stream>>>(logits, t, n_experts, top_k, ids, weights);
    return hipGetLastError();
}

int64_t qmm_moe_sort_scratch_ints(int64_t pairs, int n_experts) {
    int64_t chunks = (pairs + kSortChunk - 1) / kSortChunk;
    if (chunks < 1) chunks = 1;
    return chunks * n_experts;
}

hipError_t qmm_launch_moe_sort(const int32_t* ids, int64_t pairs, int n_experts, int32_t* perm,
                               int32_t* offsets, int32_t* seg_offsets, int32_t* scratch,
                               hipStream_t stream) {
    if (n_experts < 1 || n_experts > 8192) return hipErrorInvalidValue;
    int64_t chunks = (pairs + kSortChunk - 1) / kSortChunk;
    if (chunks < 1) chunks = 1;
    size_t sh = (size_t)n_experts * sizeof(int32_t);
    sort_hist_kernel<<<(unsigned)chunks, kSortChunk, sh, stream>>>(ids, pairs, n_experts, scratch);
    sort_scan_kernel<<<1, 256, sh, stream>>>(scratch, chunks, n_experts, offsets, seg_offsets);
    if (pairs > 0)
        sort_scatter_kernel<<<(unsigned)chunks, 128, 0, stream>>>(ids, pairs, n_experts, scratch,
                                                                  perm);
    return hipGetLastError();
}

hipError_t qmm_launch_moe_segments(const int32_t* offsets, int n_experts, int seg_rows,
                                   int32_t* seg_offsets, int32_t* seg_expert, int64_t max_segments,
                                   hipStream_t stream) {
    segments_kernel<<<1, 256, 0, stream>>>(offsets, n_experts, seg_rows, seg_offsets, seg_expert,
                                           (int)max_segments);
    return hipGetLastError();
}

hipError_t qmm_launch_moe_combine(const float* y, const float* weights, int64_t t, int top_k,
                                  int64_t hidden, float* out, hipStream_t stream) {
    int64_t total = t * hidden;
    if (total <= 0) return hipSuccess;
    combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(y, weights, t, top_k,
                                                                        hidden, out);
    return hipGetLastError();
}
