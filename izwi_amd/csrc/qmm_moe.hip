// MoE routing, expert sort and weighted combine.  All index work is integer
// arithmetic with a fixed order, so ids / perm / offsets do not depend on
// scheduling: same input, same bits.
#include <hip/hip_runtime.h>

#include "qmm_internal.h"
#include "qmm_gemv_blocks.h"
#include "qmm_moe_route.h"

namespace {

constexpr int kSortChunk = 256; // pairs per chunk of the sort

using moe_route::route_token;

// The x blocks of one token row, for weights of block type `dot_dtype` (a wave; xb.xq == nullptr:
// nothing).  The loads are issued before the routing and used after it.
__device__ __forceinline__ void token_x_issue(const float* __restrict__ x, int64_t tok, int k, const XBlocks& xb,
                                              XRowLoads& ld) {
    if (xb.xq == nullptr) return; // uniform
    x_row_issue(x, tok, k, (k + 255) >> 8, ld);
}
__device__ __forceinline__ void token_to_x_blocks(const float* __restrict__ x, int64_t tok, int k, int dot_dtype,
                                                  const XBlocks& xb, const XRowLoads& ld) {
    if (xb.xq == nullptr) return; // uniform
    const int k_units = (k + 255) >> 8;
    if (dot_dtype == QMM_Q8_0) x_row_to_blocks<QMM_Q8_0>(x, tok, k, k_units, xb, ld);
    else if (dot_dtype == QMM_Q6_K) x_row_to_blocks<QMM_Q6_K>(x, tok, k, k_units, xb, ld);
    else x_row_to_blocks<QMM_Q4_K>(x, tok, k, k_units, xb, ld);
}

// One wavefront per token.  With x blocks to fill, a second wavefront per token (the second half of
// the workgroup) quantizes the token's activation row meanwhile (the rows the expert-grouped decode
// kernel would otherwise quantize in every workgroup of a segment; one wave doing both in turn made
// the launch as long as their sum, and the sort waits for this launch to end).
template <int PER_LANE>
__global__ void route_kernel(const float* __restrict__ logits, int64_t t, int n_experts, int top_k,
                             int32_t* __restrict__ ids, float* __restrict__ weights,
                             const float* __restrict__ x, int k, int dot_dtype, XBlocks xb) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tokens_per_block = xb.xq != nullptr ? blockDim.x >> 7 : blockDim.x >> 6;
    const bool quantizes = wave >= tokens_per_block; // (uniform per wave)
    const int64_t tok = (int64_t)blockIdx.x * tokens_per_block + (quantizes ? wave - tokens_per_block : wave);
    if (tok >= t) return; // whole waves leave together
    if (quantizes) {
        XRowLoads ld;
        token_x_issue(x, tok, k, xb, ld);
        token_to_x_blocks(x, tok, k, dot_dtype, xb, ld);
        return;
    }
    int id;
    float w;
    route_token<PER_LANE>(logits + tok * n_experts, n_experts, top_k, lane, id, w);
    if (lane < top_k) {
        ids[tok * top_k + lane] = id;
        weights[tok * top_k + lane] = w;
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
                                 int32_t* __restrict__ offsets, int32_t* __restrict__ seg_offsets, int seg_rows,
                                 int32_t* __restrict__ seg_expert, int max_segments) {
    extern __shared__ int32_t sh[]; // totals[n_experts]
    __shared__ int32_t total_segments;
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        int32_t tot = 0;
        for (int64_t c = 0; c < chunks; c++) tot += hist[c * n_experts + e];
        sh[e] = tot;
    }
    __syncthreads();
    if (n_experts <= (int)blockDim.x) {
        // few experts: thread e sums the totals before it (LDS broadcast reads), no serial chain
        const int e = threadIdx.x;
        int32_t run = 0, seg = 0;
        for (int i = 0; i < e && i < n_experts; i++) {
            const int32_t c = sh[i];
            run += c;
            seg += (c + seg_rows - 1) / seg_rows;
        }
        __syncthreads();
        if (e < n_experts) {
            offsets[e] = run;
            if (seg_offsets) seg_offsets[e] = seg;
            const int32_t c = sh[e];
            if (seg_expert)
                for (int i = 0, n = (c + seg_rows - 1) / seg_rows; i < n && seg + i < max_segments; i++) seg_expert[seg + i] = e;
            if (e == n_experts - 1) {
                offsets[n_experts] = run + c;
                if (seg_offsets) seg_offsets[n_experts] = seg + (c + seg_rows - 1) / seg_rows;
                total_segments = seg + (c + seg_rows - 1) / seg_rows;
            }
            sh[e] = run;
        }
    } else if (threadIdx.x == 0) {
        int32_t run = 0, seg = 0;
        for (int e = 0; e < n_experts; e++) {
            int32_t c = sh[e];
            offsets[e] = run;
            if (seg_offsets) seg_offsets[e] = seg;
            sh[e] = run;
            run += c;
            if (seg_expert)
                for (int i = 0, n = (c + seg_rows - 1) / seg_rows; i < n && seg + i < max_segments; i++) seg_expert[seg + i] = e;
            seg += (c + seg_rows - 1) / seg_rows;
        }
        offsets[n_experts] = run;
        if (seg_offsets) seg_offsets[n_experts] = seg;
        total_segments = seg;
    }
    __syncthreads();
    if (seg_expert) // entries past the last segment say so
        for (int i = total_segments + (int)threadIdx.x; i < max_segments; i += blockDim.x) seg_expert[i] = -1;
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

// Rank of every lane's id among the equal ids of earlier lanes of its wave, and the number of lanes
// that hold it: the lanes OR their bit into a 64-bit mask per expert in LDS (an OR is order-free), then
// count the bits below their own.  `masks` = the wave's own [n_experts] pairs of 32-bit words, zeroed here.
__device__ __forceinline__ void wave_ranks(int e, int n_experts, int lane, uint32_t* masks, int& rank, int& total) {
    for (int i = lane; i < 2 * n_experts; i += 64) masks[i] = 0u;
    __builtin_amdgcn_wave_barrier();
    const bool ok = e >= 0 && e < n_experts;
    if (ok) atomicOr(&masks[2 * e + (lane >> 5)], 1u << (lane & 31));
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const uint32_t lo = ok ? masks[2 * e] : 0u, hi = ok ? masks[2 * e + 1] : 0u;
    const uint32_t below_lo = lane < 32 ? lo & ((1u << lane) - 1u) : lo;
    const uint32_t below_hi = lane < 32 ? 0u : hi & ((1u << (lane & 31)) - 1u);
    rank = __popc(below_lo) + __popc(below_hi);
    total = __popc(lo) + __popc(hi);
    __builtin_amdgcn_wave_barrier(); // the masks are reused by the wave's next run
}

// inclusive sum over the 64 lanes of a wave: shifts inside the 16-lane rows, then the last lane of a
// row broadcast to the rows behind it (data-parallel primitives on the vector ALU: six adds; the
// shuffle form goes through the LDS crossbar six times).  All lanes must be active.
__device__ __forceinline__ int wave_inclusive_sum(int v, int lane) {
    (void)lane;
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false); // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false); // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false); // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false); // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false); // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false); // row_bcast:31 into rows 2 and 3
    return v;
}

// The whole stable counting sort in ONE workgroup (pairs up to 16384, n_experts up to 1024 as far as
// LDS holds runs x experts counters): pairs are cut into runs of 64 (one wave each); a lane finds its
// rank among the equal ids of its run through per-expert bit masks; the runs' per-expert counts are
// scanned run by run (a wave per expert, a lane per run) and over the experts (wave scans); every
// pair goes to offsets[e] + (pairs of e in earlier runs) + rank.  Integer arithmetic whose result does
// not depend on the order of execution: the same perm / offsets as the three-kernel sort.
// `ids`: the pairs' experts, in global memory or in LDS (the one-launch plan of small batches routes
// them there first).  `sh`: block_sort_lds_ints(pairs, n_experts) ints of LDS.  Called by all
// kBlockSortThreads threads of the workgroup.
constexpr int kBlockSortThreads = 1024, kBlockSortMaxRuns = 16; // runs per wave
constexpr int kBlockSortMaxLds = 152 * 1024; // (of the CU's 160 KB: 16384 pairs of 128 experts take 149 KB)
__host__ __device__ inline int64_t block_sort_lds_ints(int64_t pairs, int n_experts) {
    return ((pairs + 63) / 64) * (n_experts | 1) + n_experts + 1 + (int64_t)2 * n_experts * (kBlockSortThreads / 64);
}
__device__ __forceinline__ void block_sort_body(const int32_t* ids, int pairs, int n_experts, int32_t* __restrict__ perm,
                                                int32_t* __restrict__ offsets, int32_t* __restrict__ seg_offsets,
                                                int seg_rows, int32_t* __restrict__ seg_expert, int max_segments,
                                                int32_t* sh, int32_t* __restrict__ expert_order = nullptr) {
    // hist[runs][stride] | start[n_experts + 1] | masks[waves][2 * n_experts]; the rows of hist have an odd
    // stride: a wave that reads one expert's count of 64 runs would otherwise hit one LDS bank 64 times
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = kBlockSortThreads / 64;
    const int runs = (pairs + 63) / 64;
    const int stride = n_experts | 1;
    int32_t* start = sh + runs * stride;
    uint32_t* masks = reinterpret_cast<uint32_t*>(start + n_experts + 1) + wave * 2 * n_experts;
    __shared__ int32_t wave_tot[16], wave_seg[16], total_segments;
    int my_e[kBlockSortMaxRuns], my_rank[kBlockSortMaxRuns];
    // all ids of the wave's runs are requested before anything waits for one
#pragma unroll
    for (int j = 0; j < kBlockSortMaxRuns; j++) {
        const int p = (wave + j * waves) * 64 + lane;
        my_e[j] = p < pairs ? ids[p] : -1;
    }
    for (int i = threadIdx.x; i < runs * stride; i += kBlockSortThreads) sh[i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kBlockSortMaxRuns; j++) {
        const int run = wave + j * waves;
        my_rank[j] = 0;
        if (run >= runs) continue; // uniform per wave
        const int e = my_e[j];
        int rank, total;
        wave_ranks(e, n_experts, lane, masks, rank, total);
        my_rank[j] = rank;
        if (e >= 0 && e < n_experts && rank == 0) sh[run * stride + e] = total; // the first of its expert in the run
    }
    __syncthreads();
    // per expert (a wave each, in turn): the runs' counts become the number of earlier pairs of the
    // expert; lane = run, 64 runs per step
    // (few runs: a thread per expert walks them - consecutive experts, consecutive LDS words - instead
    // of eight wave scans in a row per wave with two lanes in use)
    if (runs <= 64) {
        for (int e = threadIdx.x; e < n_experts; e += kBlockSortThreads) {
            int carry = 0;
            for (int r = 0; r < runs; r++) {
                const int h = sh[r * stride + e];
                sh[r * stride + e] = carry;
                carry += h;
            }
            start[e] = carry;
        }
    } else {
        for (int e = wave; e < n_experts; e += waves) {
            int carry = 0;
            for (int r0 = 0; r0 < runs; r0 += 64) {
                const int r = r0 + lane;
                const int h = r < runs ? sh[r * stride + e] : 0;
                const int inc = wave_inclusive_sum(h, lane);
                if (r < runs) sh[r * stride + e] = carry + inc - h;
                carry += __shfl(inc, 63);
            }
            if (lane == 0) start[e] = carry; // the expert's total, for now
        }
    }
    __syncthreads();
    // exclusive scan over the experts: thread e holds expert e (n_experts <= 1024), wave scans, then the
    // waves' totals
    const int e0 = threadIdx.x;
    const int c = e0 < n_experts ? start[e0] : 0;
    const int sg = (c + seg_rows - 1) / seg_rows;
    const int inc_c = wave_inclusive_sum(c, lane), inc_s = wave_inclusive_sum(sg, lane);
    if (lane == 63) wave_tot[wave] = inc_c, wave_seg[wave] = inc_s;
    __syncthreads();
    int base_c = 0, base_s = 0;
    for (int w = 0; w < wave; w++) base_c += wave_tot[w], base_s += wave_seg[w];
    if (e0 <= n_experts) {
        // (thread n_experts holds the grand totals: its own c is 0)
        offsets[e0] = base_c + inc_c - c;
        if (seg_offsets) seg_offsets[e0] = base_s + inc_s - sg;
        start[e0] = base_c + inc_c - c;
        // segment -> expert (the segments of expert e0 are consecutive)
        if (seg_expert)
            for (int i = 0, first = base_s + inc_s - sg; i < sg && first + i < max_segments; i++) seg_expert[first + i] = e0;
        if (e0 == n_experts) total_segments = base_s + inc_s;
    }
    int32_t* counts = start + n_experts + 1; // (the first wave's bit masks: done with) counts | ranks
    if (expert_order && e0 < n_experts) counts[e0] = sg, counts[n_experts + e0] = 0;
    __syncthreads();
    // entries past the last segment say so (the grouped decode launch has one workgroup per entry)
    if (seg_expert)
        for (int i = total_segments + (int)threadIdx.x; i < max_segments; i += kBlockSortThreads) seg_expert[i] = -1;
#pragma unroll
    for (int j = 0; j < kBlockSortMaxRuns; j++) {
        const int run = wave + j * waves;
        if (run >= runs) continue;
        const int e = my_e[j];
        if (e >= 0 && e < n_experts) perm[start[e] + sh[run * stride + e] + my_rank[j]] = run * 64 + lane;
    }
    // the experts by falling segment count, ties by index (behind the stores above, which drain
    // meanwhile): all threads share the comparisons, thread (expert, slice of the experts) adds its
    // part of the expert's rank (integer adds: order-free)
    if (expert_order) { // (uniform)
        const int slices = max(1, kBlockSortThreads / n_experts), per = (n_experts + slices - 1) / slices;
        const int e = (int)threadIdx.x % n_experts, slice = (int)threadIdx.x / n_experts;
        if (slice < slices) {
            const int mine = counts[e];
            int part = 0;
            for (int o = slice * per, o_end = min(n_experts, o + per); o < o_end; o++) {
                const int co = counts[o];
                part += (co > mine || (co == mine && o < e)) ? 1 : 0;
            }
            if (part) atomicAdd(&counts[n_experts + e], part);
        }
        __syncthreads();
        if (e0 < n_experts) {
            // (a permutation: every slot is written once) the expert and where its segments and pairs sit
            int32_t* d = expert_order + 8 * counts[n_experts + e0];
            d[0] = e0, d[1] = base_s + inc_s - sg, d[2] = sg, d[3] = base_c + inc_c - c, d[4] = base_c + inc_c;
        }
    }
}

__global__ __launch_bounds__(kBlockSortThreads) void sort_block_kernel(const int32_t* __restrict__ ids, int pairs,
                                                                       int n_experts, int32_t* __restrict__ perm,
                                                                       int32_t* __restrict__ offsets,
                                                                       int32_t* __restrict__ seg_offsets, int seg_rows,
                                                                       int32_t* __restrict__ seg_expert, int max_segments,
                                                                       int32_t* __restrict__ expert_order) {
    extern __shared__ int32_t sh[];
    block_sort_body(ids, pairs, n_experts, perm, offsets, seg_offsets, seg_rows, seg_expert, max_segments, sh, expert_order);
}

bool block_sort_fits(int64_t pairs, int n_experts) {
    if (pairs < 1 || n_experts >= kBlockSortThreads) return false;
    const int64_t runs = (pairs + 63) / 64;
    return runs <= (int64_t)kBlockSortMaxRuns * (kBlockSortThreads / 64) && block_sort_lds_ints(pairs, n_experts) * 4 <= kBlockSortMaxLds;
}

// seg_offsets[e] = sum over e' < e of ceil(count(e') / seg_rows).  One block:
// every thread sums a contiguous run of experts, the runs are scanned in LDS.
// With seg_expert: seg_expert[s] = expert of segment s, -1 for s past the last
// segment (up to max_segments entries).
// With expert_order (n_experts <= kSegmentsRankedExperts): the table of the ranked experts that the
// one-workgroup sort writes (see block_sort_body).
constexpr int kSegmentsRankedExperts = 512;
__global__ void segments_kernel(const int32_t* __restrict__ offsets, int n_experts, int seg_rows,
                                int32_t* __restrict__ seg_offsets, int32_t* __restrict__ seg_expert,
                                int max_segments, int32_t* __restrict__ expert_order) {
    __shared__ int32_t part[256];
    __shared__ int32_t counts[kSegmentsRankedExperts];
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
        if (expert_order) counts[e] = n;
        run += n;
    }
    if (expert_order) { // (uniform) the experts by falling segment count, ties by index
        __syncthreads();
        int32_t first = part[threadIdx.x] - sum;
        for (int e = e0; e < e1; e++) {
            const int32_t n = counts[e];
            int rank = 0;
            for (int o = 0; o < n_experts; o++) {
                const int co = counts[o];
                rank += (co > n || (co == n && o < e)) ? 1 : 0;
            }
            int32_t* d = expert_order + 8 * rank;
            d[0] = e, d[1] = first, d[2] = n, d[3] = offsets[e], d[4] = offsets[e + 1];
            first += n;
        }
    }
    const int32_t total = part[255];
    if (threadIdx.x == 255) seg_offsets[n_experts] = total;
    if (seg_expert)
        for (int s = total + threadIdx.x; s < max_segments; s += 256) seg_expert[s] = -1;
}

// Small batches (up to kPlanMaxTokens tokens): routing, stable counting sort and the segment tables of
// the grouped decode kernel in ONE workgroup and launch: a wave routes a token (all tokens at once), the
// ids stay in LDS and go through the one-workgroup sort above.  Results equal route_kernel + sort_* +
// segments_kernel bit for bit (same routing function, integer-only sort).  (A first version ran four
// waves, routed the tokens four at a time and ranked every pair against all earlier ones: 17.6 us at 16
// tokens, 54 us at 64, where routing and sort as two launches take 10.)
constexpr int kPlanMaxTokens = kBlockSortThreads / 64, kPlanMaxExperts = 256;
template <int PER_LANE>
__global__ __launch_bounds__(kBlockSortThreads) void moe_plan_small_kernel(
    const float* __restrict__ logits, int t, int n_experts, int top_k, int max_segments,
    int32_t* __restrict__ ids, float* __restrict__ weights, int32_t* __restrict__ perm,
    int32_t* __restrict__ offsets, int32_t* __restrict__ seg_offsets, int32_t* __restrict__ seg_expert) {
    extern __shared__ int32_t sh[]; // the sort's counters | the ids
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pairs = t * top_k;
    int32_t* s_ids = sh + block_sort_lds_ints(pairs, n_experts);
    if (wave < t) { // uniform per wave
        int id;
        float w;
        route_token<PER_LANE>(logits + (int64_t)wave * n_experts, n_experts, top_k, lane, id, w);
        if (lane < top_k) {
            ids[wave * top_k + lane] = id;
            weights[wave * top_k + lane] = w;
            s_ids[wave * top_k + lane] = id;
        }
    }
    __syncthreads();
    block_sort_body(s_ids, pairs, n_experts, perm, offsets, seg_offsets, QMM_MOE_SEG_ROWS, seg_expert, max_segments, sh);
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

// The same sums, four columns per thread, the loads of eight slots requested before the first is
// used (the loop above waits for one slot's load per step: eight round trips in a row).  The slots
// are still added in order s = 0, 1, ..: the same bits.
__global__ void combine4_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                                int64_t t, int top_k, int64_t hidden4, float* __restrict__ out) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= t * hidden4) return;
    const int64_t tok = idx / hidden4, c4 = idx - tok * hidden4;
    const float4* yr = reinterpret_cast<const float4*>(y) + tok * top_k * hidden4 + c4;
    const float* w = weights + tok * top_k;
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int s0 = 0; s0 < top_k; s0 += 8) {
        float4 v[8];
        float ww[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int s = s0 + i < top_k ? s0 + i : top_k - 1; // (a slot past the end: a valid address, unused)
            v[i] = yr[s * hidden4];
            ww[i] = w[s];
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (s0 + i < top_k) { // uniform
                acc.x += ww[i] * v[i].x, acc.y += ww[i] * v[i].y;
                acc.z += ww[i] * v[i].z, acc.w += ww[i] * v[i].w;
            }
        }
    }
    reinterpret_cast<float4*>(out)[idx] = acc;
}

} // namespace

size_t qmm_x_blocks_bytes(int64_t rows, int64_t k) { return x_blocks_bytes(rows, (k + 255) / 256); }

hipError_t qmm_launch_moe_route(const float* logits, int64_t t, int n_experts, int top_k,
                                int32_t* ids, float* weights, hipStream_t stream,
                                const float* x, int64_t k, int dot_dtype, void* x_blocks) {
    if (t <= 0) return hipSuccess;
    if (x_blocks && (!x || k <= 0 || k > 0x3fffffff || k % 32)) return hipErrorInvalidValue;
    const XBlocks xb = x_blocks ? x_blocks_carve(x_blocks, t, (k + 255) / 256) : XBlocks{nullptr, nullptr, nullptr};
    if (n_experts < 1 || n_experts > 1024 || top_k < 1 || top_k > 64 || top_k > n_experts)
        return hipErrorInvalidValue;
    const int tokens_per_block = 4;
    unsigned grid = (unsigned)((t + tokens_per_block - 1) / tokens_per_block);
    const unsigned block = 64 * tokens_per_block * (x_blocks ? 2 : 1); // (a quantizing wave beside every routing wave)
    int per_lane = (n_experts + 63) / 64;
    if (per_lane <= 2)
        route_kernel<2><<<grid, block, 0, stream>>>(logits, t, n_experts, top_k, ids, weights, x, (int)k, dot_dtype, xb);
    else if (per_lane <= 4)
        route_kernel<4><<<grid, block, 0, stream>>>(logits, t, n_experts, top_k, ids, weights, x, (int)k, dot_dtype, xb);
    else
        route_kernel<16><<<grid, block, 0, stream>>>(logits, t, n_experts, top_k, ids, weights, x, (int)k, dot_dtype, xb);
    return hipGetLastError();
}

int64_t qmm_moe_sort_scratch_ints(int64_t pairs, int n_experts) {
    int64_t chunks = (pairs + kSortChunk - 1) / kSortChunk;
    if (chunks < 1) chunks = 1;
    return chunks * n_experts;
}

hipError_t qmm_launch_moe_sort(const int32_t* ids, int64_t pairs, int n_experts, int32_t* perm,
                               int32_t* offsets, int32_t* seg_offsets, int32_t* scratch,
                               hipStream_t stream, int seg_rows, int32_t* seg_expert, int64_t max_segments,
                               int32_t* expert_order) {
    if (seg_rows < 1 || max_segments > 0x7fffffff) return hipErrorInvalidValue;
    if (n_experts < 1 || n_experts > 8192) return hipErrorInvalidValue;
    if (expert_order && !block_sort_fits(pairs, n_experts)) return hipErrorInvalidValue; // (qmm_moe_sort_ranks_experts)
    if (block_sort_fits(pairs, n_experts)) {
        const size_t lds = (size_t)block_sort_lds_ints(pairs, n_experts) * sizeof(int32_t);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sort_block_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kBlockSortMaxLds);
            if (e != hipSuccess) return e;
        }
        sort_block_kernel<<<1, kBlockSortThreads, lds, stream>>>(ids, (int)pairs, n_experts, perm, offsets, seg_offsets, seg_rows, seg_expert, (int)max_segments, expert_order);
        return hipGetLastError();
    }
    int64_t chunks = (pairs + kSortChunk - 1) / kSortChunk;
    if (chunks < 1) chunks = 1;
    size_t sh = (size_t)n_experts * sizeof(int32_t);
    sort_hist_kernel<<<(unsigned)chunks, kSortChunk, sh, stream>>>(ids, pairs, n_experts, scratch);
    sort_scan_kernel<<<1, 256, sh, stream>>>(scratch, chunks, n_experts, offsets, seg_offsets, seg_rows, seg_expert,
                                             (int)max_segments);
    if (pairs > 0)
        sort_scatter_kernel<<<(unsigned)chunks, 128, 0, stream>>>(ids, pairs, n_experts, scratch,
                                                                  perm);
    return hipGetLastError();
}

bool qmm_moe_sort_ranks_experts(int64_t pairs, int n_experts) { return block_sort_fits(pairs, n_experts); }

bool qmm_moe_segments_rank_experts(int n_experts) { return n_experts <= kSegmentsRankedExperts; }

hipError_t qmm_launch_moe_segments(const int32_t* offsets, int n_experts, int seg_rows,
                                   int32_t* seg_offsets, int32_t* seg_expert, int64_t max_segments,
                                   hipStream_t stream, int32_t* expert_order) {
    if (expert_order && !qmm_moe_segments_rank_experts(n_experts)) return hipErrorInvalidValue;
    segments_kernel<<<1, 256, 0, stream>>>(offsets, n_experts, seg_rows, seg_offsets, seg_expert,
                                           (int)max_segments, expert_order);
    return hipGetLastError();
}

bool qmm_moe_plan_small_supported(int64_t t, int n_experts, int top_k) {
    return t > 0 && t <= kPlanMaxTokens && n_experts <= kPlanMaxExperts && top_k <= 64 && top_k <= n_experts &&
           block_sort_fits(t * top_k, n_experts) && (block_sort_lds_ints(t * top_k, n_experts) + t * top_k) * 4 <= 64 * 1024;
}

hipError_t qmm_launch_moe_plan_small(const float* logits, int64_t t, int n_experts, int top_k, int seg_rows,
                                     int64_t max_segments, int32_t* ids, float* weights, int32_t* perm,
                                     int32_t* offsets, int32_t* seg_offsets, int32_t* seg_expert,
                                     hipStream_t stream) {
    if (!qmm_moe_plan_small_supported(t, n_experts, top_k) || max_segments > 0x7fffffff || seg_rows != QMM_MOE_SEG_ROWS)
        return hipErrorInvalidValue;
    const size_t lds = (size_t)(block_sort_lds_ints(t * top_k, n_experts) + t * top_k) * sizeof(int32_t);
    const void* fn = n_experts <= 128 ? reinterpret_cast<const void*>(&moe_plan_small_kernel<2>)
                                      : reinterpret_cast<const void*>(&moe_plan_small_kernel<4>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
        if (e != hipSuccess) return e;
    }
    if (n_experts <= 128)
        moe_plan_small_kernel<2><<<1, kBlockSortThreads, lds, stream>>>(logits, (int)t, n_experts, top_k, (int)max_segments,
                                                                       ids, weights, perm, offsets, seg_offsets, seg_expert);
    else
        moe_plan_small_kernel<4><<<1, kBlockSortThreads, lds, stream>>>(logits, (int)t, n_experts, top_k, (int)max_segments,
                                                                       ids, weights, perm, offsets, seg_offsets, seg_expert);
    return hipGetLastError();
}

hipError_t qmm_launch_moe_combine(const float* y, const float* weights, int64_t t, int top_k,
                                  int64_t hidden, float* out, hipStream_t stream) {
    int64_t total = t * hidden;
    if (total <= 0) return hipSuccess;
    if (hidden % 4 == 0 && ((uintptr_t)y | (uintptr_t)out) % 16 == 0) {
        // (64 threads per workgroup: a few tokens still spread over many CUs)
        const int64_t total4 = total / 4;
        combine4_kernel<<<(unsigned)((total4 + 63) / 64), 64, 0, stream>>>(y, weights, t, top_k, hidden / 4, out);
        return hipGetLastError();
    }
    combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(y, weights, t, top_k,
                                                                        hidden, out);
    return hipGetLastError();
}
