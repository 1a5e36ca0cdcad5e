// Decode kernel: fused activation-quantize + block dot products, M = 1, 2 and
// the expert-grouped segments of up to four rows.
//
// The arithmetic is candle-core's CPU `matmul` (quantize each activation row to
// the weight type's dot type, integer block dots, f32 scaling); only the f32
// summation order differs.  The work is bounded by streaming the weight bytes
// from HBM once:
//   * a wavefront reads a panel (16 rows x S units of 256 k-elements) as one
//     16 B/lane coalesced load for the headers plus 8 (Q4_K), 13 (Q6_K) or
//     16 (Q8_0) for the quants; lane (u, r) owns unit u of row r, so no weight byte is
//     shuffled between lanes and all nibble / int8 products run on
//     v_dot4_i32_i8 (about 0.7 VALU lane-ops per weight element);
//   * a wave issues its activation loads and then all loads of its panel before
//     anything else, unconditionally and in one basic block, so that the waits
//     can be counted: the activations are quantized while the panel flies, the
//     panel is multiplied chunk by chunk while its rest arrives;
//   * the workgroup quantizes the activations once into LDS (16 lanes per
//     256-value block, reductions on DPP); lanes of one 16-row group read the
//     same LDS words (broadcast), the unit stride is padded by 16 B so the S
//     groups hit different banks;
//   * the S partial sums of a row are combined with two cross-lane steps, the
//     k-split between the waves of a workgroup through LDS.
// The launch bound of 768 threads caps a wave at 168 registers (three waves per
// SIMD): a 28 MB matrix then fits in one round of 12-wave workgroups.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <type_traits>

#include "qmm_internal.h"

#include "qmm_gemv_blocks.h"
#include "qmm_moe_route.h"

namespace {

// The first 64 bytes hold everything a wave needs to issue its first loads, so
// that one scalar load fetches them.
struct GemvParams {
    const uint8_t* w;  // tiled matrix (expert 0 of a stack)
    const float* x;    // [m, k]            (grouped: [tokens, k] or [pairs, k])
    float* y;          // [m, n]            (grouped: [pairs, n])
    int m, n, k;
    int k_groups, slots; // the kernel derives k_units = ceil(k / 256) and s = slots / 16
    int row_tiles, panel_bytes;
    // split of the workgroup's waves: nwk along k times nwr row-tiles side by side
    int nwk, nwr;
    int wave_magic; // ceil(65536 / nwk): wave / nwk == (wave * wave_magic) >> 16
    // ---- 64 bytes ----
    int k_units;
    const uint8_t* w2; // gated form only: the second stack ("up"), same layout as w
    int64_t matrix_bytes;
    int kpw;        // ceil(k_groups / nwk): panels per row-tile for every wave
    int rt_groups;  // ceil(row_tiles / nwr)
    // grouped (expert) form: blockIdx.y is a segment of up to QMM_MOE_SEG_ROWS
    // sorted pairs that share one expert
    const int32_t* perm;
    const int32_t* offsets;     // [n_experts + 1]
    const int32_t* seg_offsets; // [n_experts + 1]
    const int32_t* seg_expert;  // [max segments]: expert of the segment, -1 past the last
    int n_experts;
    int x_div; // x row of pair p is p / x_div
    // several weights of equal k and type on the same activations in one launch:
    // workgroup b belongs to weight i with rtg_end[i - 1] <= b < rtg_end[i]
    int n_weights; // 0 or 1: just w / y / n / row_tiles above
    int rtg_end[QMM_MAX_GROUP];
    int nv[QMM_MAX_GROUP], row_tiles_v[QMM_MAX_GROUP];
    const uint8_t* wv[QMM_MAX_GROUP];
    float* yv[QMM_MAX_GROUP];
    // plain form only: y = sums (+ residual), stored as f32 or bf16 (P.y then points to bf16)
    QmmEpilogue ep;
    // NORM variants: the activations are RMS-normalized on the way in (weight norm_w[k], eps)
    const float* norm_w;
    float norm_eps;
    // expert-grouped form: the token rows quantized ahead of the launch (x blocks of row p / x_div for
    // pair p); xb.xq == nullptr: the workgroups quantize their rows themselves
    XBlocks xb;
    // TILEMAP variant (selected rows): row-tile i of the launch reads the weight's row-tile
    // tile_ids[i]; row_tiles, rt_groups and n count the selected tiles, y is [m, 16 * tiles]
    const int32_t* tile_ids;
};
static_assert(offsetof(GemvParams, k_units) == 64, "first-load fields must fill one 64-byte line");

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// MT rows per pass.  GATED: two weight stacks share x and the result is
// silu(w x) * (w2 x) (the expert MLP's gate/up pair); the second half of the
// workgroup's waves works on the second stack, so that the panels of both are
// in flight together, and the two are combined where the k-split is summed.  GROUPED: rows are sorted
// (token, slot) pairs of one expert.  ONESHOT: the launch gives every wave exactly
// one panel (one pass of rows, one row-tile group per workgroup, one k step), so
// the three loops below run once and the kernel is straight-line code from its
// entry to the first load.
// IO: 0 = f32 activations and a plain f32 store; 1 = f32 activations, 2 = bf16 activations, both
// with the epilogue of P.ep (residual add, f32 or bf16 store).
// NORM: x is replaced by rms_norm(x) * norm_w.  The workgroup reads all of x anyway: every 16-lane
// group adds the squares of its 256 raw values while it quantizes x * norm_w, and because the
// quantizers are invariant under a positive scale of their input (the quants stay, the block scale
// moves), the row's factor rsqrt(mean(x^2) + eps) multiplies the finished sums instead.
// The weight of a wave's row-tile in a group launch (straight-line form), looked up BEHIND the
// activation loads: those need nothing from the tables, so the tables' round trip hides behind them.
// The launch's row-tiles are counted over all weights, rtg_end[i] = the end of weight i's row-tiles,
// and every WAVE finds the weight of its own row-tile (a workgroup may straddle two weights; its
// waves only share the quantized activations and the LDS of the k-split).  The tables are read
// whole (independent scalar loads, one round trip) and the entry is picked with selects; rtg_end
// ascends, so the entry is the number of ends at or below the row-tile's index.  Entries past
// n_weights hold whatever the host left there and are never picked.
struct NoGroupPick {
    static constexpr bool kActive = false;
    __device__ __forceinline__ void operator()(int, const uint8_t*&, float*&, int&, int&, int&) const {}
};
struct GroupPick {
    static constexpr bool kActive = true;
    const GemvParams& P0;
    int n_weights;
    // b: the wave's row-tile counted over the launch
    __device__ __forceinline__ void operator()(int b, const uint8_t*& w_first, float*& y_out, int& n_rows, int& row_tiles,
                                               int& item_bias) const {
        if (n_weights <= 1) return; // uniform
        static_assert(QMM_MAX_GROUP == 4, "the selects below name four entries");
        const int e0 = P0.rtg_end[0], e1 = P0.rtg_end[1], e2 = P0.rtg_end[2];
        const bool c1 = b >= e0, c2 = n_weights > 2 && b >= e1, c3 = n_weights > 3 && b >= e2;
        auto pick = [c1, c2, c3](auto v0, auto v1, auto v2, auto v3) {
            auto v = c1 ? v1 : v0;
            v = c2 ? v2 : v;
            return c3 ? v3 : v;
        };
        item_bias = -pick(0, e0, e1, e2);
        w_first = pick(P0.wv[0], P0.wv[1], P0.wv[2], P0.wv[3]);
        y_out = pick(P0.yv[0], P0.yv[1], P0.yv[2], P0.yv[3]);
        n_rows = pick(P0.nv[0], P0.nv[1], P0.nv[2], P0.nv[3]);
        row_tiles = pick(P0.row_tiles_v[0], P0.row_tiles_v[1], P0.row_tiles_v[2], P0.row_tiles_v[3]);
    }
};

// XBLK (expert-grouped form): the rows' x blocks were made ahead of the launch and are copied.
template <int QT, int MT, bool GATED, bool GROUPED, bool ONESHOT, int IO = 0, bool NORM = false, bool TILEMAP = false,
          bool XBLK = false, class Pick = NoGroupPick>
__device__ __forceinline__ void gemv_body(const GemvParams& P, int m_begin, int m_end, const uint8_t* w_first,
                                          float* y_out, int n_rows, int row_tiles, int rtg0, uint8_t* smem,
                                          int item_bias = 0, Pick group_pick = Pick{}) {
    static_assert(!Pick::kActive || (ONESHOT && !GATED && !GROUPED && !TILEMAP), "group launches are dense straight-line launches");
    constexpr bool XB = IO == 2, EP = IO != 0;
    const int lane0 = threadIdx.x & 63;
    // wave-uniform by construction; said so, the row-tile, panel offset and output row that
    // derive from it live in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int stack_waves = P.nwk * P.nwr;               // waves per weight stack
    const int waves = GATED ? 2 * stack_waves : stack_waves; // = blockDim.x / 64, without the dispatch packet read
    const int stack = GATED && wave >= stack_waves ? 1 : 0;
    const int sw = wave - stack * stack_waves;
    const int wr = (sw * P.wave_magic) >> 16;
    const int wk = sw - wr * P.nwk;
    const bool lane_active = lane0 < P.slots;
    const int k_units = (P.k + 255) >> 8, s_units = P.slots >> 4;
    const uint8_t* wbase_init = stack ? P.w2 + (w_first - P.w) : w_first; // the second stack at the same offset
    const uint8_t* wbase = wbase_init; // (set again by a group pick)
    const XLds<QT> l = carve<QT, MT>(smem, k_units);
    float* xss = l.red + 2 * waves * MT * 16; // NORM: [MT][k_units] sums of squares, behind everything else

    for (int m0 = m_begin; ONESHOT ? m0 == m_begin : m0 < m_end; m0 += MT) {
        bool x_ready = false;
        int red_buf = 0;
        for (int rtg = rtg0; ONESHOT ? rtg == rtg0 : rtg < P.rt_groups;
             rtg += ONESHOT ? 1 : (int)gridDim.x) {
            // the wave's row-tile (item_bias: a group launch counts its row-tiles over all weights and
            // this is minus the first one of the wave's weight; uniform)
            int rt = rtg * P.nwr + wr + item_bias;
            // the weight's row-tile behind this one (uniform: a scalar load)
            int rt_w = TILEMAP ? P.tile_ids[rt < row_tiles ? rt : 0] : rt;
            float acc[MT];
#pragma unroll
            for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
            // Epilogue with a residual, k split over waves: the lane that will store requests its
            // residual value behind the first panel's loads, so that the value is there when the
            // sums are (at the end it would be one more memory round trip on the kernel's critical
            // path).  Like the other loads it is unconditional and branch-free: the aligned dword
            // that holds the value (f32, or a bf16 pair), or the start of x for lanes without one.
            uint32_t res_raw = 0;
            for (int ks = 0; ONESHOT ? ks < 1 : ks < P.kpw; ks++) {
                const int kg = ks * P.nwk + wk;
                bool ok = rt < row_tiles && kg < P.k_groups;
                int64_t off = ok ? ((int64_t)rt_w * P.k_groups + kg) * P.panel_bytes : 0;
                Panel<QT> p;
                bool active = ok && lane_active;
                if (XBLK && GROUPED && !x_ready) {
                    // the rows' x blocks were made ahead of the launch: copy them (a quarter of the f32
                    // bytes, no arithmetic); first item ahead of the panel as below
                    const int group = threadIdx.x >> 4, n_groups = 4 * waves;
                    const int items = MT * k_units;
                    auto copy_item = [&](int item) {
                        const int mi = item % MT, unit = item / MT;
                        const bool row_ok = m0 + mi < m_end;
                        const int64_t token = row_ok ? P.perm[m0 + mi] / P.x_div : 0;
                        x_blocks_to_lds<QT>(l, mi * k_units + unit, P.xb, token * k_units + unit, row_ok);
                    };
                    if (group < items) copy_item(group);
                    load_panel<QT>(p, wbase + off, P.slots, lane0, active);
                    for (int item = group + n_groups; item < items; item += n_groups) copy_item(item);
                    lds_barrier();
                    x_ready = true;
                } else if (!x_ready) {
                    // Loads return in issue order: the small activation load goes first so
                    // that it can be consumed (quantized) while the panel loads still fly.
                    const int group = threadIdx.x >> 4, n_groups = 4 * waves; // = blockDim.x / 16
                    const int items = MT * k_units;
                    const XSource xs{P.x, GROUPED ? P.perm : nullptr, P.x_div, m0, m_end, P.k, k_units};
                    float4 f[4];
                    float v[16];
                    const bool in0 = x_item_issue<MT, XB>(xs, group, group < items, f);
                    float4 fnw[4];
                    if (NORM) x16_issue<false>(P.norm_w + (group / MT) * 256 + 16 * (threadIdx.x & 15), P.norm_w, in0, fnw);
                    if (IO != 0 || NORM) __builtin_amdgcn_sched_barrier(0); // the activation loads stay in front
                    if constexpr (Pick::kActive) {
                        group_pick(rt, w_first, y_out, n_rows, row_tiles, item_bias);
                        wbase = w_first;
                        rt = rtg * P.nwr + wr + item_bias;
                        rt_w = rt;
                        ok = rt < row_tiles && kg < P.k_groups;
                        off = ok ? ((int64_t)rt_w * P.k_groups + kg) * P.panel_bytes : 0;
                        active = ok && lane_active;
                    }
                    load_panel<QT>(p, wbase + off, P.slots, lane0, active);
                    if (EP && ks == 0) {
                        // (the lanes and conditions of the store at the end)
                        const int mi = lane0 >> 4, row = rt * 16 + (lane0 & 15);
                        const bool have = P.ep.residual != nullptr && P.nwk != 1 && wk == 0 && lane0 < 16 * MT &&
                                          rt < row_tiles && row < n_rows && m0 + mi < m_end;
                        const int64_t byte = ((int64_t)(m0 + mi) * n_rows + row) * (P.ep.y_bf16 ? 2 : 4);
                        const uint8_t* rp = have ? static_cast<const uint8_t*>(P.ep.residual) + (byte & ~(int64_t)3)
                                                 : reinterpret_cast<const uint8_t*>(P.x);
                        res_raw = *reinterpret_cast<const uint32_t*>(rp);
                    }
                    if (m0 != m_begin) lds_barrier(); // the previous rows' readers are done
                    // one row of whole 256-value units: an item that exists is in range, and only those are quantized
                    constexpr bool kWhole = MT == 1 && QT != QMM_Q8_0 && !GATED; // (the gated form measured no faster with it)
                    x16_finish<XB, kWhole>(f, in0, v);
                    // NORM: sum of the raw squares of the item (all 16 lanes of the group), then x * norm_w
                    auto norm_item = [&](int item, bool in_range, const float4 (&fw)[4]) {
                        float wv[16], ss = 0.0f;
                        x16_finish<false>(fw, in_range, wv);
#pragma unroll
                        for (int i = 0; i < 16; i++) ss += v[i] * v[i], v[i] *= wv[i];
                        ss = row16_sum(ss);
                        if ((threadIdx.x & 15) == 0) xss[(item % MT) * k_units + item / MT] = ss;
                    };
                    if (NORM && group < items) norm_item(group, in0, fnw);
                    if (group < items) x_item_quantize<QT, MT>(l, k_units, group, v);
                    for (int item = group + n_groups; item < items; item += n_groups) {
                        const bool in1 = x_item_issue<MT, XB>(xs, item, true, f);
                        if (NORM) x16_issue<false>(P.norm_w + (item / MT) * 256 + 16 * (threadIdx.x & 15), P.norm_w, in1, fnw);
                        x16_finish<XB, kWhole>(f, in1, v);
                        if (NORM) norm_item(item, in1, fnw);
                        x_item_quantize<QT, MT>(l, k_units, item, v);
                    }
                    // One row, one row-tile per workgroup, four units per panel: wave wk has just
                    // quantized exactly the units 4 wk .. 4 wk + 3 that its own panel multiplies
                    // (LDS serves a wave's accesses in order), so no wave waits for another here.
                    const bool own_units = ONESHOT && MT == 1 && !GATED && !GROUPED && P.nwr == 1 && P.slots == 64;
                    if (!own_units) lds_barrier();
                    x_ready = true;
                } else {
                    load_panel<QT>(p, wbase + off, P.slots, lane0, active);
                }
                // the lane index again, from the hardware: nothing lane-derived has to stay in a
                // register across the quantizer
                const int lane_m = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
                mask_panel<QT>(p, ok && lane_m < P.slots);
                const int unit = min(kg * s_units + (lane_m >> 4), k_units - 1);
                multiply_panel<QT, MT>(p, l, unit, k_units, acc);
            }
            const int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); // as above
            // row-tile finished: combine the S units of a row, then the waves that split k
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                acc[mi] += __shfl_xor(acc[mi], 16);
                acc[mi] += __shfl_xor(acc[mi], 32);
            }
            if (P.nwk == 1 && !GATED) {
                const int row = rt * 16 + lane;
                if (lane < 16 && rt < row_tiles && row < n_rows) {
#pragma unroll
                    for (int mi = 0; mi < MT; mi++) {
                        if (m0 + mi < m_end) {
                            int64_t yr = GROUPED ? P.perm[m0 + mi] : m0 + mi;
                            if (NORM) {
                                float ssq = 0.0f;
                                for (int u = 0; u < k_units; u++) ssq += xss[mi * k_units + u];
                                acc[mi] *= 1.0f / sqrtf(ssq / (float)P.k + P.norm_eps);
                            }
                            if (EP) qmm_store(y_out, P.ep, yr * n_rows + row, acc[mi]);
                            else y_out[yr * n_rows + row] = acc[mi];
                        }
                    }
                }
            } else {
                float* red = l.red + red_buf * (waves * MT * 16);
                if (lane < 16) {
#pragma unroll
                    for (int mi = 0; mi < MT; mi++) red[(wave * MT + mi) * 16 + lane] = acc[mi];
                }
                __syncthreads();
                if (wk == 0 && stack == 0 && lane < 16 * MT) {
                    const int mi = lane >> 4, r = lane & 15;
                    float sum = 0.0f, sum2 = 0.0f;
                    for (int w2 = 0; w2 < P.nwk; w2++) {
                        sum += red[((wr * P.nwk + w2) * MT + mi) * 16 + r];
                        if (GATED) sum2 += red[((stack_waves + wr * P.nwk + w2) * MT + mi) * 16 + r];
                    }
                    const int row = rt * 16 + r;
                    if (NORM) {
                        float ssq = 0.0f;
                        for (int u = 0; u < k_units; u++) ssq += xss[mi * k_units + u];
                        const float ns = 1.0f / sqrtf(ssq / (float)P.k + P.norm_eps);
                        sum *= ns;
                        sum2 *= ns;
                    }
                    if (rt < row_tiles && row < n_rows && m0 + mi < m_end) {
                        int64_t yr = GROUPED ? P.perm[m0 + mi] : m0 + mi;
                        if (EP) {
                            const int64_t idx = yr * n_rows + row;
                            const float res = P.ep.residual == nullptr ? 0.0f
                                              : P.ep.y_bf16 ? qmm_bf16_bits_to_f32((uint16_t)(res_raw >> (16 * (int)(idx & 1))))
                                                            : __uint_as_float(res_raw);
                            qmm_store(y_out, QmmEpilogue{nullptr, P.ep.y_bf16}, idx, sum + res);
                        } else {
                            y_out[yr * n_rows + row] = GATED ? silu(sum) * sum2 : sum;
                        }
                    }
                }
                red_buf ^= 1;
            }
        }
    }
}

// The grouped straight-line form picks the row count of its segment (1, 2 or up to
// QMM_MOE_SEG_ROWS rows; uniform for the workgroup) at run time: most segments of a
// small batch hold one or two pairs, and a row costs its share of the arithmetic
// whether it exists or not.
// The dense straight-line single-row Q4_K form is held to 80 registers: six waves per SIMD,
// i.e. two 12-wave workgroups per CU.
template <int QT, int MT, bool GATED, bool GROUPED, bool ONESHOT, int IO, bool NORM, bool TILEMAP, bool XBLK = false>
__device__ __forceinline__ void gemv_entry(const GemvParams& P, const GemvParams& P0, int n_weights) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int m_begin = 0, m_end = P.m;
    int64_t w_offset = 0;
    if (GROUPED) {
        const int seg = blockIdx.y;
        const int lo = P.seg_expert[seg]; // uniform for the block
        if (lo < 0) return;               // past the last segment
        m_begin = P.offsets[lo] + (seg - P.seg_offsets[lo]) * QMM_MOE_SEG_ROWS;
        m_end = min(P.offsets[lo + 1], m_begin + QMM_MOE_SEG_ROWS);
        w_offset = (int64_t)lo * P.matrix_bytes;
    }
    const uint8_t* w_first = P.w + w_offset;
    float* y_out = P.y;
    int n_rows = P.n, row_tiles = P.row_tiles, rtg0 = blockIdx.x;
    if (GROUPED && ONESHOT && MT == 4) {
        const int rows = m_end - m_begin;
        if (rows == 1)
            gemv_body<QT, 1, GATED, GROUPED, ONESHOT, 0, false, false, XBLK>(P, m_begin, m_end, w_first, y_out, n_rows, row_tiles, rtg0, smem);
        else if (rows == 2)
            gemv_body<QT, 2, GATED, GROUPED, ONESHOT, 0, false, false, XBLK>(P, m_begin, m_end, w_first, y_out, n_rows, row_tiles, rtg0, smem);
        else
            gemv_body<QT, 4, GATED, GROUPED, ONESHOT, 0, false, false, XBLK>(P, m_begin, m_end, w_first, y_out, n_rows, row_tiles, rtg0, smem);
    } else {
        if constexpr (!GROUPED && !GATED && ONESHOT && !TILEMAP)
            gemv_body<QT, MT, GATED, GROUPED, ONESHOT, IO, NORM, TILEMAP, XBLK, GroupPick>(
                P, m_begin, m_end, w_first, y_out, n_rows, row_tiles, rtg0, smem, 0, GroupPick{P0, n_weights});
        else
            gemv_body<QT, MT, GATED, GROUPED, ONESHOT, IO, NORM, TILEMAP, XBLK>(P, m_begin, m_end, w_first, y_out, n_rows, row_tiles, rtg0, smem);
    }
}

// The dense launches.  What the first loads' addresses need comes in the 14 leading argument
// dwords, which the command processor writes into scalar registers when it starts a wave
// (kernel-argument preload): the first load does not wait for a read of the argument block.
// The rest of the parameter block is read from memory when its first use comes (the tables
// of a group of weights are indexed in the block itself, P0).
template <int QT, int MT, bool GATED, bool GROUPED, bool ONESHOT = false, int IO = 0, bool NORM = false, bool TILEMAP = false>
__global__ __launch_bounds__(64 * kMaxWaves)
__attribute__((amdgpu_waves_per_eu(NORM ? 3 : (ONESHOT && MT == 1 && QT == QMM_Q4_K) ? 6 : 3)))
void gemv_kernel(const uint8_t* w_arg, const float* x_arg, float* y_arg, int m_arg, int n_arg, int k_arg, int k_groups_arg,
                 int panel_bytes_arg, int row_tiles_arg, int split_arg, int wave_magic_arg, GemvParams P0) {
    static_assert(!GROUPED, "the expert-grouped launches go through gemv_grouped_kernel");
    GemvParams P = P0;
    P.w = w_arg, P.x = x_arg, P.y = y_arg, P.m = m_arg, P.n = n_arg, P.k = k_arg, P.k_groups = k_groups_arg;
    P.panel_bytes = panel_bytes_arg, P.row_tiles = row_tiles_arg, P.wave_magic = wave_magic_arg;
    P.nwk = split_arg & 255, P.nwr = (split_arg >> 8) & 255, P.slots = (split_arg >> 16) & 255;
    gemv_entry<QT, MT, GATED, false, ONESHOT, IO, NORM, TILEMAP>(P, P0, split_arg >> 24);
}

// The expert-grouped launches: thousands of short workgroups, whose waves start faster with
// fewer scalar registers to fill (measured: 1 us of 19 - 30 lost with preloaded arguments), so
// the parameter block stays one block in memory.
template <int QT, int MT, bool GATED, bool ONESHOT, bool XBLK = false>
__global__ __launch_bounds__(64 * kMaxWaves) __attribute__((amdgpu_waves_per_eu(3))) void gemv_grouped_kernel(GemvParams P) {
    gemv_entry<QT, MT, GATED, true, ONESHOT, 0, false, false, XBLK>(P, P, 0);
}

// The launch of a gemv_kernel: its leading arguments are the fields of P that the first loads need.
template <class Kernel>
void launch_gemv(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const GemvParams& P) {
    kernel<<<grid, block, lds, stream>>>(P.w, P.x, P.y, P.m, P.n, P.k, P.k_groups, P.panel_bytes, P.row_tiles,
                                         P.nwk | (P.nwr << 8) | (P.slots << 16) | (P.n_weights << 24), P.wave_magic, P);
}

// Waves per workgroup and their split: as many waves along k as there are
// panels per row-tile (up to kMaxWaves) so that every panel of a row-tile is in
// flight at once, times as many row-tiles side by side as still leave one
// workgroup per CU: the activations are quantized once per workgroup, so
// taller workgroups amortize that work and its L2 traffic.
void choose_split(const QmmLayout& L, int n_cus, int grid_y, bool gated, GemvParams& P, int& waves) {
    // Waves per weight stack.  The grouped (expert) launches run many short workgroups
    // one after the other on a CU: small workgroups fill the wave slots that the
    // register count leaves (several side by side, one loads while another multiplies).
    const int total = grid_y > 1 ? 4 : kMaxWaves;
    const int budget = gated ? total / 2 : total;
    int nwk = (int)(L.k_groups < budget ? L.k_groups : budget);
    int nwr_max = budget / nwk;
    // Dense launches: as few workgroups as CUs where the waves allow it, i.e. ceil(row-tiles / CUs)
    // row-tiles side by side (measured, k = 4096, one row: 384 row-tiles as 192 workgroups of two
    // 5.05 us, as 384 of one 5.78 - the second workgroup of a CU starts late and quantizes the
    // activations again; 576..704 row-tiles as workgroups of three 6.3 - 7.0 us, of two 6.9 - 7.5).
    const int64_t cus = n_cus > 0 ? n_cus : 1;
    int64_t want = grid_y == 1 ? (L.row_tiles + cus - 1) / cus : L.row_tiles * grid_y / cus;
    int nwr = (int)(want < 1 ? 1 : (want > nwr_max ? nwr_max : want));
    // More than one full workgroup per CU (gate|up group): the register count lets 20 waves
    // share a CU, so two 8-wave workgroups run side by side (one loads while the other
    // multiplies) where a second 12-wave workgroup would wait for the first to end.
    if (grid_y == 1 && nwk * nwr > 8 && nwk <= 4 && L.row_tiles > (int64_t)nwr * n_cus) nwr = 8 / nwk;
    if (grid_y == 1 && L.row_tiles >= 16 * (int64_t)n_cus) {
        // very tall (LM head): whole row-tiles per wave, no barrier per row-tile
        nwk = 1;
        nwr = 4;
    }
    waves = nwk * nwr;
    P.nwk = nwk;
    P.nwr = nwr;
    P.kpw = (int)((L.k_groups + nwk - 1) / nwk);
    P.rt_groups = (int)((L.row_tiles + nwr - 1) / nwr);
    P.wave_magic = (65536 + nwk - 1) / nwk;
}

template <int QT, int MT, bool GATED, bool GROUPED, int IO = 0, bool NORM = false>
hipError_t launch_mt(const GemvParams& P, int waves, int n_cus, int grid_y, hipStream_t stream) {
    const int all_waves = GATED ? 2 * waves : waves;
    size_t lds = lds_bytes<QT, MT>(P.k_units, all_waves) + (NORM ? (size_t)MT * P.k_units * sizeof(float) : 0);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    int64_t cap = (int64_t)n_cus * 32;
    if (grid_y > 1) cap = cap / grid_y > 64 ? cap / grid_y : 64;
    int64_t grid = P.rt_groups < cap ? P.rt_groups : cap;
    if (grid < 1) grid = 1;
    // straight-line form: one pass of rows (a segment never has more than MT rows in the
    // grouped form), one row-tile group per workgroup, one k step
    constexpr bool kCanOneshot = GROUPED ? MT == QMM_MOE_SEG_ROWS : true;
    const bool oneshot = kCanOneshot && (GROUPED || P.m <= MT) && P.kpw == 1 && grid == P.rt_groups;
    const dim3 g((unsigned)grid, (unsigned)grid_y), b(64 * all_waves);
    if constexpr (GROUPED) {
        static_assert(IO == 0 && !NORM, "the grouped form has no epilogue and no folded norm");
        const void* fn = oneshot ? reinterpret_cast<const void*>(&gemv_grouped_kernel<QT, MT, GATED, kCanOneshot>)
                                 : reinterpret_cast<const void*>(&gemv_grouped_kernel<QT, MT, GATED, false>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        // (x blocks: gate / up of the straight-line form copies them; every other form quantizes P.x itself)
        if (GATED && oneshot && P.xb.xq != nullptr) {
            if (lds > 48 * 1024) {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_grouped_kernel<QT, MT, GATED, kCanOneshot, GATED>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
            }
            gemv_grouped_kernel<QT, MT, GATED, kCanOneshot, GATED><<<g, b, lds, stream>>>(P);
        } else if (oneshot) gemv_grouped_kernel<QT, MT, GATED, kCanOneshot><<<g, b, lds, stream>>>(P);
        else gemv_grouped_kernel<QT, MT, GATED, false><<<g, b, lds, stream>>>(P);
    } else {
        const void* fn = oneshot ? reinterpret_cast<const void*>(&gemv_kernel<QT, MT, GATED, false, kCanOneshot, IO, NORM>)
                                 : reinterpret_cast<const void*>(&gemv_kernel<QT, MT, GATED, false, false, IO, NORM>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        if (oneshot) launch_gemv(gemv_kernel<QT, MT, GATED, false, kCanOneshot, IO, NORM>, g, b, lds, stream, P);
        else launch_gemv(gemv_kernel<QT, MT, GATED, false, false, IO, NORM>, g, b, lds, stream, P);
    }
    return hipGetLastError();
}

// f(std::integral_constant<int, block type>) for the layout's block type
template <class F>
hipError_t with_block_type(int dtype, F&& f) {
    if (dtype == QMM_Q4_K) return f(std::integral_constant<int, QMM_Q4_K>{});
    if (dtype == QMM_Q6_K) return f(std::integral_constant<int, QMM_Q6_K>{});
    return f(std::integral_constant<int, QMM_Q8_0>{});
}

template <int QT>
hipError_t launch_plain(const GemvParams& P, int waves, int n_cus, int io, hipStream_t stream) {
    if (P.norm_w != nullptr) { // folded RMSNorm: f32 activations, plain store, one or two rows
        if (io != 0 || P.m > 2) return hipErrorNotSupported;
        if (P.m == 2 && lds_bytes<QT, 2>(P.k_units, waves) <= 64 * 1024)
            return launch_mt<QT, 2, false, false, 0, true>(P, waves, n_cus, 1, stream);
        if (P.m == 2) return hipErrorNotSupported;
        return launch_mt<QT, 1, false, false, 0, true>(P, waves, n_cus, 1, stream);
    }
    // the widest row tile whose quantized activations fit comfortably in LDS
    int mt = P.m >= 3 ? 4 : (P.m == 2 ? 2 : 1);
    if (mt == 4 && lds_bytes<QT, 4>(P.k_units, waves) > 64 * 1024) mt = 2;
    if (mt == 2 && lds_bytes<QT, 2>(P.k_units, waves) > 64 * 1024) mt = 1;
    if (io == 2) { // bf16 activations: the one- and two-row forms only
        if (P.m > 2) return hipErrorNotSupported;
        if (mt == 2) return launch_mt<QT, 2, false, false, 2>(P, waves, n_cus, 1, stream);
        return launch_mt<QT, 1, false, false, 2>(P, waves, n_cus, 1, stream);
    }
    if (io == 1) {
        if (mt == 4) return launch_mt<QT, 4, false, false, 1>(P, waves, n_cus, 1, stream);
        if (mt == 2) return launch_mt<QT, 2, false, false, 1>(P, waves, n_cus, 1, stream);
        return launch_mt<QT, 1, false, false, 1>(P, waves, n_cus, 1, stream);
    }
    if (mt == 4) return launch_mt<QT, 4, false, false>(P, waves, n_cus, 1, stream);
    if (mt == 2) return launch_mt<QT, 2, false, false>(P, waves, n_cus, 1, stream);
    return launch_mt<QT, 1, false, false>(P, waves, n_cus, 1, stream);
}

// false when a dimension does not fit the kernel's 32-bit index arithmetic
bool make_params(const QmmLayout& L, const void* tiled, const float* x, int64_t m, float* y,
                 GemvParams& P) {
    if (L.n > 0x7fffffff / 2 || L.k > 0x7fffffff / 2 || m > 0x7fffffff / 2 ||
        L.row_tiles * L.k_groups > 0x7fffffff || L.panel_bytes > 0x7fffffff)
        return false;
    P.w = (const uint8_t*)tiled;
    P.w2 = nullptr;
    P.x = x;
    P.y = y;
    P.m = (int)m;
    P.n = (int)L.n;
    P.k = (int)L.k;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.slots = L.slots;
    P.row_tiles = (int)L.row_tiles;
    P.panel_bytes = (int)L.panel_bytes;
    P.matrix_bytes = L.matrix_bytes;
    P.perm = nullptr;
    P.offsets = nullptr;
    P.seg_offsets = nullptr;
    P.seg_expert = nullptr;
    P.n_experts = 0;
    P.x_div = 1;
    P.n_weights = 0;
    P.ep.residual = nullptr;
    P.ep.y_bf16 = 0;
    P.norm_w = nullptr;
    P.norm_eps = 0.0f;
    P.xb = XBlocks{nullptr, nullptr, nullptr};
    P.tile_ids = nullptr;
    return true;
}

// ---- export of the activation quantizer ---------------------------------------
template <int QT>
__global__ void quantize_export_kernel(const float* __restrict__ x, int64_t m, int64_t k,
                                       int64_t k_units, uint8_t* __restrict__ out) {
    const int64_t group = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    if (group >= m * k_units) return; // whole 16-lane groups leave together
    int64_t mi = group / k_units, unit = group - mi * k_units;
    float v[16];
    {
        const int64_t k0 = unit * 256 + 16 * j;
        const bool in_range = k0 + 16 <= k;
        float4 f[4];
        x16_issue(x + mi * k + k0, x, in_range, f);
        x16_finish(f, in_range, v);
    }
    uint32_t q[4];
    if (QT == QMM_Q4_K) {
        float d;
        int s16;
        quantize_q8k_lane(v, j, q, d, s16);
        uint8_t* blk = out + group * 292;
        if (j == 0) *reinterpret_cast<float*>(blk) = d;
        uint32_t* qs = reinterpret_cast<uint32_t*>(blk + 4 + 16 * j);
        qs[0] = q[0];
        qs[1] = q[1];
        qs[2] = q[2];
        qs[3] = q[3];
        *reinterpret_cast<int16_t*>(blk + 260 + 2 * j) = (int16_t)s16;
    } else {
        float d;
        uint16_t bits;
        quantize_q80_lane(v, q, d, bits);
        int64_t kb = unit * 8 + (j >> 1);
        if (kb < k / 32) {
            uint8_t* blk = out + (mi * (k / 32) + kb) * 34;
            if ((j & 1) == 0) *reinterpret_cast<uint16_t*>(blk) = bits;
            uint16_t* qs = reinterpret_cast<uint16_t*>(blk + 2 + 16 * (j & 1));
#pragma unroll
            for (int w = 0; w < 4; w++) {
                qs[2 * w] = (uint16_t)(q[w] & 0xffffu);
                qs[2 * w + 1] = (uint16_t)(q[w] >> 16);
            }
        }
    }
}

} // namespace

hipError_t qmm_launch_gemv(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                           float* y, int n_cus, hipStream_t stream, const QmmIo* io, const QmmNorm* norm) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    GemvParams P;
    if (!make_params(L, tiled, x, m, y, P)) return hipErrorInvalidValue;
    if (norm) P.norm_w = norm->weight, P.norm_eps = norm->eps;
    // kernel variant: plain, or with the epilogue (and f32 / bf16 activations)
    const int iom = !io ? 0 : (io->x_bf16 ? 2 : (io->residual || io->y_bf16 ? 1 : 0));
    if (io) P.ep = QmmEpilogue{io->residual, io->y_bf16};
    int waves;
    choose_split(L, n_cus, 1, false, P, waves);
    if (L.dtype == QMM_Q6_K) return launch_plain<QMM_Q6_K>(P, waves, n_cus, iom, stream);
    return L.dtype == QMM_Q4_K ? launch_plain<QMM_Q4_K>(P, waves, n_cus, iom, stream)
                               : launch_plain<QMM_Q8_0>(P, waves, n_cus, iom, stream);
}

namespace {

// Selected rows: the looped form of the decode kernel over a list of row-tiles.
template <int QT, int MT>
hipError_t launch_rows_mt(const GemvParams& P, int waves, int n_cus, hipStream_t stream) {
    const size_t lds = lds_bytes<QT, MT>(P.k_units, waves);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    const int64_t cap = (int64_t)n_cus * 32;
    const int64_t grid = P.rt_groups < cap ? P.rt_groups : cap;
    const void* fn = reinterpret_cast<const void*>(&gemv_kernel<QT, MT, false, false, false, 0, false, true>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    launch_gemv(gemv_kernel<QT, MT, false, false, false, 0, false, true>, dim3((unsigned)grid), dim3(64 * waves), lds, stream, P);
    return hipGetLastError();
}

template <int QT>
hipError_t launch_rows(const GemvParams& P, int waves, int n_cus, hipStream_t stream) {
    // the row count per pass that the full product takes for this m (launch_plain)
    if (P.m == 2 && lds_bytes<QT, 2>(P.k_units, waves) <= 64 * 1024) return launch_rows_mt<QT, 2>(P, waves, n_cus, stream);
    return launch_rows_mt<QT, 1>(P, waves, n_cus, stream);
}

// tile_ids[i] = row-tile of token i (clamped into the matrix)
__global__ void rows_prepare_kernel(const uint32_t* __restrict__ token_ids, int64_t count, int64_t n,
                                    int32_t* __restrict__ tile_ids) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const uint32_t t = token_ids[i];
    tile_ids[i] = (int32_t)(((int64_t)t < n ? (int64_t)t : n - 1) >> 4);
}

// out[mi, i] = tiles[mi, 16 i + token_i % 16]; NaN for a token outside the matrix
__global__ void rows_gather_kernel(const float* __restrict__ tiles, const uint32_t* __restrict__ token_ids,
                                   int64_t count, int64_t n, int m, float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const uint32_t t = token_ids[i];
    for (int mi = 0; mi < m; mi++)
        out[mi * count + i] = (int64_t)t < n ? tiles[(mi * count + i) * 16 + (t & 15)] : __uint_as_float(0x7fc00000u);
}

} // namespace

size_t qmm_gemv_rows_workspace_bytes(int64_t m, int64_t count) {
    return (size_t)(((count * 4 + 255) & ~(int64_t)255) + m * count * 16 * 4);
}

hipError_t qmm_launch_gemv_rows(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                                const uint32_t* token_ids, int64_t count, float* out, void* workspace, int n_cus,
                                hipStream_t stream) {
    if (m <= 0 || count <= 0 || L.n == 0) return hipSuccess;
    if (m > 2) return hipErrorNotSupported;
    if (count > 0x7fffffff / 64) return hipErrorInvalidValue;
    GemvParams P;
    if (!make_params(L, tiled, x, m, nullptr, P)) return hipErrorInvalidValue;
    int waves;
    choose_split(L, n_cus, 1, false, P, waves); // the split along k of the full product: same sums
    int32_t* tile_ids = static_cast<int32_t*>(workspace);
    float* tiles = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + ((count * 4 + 255) & ~(int64_t)255));
    P.tile_ids = tile_ids;
    P.y = tiles;
    P.row_tiles = (int)count;
    P.n = (int)count * 16;
    P.rt_groups = (int)((count + P.nwr - 1) / P.nwr);
    const unsigned blocks = (unsigned)((count + 255) / 256);
    rows_prepare_kernel<<<blocks, 256, 0, stream>>>(token_ids, count, L.n, tile_ids);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    e = with_block_type(L.dtype, [&](auto qt) { return launch_rows<decltype(qt)::value>(P, waves, n_cus, stream); });
    if (e != hipSuccess) return e;
    rows_gather_kernel<<<blocks, 256, 0, stream>>>(tiles, token_ids, count, L.n, (int)m, out);
    return hipGetLastError();
}

namespace {

__global__ void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                float* __restrict__ out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) out[i] = silu(gate[i]) * up[i];
}

} // namespace

hipError_t qmm_launch_silu_mul(const float* gate, const float* up, float* out, int64_t count,
                               hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    const int64_t grid = (count + 255) / 256;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    silu_mul_kernel<<<(unsigned)grid, 256, 0, stream>>>(gate, up, out, count);
    return hipGetLastError();
}

hipError_t qmm_launch_gemv_gated(const QmmLayout& L, const void* tiled_gate, const void* tiled_up,
                                 const float* x, int64_t m, float* y, int n_cus, hipStream_t stream,
                                 const QmmNorm* norm) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    if (m > 2) return hipErrorNotSupported;
    GemvParams P;
    if (!make_params(L, tiled_gate, x, m, y, P)) return hipErrorInvalidValue;
    P.w2 = (const uint8_t*)tiled_up;
    int waves;
    choose_split(L, n_cus, 1, true, P, waves);
    if (norm) P.norm_w = norm->weight, P.norm_eps = norm->eps;
    return with_block_type(L.dtype, [&](auto QT) {
        constexpr int qt = decltype(QT)::value;
        if (norm)
            return m == 2 ? launch_mt<qt, 2, true, false, 0, true>(P, waves, n_cus, 1, stream)
                          : launch_mt<qt, 1, true, false, 0, true>(P, waves, n_cus, 1, stream);
        return m == 2 ? launch_mt<qt, 2, true, false>(P, waves, n_cus, 1, stream)
                      : launch_mt<qt, 1, true, false>(P, waves, n_cus, 1, stream);
    });
}

hipError_t qmm_launch_gemv_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                 const float* x, int64_t m, float* const* ys, int n_cus,
                                 hipStream_t stream, const QmmNorm* norm) {
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP || m < 1 || m > 4) return hipErrorInvalidValue;
    if (norm && m > 2) return hipErrorNotSupported; // (the folded norm: one or two rows)
    const QmmLayout& L0 = *layouts[0];
    int64_t total_row_tiles = 0;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        if (L.dtype != L0.dtype || L.k != L0.k || L.n_stacked != 1 || L.n == 0) return hipErrorInvalidValue;
        total_row_tiles += L.row_tiles;
    }
    if (L0.k_groups > kMaxWaves) return hipErrorNotSupported; // no single-launch form: the caller launches one by one
    GemvParams P;
    if (!make_params(L0, tiled[0], x, m, ys[0], P)) return hipErrorInvalidValue;
    // the split of a single matrix with all the row-tiles
    QmmLayout all = L0;
    all.row_tiles = total_row_tiles;
    int waves;
    choose_split(all, n_cus, 1, false, P, waves);
    if (P.kpw != 1) return hipErrorNotSupported;
    P.n_weights = n_weights;
    int64_t tiles_all = 0;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        if (L.n > 0x3fffffff) return hipErrorInvalidValue;
        tiles_all += L.row_tiles;
        P.rtg_end[i] = (int)tiles_all; // in row-tiles, not workgroups: see the kernel
        P.nv[i] = (int)L.n;
        P.row_tiles_v[i] = (int)L.row_tiles;
        P.wv[i] = (const uint8_t*)tiled[i];
        P.yv[i] = ys[i];
    }
    const int64_t groups = (tiles_all + P.nwr - 1) / P.nwr;
    if (groups > (int64_t)n_cus * 32) return hipErrorNotSupported;
    P.rt_groups = (int)groups;
    const int mt = m > 2 ? 4 : (m == 2 ? 2 : 1); // rows per pass: one pass
    if (norm) P.norm_w = norm->weight, P.norm_eps = norm->eps;
    const dim3 g((unsigned)groups), b(64 * waves);
    return with_block_type(L0.dtype, [&](auto QT) {
        constexpr int qt = decltype(QT)::value;
        size_t need = mt == 4 ? lds_bytes<qt, 4>(P.k_units, waves) : mt == 2 ? lds_bytes<qt, 2>(P.k_units, waves) : lds_bytes<qt, 1>(P.k_units, waves);
        if (norm) need += (size_t)mt * P.k_units * sizeof(float);
        if (need > 48 * 1024) return hipErrorNotSupported;
        if (mt == 4) {
            launch_gemv(gemv_kernel<qt, 4, false, false, true>, g, b, need, stream, P);
            return hipGetLastError();
        }
        if (norm) {
            if (mt == 2) launch_gemv(gemv_kernel<qt, 2, false, false, true, 0, true>, g, b, need, stream, P);
            else launch_gemv(gemv_kernel<qt, 1, false, false, true, 0, true>, g, b, need, stream, P);
        } else {
            if (mt == 2) launch_gemv(gemv_kernel<qt, 2, false, false, true>, g, b, need, stream, P);
            else launch_gemv(gemv_kernel<qt, 1, false, false, true>, g, b, need, stream, P);
        }
        return hipGetLastError();
    });
}

// ---- expert MLP of a small batch in two launches --------------------------------------------
// Launch 1: every workgroup routes its own token (a wave, 128 logits: cheaper than a launch of
// its own), then runs the gated single-row decode body on the expert of its (token, slot) pair:
// h[pair] = silu(W_gate[e] x_t) * (W_up[e] x_t).  blockIdx.y = pair.
namespace {

template <int QT, int PER_LANE>
__global__ __launch_bounds__(64 * kMaxWaves) __attribute__((amdgpu_waves_per_eu(3)))
void moe_small_gate_up_kernel(GemvParams P, const float* __restrict__ logits, int n_experts, int top_k,
                              int32_t* __restrict__ ids, float* __restrict__ weights, int32_t* __restrict__ ids_out,
                              float* __restrict__ weights_out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int expert_sh;
    const int pair = blockIdx.y;
    const int tok = pair / top_k, slot = pair - tok * top_k;
    if (threadIdx.x < 64) {
        int id;
        float w;
        // (only the workgroup that writes the token's routing needs all slots and their weights; the
        // others stop behind their own slot: the arg-max rounds stand in front of every load of weights)
        const bool writes_routing = blockIdx.x == 0 && slot == 0;
        moe_route::route_token<PER_LANE>(logits + (int64_t)tok * n_experts, n_experts, top_k, (int)threadIdx.x, id, w,
                                         writes_routing ? -1 : slot + 1);
        if ((int)threadIdx.x == slot) expert_sh = id;
        if (writes_routing && (int)threadIdx.x < top_k) { // once per token: the routing for launch 2
            ids[tok * top_k + threadIdx.x] = id;
            weights[tok * top_k + threadIdx.x] = w;
            if (ids_out) ids_out[tok * top_k + threadIdx.x] = id;
            if (weights_out) weights_out[tok * top_k + threadIdx.x] = w;
        }
    }
    __syncthreads();
    const int e = expert_sh;
    GemvParams Q = P;
    Q.x = P.x + (int64_t)tok * P.k;
    gemv_body<QT, 1, true, false, true>(Q, 0, 1, P.w + (int64_t)e * P.matrix_bytes, P.y + (int64_t)pair * P.n, P.n,
                                        P.row_tiles, blockIdx.x, smem);
}

// Launch 2: out[t] = sum over slots s (in order) of weights[t, s] * (W_down[e_s] h[t, s]).  A
// workgroup is one 16-row tile of one token, a wave is one slot: it quantizes its h row, multiplies
// its expert's panel (k fits one panel), and the slots are added in order through LDS, the sums and
// products of the grouped decode kernel followed by the combine kernel.
struct MoeSmallDown {
    const uint8_t* w;
    const float* h;        // [pairs, k]
    const int32_t* ids;    // [pairs]
    const float* weights;  // [pairs]
    float* out;            // [t, n]
    int n, k, k_units, slots, row_tiles, top_k;
    int panel_bytes;
    int64_t matrix_bytes;
};

template <int QT>
__global__ __launch_bounds__(64 * kMaxWaves) void moe_small_down_kernel(MoeSmallDown P) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int rt = blockIdx.x, tok = blockIdx.y;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int pair = tok * P.top_k + wave;
    const int e = P.ids[pair];
    const size_t per_wave = (lds_bytes<QT, 1>(P.k_units, 0) + 15) & ~(size_t)15;
    float* ysum = reinterpret_cast<float*>(smem + per_wave * P.top_k); // [top_k][16]
    const XLds<QT> l = carve<QT, 1>(smem + per_wave * wave, P.k_units);
    // activations first, the panel behind them
    const int item = lane >> 4, j = lane & 15;
    const bool item_ok = item < P.k_units;
    const int k0 = item * 256 + 16 * j;
    const bool in_range = item_ok && k0 + 16 <= P.k;
    float4 f[4];
    x16_issue<false>(P.h + (int64_t)pair * P.k + k0, P.h, in_range, f);
    Panel<QT> p;
    const bool active = lane < P.slots;
    load_panel<QT>(p, P.w + (int64_t)e * P.matrix_bytes + (int64_t)rt * P.panel_bytes, P.slots, lane, active);
    float v[16];
    x16_finish<false>(f, in_range, v);
    if (item_ok) x_item_quantize<QT, 1>(l, P.k_units, item, v);
    for (int it = item + 4; it < P.k_units; it += 4) { // more than four units (k > 1024): not reached, k fits a panel
        const int k1 = it * 256 + 16 * j;
        const bool ok1 = k1 + 16 <= P.k;
        x16_issue<false>(P.h + (int64_t)pair * P.k + k1, P.h, ok1, f);
        x16_finish<false>(f, ok1, v);
        x_item_quantize<QT, 1>(l, P.k_units, it, v);
    }
    // the wave reads back what its own lanes wrote: LDS serves a wave's accesses in order
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    mask_panel<QT>(p, active);
    float acc[1] = {0.0f};
    multiply_panel<QT, 1>(p, l, min(lane >> 4, P.k_units - 1), P.k_units, acc);
    acc[0] += __shfl_xor(acc[0], 16);
    acc[0] += __shfl_xor(acc[0], 32);
    if (lane < 16) ysum[wave * 16 + lane] = acc[0];
    __syncthreads();
    if (wave == 0 && lane < 16) {
        const int row = rt * 16 + lane;
        float o = 0.0f;
        for (int s = 0; s < P.top_k; s++) o += P.weights[tok * P.top_k + s] * ysum[s * 16 + lane];
        if (row < P.n) P.out[(int64_t)tok * P.n + row] = o;
    }
}

} // namespace

bool qmm_moe_small_supported(const QmmLayout& G, const QmmLayout& D, int64_t t, int n_experts, int top_k) {
    // one panel per row tile of the down projection (k = inter <= 1024), a wave per slot
    return t >= 1 && t * top_k <= 64 && top_k <= kMaxWaves && n_experts <= 256 && D.k_groups == 1 && D.k_units <= 4 &&
           G.k_groups <= kMaxWaves / 2;
}

hipError_t qmm_launch_moe_small(const QmmLayout& G, const void* gate, const void* up, const QmmLayout& D, const void* down,
                                const float* logits, const float* x, int64_t t, int n_experts, int top_k, float* h,
                                int32_t* ids, float* weights, int32_t* ids_out, float* weights_out, float* out,
                                int64_t max_segments, int n_cus, hipStream_t stream) {
    if (!qmm_moe_small_supported(G, D, t, n_experts, top_k)) return hipErrorNotSupported;
    const int pairs = (int)(t * top_k);
    GemvParams P;
    if (!make_params(G, gate, x, 1, h, P)) return hipErrorInvalidValue;
    P.w2 = (const uint8_t*)up;
    int waves;
    // the split of the grouped launch this replaces: same sums
    choose_split(G, n_cus, (int)max_segments, true, P, waves);
    if (P.kpw != 1 || P.rt_groups > n_cus * 32) return hipErrorNotSupported;
    hipError_t e = with_block_type(G.dtype, [&](auto QT) {
        constexpr int qt = decltype(QT)::value;
        const size_t lds = lds_bytes<qt, 1>(P.k_units, 2 * waves);
        if (lds > 48 * 1024) return hipErrorNotSupported;
        const dim3 grid((unsigned)P.rt_groups, (unsigned)pairs), block(64 * 2 * waves);
        if (n_experts <= 128)
            moe_small_gate_up_kernel<qt, 2><<<grid, block, lds, stream>>>(P, logits, n_experts, top_k, ids, weights, ids_out, weights_out);
        else
            moe_small_gate_up_kernel<qt, 4><<<grid, block, lds, stream>>>(P, logits, n_experts, top_k, ids, weights, ids_out, weights_out);
        return hipGetLastError();
    });
    if (e != hipSuccess) return e;
    MoeSmallDown Q;
    Q.w = (const uint8_t*)down;
    Q.h = h;
    Q.ids = ids;
    Q.weights = weights;
    Q.out = out;
    Q.n = (int)D.n, Q.k = (int)D.k, Q.k_units = (int)D.k_units, Q.slots = D.slots, Q.row_tiles = (int)D.row_tiles;
    Q.top_k = top_k;
    Q.panel_bytes = (int)D.panel_bytes;
    Q.matrix_bytes = D.matrix_bytes;
    return with_block_type(D.dtype, [&](auto QT) {
        constexpr int qt = decltype(QT)::value;
        const size_t per_wave = (lds_bytes<qt, 1>(Q.k_units, 0) + 15) & ~(size_t)15;
        const size_t lds = per_wave * top_k + (size_t)top_k * 16 * sizeof(float);
        if (lds > 48 * 1024) return hipErrorNotSupported;
        moe_small_down_kernel<qt><<<dim3((unsigned)D.row_tiles, (unsigned)t), dim3(64 * top_k), lds, stream>>>(Q);
        return hipGetLastError();
    });
}

hipError_t qmm_launch_gemv_grouped(const QmmLayout& L, const void* tiled, const void* tiled2,
                                   const float* x, int x_div, float* y, const int32_t* perm,
                                   const int32_t* offsets, const int32_t* seg_offsets,
                                   const int32_t* seg_expert, int n_experts, int64_t max_segments,
                                   int n_cus, hipStream_t stream, const void* x_blocks, int64_t x_rows) {
    if (max_segments <= 0 || L.n == 0) return hipSuccess;
    if (max_segments > 65535) return hipErrorInvalidValue;
    GemvParams P;
    if (!make_params(L, tiled, x, 0, y, P)) return hipErrorInvalidValue;
    P.w2 = (const uint8_t*)tiled2;
    P.perm = perm;
    P.offsets = offsets;
    P.seg_offsets = seg_offsets;
    P.seg_expert = seg_expert;
    P.n_experts = n_experts;
    P.x_div = x_div;
    if (x_blocks) P.xb = x_blocks_carve(const_cast<void*>(x_blocks), x_rows, L.k_units);
    const bool gated = tiled2 != nullptr;
    int waves;
    choose_split(L, n_cus, (int)max_segments, gated, P, waves);
    if (L.dtype == QMM_Q4_K)
        return gated ? launch_mt<QMM_Q4_K, 4, true, true>(P, waves, n_cus, (int)max_segments, stream)
                     : launch_mt<QMM_Q4_K, 4, false, true>(P, waves, n_cus, (int)max_segments, stream);
    if (L.dtype == QMM_Q6_K)
        return gated ? launch_mt<QMM_Q6_K, 4, true, true>(P, waves, n_cus, (int)max_segments, stream)
                     : launch_mt<QMM_Q6_K, 4, false, true>(P, waves, n_cus, (int)max_segments, stream);
    return gated ? launch_mt<QMM_Q8_0, 4, true, true>(P, waves, n_cus, (int)max_segments, stream)
                 : launch_mt<QMM_Q8_0, 4, false, true>(P, waves, n_cus, (int)max_segments, stream);
}

hipError_t qmm_launch_quantize_activations(int weight_dtype, const float* x, int64_t m, int64_t k,
                                           void* out_blocks, hipStream_t stream) {
    int64_t k_units = (k + 255) / 256;
    int64_t threads = m * k_units * 16;
    if (threads == 0) return hipSuccess;
    unsigned grid = (unsigned)((threads + 255) / 256);
    if (weight_dtype == QMM_Q4_K || weight_dtype == QMM_Q6_K) // both dot types are Q8_K
        quantize_export_kernel<QMM_Q4_K>
            <<<grid, 256, 0, stream>>>(x, m, k, k_units, (uint8_t*)out_blocks);
    else
        quantize_export_kernel<QMM_Q8_0>
            <<<grid, 256, 0, stream>>>(x, m, k, k_units, (uint8_t*)out_blocks);
    return hipGetLastError();
}
