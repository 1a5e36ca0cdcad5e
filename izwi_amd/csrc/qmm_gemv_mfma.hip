// Batched decode kernels (M = 3..64): the same arithmetic as the M <= 2 kernel
// (candle-core's integer block dots on Q8-quantized activations), with the
// int8 products on v_mfma_i32_16x16x32_i8 so that the cost per weight byte does
// not grow with M.
//
// Two launches:
//  1. the activations are quantized ONCE into a workspace of self-contained
//     unit records (256 k-values of 16 rows): 4096 B of int8 laid out exactly as
//     the MFMA A operand wants them ([sub-block pair][octet][row][16 B]) followed by
//     the unit's side information (row scales; for Q4_K also the sub-block sums
//     as two int8 planes), so the matmul workgroups move a run of units to LDS
//     verbatim with LDS-direct loads;
//  2. a wave streams weight panels (16 rows x S units) as in the M <= 2 kernel.
//     A panel lane holds one (row, unit); the MFMA B operand wants (row, 8-element
//     octet) per lane, so the quants are transposed between the four 16-lane rows
//     in registers (v_permlane32_swap + v_permlane16_swap, two swaps per dword).
//     One MFMA per 32-element sub-block: D[m][row] are the block dots of 16
//     activation rows at once; the 6-bit sub-block scales are applied on integers
//     (v_mad_i32_i24), the Q4_K min term is itself a matmul over the sub-block
//     index (two MFMAs per unit).  The panel is consumed chunk pair by chunk pair
//     in load order, so the arithmetic runs while the rest of the panel arrives.
//
// Two forms of launch 2:
//  * one-shot: every wave owns exactly one panel, all panels of the matrix are
//    requested at once (after the first activation window); a workgroup is nwk
//    waves along k times nwr row-tiles.  Activation windows (up to 32 units) that
//    do not fit LDS together follow one another, the panels stay in registers;
//  * streaming (very tall matrices): a wave owns whole row-tiles and walks their
//    panels, the activation window stays in LDS for all of them.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>

#include "qmm_internal.h"
#include "qmm_moe_route.h"
#include "qmm_records.h"

// Timing-only ablations of the Q4_K single-tile arithmetic (results are WRONG when set; never defined
// in the library's build): bit 0 drops the integer scale multiply-adds (the matrix instruction
// accumulates instead), bit 1 the in-register transposition, bit 2 the nibble split, bit 3 the f32
// finish and the min term, bit 4 the copy of the activation window into LDS, bit 5 the stores; bit 6
// restores the one-wave k-split finish; bit 7 (Q4_K expert form) keeps a panel's load and preparation
// and drops its arithmetic against the tiles.
#ifndef QMM_MFMA_ABL
#define QMM_MFMA_ABL 0
#endif

// Measurement build only (-DQMM_EXPERT_TRACE, never defined in the library's build): the Q4_K expert
// kernel records, per work item and wave, the 100 MHz clock at the item's start, when its tiles had
// landed and at its end, with the CU it ran on; izwi_qmm_expert_trace_read copies the records out
// (izwi_amd/csrc/expert_trace.py prints a summary).  Record (w, i) of 8 words sits at ((launch kind *
// 512 + round * 256 + workgroup) * 8 + wave) * 8; launch kind 0: four-unit panels, 1: three-unit panels.
#ifdef QMM_EXPERT_TRACE
__device__ unsigned long long g_expert_trace[8 * 8192];
extern "C" int izwi_qmm_expert_trace_read(void* dst, size_t bytes) {
    if (bytes > sizeof(unsigned long long) * 8 * 8192) return -1;
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_expert_trace), bytes, 0, hipMemcpyDeviceToHost);
}
#endif

namespace {

constexpr int kMaxWaves = 12;
constexpr uint32_t kNib = 0x0f0f0f0fu;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef long i64x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kWindowUnits = 32; // activation units resident in LDS at a time

__host__ __device__ inline int unit_bytes(int qt) { return qt == QMM_Q8_0 ? Unit<QMM_Q8_0>::kBytes : Unit<QMM_Q4_K>::kBytes; }

// Workgroup barrier that orders LDS traffic only (the compiler's own barrier also
// waits for every outstanding global load of the wave).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Sixteen consecutive values of a row (k is a multiple of 32: the run is inside
// the row or past its end), zeros when out of range.
// XB: the values are bf16 (widened exactly).
template <bool XB = false>
__device__ __forceinline__ void load_run16(const void* __restrict__ src, const void* __restrict__ safe,
                                           bool in_range, float (&v)[16]) {
    if (XB) {
        const uint4* p = reinterpret_cast<const uint4*>(in_range ? src : safe);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint4 f = p[i];
            const uint32_t w[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                v[8 * i + 2 * c] = in_range ? __uint_as_float(w[c] << 16) : 0.0f;
                v[8 * i + 2 * c + 1] = in_range ? __uint_as_float(w[c] & 0xffff0000u) : 0.0f;
            }
        }
        return;
    }
    const float4* p = reinterpret_cast<const float4*>(in_range ? src : safe);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 f = p[i];
        v[4 * i] = in_range ? f.x : 0.0f, v[4 * i + 1] = in_range ? f.y : 0.0f;
        v[4 * i + 2] = in_range ? f.z : 0.0f, v[4 * i + 3] = in_range ? f.w : 0.0f;
    }
}

template <int QT, bool XB = false>
__global__ void quantize_ws_kernel(const void* __restrict__ x, int m, int k, int k_units, int n_tiles,
                                   uint8_t* __restrict__ ws) {
    // (a workgroup of 256 threads = the 16 rows of one (tile, unit): it writes that unit record whole)
    const int group = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    const int rows = n_tiles * 16;
    if (group >= rows * k_units) return; // whole 16-lane groups leave together
    const int mr = group & 15, tu = group >> 4;
    const int tile = tu / k_units, unit = tu - tile * k_units;
    const int row = tile * 16 + mr;
    float v[16];
    const int k0 = unit * 256 + 16 * j;
    if (XB) load_run16<true>(static_cast<const uint16_t*>(x) + (int64_t)row * k + k0, x, row < m && k0 + 16 <= k, v);
    else load_run16<false>(static_cast<const float*>(x) + (int64_t)row * k + k0, x, row < m && k0 + 16 <= k, v);
    quantize_into_record<QT>(v, j, mr, ws + ((int64_t)tile * k_units + unit) * Unit<QT>::kBytes);
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }

// The same quantizer on silu(gate) * up (the MLP's activation, worked out on the way in).
template <int QT>
__global__ void quantize_silu_mul_ws_kernel(const float* __restrict__ gate, const float* __restrict__ up, int m, int k,
                                            int k_units, int n_tiles, uint8_t* __restrict__ ws) {
    const int group = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    const int rows = n_tiles * 16;
    if (group >= rows * k_units) return; // whole 16-lane groups leave together
    const int mr = group & 15, tu = group >> 4; // (a workgroup = the 16 rows of one (tile, unit), as above)
    const int tile = tu / k_units, unit = tu - tile * k_units;
    const int row = tile * 16 + mr;
    float g[16], u[16];
    const int k0 = unit * 256 + 16 * j;
    const bool ok = row < m && k0 + 16 <= k;
    load_run16<false>(gate + (int64_t)row * k + k0, gate, ok, g);
    load_run16<false>(up + (int64_t)row * k + k0, up, ok, u);
#pragma unroll
    for (int i = 0; i < 16; i++) g[i] = silu_f(g[i]) * u[i];
    quantize_into_record<QT>(g, j, mr, ws + ((int64_t)tile * k_units + unit) * Unit<QT>::kBytes);
}

// Expert-grouped form: tile g of the list belongs to the expert e with
// tile_offsets[e] <= g < tile_offsets[e + 1]; its row r is sorted pair
// offsets[e] + 16 (g - tile_offsets[e]) + r (rows past the expert's end are zero),
// pair p = perm[..] reads activation row p / x_div; with x2 the value is
// silu(x) * x2 (the expert MLP's gate/up product feeding the down projection).
template <int QT>
__global__ void quantize_grouped_kernel(const float* __restrict__ x, const float* __restrict__ x2, int x_div,
                                        int k, int k_units, const int32_t* __restrict__ perm,
                                        const int32_t* __restrict__ offsets,
                                        const int32_t* __restrict__ tile_offsets, int n_experts,
                                        const int32_t* __restrict__ tile_expert, uint8_t* __restrict__ ws) {
    // a workgroup of 256 threads = the 16 rows of one (tile, unit): it writes that unit record whole
    // (with a row's units side by side in a workgroup, every record was put together from the 8-byte
    // pieces of 16 workgroups)
    const int64_t group = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    const int mr = (int)(group & 15);
    const int64_t tu = group >> 4;
    const int tile = (int)(tu / k_units);
    const int unit = (int)(tu - (int64_t)tile * k_units);
    if (tile >= tile_offsets[n_experts]) return; // whole 16-lane groups leave together
    int lo = 0, hi = n_experts; // last e with tile_offsets[e] <= tile: from the table, or searched for
    if (tile_expert) {
        lo = tile_expert[tile];
    } else {
        while (hi - lo > 1) { // seven dependent loads at 128 experts
            const int mid = (lo + hi) >> 1;
            if (tile_offsets[mid] <= tile) lo = mid;
            else hi = mid;
        }
    }
    const int pos = offsets[lo] + (tile - tile_offsets[lo]) * 16 + mr;
    const bool row_ok = pos < offsets[lo + 1];
    const int64_t src_row = row_ok ? perm[pos] / x_div : 0;
    const int k0 = unit * 256 + 16 * j;
    const bool in_range = row_ok && k0 + 16 <= k;
    float v[16];
    load_run16(x + src_row * k + k0, x, in_range, v);
    if (x2 != nullptr) {
        float u[16];
        load_run16(x2 + src_row * k + k0, x2, in_range, u);
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = silu_f(v[i]) * u[i];
    }
    quantize_into_record<QT>(v, j, mr, ws + ((int64_t)tile * k_units + unit) * Unit<QT>::kBytes);
}

// Row records (see kRowUnitBytes): rows [0, rows) of x, or of silu(x) * x2, one 16-lane group per
// (row, unit), no index tables.
template <int QT>
__global__ void quantize_rows_kernel(const float* __restrict__ x, const float* __restrict__ x2, int64_t rows, int k,
                                     int k_units, uint8_t* __restrict__ out) {
    const int64_t group = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    if (group >= rows * k_units) return; // whole 16-lane groups leave together
    const int64_t row = group / k_units;
    const int unit = (int)(group - row * k_units);
    const int k0 = unit * 256 + 16 * j;
    const bool in_range = k0 + 16 <= k;
    float v[16];
    load_run16(x + row * k + k0, x, in_range, v);
    if (x2 != nullptr) {
        float u[16];
        load_run16(x2 + row * k + k0, x2, in_range, u);
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = silu_f(v[i]) * u[i];
    }
    quantize_into_record<QT, true>(v, j, 0, out + group * kRowUnitBytes);
}

// Routing of the tokens with the row records of their activation rows: the routing kernel of
// qmm_moe.hip with the matrix-core kernels' quantizer.  Two wavefronts per token, in the two halves
// of the workgroup: one routes, the other quantizes the token's row meanwhile (one wave doing both in
// turn made the launch as long as their sum, and the sort waits for this launch to end).
template <int PER_LANE, int QT>
__global__ void route_rows_kernel(const float* __restrict__ logits, int64_t t, int n_experts, int top_k,
                                  int32_t* __restrict__ ids, float* __restrict__ weights,
                                  const float* __restrict__ x, int k, int k_units, uint8_t* __restrict__ out) {
    const int lane = threadIdx.x & 63, j = lane & 15;
    const int wave = threadIdx.x >> 6, tokens_per_block = blockDim.x >> 7;
    const bool quantizes = wave >= tokens_per_block; // (uniform per wave)
    const int64_t tok = (int64_t)blockIdx.x * tokens_per_block + (quantizes ? wave - tokens_per_block : wave);
    if (tok >= t) return; // whole waves leave together
    if (!quantizes) {
        int id;
        float w;
        moe_route::route_token<PER_LANE>(logits + tok * n_experts, n_experts, top_k, lane, id, w);
        if (lane < top_k) {
            ids[tok * top_k + lane] = id;
            weights[tok * top_k + lane] = w;
        }
        return;
    }
    uint8_t* rec = out + tok * k_units * kRowUnitBytes;
    for (int unit = lane >> 4; unit < k_units; unit += 4) {
        const int k0 = unit * 256 + 16 * j;
        float v[16];
        load_run16(x + tok * k + k0, x, k0 + 16 <= k, v);
        quantize_into_record<QT, true>(v, j, 0, rec + unit * kRowUnitBytes);
    }
}

// ---- launch 2 ------------------------------------------------------------------
struct MfmaParams {
    const uint8_t* w;
    const uint8_t* ws; // unit records [n_tiles][k_units]
    float* y;
    const uint8_t* w2; // grouped and expert forms: second stack and its output
    float* y2;
    int double_buf;    // two LDS windows
    // several weights of equal k and type on the same records in one launch (SINGLE form):
    // workgroup b belongs to weight i with rtg_end[i - 1] <= b < rtg_end[i]
    int n_weights; // 0 or 1: just w / y / n / row_tiles above
    int rtg_end[QMM_MAX_GROUP];
    int nv[QMM_MAX_GROUP], row_tiles_v[QMM_MAX_GROUP];
    const uint8_t* wv[QMM_MAX_GROUP];
    float* yv[QMM_MAX_GROUP];
    int m, n;
    int k_units, k_groups, slots;
    int row_tiles, panel_bytes;
    int nwk, nwr, wave_magic;
    int n_tiles;
    int window_units; // multiple of s, <= kWindowUnits
    int rt_groups;
    // expert-grouped form: a one-dimensional grid; a workgroup's (expert, stack, row-tile group)
    // is decoded so that all workgroups of an expert run on one XCD (see the kernel)
    int n_experts, stacks;
    int parts; // expert forms: the row tiles of a stack are shared out to this many items
    // expert forms on row records (row_div > 0): ws holds one record per (source row, unit) and sorted
    // pair p reads source row perm[p] / row_div = (perm[p] * row_magic) >> 32
    int row_div;
    uint32_t row_magic;
    // expert forms: the experts by falling tile count with their ranges (8 ints per rank: expert, first
    // tile, tiles, first and last + 1 sorted pair), or NULL (ranked in the kernel, ranges from the tables)
    const int32_t* expert_order;
    const int32_t* perm;
    const int32_t* offsets;      // sorted pairs of expert e: [offsets[e], offsets[e + 1])
    const int32_t* tile_offsets; // its 16-row tiles (records): [tile_offsets[e], tile_offsets[e + 1])
    int64_t matrix_bytes;
    // dense forms only: y = sums (+ residual), stored as f32 or bf16 (y then points to bf16)
    QmmEpilogue ep;
};

// The matrix-core kernels take the fields that their first loads need as leading scalar arguments
// (14 dwords): those arrive in scalar registers with the wave (kernel-argument preload), the
// rest of the parameter block is read from memory.  with_leading_args puts them back into a
// copy of the block; the tables of a group of weights are indexed in the block itself (P0).
__device__ __forceinline__ MfmaParams with_leading_args(const MfmaParams& P0, const uint8_t* w, const uint8_t* ws, float* y,
                                                        int k_units, int k_groups, int row_tiles, int panel_bytes,
                                                        int split, int wave_magic, int n_tiles, int window) {
    MfmaParams P = P0;
    P.w = w, P.ws = ws, P.y = y, P.k_units = k_units, P.k_groups = k_groups, P.row_tiles = row_tiles;
    P.panel_bytes = panel_bytes, P.wave_magic = wave_magic, P.n_tiles = n_tiles;
    P.nwk = split & 255, P.nwr = (split >> 8) & 255, P.slots = (split >> 16) & 255, P.n_weights = split >> 24;
    P.window_units = window & 0xffff, P.double_buf = window >> 16;
    return P;
}

template <class Kernel>
void launch_mfma(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const MfmaParams& P) {
    kernel<<<grid, block, lds, stream>>>(P.w, P.ws, P.y, P.k_units, P.k_groups, P.row_tiles, P.panel_bytes,
                                         P.nwk | (P.nwr << 8) | (P.slots << 16) | (P.n_weights << 24), P.wave_magic, P.n_tiles,
                                         P.window_units | (P.double_buf << 16), P);
}

// The entry of a group of weights for workgroup b: the tables are read whole (independent scalar
// loads, one round trip) and the entry is picked with selects; rtg_end ascends, so the entry is
// the number of ends at or below b.  Entries past n_weights hold whatever the host left there
// and are never picked.
__device__ __forceinline__ void pick_group_entry(const MfmaParams& P0, int n_weights, int b, int& rtg, const uint8_t*& wbase,
                                                 float*& yout, int& n_rows, int& row_tiles) {
    static_assert(QMM_MAX_GROUP == 4, "the selects below name four entries");
    const int e0 = P0.rtg_end[0], e1 = P0.rtg_end[1], e2 = P0.rtg_end[2];
    const bool c1 = b >= e0, c2 = n_weights > 2 && b >= e1, c3 = n_weights > 3 && b >= e2;
    auto pick = [c1, c2, c3](auto v0, auto v1, auto v2, auto v3) {
        auto v = c1 ? v1 : v0;
        v = c2 ? v2 : v;
        return c3 ? v3 : v;
    };
    rtg = b - pick(0, e0, e1, e2);
    wbase = pick(P0.wv[0], P0.wv[1], P0.wv[2], P0.wv[3]);
    yout = pick(P0.yv[0], P0.yv[1], P0.yv[2], P0.yv[3]);
    n_rows = pick(P0.nv[0], P0.nv[1], P0.nv[2], P0.nv[3]);
    row_tiles = pick(P0.row_tiles_v[0], P0.row_tiles_v[1], P0.row_tiles_v[2], P0.row_tiles_v[3]);
}

// 4x4 transpose of one dword between the four 16-lane rows: on entry row u
// holds X_u[t] in r[t]; on exit row t holds X_u[t] in r[u].
__device__ __forceinline__ void transpose_rows(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
    u32x2 a = __builtin_amdgcn_permlane32_swap(r0, r2, false, false);
    u32x2 b = __builtin_amdgcn_permlane32_swap(r1, r3, false, false);
    u32x2 c = __builtin_amdgcn_permlane16_swap(a.x, b.x, false, false);
    u32x2 d = __builtin_amdgcn_permlane16_swap(a.y, b.y, false, false);
    r0 = c.x, r1 = c.y, r2 = d.x, r3 = d.y;
}

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi) {
    return (long)(((unsigned long)hi << 32) | lo);
}

// (row, unit) per lane -> (row, octet) per lane for chunk pair b: afterwards unit u of
// the pair sits in dwords (x,y) / (z,w) of q[2b] / q[2b+1]:
//   u = 0: q[2b].xy   u = 1: q[2b].zw   u = 2: q[2b+1].xy   u = 3: q[2b+1].zw
__device__ __forceinline__ void transpose_pair(u32x4& q0, u32x4& q1) {
    uint32_t a0 = q0.x, a1 = q0.z, a2 = q1.x, a3 = q1.z;
    uint32_t b0 = q0.y, b1 = q0.w, b2 = q1.y, b3 = q1.w;
    transpose_rows(a0, a1, a2, a3);
    transpose_rows(b0, b1, b2, b3);
    q0 = u32x4{a0, b0, a1, b1};
    q1 = u32x4{a2, b2, a3, b3};
}

template <int QT>
struct WPanel {
    // quant chunks held per lane: Q6_K's are the 8 of low nibbles and the 4 of high bit pairs
    static constexpr int QC = QT == QMM_Q4_K ? 8 : (QT == QMM_Q6_K ? 12 : 16);
    static constexpr int kLoads = QC + 4 + (QT == QMM_Q6_K ? 4 : 0); // vector loads of one panel
    u32x4 hdr[4]; // headers of the four units of row j
    u32x4 q[QC];
    u32x4 dch[QT == QMM_Q6_K ? 4 : 1]; // Q6_K: the chunks that hold d of the four units of row j
};

// Unconditional loads (one basic block, so the waits can be counted): a lane
// without a slot reads slot 0, units past s re-read unit 0's header; neither is
// used afterwards.
template <int QT>
__device__ __forceinline__ void load_wpanel(WPanel<QT>& p, const uint8_t* __restrict__ base, int slots,
                                            int lane, int j) {
    const u32x4* b = reinterpret_cast<const u32x4*>(base);
    const int ln = lane < slots ? lane : 0;
    // Addresses as the uniform `base` plus a 32-bit lane offset (the scalar-base form of the load).  The
    // empty statements keep the offsets' widening to 64 bits in this block: moved out of a caller's
    // loop, the widened offsets are a register pair and a 64-bit add per load.
    uint32_t j16 = (uint32_t)j * 16u, ln16 = (uint32_t)ln * 16u;
    asm volatile("" : "+v"(j16));
    asm volatile("" : "+v"(ln16));
#pragma unroll
    for (int u = 0; u < 4; u++)
        p.hdr[u] = *reinterpret_cast<const u32x4*>(base + ((uint32_t)(u * 16 < slots ? u * 256 : 0) + j16));
    if (QT == QMM_Q6_K) {
        // in the order panel_dot consumes them (loads return in order): per half of the units' 256
        // elements first its two chunks of bit pairs, then its four of nibbles; d last
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int c = 0; c < 2; c++) p.q[8 + 2 * h + c] = __builtin_nontemporal_load(b + (size_t)(9 + 2 * h + c) * slots + ln);
#pragma unroll
            for (int c = 0; c < 4; c++) p.q[4 * h + c] = __builtin_nontemporal_load(b + (size_t)(1 + 4 * h + c) * slots + ln);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) p.dch[u] = b[(size_t)13 * slots + (u * 16 < slots ? u * 16 : 0) + j];
        return;
    }
    // (a uniform chunk address plus one 32-bit lane offset for all chunks: the scalar-base form of the
    // load, where a 64-bit address per lane and chunk costs two registers and an add each)
#pragma unroll
    for (int c = 0; c < WPanel<QT>::QC; c++) {
        const uint32_t off = (uint32_t)((1 + c) * slots * 16) + ln16; // (a panel is under 32 KiB)
        p.q[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + off));
    }
}

// sum + s0 * d0 + s1 * d1 (24-bit factors) as two multiply-adds.  The empty statement behind each
// keeps the compiler from regrouping the sums into two multiplies and a three-operand add: three
// instructions where two do (the scale multiplies are the largest share of these kernels' vector
// instructions).  It names only `sum`, the result of a vector instruction.
__device__ __forceinline__ int scaled_pair_sum(int s0, int d0, int s1, int d1, int sum) {
    sum = __mul24(s0, d0) + sum;
    asm volatile("" : "+v"(sum));
    sum = __mul24(s1, d1) + sum;
    asm volatile("" : "+v"(sum));
    return sum;
}

// The Q4_K arithmetic of one panel against one 16-row tile of activations, shared by the LDS forms
// and the register-direct form.  `a_of(u, b)` returns the tile's two matrix-core operands of unit u,
// sub-block pair b (16 bytes per lane), `side_of(u, bs_lo, bs_hi, dx)` the unit's sub-block sum planes
// (k slots of the first 16-lane row only) and this lane group's four row scales.
// NU: the number of the panel's units that exist as a compile-time constant - straight-line code, in
// which the LDS reads, the matrix instructions and the integer scale multiply-adds of different units
// interleave (a wave that is alone on its SIMD has nothing else to hide their latencies) - or 0:
// `n_units` (uniform) at run time, with a branch around every unit.
// FIRST: the quants are still in load layout and are transposed pair by pair, in load order.
template <bool FIRST, int NU, class AFetch, class SFetch>
__device__ __forceinline__ void q4k_panel_dot(WPanel<QMM_Q4_K>& p, int n_units, AFetch&& a_of, SFetch&& side_of,
                                              float (&acc)[4]) {
    const int nu = NU ? NU : n_units;
    // 6-bit scales of the four units (byte i of sc_lo / sc_hi = scale i / i + 4); the mins are only
    // needed at the end and are unpacked there
    uint32_t sc_lo[4], sc_hi[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        sc_lo[u] = p.hdr[u].y & 0x3f3f3f3fu;
        sc_hi[u] = (p.hdr[u].w & 0x0f0f0f0fu) | (((p.hdr[u].y >> 6) & 0x03030303u) << 4);
    }
    int isum[4][4];
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
        for (int r = 0; r < 4; r++) isum[u][r] = 0;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        if (FIRST && !(QMM_MFMA_ABL & 2)) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            // two units at a time: their four matrix instructions are issued back to back and the
            // results consumed afterwards (the matrix pipe's latency is paid once)
            const u32x4 qq = p.q[2 * b + h];
            i32x4 dlo[2], dhi[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int u = 2 * h + e;
                if (u >= nu) continue; // compile-time, or uniform
                const uint32_t w0 = e ? qq.z : qq.x, w1 = e ? qq.w : qq.y;
                const i64x2 aa = a_of(u, b);
                if (QMM_MFMA_ABL & 5) { // timing only: no scale products (the sums chain through the matrix
                                        // instructions) and / or no nibble split
                    const long blo = (QMM_MFMA_ABL & 4) ? pack64(w0, w1) : pack64(w0 & kNib, w1 & kNib);
                    const long bhi = (QMM_MFMA_ABL & 4) ? pack64(w1, w0) : pack64((w0 >> 4) & kNib, (w1 >> 4) & kNib);
                    const i32x4 c0 = (QMM_MFMA_ABL & 1) ? i32x4{isum[u][0], isum[u][1], isum[u][2], isum[u][3]} : i32x4{0, 0, 0, 0};
                    dlo[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.x, blo, c0, 0, 0, 0);
                    dhi[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.y, bhi, (QMM_MFMA_ABL & 1) ? dlo[e] : i32x4{0, 0, 0, 0}, 0, 0, 0);
                    if (QMM_MFMA_ABL & 1) {
#pragma unroll
                        for (int r = 0; r < 4; r++) isum[u][r] = dhi[e][r];
                    }
                    continue;
                }
                dlo[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.x, pack64(w0 & kNib, w1 & kNib), i32x4{0, 0, 0, 0}, 0, 0, 0);
                dhi[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.y, pack64((w0 >> 4) & kNib, (w1 >> 4) & kNib),
                                                               i32x4{0, 0, 0, 0}, 0, 0, 0);
            }
            if (QMM_MFMA_ABL & 1) continue;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int u = 2 * h + e;
                if (u >= nu) continue;
                const int sc0 = (int)qmm_byte_of(sc_lo[u], sc_hi[u], 2 * b);
                const int sc1 = (int)qmm_byte_of(sc_lo[u], sc_hi[u], 2 * b + 1);
#pragma unroll
                for (int r = 0; r < 4; r++) // |dot| < 2^17, scale < 64
                    isum[u][r] = scaled_pair_sum(sc0, dlo[e][r], sc1, dhi[e][r], isum[u][r]);
            }
        }
    }
    if (QMM_MFMA_ABL & 8) { // timing only: no min term, no f32 finish
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += __int_as_float(isum[u][r] + (int)p.hdr[u].x);
        return;
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
        if (u >= nu) continue;
        const float d = qmm_f16_bits_to_f32((uint16_t)(p.hdr[u].x & 0xffffu));
        const float dmin = qmm_f16_bits_to_f32((uint16_t)(p.hdr[u].x >> 16));
        const uint32_t mn_lo = p.hdr[u].z & 0x3f3f3f3fu;
        const uint32_t mn_hi = ((p.hdr[u].w >> 4) & 0x0f0f0f0fu) | (((p.hdr[u].z >> 6) & 0x03030303u) << 4);
        // min term: sum_s min_s * bsum_s as two matrix instructions over k = sub-block index; only
        // the first 16-lane row carries data (k slots 0..7), the rest multiply zeros
        long bs_lo, bs_hi;
        float4 dx;
        side_of(u, bs_lo, bs_hi, dx);
        const long bmn = pack64(mn_lo, mn_hi);
        const i32x4 m_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_lo, bmn, i32x4{0, 0, 0, 0}, 0, 0, 0);
        const i32x4 m_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_hi, bmn, i32x4{0, 0, 0, 0}, 0, 0, 0);
        const float dxs[4] = {dx.x, dx.y, dx.z, dx.w};
#pragma unroll
        for (int r = 0; r < 4; r++) {
            // (d isum - dmin msum) dx: both integers are exact in f32 (|isum| < 2^26 only in theory:
            // 2^24 needs every product of a block at its extreme), two roundings per unit
            const int msum = m_lo[r] + (m_hi[r] << 7);
            acc[r] = fmaf(fmaf(-dmin, (float)msum, d * (float)isum[u][r]), dxs[r], acc[r]);
        }
    }
}


// A Q4_K panel prepared for several tiles of activations (the multi-stage forms: an expert's tiles, a
// batch of more than 16 rows walked inside one workgroup): what does not depend on the activations is done once per panel
// instead of once per (panel, tile) - the nibbles split into the two matrix-core operands of every
// (unit, sub-block pair), the 6-bit scales and mins unpacked, d and dmin converted.  Twice the
// registers of the packed quants, so the units are walked one after the other (four running sums
// instead of sixteen).  Same integers and the same f32 operations as q4k_panel_dot: same bits.
template <int NU>
struct Q4Prepared {
    long lo[NU][4], hi[NU][4]; // [unit][pair]: quants of sub-block 2b / 2b + 1, this lane's octet
    uint32_t sc_lo[NU], sc_hi[NU];
    long bmn[NU];
    float d[NU], dmin[NU];
};

// `p` transposed already (transpose_pair on every chunk pair).
template <int NU>
__device__ __forceinline__ void q4k_prepare(const WPanel<QMM_Q4_K>& p, Q4Prepared<NU>& t, int grp) {
#pragma unroll
    for (int u = 0; u < NU; u++) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const u32x4 qq = p.q[2 * b + (u >> 1)];
            const uint32_t w0 = (u & 1) ? qq.z : qq.x, w1 = (u & 1) ? qq.w : qq.y;
            t.lo[u][b] = pack64(w0 & kNib, w1 & kNib);
            t.hi[u][b] = pack64((w0 >> 4) & kNib, (w1 >> 4) & kNib);
        }
        t.sc_lo[u] = p.hdr[u].y & 0x3f3f3f3fu;
        t.sc_hi[u] = (p.hdr[u].w & 0x0f0f0f0fu) | (((p.hdr[u].y >> 6) & 0x03030303u) << 4);
        const uint32_t mn_lo = p.hdr[u].z & 0x3f3f3f3fu;
        const uint32_t mn_hi = ((p.hdr[u].w >> 4) & 0x0f0f0f0fu) | (((p.hdr[u].z >> 6) & 0x03030303u) << 4);
        // the min term's matrix instructions use k slots 0..7 (the first 16-lane row); the other rows'
        // slots are made zero HERE, once per panel, so that the activation side needs no select per tile
        t.bmn[u] = grp == 0 ? pack64(mn_lo, mn_hi) : 0L;
        t.d[u] = qmm_f16_bits_to_f32((uint16_t)(p.hdr[u].x & 0xffffu));
        t.dmin[u] = qmm_f16_bits_to_f32((uint16_t)(p.hdr[u].x >> 16));
    }
}

template <int NU, class AFetch, class SFetch>
__device__ __forceinline__ void q4k_tile_dot(const Q4Prepared<NU>& t, AFetch&& a_of, SFetch&& side_of, float (&acc)[4]) {
#pragma unroll
    for (int u = 0; u < NU; u++) {
        int isum[4] = {0, 0, 0, 0};
#pragma unroll
        for (int b2 = 0; b2 < 2; b2++) {
            i32x4 dlo[2], dhi[2];
#pragma unroll
            for (int bb = 0; bb < 2; bb++) {
                const int b = 2 * b2 + bb;
                const i64x2 aa = a_of(u, b);
                dlo[bb] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.x, t.lo[u][b], i32x4{0, 0, 0, 0}, 0, 0, 0);
                dhi[bb] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aa.y, t.hi[u][b], i32x4{0, 0, 0, 0}, 0, 0, 0);
            }
#pragma unroll
            for (int bb = 0; bb < 2; bb++) {
                const int b = 2 * b2 + bb;
                const int sc0 = (int)qmm_byte_of(t.sc_lo[u], t.sc_hi[u], 2 * b);
                const int sc1 = (int)qmm_byte_of(t.sc_lo[u], t.sc_hi[u], 2 * b + 1);
#pragma unroll
                for (int r = 0; r < 4; r++) isum[r] = scaled_pair_sum(sc0, dlo[bb][r], sc1, dhi[bb][r], isum[r]);
            }
        }
        long bs_lo, bs_hi;
        float4 dx;
        side_of(u, bs_lo, bs_hi, dx);
        const i32x4 m_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_lo, t.bmn[u], i32x4{0, 0, 0, 0}, 0, 0, 0);
        const i32x4 m_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_hi, t.bmn[u], i32x4{0, 0, 0, 0}, 0, 0, 0);
        const float dxs[4] = {dx.x, dx.y, dx.z, dx.w};
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int msum = m_lo[r] + (m_hi[r] << 7);
            acc[r] = fmaf(fmaf(-t.dmin[u], (float)msum, t.d[u] * (float)isum[r]), dxs[r], acc[r]);
        }
    }
}

// acc[r] += block dots of the panel's units against activation rows 4 grp + r of
// the tile whose unit records start at `xu0` (LDS, record of the panel's unit 0).
// FIRST: the quants are still in load layout and are transposed pair by pair, in
// load order.  `n_units` (uniform) is the number of the panel's units that exist.
template <int QT, bool FIRST, int NU = 0>
__device__ __forceinline__ void panel_dot(WPanel<QT>& p, const uint8_t* xu0, int n_units, int j, int grp,
                                          float (&acc)[4]) {
    constexpr int UB = Unit<QT>::kBytes;
    const int lane16 = (grp * 16 + j) * 16; // this lane's 16 bytes of a sub-block pair
    // Q8_0 / Q6_K: units of the panel that do not exist (ragged k, S < 4) get unit 0's
    // activations as their address and a weight scale multiplied by zero wherever the
    // compiler keeps their arithmetic.  (Their header is zero padding or a copy of unit
    // 0's, so every factor is finite.)
    int xo[4];
    float ef[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const bool exists = u < n_units; // uniform
        xo[u] = exists ? u * UB : 0;
        ef[u] = exists ? 1.0f : 0.0f;
    }
    if constexpr (QT == QMM_Q4_K) {
        q4k_panel_dot<FIRST, NU>(
            p, n_units,
            [&](int u, int b) { return *reinterpret_cast<const i64x2*>(xu0 + u * UB + lane16 + b * 1024); },
            [&](int u, long& bs_lo, long& bs_hi, float4& dx) {
                const uint8_t* side = xu0 + u * UB + Unit<QT>::kQuant;
                const i64x2 planes = *reinterpret_cast<const i64x2*>(side + 64 + j * 16);
                bs_lo = grp == 0 ? planes.x : 0L;
                bs_hi = grp == 0 ? planes.y : 0L;
                dx = *reinterpret_cast<const float4*>(side + grp * 16);
            },
            acc);
    } else if constexpr (QT == QMM_Q6_K) {
        // Sub-block t = 4 h + g of a unit (32 elements) is nibble g / 2 of the nibble chunk pair
        // 2 h + g % 2 with bit pair g of the bit-pair chunk pair h; each of its two 16-element
        // groups has its own signed scale, and the matrix instruction sums 32: it runs twice, once
        // with the upper two octets of the B operand zeroed and once with the lower two.
        int isum[4][4];
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) isum[u][r] = 0;
#pragma unroll
        for (int cp = 0; cp < 4; cp++) {
            const int h = cp >> 1, gb = cp & 1;
            if (FIRST) {
                if (gb == 0) transpose_pair(p.q[8 + 2 * h], p.q[9 + 2 * h]);
                transpose_pair(p.q[2 * cp], p.q[2 * cp + 1]);
            }
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                const int g = gb + 2 * hi, t = 4 * h + g;
#pragma unroll
                for (int up = 0; up < 2; up++) {
                    const u32x4 ql = p.q[2 * cp + up], qh = p.q[8 + 2 * h + up];
                    i32x4 dlo[2], dhi[2];
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const int u = 2 * up + e;
                        if (u >= n_units) continue; // uniform
                        const uint32_t w0 = e ? ql.z : ql.x, w1 = e ? ql.w : ql.y;
                        const uint32_t h0 = e ? qh.z : qh.x, h1 = e ? qh.w : qh.y;
                        // six-bit quants, then q - 32 as int8 in every byte without a borrow
                        const uint32_t v0 = ((w0 >> (4 * hi)) & kNib) | (((h0 >> (2 * g)) & 0x03030303u) << 4);
                        const uint32_t v1 = ((w1 >> (4 * hi)) & kNib) | (((h1 >> (2 * g)) & 0x03030303u) << 4);
                        const uint32_t s0 = ((v0 | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
                        const uint32_t s1 = ((v1 | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
                        const long bq = pack64(s0, s1);
                        const long b_lo = grp < 2 ? bq : 0L, b_hi = grp < 2 ? 0L : bq;
                        const long a = *reinterpret_cast<const long*>(xu0 + xo[u] + lane16 + (t >> 1) * 1024 + (t & 1) * 8);
                        dlo[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b_lo, i32x4{0, 0, 0, 0}, 0, 0, 0);
                        dhi[e] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b_hi, i32x4{0, 0, 0, 0}, 0, 0, 0);
                    }
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const int u = 2 * up + e;
                        if (u >= n_units) continue;
                        const uint32_t hw = t < 2 ? p.hdr[u].x : t < 4 ? p.hdr[u].y : t < 6 ? p.hdr[u].z : p.hdr[u].w;
                        const int sc_lo = (int)(int8_t)((hw >> (16 * (t & 1))) & 0xffu);
                        const int sc_hi = (int)(int8_t)((hw >> (16 * (t & 1) + 8)) & 0xffu);
#pragma unroll
                        for (int r = 0; r < 4; r++) // |dot| <= 16 * 32 * 128, |scale| <= 128
                            isum[u][r] = scaled_pair_sum(sc_lo, dlo[e][r], sc_hi, dhi[e][r], isum[u][r]);
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (u >= n_units) continue;
            const float d = qmm_f16_bits_to_f32((uint16_t)(p.dch[u].x & 0xffffu)) * ef[u];
            const float4 dx = *reinterpret_cast<const float4*>(xu0 + xo[u] + Unit<QT>::kQuant + grp * 16);
            acc[0] += (d * dx.x) * (float)isum[u][0];
            acc[1] += (d * dx.y) * (float)isum[u][1];
            acc[2] += (d * dx.z) * (float)isum[u][2];
            acc[3] += (d * dx.w) * (float)isum[u][3];
        }
    } else {
#pragma unroll
        for (int b = 0; b < 8; b++) {
            if (FIRST) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
            i32x4 dd[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (u >= n_units) continue; // uniform
                const u32x4 qq = p.q[2 * b + (u >> 1)];
                const uint32_t w0 = (u & 1) ? qq.z : qq.x, w1 = (u & 1) ? qq.w : qq.y;
                const long a = *reinterpret_cast<const long*>(xu0 + xo[u] + lane16 + (b >> 1) * 1024 + (b & 1) * 8);
                dd[u] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, pack64(w0, w1), i32x4{0, 0, 0, 0}, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (u >= n_units) continue;
                const uint32_t hw = b < 2 ? p.hdr[u].x : b < 4 ? p.hdr[u].y : b < 6 ? p.hdr[u].z : p.hdr[u].w;
                const float dw = qmm_f16_bits_to_f32((uint16_t)((hw >> (16 * (b & 1))) & 0xffffu)) * ef[u];
                const float4 dx = *reinterpret_cast<const float4*>(xu0 + xo[u] + Unit<QT>::kQuant +
                                                                   (b * 16 + grp * 4) * 4);
                acc[0] += ((float)dd[u][0] * dw) * dx.x;
                acc[1] += ((float)dd[u][1] * dw) * dx.y;
                acc[2] += ((float)dd[u][2] * dw) * dx.z;
                acc[3] += ((float)dd[u][3] * dw) * dx.w;
            }
        }
    }
}

// Moves `n_units` unit records of a tile from the workspace to LDS, 1 KiB pieces
// spread over the workgroup's waves, 16 B per lane, without passing through
// registers.  Completion is the caller's business (vmcnt, then a barrier).
// The LDS-direct load is issued from inline assembly on purpose: for the
// compiler's own form it conservatively waits for ALL outstanding vector loads
// before the first LDS read that follows, which would put the whole weight panel
// in front of the arithmetic; the callers order these copies explicitly.
template <int QT>
__device__ __forceinline__ void issue_window_copy(const uint8_t* __restrict__ src, uint8_t* lds, int n_units,
                                                  int wave, int waves, int lane) {
    const int bytes = n_units * Unit<QT>::kBytes; // a multiple of 64
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds; // LDS byte address (uniform)
    for (int piece = wave; piece * 1024 < bytes; piece += waves) {
        const int off = piece * 1024 + lane * 16;
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + piece * 1024);
        if (off < bytes)
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src + off)
                         : "memory", "m0");
    }
}

// The same window put together from row records: the unit records of up to TC tiles whose sixteen
// rows each are rows of `rows` (row_off: the lane's byte offsets of the rows lane % 16 of the tiles).
// A unit record is six pieces of one instruction each: the four KiB of quants (lane = (octet, row):
// the row's chunk of that octet), and the side data - Q4_K records: the sixteen scales (a dword from
// each row, lanes 0 - 15) and the sixteen rows of sum bytes (16 B from each row, lanes 0 - 15); Q8_0:
// twice four blocks' scales of the sixteen rows (a dword per lane).
template <int QT, int TC>
__device__ __forceinline__ void issue_window_gather(const uint8_t* __restrict__ rows, const uint32_t (&row_off)[TC],
                                                    uint8_t* lds, int nt, int k_units, int wave, int waves, int lane) {
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds; // LDS byte address (uniform)
    const uint32_t grp16 = (uint32_t)(lane >> 4) * 16u;
#pragma unroll
    for (int t = 0; t < TC; t++) {
        if (t >= nt) continue; // uniform
        const uint8_t* src_row = rows + row_off[t];
        for (int piece = wave; piece < k_units * 6; piece += waves) {
            const int u = piece / 6, sub = piece - 6 * u; // (uniform)
            const uint32_t unit_lds = lds_base + (uint32_t)(t * k_units + u) * Unit<QT>::kBytes;
            const uint8_t* src = src_row + u * kRowUnitBytes;
            if (sub < 4) {
                const uint32_t dst = __builtin_amdgcn_readfirstlane(unit_lds + sub * 1024);
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src + sub * 64 + grp16)
                             : "memory", "m0");
            } else if (QT == QMM_Q8_0) {
                const uint32_t dst = __builtin_amdgcn_readfirstlane(unit_lds + Unit<QT>::kQuant + (sub - 4) * 256);
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(dst), "v"(src + 256 + (sub - 4) * 16 + (grp16 >> 2))
                             : "memory", "m0");
            } else if (sub == 4) {
                const uint32_t dst = __builtin_amdgcn_readfirstlane(unit_lds + Unit<QT>::kQuant);
                if (lane < 16)
                    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(dst), "v"(src + 272) : "memory", "m0");
            } else {
                const uint32_t dst = __builtin_amdgcn_readfirstlane(unit_lds + Unit<QT>::kQuant + 64);
                if (lane < 16)
                    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src + 256) : "memory", "m0");
            }
        }
    }
}

// The lane's row offsets for issue_window_gather, in two steps (a kernel puts the loads it can
// request without them in between): the pairs of row lane % 16 of the tiles t0 .. t0 + TC - 1 of the
// expert whose sorted pairs are [pos_begin, pos_end) - a row past the end reads the expert's first
// row, its sums are never stored - and from them the byte offsets of their source rows.
template <int TC>
__device__ __forceinline__ void gather_pairs(const int32_t* __restrict__ perm, int pos_begin, int pos_end, int t0, int nt,
                                             int lane, uint32_t (&pair)[TC]) {
#pragma unroll
    for (int t = 0; t < TC; t++) {
        const int pos = pos_begin + (t0 + t) * 16 + (lane & 15);
        pair[t] = (uint32_t)perm[t < nt && pos < pos_end ? pos : pos_begin];
    }
}
template <int TC>
__device__ __forceinline__ void gather_row_offsets(uint32_t (&pair)[TC], int row_div, uint32_t row_magic, uint32_t row_bytes) {
#pragma unroll
    for (int t = 0; t < TC; t++) pair[t] = (row_div == 1 ? pair[t] : __umulhi(pair[t], row_magic)) * row_bytes;
}

// Several 16-row tiles of activations on the single-stage forms: one workgroup per (row-tile group,
// tile), each exactly the workgroup of a call of up to 16 rows.  The launch is one-dimensional and
// index = ((group / 8) * n_tiles + tile) * 8 + group % 8: workgroups go to the eight XCDs round-robin
// by their index, so the n_tiles workgroups that read the same weight panels sit on one XCD, eight
// positions apart in the order of placement, and all but the first find the panels in that XCD's L2.
// Returns false for the padding past the last group (uniform).
__device__ __forceinline__ bool tile_parallel_decode(int n_tiles, int rt_groups, int& rtg, int& tile) {
    const int slot = blockIdx.x >> 3, hi = slot / n_tiles;
    tile = slot - hi * n_tiles;
    rtg = hi * 8 + (int)(blockIdx.x & 7);
    return rtg < rt_groups;
}

// One-shot form: wave (wr, wk) owns panel wk of row-tile blockIdx.x * nwr + wr.
// SINGLE: one tile of rows and one activation window, i.e. straight-line code.
// GROUPED: the workgroup belongs to an expert; its weights are that matrix of the
// stack, its rows the expert's tiles of sorted pairs, output row = pair index.
// EP: the sums go through the epilogue of P.ep (residual add, f32 or bf16 store).
// (the compact single-stage Q4_K form is held to the 80 registers of six waves per SIMD: two 12-wave
// workgroups per CU keep every panel of gate | up in flight at once)
template <int QT, bool SINGLE, bool GROUPED, bool EP, int NU>
__device__ __forceinline__ void oneshot_body(const MfmaParams& P, const MfmaParams& P0) {
    constexpr int UB = Unit<QT>::kBytes;
    constexpr int NL = WPanel<QT>::kLoads; // loads of one panel
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* lds_x = smem;                                                       // window_units * UB
    // the sums of the k-split (waves * 256 floats): behind the window(s); in the single-stage form
    // over the window itself, which nobody reads any more by then (two workgroups then fit a CU)
    float* lds_red = SINGLE ? reinterpret_cast<float*>(smem)
                            : reinterpret_cast<float*>(smem + (size_t)(P.double_buf ? 2 : 1) * P.window_units * UB);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // wave-uniform by construction
    const int waves = P.nwk * P.nwr;
    const int wr = (wave * P.wave_magic) >> 16;
    const int wk = wave - wr * P.nwk;
    const int j = lane & 15, grp = lane >> 4;
    const int s_units = P.slots >> 4;
    const uint8_t* wbase = P.w;
    float* yout = P.y;
    int n_rows = P.n, row_tiles = P.row_tiles, rtg = blockIdx.x, tile0 = 0;
    if (SINGLE && P.n_tiles > 1 && !tile_parallel_decode(P.n_tiles, P.rt_groups, rtg, tile0)) return;
    const int group_index = rtg; // (over all weights of a group)
    // GROUPED: workgroups go to the eight XCDs round-robin by their linear index, and every XCD has
    // its own L2: index = 8 * slot + (expert % 8), so the 2 * rt_groups workgroups of an expert share
    // one L2 and all but the first find the expert's activation records there (measured neutral at
    // T = 512: the records' first touch is not what a workgroup waits for longest).
    int g_expert = 0, g_stack = 0;
    if (GROUPED) {
        const int per_expert = P.rt_groups * P.stacks;
        const int slot = blockIdx.x >> 3;
        const int e_hi = slot / per_expert, within = slot - e_hi * per_expert;
        g_expert = e_hi * 8 + (int)(blockIdx.x & 7);
        if (g_expert >= P.n_experts) return; // uniform for the workgroup
        g_stack = within / P.rt_groups;
        rtg = within - g_stack * P.rt_groups;
    }
    const int unit0 = wk * s_units;                       // first unit of this wave's panel
    const int n_units = min(s_units, P.k_units - unit0);  // its units that exist (>= 1)

    const uint8_t* records = P.ws + (size_t)tile0 * P.k_units * UB;
    int n_tiles = P.n_tiles, pos_begin = 0, pos_end = 0;
    if (GROUPED) {
        const int e = g_expert;
        if (g_stack != 0) wbase = P.w2, yout = P.y2; // second weight stack on the same activations
        const int tile_begin = P.tile_offsets[e];
        n_tiles = P.tile_offsets[e + 1] - tile_begin;
        if (n_tiles == 0) return; // uniform for the workgroup: nobody reaches a barrier
        pos_begin = P.offsets[e];
        pos_end = P.offsets[e + 1];
        wbase += (int64_t)e * P.matrix_bytes;
        records += (size_t)tile_begin * P.k_units * UB;
    }

    // the first activation window goes first (loads return in order), then the panel
    const int w0_units = min(P.window_units, P.k_units);
    if (!(QMM_MFMA_ABL & 16)) issue_window_copy<QT>(records, lds_x, w0_units, wave, waves, lane);
    // A CU's loads return in the order they were issued, for all its waves together: without this
    // barrier the last wave's window pieces queue behind the other waves' panels, and the barrier
    // below - the start of all arithmetic - waits for nearly the whole workgroup's weights.
    asm volatile("s_barrier" ::: "memory");
    // (a group's tables are read here, behind the window copies: those need nothing from them)
    if (!GROUPED && P.n_weights > 1) pick_group_entry(P0, P.n_weights, group_index, rtg, wbase, yout, n_rows, row_tiles);
    const int rt = rtg * P.nwr + wr;
    const bool rt_ok = rt < row_tiles;
    const int row = rt * 16 + j;
    WPanel<QT> p;
    load_wpanel<QT>(p, wbase + (int64_t)((rt_ok ? rt : 0) * P.k_groups + wk) * P.panel_bytes, P.slots, lane, j);
    // The window has landed.  The single-stage form lets the panel fly on: its arithmetic starts on the
    // first chunk pair, and all NL loads of the panel are behind the window.  That count is right only
    // while the compiler keeps every load of the panel: it drops a load whose value no path uses (the
    // fourth header of a panel instantiated for three units), and the wait is then one short.  So the
    // counted wait is taken only where every loaded register is used on some path - the unit count a
    // run-time value (NU = 0: Q8_0, Q6_K, compact Q4_K) or all four units present (NU = 4) - and every
    // other instantiation waits for everything, as the multi-stage forms do anyway (they transpose the
    // whole panel before their first stage).
    constexpr bool kEveryPanelLoadUsed = NU == 0 || NU == 4;
    if (SINGLE && kEveryPanelLoadUsed) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();

    // several stages reuse the panel: its activation-independent part once, up front
    constexpr bool PREP = QT == QMM_Q4_K && !SINGLE && NU > 0;
    Q4Prepared<PREP ? NU : 1> prep;
    if constexpr (PREP) {
#pragma unroll
        for (int b = 0; b < WPanel<QT>::QC / 2; b++) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
        q4k_prepare<NU>(p, prep, grp);
    }

    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // (row tile, window) stages in order; with two LDS buffers the next stage's window is
    // copied while this one is multiplied
    const int n_win = SINGLE ? 1 : (P.k_units + P.window_units - 1) / P.window_units;
    const int n_stages = SINGLE ? 1 : n_tiles * n_win;
    const size_t buf_bytes = (size_t)P.window_units * UB;
    bool transposed = false;
    int tile = tile0, win = 0;
    for (int s = 0; s < n_stages; s++) {
        const int wu0 = win * P.window_units;
        const int wn = min(P.window_units, P.k_units - wu0);
        uint8_t* cur = lds_x + (P.double_buf ? (s & 1) * buf_bytes : 0);
        int ntile = tile, nwin = win + 1;
        if (nwin == n_win) nwin = 0, ntile = tile + 1;
        const bool more = !SINGLE && s + 1 < n_stages;
        const uint8_t* next_src = records + ((size_t)ntile * P.k_units + (size_t)nwin * P.window_units) * UB;
        const int next_n = min(P.window_units, P.k_units - nwin * P.window_units);
        if (more && P.double_buf)
            issue_window_copy<QT>(next_src, lds_x + ((s + 1) & 1) * buf_bytes, next_n, wave, waves, lane);
        if (SINGLE || (unit0 >= wu0 && unit0 < wu0 + wn)) {
            const uint8_t* xu0 = cur + (size_t)(unit0 - wu0) * UB;
            if constexpr (SINGLE) {
                panel_dot<QT, true, NU>(p, xu0, n_units, j, grp, acc);
            } else if constexpr (PREP) {
                const int lane16 = lane * 16;
                q4k_tile_dot<NU>(
                    prep, [&](int u, int b) { return *reinterpret_cast<const i64x2*>(xu0 + u * UB + lane16 + b * 1024); },
                    [&](int u, long& bs_lo, long& bs_hi, float4& dx) {
                        const uint8_t* side = xu0 + u * UB + Unit<QT>::kQuant;
                        const i64x2 planes = *reinterpret_cast<const i64x2*>(side + 64 + j * 16);
                        bs_lo = planes.x, bs_hi = planes.y; // (every lane row: the prepared mins are zero past the first)
                        dx = *reinterpret_cast<const float4*>(side + grp * 16);
                    },
                    acc);
            } else {
                // several stages reuse the panel: transpose it once, up front (one copy of
                // the arithmetic in the code keeps the register count down)
                if (!transposed) {
#pragma unroll
                    for (int b = 0; b < WPanel<QT>::QC / 2; b++) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
                }
                transposed = true;
                panel_dot<QT, false>(p, xu0, n_units, j, grp, acc);
            }
        }
        if (win == n_win - 1) {
            // ---- row tile finished: combine the waves that split k, write
            // y[tile*16 + 4*grp + r][rt*16 + j] (grouped: the row is a sorted position of the
            // expert, the y row its pair index)
            auto store = [&](int r, float v) {
                if ((QMM_MFMA_ABL & 32) && v != 12345.0f) return; // timing only: (almost) nothing is stored
                const int mm = tile * 16 + grp * 4 + r;
                if (GROUPED) {
                    if (pos_begin + mm < pos_end) yout[(int64_t)P.perm[pos_begin + mm] * n_rows + row] = v;
                } else if (mm < P.m) {
                    if (EP) qmm_store(yout, P.ep, (int64_t)mm * n_rows + row, v);
                    else yout[(int64_t)mm * n_rows + row] = v;
                }
            };
            if (P.nwk == 1) {
                if (rt_ok && row < n_rows) {
#pragma unroll
                    for (int r = 0; r < 4; r++) store(r, acc[r]);
                }
            } else if (!GROUPED && !(QMM_MFMA_ABL & 64)) {
                // Dense forms: every thread of the workgroup finishes outputs - one (activation row, weight
                // row) pair at a time, the nwk partial sums added in the order wave wk = 0 adds them - and
                // consecutive threads store consecutive weight rows of one activation row: nwr * 64 bytes
                // in one piece (a wave of the k-split storing its own tile writes 64-byte pieces, and the
                // other nwk - 1 waves of the tile stand by meanwhile).
                if (SINGLE || tile != 0) lds_barrier(); // the window / the previous tile's sums have been read
#pragma unroll
                for (int r = 0; r < 4; r++) lds_red[(wave * 4 + r) * 64 + lane] = acc[r];
                lds_barrier();
                const int cols = P.nwr * 16;
                for (int o = (int)threadIdx.x; o < cols * 16; o += waves * 64) {
                    const int mrow = o / cols, c = o - mrow * cols;
                    const int wr2 = c >> 4, j2 = c & 15;
                    const float* part = lds_red + ((wr2 * P.nwk) * 4 + (mrow & 3)) * 64 + (mrow >> 2) * 16 + j2;
                    float sum = 0.0f;
                    for (int w2 = 0; w2 < P.nwk; w2++) sum += part[w2 * 256];
                    const int rt2 = rtg * P.nwr + wr2, col = rt2 * 16 + j2, mm = tile * 16 + mrow;
                    if (rt2 < row_tiles && col < n_rows && mm < P.m) {
                        if (EP) qmm_store(yout, P.ep, (int64_t)mm * n_rows + col, sum);
                        else yout[(int64_t)mm * n_rows + col] = sum;
                    }
                }
            } else {
                if (SINGLE || tile != 0) lds_barrier(); // the window / the previous tile's sums have been read
#pragma unroll
                for (int r = 0; r < 4; r++) lds_red[(wave * 4 + r) * 64 + lane] = acc[r];
                lds_barrier();
                if (wk == 0 && rt_ok && row < n_rows) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        float sum = 0.0f;
                        for (int w2 = 0; w2 < P.nwk; w2++) sum += lds_red[((wr * P.nwk + w2) * 4 + r) * 64 + lane];
                        store(r, sum);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = 0.0f;
        }
        if (more) {
            if (!P.double_buf) {
                lds_barrier(); // every wave is done with this window
                issue_window_copy<QT>(next_src, lds_x, next_n, wave, waves, lane);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier(); // the next window has landed; with two buffers: and this one is free
        }
        tile = ntile, win = nwin;
    }
}
// The dense launches of the one-shot form: leading scalar arguments (see with_leading_args).
template <int QT, bool SINGLE, bool GROUPED = false, bool EP = false, int NU = 0>
__global__ __launch_bounds__(64 * kMaxWaves, (QT == QMM_Q4_K && SINGLE && NU == 0) ? 6 : 3) void gemv_mfma_oneshot_kernel(
        const uint8_t* w_arg, const uint8_t* ws_arg, float* y_arg, int k_units_arg, int k_groups_arg, int row_tiles_arg, int panel_bytes_arg,
        int split_arg, int wave_magic_arg, int n_tiles_arg, int window_arg, MfmaParams P0) {
    static_assert(!GROUPED, "the expert-grouped launches go through gemv_mfma_grouped_kernel");
    const MfmaParams P = with_leading_args(P0, w_arg, ws_arg, y_arg, k_units_arg, k_groups_arg, row_tiles_arg, panel_bytes_arg, split_arg,
                                             wave_magic_arg, n_tiles_arg, window_arg);
    oneshot_body<QT, SINGLE, false, EP, NU>(P, P0);
}

// The expert-grouped launches: thousands of short workgroups, whose waves start faster with
// fewer scalar registers to fill (measured: the grouped one-row kernels lost 1 us of 19 - 30
// with preloaded arguments), so the parameter block stays one block in memory.
template <int QT, int NU = 0>
__global__ __launch_bounds__(64 * kMaxWaves, 3) void gemv_mfma_grouped_kernel(MfmaParams P) {
    oneshot_body<QT, false, true, false, NU>(P, P);
}

// Register-direct form (Q4_K, one row tile of activations, one row-tile of weights per
// workgroup): wave wk multiplies panel wk, which needs only units 4 wk .. 4 wk + 3 of the
// activations, and no other wave of the workgroup needs them.  Staging them in LDS would buy no
// reuse and cost a barrier, so every lane loads its share of the MFMA A operands (and the
// units' side information) straight into registers, ahead of the panel: no LDS, no barrier
// before the arithmetic, and k of any length (the LDS forms need several windows from 32
// units on).  Returns acc[r] for activation rows 4 grp + r.
template <int NU>
__device__ __forceinline__ void panel_dot_direct_q4k(WPanel<QMM_Q4_K>& p, const i64x2 (&a)[4][4],
                                                     const long (&bs_lo)[4], const long (&bs_hi)[4],
                                                     const float4 (&dx)[4], int n_units, float (&acc)[4]) {
    q4k_panel_dot<true, NU>(
        p, n_units, [&](int u, int b) { return a[u][b]; },
        [&](int u, long& lo, long& hi, float4& d4) { lo = bs_lo[u], hi = bs_hi[u], d4 = dx[u]; }, acc);
}

template <bool EP = false, int NU = 0>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_mfma_direct_q4k_kernel(
        const uint8_t* w_arg, const uint8_t* ws_arg, float* y_arg, int k_units_arg, int k_groups_arg, int row_tiles_arg, int panel_bytes_arg,
        int split_arg, int wave_magic_arg, int n_tiles_arg, int window_arg, MfmaParams P0) {
    const MfmaParams P = with_leading_args(P0, w_arg, ws_arg, y_arg, k_units_arg, k_groups_arg, row_tiles_arg, panel_bytes_arg, split_arg,
                                             wave_magic_arg, n_tiles_arg, window_arg);
    constexpr int QT = QMM_Q4_K;
    constexpr int UB = Unit<QT>::kBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float* lds_red = reinterpret_cast<float*>(smem); // the sums of the k-split: waves * 256 floats

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = (wave * P.wave_magic) >> 16;
    const int wk = wave - wr * P.nwk;
    const int j = lane & 15, grp = lane >> 4;
    const int s_units = P.slots >> 4;
    const uint8_t* wbase = P.w;
    float* yout = P.y;
    int n_rows = P.n, row_tiles = P.row_tiles, rtg = blockIdx.x, tile0 = 0;
    if (P.n_tiles > 1 && !tile_parallel_decode(P.n_tiles, P.rt_groups, rtg, tile0)) return;
    if (P.n_weights > 1) pick_group_entry(P0, P.n_weights, rtg, rtg, wbase, yout, n_rows, row_tiles);
    const uint8_t* records = P.ws + (size_t)tile0 * P.k_units * UB;
    const int m_base = tile0 * 16; // the tile's first activation row
    const int rt = rtg * P.nwr + wr;
    const bool rt_ok = rt < row_tiles;
    const int unit0 = wk * s_units;
    const int n_units = min(s_units, P.k_units - unit0); // uniform, >= 1
    const int row = rt * 16 + j;

    // the activations first (they come from the L2 and return first), then the panel
    i64x2 a[4][4];
    long bs_lo[4], bs_hi[4];
    float4 dx[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const uint8_t* rec = records + (size_t)(unit0 + (u < n_units ? u : 0)) * UB; // missing units re-read unit 0
#pragma unroll
        for (int b = 0; b < 4; b++) a[u][b] = *reinterpret_cast<const i64x2*>(rec + b * 1024 + lane * 16);
        const uint8_t* side = rec + Unit<QT>::kQuant;
        // the sub-block sums occupy k slots 0..7 of the min-term MFMA: the first 16-lane row only
        const i64x2 planes = *reinterpret_cast<const i64x2*>(side + 64 + j * 16);
        bs_lo[u] = grp == 0 ? planes.x : 0L;
        bs_hi[u] = grp == 0 ? planes.y : 0L;
        dx[u] = *reinterpret_cast<const float4*>(side + grp * 16);
    }
    WPanel<QT> p;
    load_wpanel<QT>(p, wbase + (int64_t)((rt_ok ? rt : 0) * P.k_groups + wk) * P.panel_bytes, P.slots, lane, j);

    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    panel_dot_direct_q4k<NU>(p, a, bs_lo, bs_hi, dx, n_units, acc);

    // combine the waves that split k, write y[4 grp + r][rt * 16 + j]
    if (P.nwk == 1) {
        if (rt_ok && row < n_rows) {
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (m_base + grp * 4 + r < P.m) {
                    if (EP) qmm_store(yout, P.ep, (int64_t)(m_base + grp * 4 + r) * n_rows + row, acc[r]);
                    else yout[(int64_t)(m_base + grp * 4 + r) * n_rows + row] = acc[r];
                }
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < 4; r++) lds_red[(wave * 4 + r) * 64 + lane] = acc[r];
    lds_barrier();
    // every thread finishes outputs (see the one-shot form): the partial sums of a pair added in wave
    // order, consecutive threads storing consecutive weight rows of one activation row
    const int cols = P.nwr * 16, threads = P.nwk * P.nwr * 64;
    for (int o = (int)threadIdx.x; o < cols * 16; o += threads) {
        const int mrow = o / cols, c = o - mrow * cols;
        const int wr2 = c >> 4, j2 = c & 15;
        const float* part = lds_red + ((wr2 * P.nwk) * 4 + (mrow & 3)) * 64 + (mrow >> 2) * 16 + j2;
        float sum = 0.0f;
        for (int w2 = 0; w2 < P.nwk; w2++) sum += part[w2 * 256];
        const int rt2 = rtg * P.nwr + wr2, col = rt2 * 16 + j2, mm = m_base + mrow;
        if (rt2 < row_tiles && col < n_rows && mm < P.m) {
            if (EP) qmm_store(yout, P.ep, (int64_t)mm * n_rows + col, sum);
            else yout[(int64_t)mm * n_rows + col] = sum;
        }
    }
}

// Two to four tiles of rows: one single-stage workgroup per tile (tile_parallel_decode) instead of one
// workgroup that walks the tiles stage by stage.  IZWI_QMM_MFMA_TILE_PARALLEL=0 / 1 forces the choice
// (tuning aid).
bool tile_parallel_applies(int n_tiles) {
    static const int mode = [] {
        const char* e = getenv("IZWI_QMM_MFMA_TILE_PARALLEL");
        return e && (e[0] == '0' || e[0] == '1') ? e[0] - '0' : -1;
    }();
    if (n_tiles < 2 || n_tiles > 4) return false;
    return mode != 0;
}

// One row tile of activations (m <= 16), one row-tile of weights per workgroup, Q4_K, and k
// longer than one LDS window (measured on the 8B shapes at m = 16: 4096 x 12288 17.0 -> 15.4 us
// per call; with k = 4096 the single-window LDS form is the faster one, 10.2 against 10.4 us
// and 11.9 against 12.7 us for the q|k|v group).  IZWI_QMM_MFMA_DIRECT=0 keeps the LDS forms
// (tuning aid).
bool direct_form_applies(int dtype, int n_tiles, int nwr, bool one_window) {
    static const int mode = [] {
        const char* e = getenv("IZWI_QMM_MFMA_DIRECT");
        return e && e[0] >= '0' && e[0] <= '2' ? e[0] - '0' : 1;
    }();
    if (mode == 0 || dtype != QMM_Q4_K || n_tiles != 1) return false;
    if (mode == 2) return true; // every single-tile Q4_K call (tuning aid: measured slower where one window covers k)
    return nwr == 1 && !one_window;
}

// Streaming form: wave `wave` of workgroup b owns row-tiles (b * waves + wave),
// + gridDim.x * waves, ... and walks all their panels; the activation window
// stays in LDS meanwhile.  Windows that split k accumulate into y (the same
// wave adds the same row-tile's windows in order, so the result is deterministic).
template <int QT, bool EP = false>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_mfma_stream_kernel(MfmaParams P) {
    constexpr int UB = Unit<QT>::kBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* lds_x = smem;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = P.nwr;
    const int j = lane & 15, grp = lane >> 4;
    const int s_units = P.slots >> 4;
    const int window_groups = P.window_units / s_units;

    for (int tile = 0; tile < P.n_tiles; tile++) {
        for (int wu0 = 0; wu0 < P.k_units; wu0 += P.window_units) {
            const int wn = min(P.window_units, P.k_units - wu0);
            if (tile != 0 || wu0 != 0) lds_barrier();
            issue_window_copy<QT>(P.ws + ((size_t)tile * P.k_units + wu0) * UB, lds_x, wn, wave, waves, lane);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier();
            const int kg0 = wu0 / s_units;
            const int kg1 = min(P.k_groups, kg0 + window_groups);
            for (int rt = blockIdx.x * waves + wave; rt < P.row_tiles; rt += gridDim.x * waves) {
                float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                for (int kg = kg0; kg < kg1; kg++) {
                    WPanel<QT> p;
                    load_wpanel<QT>(p, P.w + (int64_t)(rt * P.k_groups + kg) * P.panel_bytes, P.slots, lane, j);
                    const int unit0 = kg * s_units;
                    panel_dot<QT, true>(p, lds_x + (size_t)(unit0 - wu0) * UB, min(s_units, P.k_units - unit0),
                                        j, grp, acc);
                }
                const int row = rt * 16 + j;
                if (row < P.n) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int mm = tile * 16 + grp * 4 + r;
                        if (mm < P.m) {
                            // one window covers k: the sums are final (the launcher folds the
                            // epilogue only then); otherwise y accumulates the windows in f32
                            float* dst = P.y + (int64_t)mm * P.n + row;
                            if (EP && P.k_units <= P.window_units) qmm_store(P.y, P.ep, (int64_t)mm * P.n + row, acc[r]);
                            else *dst = wu0 == 0 ? acc[r] : *dst + acc[r];
                        }
                    }
                }
            }
        }
    }
}

// ---- the expert forms' work items ------------------------------------------------------------
// An item is (expert, weight stack, part of the stack's row tiles).  Where the items are two per CU, a
// launch is one workgroup per CU that takes two items in turn; two things decide how evenly the CUs
// finish:
//   * an item lives in proportion to its expert's tile count (measured at 128 experts, top-8, 512
//     tokens, gate | up: 36 us with two tiles, 47 with three), and
//   * a grid of one workgroup per ITEM leaves the pairing of items on a CU to the order in which
//     workgroups happen to end, and the hardware places the workgroups of the second round slowly
//     (measured: CUs idle for 2 - 15 us between their two workgroups, finishing 60 - 101 us after the
//     launch's start).
// So the experts are ranked by falling tile count (ties by index) and the items numbered in that
// order; workgroup c of G takes items c and 2G - 1 - c: a heavy and a light item on every CU.  Every
// workgroup ranks the experts itself (counts in LDS, one thread per expert against all: under a
// microsecond up to kRankedExperts experts; past that the experts keep their own order).
constexpr int kRankedExperts = 512;
constexpr int kExpertRounds = 2; // items a workgroup takes at most (the kernels' round loops are unrolled)

// order[r] = the expert of rank r.  Returns whether the experts were ranked.  Contains barriers.
__device__ __forceinline__ bool rank_experts(const int32_t* __restrict__ tile_offsets, int n_experts, int* order, int* scratch) {
    if (n_experts > kRankedExperts) return false;
    for (int i = threadIdx.x; i < n_experts; i += blockDim.x) scratch[i] = tile_offsets[i + 1] - tile_offsets[i];
    __syncthreads();
    for (int i = threadIdx.x; i < n_experts; i += blockDim.x) {
        const int c = scratch[i];
        int rank = 0;
        for (int o = 0; o < n_experts; o++) {
            const int co = scratch[o];
            rank += (co > c || (co == c && o < i)) ? 1 : 0;
        }
        order[rank] = i; // a permutation: every slot is written once
    }
    __syncthreads(); // (also: `scratch` may be overwritten from here on)
    return true;
}

// The item of this workgroup in round `round`: -1 when the rounds are over, -2 when this round has none.
// Workgroups go to the eight XCDs round-robin by their index, and every XCD has its own L2: the
// per_expert items of an expert (its stacks and parts, which all copy the same activation tiles) are
// given to workgroups of one XCD, so that all but the first find the tiles in that L2 - position
// c = x + 8 (q + per_expert * j) takes item (8 j + x) * per_expert + q.  The second item of a workgroup,
// 2G - 1 - (its first), then belongs to one expert for the same per_expert workgroups as well.
__device__ __forceinline__ int expert_item(int round, int n_items, int per_expert) {
    const int g = gridDim.x, base = round * g;
    if (base >= n_items) return -1;
    int c = blockIdx.x;
    if (g % (8 * per_expert) == 0) {
        const int x = c & 7, y = c >> 3;
        const int j = y / per_expert, q = y - j * per_expert;
        c = (8 * j + x) * per_expert + q;
    }
    const int item = base + ((round & 1) ? g - 1 - c : c);
    return item < n_items ? item : -2;
}

// Expert form: a work item belongs to one expert and one of the two weight stacks; up to TC of the
// expert's 16-row activation tiles, over all of k, sit in LDS, and every wave walks row-tiles of the
// expert's matrix on its own: load a panel, multiply it with
// every tile, next panel; no wave waits for another after the tiles have landed.  The weights are
// read once per TC tiles (an expert with more tiles takes another pass), and the waves of a CU
// keep several panels in flight where the one-shot form is one chain of round trips per workgroup.
// The Q4_K kernel for whole panels (below) runs eight waves: two per SIMD, 256 registers each - it
// requests the next panel while the current one is multiplied, which the 170 registers of twelve
// waves do not hold.
constexpr int kExpertWaves = 8;
constexpr int kExpertMaxWindowBytes = 160 * 1024 - kRankedExperts * 4 - 1024; // beside the rank table
// (this general kernel requests a panel where it multiplies it and needs about 150 registers: twelve
// waves, three per SIMD, hide a panel's round trip better than eight)
constexpr int kExpertWavesGeneral = 12;
template <int QT, int TC>
__global__ __launch_bounds__(64 * kExpertWavesGeneral) void gemv_mfma_expert_kernel(MfmaParams P) {
    constexpr int UB = Unit<QT>::kBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = P.nwr;
    const int j = lane & 15, grp = lane >> 4;
    const int s_units = P.slots >> 4;
    __shared__ int order[kRankedExperts];
    // The output rows (pair indices) of the tiles in the window, -1 past the expert's last pair: read
    // from LDS where the sums are stored.  (Read from `perm` there, every row tile of a wave ended in
    // sixteen dependent loads in front of its stores.)
    __shared__ __attribute__((aligned(16))) int tile_rows[TC * 16];
    const bool ranked = P.expert_order ? true : rank_experts(P.tile_offsets, P.n_experts, order, reinterpret_cast<int*>(smem));
    const int per_expert = P.parts * P.stacks;
    bool window_used = false;
    for (int round = 0; round < kExpertRounds; round++) {
    const int item = expert_item(round, P.n_experts * per_expert, per_expert);
    if (item == -1) break;
    if (item == -2) continue;
    const int pos = item / per_expert, stack = (item - pos * per_expert) / P.parts, part = item - pos * per_expert - stack * P.parts;
    // (uniform: scalar registers; with the sort's table one load brings the expert and its ranges)
    int e, tile_begin, n_tiles, pos_begin, pos_end;
    if (P.expert_order) {
        const int32_t* d = P.expert_order + 8 * pos;
        e = __builtin_amdgcn_readfirstlane(d[0]), tile_begin = __builtin_amdgcn_readfirstlane(d[1]);
        n_tiles = __builtin_amdgcn_readfirstlane(d[2]);
        pos_begin = __builtin_amdgcn_readfirstlane(d[3]), pos_end = __builtin_amdgcn_readfirstlane(d[4]);
    } else {
        e = __builtin_amdgcn_readfirstlane(ranked ? order[pos] : pos);
        tile_begin = P.tile_offsets[e];
        n_tiles = P.tile_offsets[e + 1] - tile_begin;
    }
    if (n_tiles == 0) { // uniform for the workgroup: nobody waits at a barrier
        if (ranked) break; // (every later item's expert has no tile either)
        continue;
    }
    if (!P.expert_order) pos_begin = P.offsets[e], pos_end = P.offsets[e + 1];
    const uint8_t* wbase = (stack ? P.w2 : P.w) + (int64_t)e * P.matrix_bytes;
    float* yout = stack ? P.y2 : P.y;
    const uint8_t* records = P.ws + (size_t)tile_begin * P.k_units * UB;

    for (int t0 = 0; t0 < n_tiles; t0 += TC) {
        const int nt = min(TC, n_tiles - t0);
        if (window_used) lds_barrier(); // every wave is done with the previous tiles
        window_used = true;
        if (P.row_div) { // (uniform)
            uint32_t row_off[TC];
            gather_pairs<TC>(P.perm, pos_begin, pos_end, t0, nt, lane, row_off);
            gather_row_offsets<TC>(row_off, P.row_div, P.row_magic, (uint32_t)P.k_units * kRowUnitBytes);
            issue_window_gather<QT, TC>(P.ws, row_off, smem, nt, P.k_units, wave, waves, lane);
        } else {
            issue_window_copy<QT>(records + (size_t)t0 * P.k_units * UB, smem, nt * P.k_units, wave, waves, lane);
        }
        if (threadIdx.x < TC * 16) { // the tiles' output rows, once per window (see tile_rows)
            const int mm = t0 * 16 + (int)threadIdx.x;
            tile_rows[threadIdx.x] = pos_begin + mm < pos_end ? P.perm[pos_begin + mm] : -1;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        int walk = 0; // panels of this wave's walk so far
        for (int rt = part * waves + wave; rt < P.row_tiles; rt += P.parts * waves) {
            float acc[TC][4];
#pragma unroll
            for (int t = 0; t < TC; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;
            for (int kg = 0; kg < P.k_groups; kg++) {
                // (the two waves of a SIMD take turns at the higher priority: see the Q4_K kernel below)
                if ((walk + (wave >> 2)) & 1) __builtin_amdgcn_s_setprio(1); // (uniform)
                else __builtin_amdgcn_s_setprio(0);
                walk++;
                WPanel<QT> p;
                load_wpanel<QT>(p, wbase + (int64_t)(rt * P.k_groups + kg) * P.panel_bytes, P.slots, lane, j);
#pragma unroll
                for (int b = 0; b < WPanel<QT>::QC / 2; b++) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
                const int unit0 = kg * s_units;
                const int n_units = min(s_units, P.k_units - unit0);
#pragma unroll
                for (int t = 0; t < TC; t++) {
                    if (t < nt) // uniform
                        panel_dot<QT, false>(p, smem + ((size_t)t * P.k_units + unit0) * UB, n_units, j, grp, acc[t]);
                }
            }
            const int row = rt * 16 + j;
            if (row < P.n) {
#pragma unroll
                for (int t = 0; t < TC; t++) {
                    if (t >= nt) continue; // uniform
                    const int4 rows4 = *reinterpret_cast<const int4*>(&tile_rows[t * 16 + grp * 4]);
                    const int out_row[4] = {rows4.x, rows4.y, rows4.z, rows4.w};
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (out_row[r] >= 0) yout[(int64_t)out_row[r] * P.n + row] = acc[t][r];
                }
            }
        }
    }
    } // rounds
}

// The expert form for Q4_K matrices whose panels all hold NU units: the panel's activation-
// independent part is prepared once and serves the TC tiles, and the next panel of the wave's walk
// (row-tile after row-tile, panel after panel) is requested before the arithmetic of the current
// one starts - its registers are free as soon as the panel is prepared - so a wave always has a
// panel in flight under its own arithmetic.
template <int TC, int NU>
__global__ __launch_bounds__(64 * kExpertWaves) void gemv_mfma_expert_q4k_kernel(MfmaParams P) {
    constexpr int QT = QMM_Q4_K;
    constexpr int UB = Unit<QT>::kBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane_id = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = P.nwr;
    __shared__ int order[kRankedExperts];
    // The output rows (pair indices) of the tiles in the window, -1 past the expert's last pair: read
    // from LDS where the sums are stored.  (Read from `perm` there, every row tile of a wave ended in
    // sixteen dependent loads in front of its stores.)
    __shared__ __attribute__((aligned(16))) int tile_rows[TC * 16];
    const bool ranked = P.expert_order ? true : rank_experts(P.tile_offsets, P.n_experts, order, reinterpret_cast<int*>(smem));
    const int per_expert = P.parts * P.stacks;
    bool window_used = false;
#pragma unroll
    for (int round = 0; round < kExpertRounds; round++) {
    // (the lane's offsets are derived anew for every item: hoisted out of this loop they would stay in
    // registers beside a panel walk that needs all 256)
    int lane = lane_id;
    asm volatile("" : "+v"(lane));
    const int j = lane & 15, grp = lane >> 4;
    const int lane16 = lane * 16;
#ifdef QMM_EXPERT_TRACE
    const unsigned long long t_start = wall_clock64();
    unsigned long long t_window = 0;
#endif
    const int item = expert_item(round, P.n_experts * per_expert, per_expert);
    if (item == -1) break;
    if (item == -2) continue;
    const int pos = item / per_expert, stack = (item - pos * per_expert) / P.parts, part = item - pos * per_expert - stack * P.parts;
    // (uniform: scalar registers; with the sort's table one load brings the expert and its ranges)
    int e, tile_begin, n_tiles, pos_begin, pos_end;
    if (P.expert_order) {
        const int32_t* d = P.expert_order + 8 * pos;
        e = __builtin_amdgcn_readfirstlane(d[0]), tile_begin = __builtin_amdgcn_readfirstlane(d[1]);
        n_tiles = __builtin_amdgcn_readfirstlane(d[2]);
        pos_begin = __builtin_amdgcn_readfirstlane(d[3]), pos_end = __builtin_amdgcn_readfirstlane(d[4]);
    } else {
        e = __builtin_amdgcn_readfirstlane(ranked ? order[pos] : pos);
        tile_begin = P.tile_offsets[e];
        n_tiles = P.tile_offsets[e + 1] - tile_begin;
    }
    if (n_tiles == 0) { // uniform for the workgroup: nobody waits at a barrier
        if (ranked) break; // (every later item's expert has no tile either)
        continue;
    }
    if (!P.expert_order) pos_begin = P.offsets[e], pos_end = P.offsets[e + 1];
    const uint8_t* wbase = (stack ? P.w2 : P.w) + (int64_t)e * P.matrix_bytes;
    float* yout = stack ? P.y2 : P.y;
    const uint8_t* records = P.ws + (size_t)tile_begin * P.k_units * UB;
    const int rt_first = part * waves + wave, rt_step = P.parts * waves;

    for (int t0 = 0; t0 < n_tiles; t0 += TC) {
        const int nt = min(TC, n_tiles - t0);
        if (window_used) lds_barrier(); // every wave is done with the previous tiles
        window_used = true;
        uint32_t row_off[TC];
        if (P.row_div) gather_pairs<TC>(P.perm, pos_begin, pos_end, t0, nt, lane, row_off); // (uniform)
        else issue_window_copy<QT>(records + (size_t)t0 * P.k_units * UB, smem, nt * P.k_units, wave, waves, lane);
        if (threadIdx.x < TC * 16) { // the tiles' output rows, once per window (see tile_rows)
            const int mm = t0 * 16 + (int)threadIdx.x;
            tile_rows[threadIdx.x] = pos_begin + mm < pos_end ? P.perm[pos_begin + mm] : -1;
        }
        WPanel<QT> p;
        if (rt_first < P.row_tiles) // (uniform) the wave's first panel, needed whole before its first tile
            load_wpanel<QT>(p, wbase + (int64_t)rt_first * P.k_groups * P.panel_bytes, P.slots, lane, j);
        if (P.row_div) { // (the rows' pairs have arrived while the panel was requested)
            gather_row_offsets<TC>(row_off, P.row_div, P.row_magic, (uint32_t)P.k_units * kRowUnitBytes);
            issue_window_gather<QT, TC>(P.ws, row_off, smem, nt, P.k_units, wave, waves, lane);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
#ifdef QMM_EXPERT_TRACE
        if (t0 == 0) t_window = wall_clock64();
#endif
        int walk = 0; // panels of this wave's walk so far
        for (int rt = rt_first; rt < P.row_tiles; rt += rt_step) {
            float acc[TC][4];
#pragma unroll
            for (int t = 0; t < TC; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;
            for (int kg = 0; kg < P.k_groups; kg++) {
                // The two waves of a SIMD take turns at the higher priority, panel by panel: at equal
                // priority the SIMD issues from the older wave whenever both are ready, and the younger
                // one of each pair finishes a quarter later (measured: waves 0 - 3 of a workgroup end an
                // item after 33.7 us, waves 4 - 7 after 42.3, alone on their SIMDs for the last 8.6 us; with
                // the turns 37.9 and 40.2.  Turns tile by tile were measured slower than none).
                if ((walk + (wave >> 2)) & 1) __builtin_amdgcn_s_setprio(1); // (uniform)
                else __builtin_amdgcn_s_setprio(0);
                walk++;
#pragma unroll
                for (int b = 0; b < WPanel<QT>::QC / 2; b++) transpose_pair(p.q[2 * b], p.q[2 * b + 1]);
                Q4Prepared<NU> prep;
                q4k_prepare<NU>(p, prep, grp);
                // the next panel of the walk, if any, into the registers just freed
                int nrt = rt, nkg = kg + 1;
                if (nkg == P.k_groups) nkg = 0, nrt = rt + rt_step;
                if (nrt < P.row_tiles)
                    load_wpanel<QT>(p, wbase + (int64_t)(nrt * P.k_groups + nkg) * P.panel_bytes, P.slots, lane, j);
                const int unit0 = kg * NU;
#pragma unroll
                for (int t = 0; t < TC; t++) {
                    if (t >= nt) continue; // uniform
                    if (QMM_MFMA_ABL & 128) { // timing only: the panel stream without the tiles' arithmetic
                        if (t == 0) {
                            long x = 0;
#pragma unroll
                            for (int u = 0; u < NU; u++)
#pragma unroll
                                for (int b = 0; b < 4; b++) x ^= prep.lo[u][b] ^ prep.hi[u][b];
                            acc[0][0] += __int_as_float((int)x ^ (int)(x >> 32)) + prep.d[0] + prep.dmin[NU - 1];
                        }
                        continue;
                    }
                    const uint8_t* xu0 = smem + ((size_t)t * P.k_units + unit0) * UB;
                    q4k_tile_dot<NU>(
                        prep, [&](int u, int b) { return *reinterpret_cast<const i64x2*>(xu0 + u * UB + lane16 + b * 1024); },
                        [&](int u, long& bs_lo, long& bs_hi, float4& dx) {
                            const uint8_t* side = xu0 + u * UB + Unit<QT>::kQuant;
                            const i64x2 planes = *reinterpret_cast<const i64x2*>(side + 64 + j * 16);
                            bs_lo = planes.x, bs_hi = planes.y; // (every lane row: the prepared mins are zero past the first)
                            dx = *reinterpret_cast<const float4*>(side + grp * 16);
                        },
                        acc[t]);
                }
            }
            const int row = rt * 16 + j;
            if (row < P.n) {
#pragma unroll
                for (int t = 0; t < TC; t++) {
                    if (t >= nt) continue; // uniform
                    const int4 rows4 = *reinterpret_cast<const int4*>(&tile_rows[t * 16 + grp * 4]);
                    const int out_row[4] = {rows4.x, rows4.y, rows4.z, rows4.w};
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (out_row[r] >= 0) yout[(int64_t)out_row[r] * P.n + row] = acc[t][r];
                }
            }
        }
    }
#ifdef QMM_EXPERT_TRACE
    if (lane == 0 && blockIdx.x < 256) {
        const unsigned hw = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (31 << 11));   // HW_ID: CU, SE
        const unsigned xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (31 << 11)); // XCC_ID
        unsigned long long* o = g_expert_trace + ((size_t)((NU == 3 ? 512 : 0) + round * 256 + blockIdx.x) * 8 + wave) * 8;
        o[0] = t_start, o[1] = t_window, o[2] = wall_clock64(), o[3] = hw, o[4] = xcc, o[5] = (unsigned)n_tiles, o[6] = (unsigned)e, o[7] = NU;
    }
#endif
    } // rounds
}

template <int TC, int NU>
hipError_t launch_expert_q4k(const MfmaParams& P, dim3 grid, int waves, size_t lds, hipStream_t stream) {
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_expert_q4k_kernel<TC, NU>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kExpertMaxWindowBytes);
        if (e != hipSuccess) return e;
    }
    gemv_mfma_expert_q4k_kernel<TC, NU><<<grid, 64 * waves, lds, stream>>>(P);
    return hipGetLastError();
}

template <int QT, int TC>
hipError_t launch_expert_form(const MfmaParams& P, dim3 grid, int waves, size_t lds, hipStream_t stream) {
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_expert_kernel<QT, TC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kExpertMaxWindowBytes);
        if (e != hipSuccess) return e;
    }
    gemv_mfma_expert_kernel<QT, TC><<<grid, 64 * waves, lds, stream>>>(P);
    return hipGetLastError();
}

} // namespace

namespace {
// form 0: one tile of rows, one activation window; 1: the general one-shot form; 2: streaming
template <int QT, bool EP>
hipError_t launch_dense_form(int form, const MfmaParams& P, unsigned grid, int waves, size_t lds, hipStream_t stream) {
    const void* fn = form == 0   ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QT, true, false, EP>)
                     : form == 1 ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QT, false, false, EP>)
                                 : reinterpret_cast<const void*>(&gemv_mfma_stream_kernel<QT, EP>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    if (form == 0) launch_mfma(gemv_mfma_oneshot_kernel<QT, true, false, EP>, grid, 64 * waves, lds, stream, P);
    else if (form == 1) launch_mfma(gemv_mfma_oneshot_kernel<QT, false, false, EP>, grid, 64 * waves, lds, stream, P);
    else gemv_mfma_stream_kernel<QT, EP><<<grid, 64 * waves, lds, stream>>>(P);
    return hipGetLastError();
}
} // namespace

namespace {
// every panel of the matrix holds four units: the kernels' straight-line Q4_K arithmetic applies
bool full_panels(const QmmLayout& L) { return L.s == 4 && L.k_units % 4 == 0; }
// the units of every panel when all panels hold the same number (3: k = 768), else 0
int uniform_panel_units(const QmmLayout& L) { return L.k_units % L.s == 0 ? L.s : 0; }

// The straight-line arithmetic needs the registers of three waves per SIMD; a launch whose waves do
// not all fit the chip at once at that occupancy (gate | up at the 8B shapes: six per SIMD) keeps
// the compact form with a branch per unit, whose 80 registers let all of them be resident.
bool straight_line_fits(int64_t groups, int waves, int n_cus) {
    return groups * waves <= (int64_t)n_cus * kMaxWaves;
}
} // namespace

hipError_t qmm_launch_quantize_ws(int dtype, const float* x, int64_t m, int64_t k, void* workspace,
                                  hipStream_t stream, bool x_bf16) {
    if (m <= 0 || k <= 0 || m > 0x3fffffff || k > 0x3fffffff) return hipErrorInvalidValue;
    const int n_tiles = (int)((m + 15) / 16);
    const int64_t k_units = (k + 255) / 256;
    const int64_t threads = (int64_t)n_tiles * 16 * k_units * 16;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (dtype == QMM_Q4_K || dtype == QMM_Q6_K) { // both dot types are Q8_K: one record format
        if (x_bf16) quantize_ws_kernel<QMM_Q4_K, true><<<grid, 256, 0, stream>>>(x, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
        else quantize_ws_kernel<QMM_Q4_K><<<grid, 256, 0, stream>>>(x, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
    } else {
        if (x_bf16) quantize_ws_kernel<QMM_Q8_0, true><<<grid, 256, 0, stream>>>(x, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
        else quantize_ws_kernel<QMM_Q8_0><<<grid, 256, 0, stream>>>(x, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
    }
    return hipGetLastError();
}

hipError_t qmm_launch_quantize_silu_mul_ws(int dtype, const float* gate, const float* up, int64_t m, int64_t k,
                                           void* workspace, hipStream_t stream) {
    if (m <= 0 || k <= 0 || m > 0x3fffffff || k > 0x3fffffff) return hipErrorInvalidValue;
    const int n_tiles = (int)((m + 15) / 16);
    const int64_t k_units = (k + 255) / 256;
    const int64_t threads = (int64_t)n_tiles * 16 * k_units * 16;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (dtype == QMM_Q8_0)
        quantize_silu_mul_ws_kernel<QMM_Q8_0><<<grid, 256, 0, stream>>>(gate, up, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
    else
        quantize_silu_mul_ws_kernel<QMM_Q4_K><<<grid, 256, 0, stream>>>(gate, up, (int)m, (int)k, (int)k_units, n_tiles, (uint8_t*)workspace);
    return hipGetLastError();
}

size_t qmm_records_bytes(int dtype, int64_t m, int64_t k) {
    return (size_t)((m + 15) / 16) * (size_t)((k + 255) / 256) * (size_t)unit_bytes(dtype);
}

size_t qmm_gemv_mfma_workspace_bytes(const QmmLayout& L, int64_t m) {
    return (size_t)((m + 15) / 16) * (size_t)L.k_units * (size_t)unit_bytes(L.dtype);
}

hipError_t qmm_launch_gemv_mfma(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                                float* y, void* workspace, int n_cus, hipStream_t stream,
                                bool quantize, const QmmIo* io) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    if (L.n > 0x3fffffff || L.k > 0x3fffffff || m > 0x3fffffff ||
        L.row_tiles * L.k_groups > 0x7fffffff)
        return hipErrorInvalidValue;
    if (n_cus <= 0) n_cus = 1;
    const int n_tiles = (int)((m + 15) / 16);
    uint8_t* ws = (uint8_t*)workspace;
    const bool epilogue = io && (io->residual || io->y_bf16);
    MfmaParams P{};
    P.ep = QmmEpilogue{nullptr, 0};
    if (io) P.ep = QmmEpilogue{io->residual, io->y_bf16};
    P.window_units = (kWindowUnits / L.s) * L.s;
    // the streaming form adds up activation windows in y itself: no folded epilogue there
    if (epilogue && !(L.k_groups <= kMaxWaves && L.row_tiles < 8 * (int64_t)n_cus) && L.k_units > P.window_units)
        return hipErrorNotSupported;
    if (quantize) {
        hipError_t e = qmm_launch_quantize_ws(L.dtype, x, m, L.k, ws, stream, io && io->x_bf16);
        if (e != hipSuccess) return e;
    }
    P.w = (const uint8_t*)tiled;
    P.ws = ws;
    P.y = y;
    P.m = (int)m;
    P.n = (int)L.n;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.slots = L.slots;
    P.row_tiles = (int)L.row_tiles;
    P.panel_bytes = (int)L.panel_bytes;
    P.n_tiles = n_tiles;
    P.perm = nullptr;
    P.offsets = nullptr;
    P.tile_offsets = nullptr;
    P.n_experts = 0;
    P.stacks = 1;
    P.matrix_bytes = 0;
    P.w2 = nullptr;
    P.y2 = nullptr;
    P.double_buf = 0;
    P.n_weights = 0;
    P.window_units = (kWindowUnits / L.s) * L.s;
    const int padded_units = (int)(L.k_groups * L.s);
    if (P.window_units > padded_units) P.window_units = padded_units;
    const size_t window_bytes = (size_t)P.window_units * unit_bytes(L.dtype);

    // Every panel in flight at once needs one wave per panel of a row-tile; very tall
    // matrices (many row-tiles per CU) amortize the activation window better when it
    // stays resident while a wave walks whole row-tiles.
    const bool oneshot = L.k_groups <= kMaxWaves && L.row_tiles < 8 * (int64_t)n_cus;
    // (tiles a workgroup walks: one when every tile has workgroups of its own)
    int oneshot_nwr = 1; // row tiles per workgroup of the one-shot forms
    if (oneshot) {
        const int nwr_max = kMaxWaves / (int)L.k_groups;
        const int64_t want = (L.row_tiles + n_cus - 1) / n_cus; // as few workgroups as CUs where the waves allow it
        oneshot_nwr = (int)(want < 1 ? 1 : (want > nwr_max ? nwr_max : want));
    }
    const bool tile_parallel = oneshot && tile_parallel_applies(n_tiles) &&
                               (L.k_units <= P.window_units || direct_form_applies(L.dtype, 1, oneshot_nwr, false));
    const int stage_tiles = tile_parallel ? 1 : n_tiles;
    size_t lds;
    unsigned grid;
    int waves;
    if (oneshot) {
        P.nwk = (int)L.k_groups;
        P.nwr = oneshot_nwr;
        waves = P.nwk * P.nwr;
        P.rt_groups = (int)((L.row_tiles + P.nwr - 1) / P.nwr);
        grid = (unsigned)P.rt_groups;
        if (tile_parallel) grid = (unsigned)(((P.rt_groups + 7) / 8) * 8 * n_tiles);
        const bool single_stage = stage_tiles == 1 && L.k_units <= P.window_units;
        P.double_buf = !single_stage && 2 * window_bytes + (size_t)waves * 256 * 4 <= 160 * 1024;
        lds = single_stage ? std::max(window_bytes, (size_t)waves * 256 * 4)
                           : (P.double_buf ? 2 : 1) * window_bytes + (size_t)waves * 256 * 4;
    } else {
        P.nwk = 1;
        P.nwr = kMaxWaves;
        waves = kMaxWaves;
        P.rt_groups = (int)((L.row_tiles + waves - 1) / waves);
        grid = (unsigned)(P.rt_groups < n_cus ? P.rt_groups : n_cus);
        lds = window_bytes;
    }
    P.wave_magic = (65536 + P.nwk - 1) / P.nwk;
    if (oneshot && direct_form_applies(L.dtype, stage_tiles, P.nwr, L.k_units <= P.window_units)) {
        const size_t red = (size_t)waves * 256 * 4;
        if (full_panels(L)) {
            if (epilogue) launch_mfma(gemv_mfma_direct_q4k_kernel<true, 4>, grid, 64 * waves, red, stream, P);
            else launch_mfma(gemv_mfma_direct_q4k_kernel<false, 4>, grid, 64 * waves, red, stream, P);
        } else {
            if (epilogue) launch_mfma(gemv_mfma_direct_q4k_kernel<true>, grid, 64 * waves, red, stream, P);
            else launch_mfma(gemv_mfma_direct_q4k_kernel<false>, grid, 64 * waves, red, stream, P);
        }
        return hipGetLastError();
    }
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    const bool single = stage_tiles == 1 && L.k_units <= P.window_units;
    const int form = oneshot ? (single ? 0 : 1) : 2;
    if (form == 1 && tile_parallel) return hipErrorInvalidValue; // (not reached: tile_parallel implies a single-stage form)
    if (L.dtype == QMM_Q4_K && form == 0 && full_panels(L) && straight_line_fits((int64_t)P.rt_groups * (tile_parallel ? n_tiles : 1), waves, n_cus)) {
        const void* fn = epilogue ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, true, 4>)
                                  : reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, false, 4>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        if (epilogue) launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, true, 4>, grid, 64 * waves, lds, stream, P);
        else launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, false, 4>, grid, 64 * waves, lds, stream, P);
        return hipGetLastError();
    }
    if (L.dtype == QMM_Q4_K && form == 1 && full_panels(L)) {
        // several tiles of rows against a resident panel: its activation-independent part once
        const void* fn = epilogue ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, true, 4>)
                                  : reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, false, 4>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        if (epilogue) launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, true, 4>, grid, 64 * waves, lds, stream, P);
        else launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, false, 4>, grid, 64 * waves, lds, stream, P);
        return hipGetLastError();
    }
    if (L.dtype == QMM_Q4_K)
        return epilogue ? launch_dense_form<QMM_Q4_K, true>(form, P, grid, waves, lds, stream)
                        : launch_dense_form<QMM_Q4_K, false>(form, P, grid, waves, lds, stream);
    if (L.dtype == QMM_Q6_K)
        return epilogue ? launch_dense_form<QMM_Q6_K, true>(form, P, grid, waves, lds, stream)
                        : launch_dense_form<QMM_Q6_K, false>(form, P, grid, waves, lds, stream);
    return epilogue ? launch_dense_form<QMM_Q8_0, true>(form, P, grid, waves, lds, stream)
                    : launch_dense_form<QMM_Q8_0, false>(form, P, grid, waves, lds, stream);
}

size_t qmm_moe_records_bytes(int dtype, int64_t max_tiles, int64_t k) {
    return (size_t)max_tiles * (size_t)((k + 255) / 256) * (size_t)unit_bytes(dtype);
}

hipError_t qmm_launch_quantize_grouped(int dtype, const float* x, const float* x2, int x_div,
                                       int64_t k, const int32_t* perm, const int32_t* offsets,
                                       const int32_t* tile_offsets, int n_experts,
                                       int64_t max_tiles, void* records, hipStream_t stream,
                                       const int32_t* tile_expert) {
    const int64_t k_units = (k + 255) / 256;
    const int64_t threads = max_tiles * 16 * k_units * 16;
    if (threads <= 0) return hipSuccess;
    if (threads > 0x7fffffff00ll || k > 0x3fffffff) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (dtype == QMM_Q4_K || dtype == QMM_Q6_K) // both dot against Q8_K activations: one record format
        quantize_grouped_kernel<QMM_Q4_K><<<grid, 256, 0, stream>>>(x, x2, x_div, (int)k, (int)k_units, perm,
                                                                    offsets, tile_offsets, n_experts, tile_expert,
                                                                    (uint8_t*)records);
    else
        quantize_grouped_kernel<QMM_Q8_0><<<grid, 256, 0, stream>>>(x, x2, x_div, (int)k, (int)k_units, perm,
                                                                    offsets, tile_offsets, n_experts, tile_expert,
                                                                    (uint8_t*)records);
    return hipGetLastError();
}

bool qmm_gemv_mfma_grouped_supported(const QmmLayout& L) { return L.k_groups <= kMaxWaves; }

namespace {
// Activation tiles of an expert that the expert form holds in LDS at a time (0: the form does not
// apply): up to four, at least two, over all of k.
int expert_form_tiles(const QmmLayout& L, int n_cus) {
    const int mode = qmm_moe_expert_form();
    const bool expert_form = mode >= 0 ? mode != 0 : true;
    if (!expert_form || n_cus <= 0) return 0;
    const size_t tile_bytes = (size_t)L.k_units * unit_bytes(L.dtype);
    return 4 * tile_bytes <= 150 * 1024 ? 4 : (2 * tile_bytes <= 150 * 1024 ? 2 : 0);
}
} // namespace

bool qmm_moe_row_records_apply(const QmmLayout& L, int n_cus, int64_t pairs, int64_t rows, int row_div) {
    // (form 2: the expert form on tile records, kept for comparison)
    if (qmm_moe_expert_form() == 2 || !qmm_gemv_mfma_grouped_supported(L) || expert_form_tiles(L, n_cus) == 0) return false;
    // (the kernel's 32-bit row offsets and its division by multiplication)
    return row_div >= 1 && pairs * row_div < ((int64_t)1 << 32) && rows * L.k_units * kRowUnitBytes < ((int64_t)1 << 32);
}

size_t qmm_row_records_bytes(int64_t rows, int64_t k) { return (size_t)rows * (size_t)((k + 255) / 256) * kRowUnitBytes; }

hipError_t qmm_launch_quantize_rows(int dtype, const float* x, const float* x2, int64_t rows, int64_t k,
                                    void* row_records, hipStream_t stream) {
    const int64_t k_units = (k + 255) / 256;
    const int64_t threads = rows * k_units * 16;
    if (threads <= 0) return hipSuccess;
    if (threads > 0x7fffffff00ll || k > 0x3fffffff || k % 32) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (dtype == QMM_Q4_K || dtype == QMM_Q6_K) // both dot against Q8_K activations: one record format
        quantize_rows_kernel<QMM_Q4_K><<<grid, 256, 0, stream>>>(x, x2, rows, (int)k, (int)k_units, (uint8_t*)row_records);
    else
        quantize_rows_kernel<QMM_Q8_0><<<grid, 256, 0, stream>>>(x, x2, rows, (int)k, (int)k_units, (uint8_t*)row_records);
    return hipGetLastError();
}

hipError_t qmm_launch_moe_route_rows(const float* logits, int64_t t, int n_experts, int top_k, int32_t* ids,
                                     float* weights, hipStream_t stream, const float* x, int64_t k, int dtype,
                                     void* row_records) {
    if (t <= 0) return hipSuccess;
    if (!x || !row_records || k <= 0 || k > 0x3fffffff || k % 32) return hipErrorInvalidValue;
    if (n_experts < 1 || n_experts > 1024 || top_k < 1 || top_k > 64 || top_k > n_experts) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)((t + 3) / 4); // four tokens per workgroup: four routing waves, four quantizing
    const int per_lane = (n_experts + 63) / 64, k_units = (int)((k + 255) / 256);
    const bool q8k = dtype == QMM_Q4_K || dtype == QMM_Q6_K;
    auto launch = [&](auto kernel) { kernel<<<grid, 512, 0, stream>>>(logits, t, n_experts, top_k, ids, weights, x, (int)k, k_units, (uint8_t*)row_records); };
    if (per_lane <= 2) q8k ? launch(route_rows_kernel<2, QMM_Q4_K>) : launch(route_rows_kernel<2, QMM_Q8_0>);
    else if (per_lane <= 4) q8k ? launch(route_rows_kernel<4, QMM_Q4_K>) : launch(route_rows_kernel<4, QMM_Q8_0>);
    else q8k ? launch(route_rows_kernel<16, QMM_Q4_K>) : launch(route_rows_kernel<16, QMM_Q8_0>);
    return hipGetLastError();
}

hipError_t qmm_launch_gemv_mfma_grouped(const QmmLayout& L, const void* tiled, const void* tiled2,
                                        const void* records, float* y, float* y2, const int32_t* perm,
                                        const int32_t* offsets, const int32_t* tile_offsets,
                                        int n_experts, int64_t pairs, hipStream_t stream, int n_cus, int row_div,
                                        const int32_t* expert_order) {
    if (L.n == 0 || n_experts <= 0) return hipSuccess;
    if (!qmm_gemv_mfma_grouped_supported(L) || n_experts > 65535 || L.n > 0x3fffffff)
        return hipErrorInvalidValue;
    if (row_div && (expert_form_tiles(L, n_cus) == 0 || row_div < 0 || pairs * row_div >= ((int64_t)1 << 32)))
        return hipErrorInvalidValue; // (row records are read by the expert form only)
    MfmaParams P{};
    P.ep = QmmEpilogue{nullptr, 0};
    P.w = (const uint8_t*)tiled;
    P.ws = (const uint8_t*)records;
    P.y = y;
    P.m = 0;
    P.n = (int)L.n;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.slots = L.slots;
    P.row_tiles = (int)L.row_tiles;
    P.panel_bytes = (int)L.panel_bytes;
    P.n_tiles = 0;
    P.window_units = (kWindowUnits / L.s) * L.s;
    const int padded_units = (int)(L.k_groups * L.s);
    if (P.window_units > padded_units) P.window_units = padded_units;
    P.nwk = (int)L.k_groups;
    int nwr = kMaxWaves / P.nwk;
    if (nwr > L.row_tiles) nwr = (int)L.row_tiles;
    P.nwr = nwr;
    P.wave_magic = (65536 + P.nwk - 1) / P.nwk;
    P.rt_groups = (int)((L.row_tiles + nwr - 1) / nwr);
    P.perm = perm;
    P.offsets = offsets;
    P.tile_offsets = tile_offsets;
    P.matrix_bytes = L.matrix_bytes;
    P.w2 = (const uint8_t*)tiled2;
    P.y2 = y2;
    P.n_weights = 0;
    {
        // The expert form wherever up to four (at least two) activation tiles of an expert over all of k
        // fit in LDS; an expert with more tiles takes another pass over its weights per four.  Measured at
        // 128 experts, top-8, per layer, expert / one-shot form: 106 / 161 us at 128 tokens, 136 / 185
        // at 256, 179 / 252 at 512, 295 / 351 at 1024, 487 / 557 at 2048, 956 / 1010 at 4096, 1756 / 1891
        // at 8192.  IZWI_QMM_MOE_EXPERT_FORM=1 / 0 or izwi_qmm_set_moe_expert_form force the choice.
        const size_t tile_bytes = (size_t)L.k_units * unit_bytes(L.dtype);
        int tc = expert_form_tiles(L, n_cus);
        // (Q6_K, a tile per expert: the kernel for two tiles at a time needs twelve registers less and is
        // the faster one, 108 against 109.5 us per layer at 64 tokens; beyond, four tiles save passes over
        // the weights: 185 against 195 us at 512 tokens)
        if (L.dtype == QMM_Q6_K && tc == 4 && pairs <= (int64_t)8 * n_experts) tc = 2;
        if (tc) {
            MfmaParams E = P;
            E.row_div = row_div;
            E.expert_order = expert_order;
            E.row_magic = row_div > 1 ? (uint32_t)((((uint64_t)1 << 32) / (uint32_t)row_div) + 1) : 0;
            const int stacks = tiled2 ? 2 : 1;
            const bool prepared_q4k = L.dtype == QMM_Q4_K && (uniform_panel_units(L) == 4 || uniform_panel_units(L) == 3);
            static const int general_waves = [] { const char* e = getenv("IZWI_QMM_EXP_GENERAL_WAVES"); int v = e ? atoi(e) : 0; return v >= 1 && v <= kExpertWavesGeneral ? v : kExpertWavesGeneral; }();
            int waves = prepared_q4k ? kExpertWaves : general_waves;
            if (waves > L.row_tiles) waves = (int)L.row_tiles;
            // Items per CU: one while every expert holds one tile (all of an expert's rows in one item: its
            // tile is copied once), two beyond 8 pairs per expert on average, where the first experts get
            // a second tile (the tile counts differ from expert to expert and a heavy and a light item
            // on each CU even the CUs out).  Measured per layer at 128 experts, top-8, one / two per CU:
            // 93.6 / 100.0 us at 64 tokens, 98.0 / 103.7 at 128, 116.8 / 112.7 at 136, 119.5 / 114.9 at 160,
            // 120.9 / 116.6 at 192, 124.2 / 124.3 at 256, 152.6 / 134.5 at 320, 183.5 / 155.9 at 512.
            // IZWI_QMM_MOE_EXPERT_WGS_PER_CU forces it.  The stacks' row tiles are shared out to `parts`
            // items so that the items are at most that many per CU; a workgroup takes up to
            // kExpertRounds items, so the launch is (items / kExpertRounds) workgroups, all resident at
            // once unless experts x stacks alone exceed two per CU.
            static const int forced_wgs_per_cu = [] { const char* e = getenv("IZWI_QMM_MOE_EXPERT_WGS_PER_CU"); int v = e ? atoi(e) : 0; return v > 0 ? v : 0; }();
            int per_cu = forced_wgs_per_cu ? forced_wgs_per_cu : (pairs <= (int64_t)8 * n_experts ? 1 : 2);
            if (per_cu > kExpertRounds) per_cu = kExpertRounds;
            int parts = (int)((int64_t)per_cu * n_cus / ((int64_t)n_experts * stacks));
            const int max_parts = (int)((L.row_tiles + waves - 1) / waves);
            if (parts > max_parts) parts = max_parts;
            if (parts < 1) parts = 1;
            E.nwr = waves; // the workgroup's waves (every wave walks all of k)
            E.n_experts = n_experts, E.stacks = stacks, E.parts = parts;
            const int64_t n_items = (int64_t)parts * stacks * n_experts;
            const dim3 grid((unsigned)(per_cu == 1 ? n_items : (n_items + kExpertRounds - 1) / kExpertRounds));
            const size_t lds = (size_t)tc * tile_bytes;
            if (L.dtype == QMM_Q4_K && uniform_panel_units(L) == 4)
                return tc == 4 ? launch_expert_q4k<4, 4>(E, grid, waves, lds, stream) : launch_expert_q4k<2, 4>(E, grid, waves, lds, stream);
            if (L.dtype == QMM_Q4_K && uniform_panel_units(L) == 3)
                return tc == 4 ? launch_expert_q4k<4, 3>(E, grid, waves, lds, stream) : launch_expert_q4k<2, 3>(E, grid, waves, lds, stream);
            if (L.dtype == QMM_Q4_K)
                return tc == 4 ? launch_expert_form<QMM_Q4_K, 4>(E, grid, waves, lds, stream)
                               : launch_expert_form<QMM_Q4_K, 2>(E, grid, waves, lds, stream);
            if (L.dtype == QMM_Q6_K)
                return tc == 4 ? launch_expert_form<QMM_Q6_K, 4>(E, grid, waves, lds, stream)
                               : launch_expert_form<QMM_Q6_K, 2>(E, grid, waves, lds, stream);
            return tc == 4 ? launch_expert_form<QMM_Q8_0, 4>(E, grid, waves, lds, stream)
                           : launch_expert_form<QMM_Q8_0, 2>(E, grid, waves, lds, stream);
        }
    }
    const int waves = P.nwk * P.nwr;
    const size_t window_bytes = (size_t)P.window_units * unit_bytes(L.dtype);
    // A second window buffer hides the next tile's copy under this tile's arithmetic.  The kernel's
    // registers (135 - 167) admit one 12-wave workgroup per CU whatever its LDS, so the buffer is free
    // where it fits (T = 512, 128 experts: 248 -> 241 us per layer; smaller workgroups, two or three per
    // CU, were measured slower: 275 - 290 us - a workgroup's time is mostly the latency of its chain of
    // round trips, which halving its work does not shorten).  IZWI_QMM_MOE_DOUBLE_BUF=1 / 0 forces the choice.
    static const int force_double = [] { const char* e = getenv("IZWI_QMM_MOE_DOUBLE_BUF"); return e ? atoi(e) : -1; }();
    const size_t red_bytes = (size_t)waves * 256 * 4;
    P.double_buf = (force_double != 0) && 2 * window_bytes + red_bytes <= 160 * 1024;
    const size_t lds = (P.double_buf ? 2 : 1) * window_bytes + red_bytes;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    const void* fn = L.dtype == QMM_Q4_K
                         ? reinterpret_cast<const void*>(&gemv_mfma_grouped_kernel<QMM_Q4_K>)
                         : L.dtype == QMM_Q6_K
                               ? reinterpret_cast<const void*>(&gemv_mfma_grouped_kernel<QMM_Q6_K>)
                               : reinterpret_cast<const void*>(&gemv_mfma_grouped_kernel<QMM_Q8_0>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    P.n_experts = n_experts;
    P.stacks = tiled2 ? 2 : 1;
    const unsigned grid = (unsigned)(((n_experts + 7) / 8) * 8 * P.rt_groups * P.stacks);
    const int nu = L.dtype == QMM_Q4_K ? uniform_panel_units(L) : 0;
    if (nu == 4 || nu == 3) {
        const void* fp = nu == 4 ? reinterpret_cast<const void*>(&gemv_mfma_grouped_kernel<QMM_Q4_K, 4>)
                                 : reinterpret_cast<const void*>(&gemv_mfma_grouped_kernel<QMM_Q4_K, 3>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fp, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        if (nu == 4) gemv_mfma_grouped_kernel<QMM_Q4_K, 4><<<grid, 64 * waves, lds, stream>>>(P);
        else gemv_mfma_grouped_kernel<QMM_Q4_K, 3><<<grid, 64 * waves, lds, stream>>>(P);
        return hipGetLastError();
    }
    if (L.dtype == QMM_Q4_K)
        gemv_mfma_grouped_kernel<QMM_Q4_K><<<grid, 64 * waves, lds, stream>>>(P);
    else if (L.dtype == QMM_Q6_K)
        gemv_mfma_grouped_kernel<QMM_Q6_K><<<grid, 64 * waves, lds, stream>>>(P);
    else
        gemv_mfma_grouped_kernel<QMM_Q8_0><<<grid, 64 * waves, lds, stream>>>(P);
    return hipGetLastError();
}

hipError_t qmm_launch_gemv_mfma_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                      int64_t m, float* const* ys, const void* workspace, int n_cus,
                                      hipStream_t stream) {
    if (n_weights < 1 || n_weights > QMM_MAX_GROUP || m < 1) return hipErrorInvalidValue;
    if (n_cus <= 0) n_cus = 1;
    const QmmLayout& L0 = *layouts[0];
    int64_t total_row_tiles = 0;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        if (L.dtype != L0.dtype || L.k != L0.k || L.n_stacked != 1 || L.n == 0 || L.n > 0x3fffffff)
            return hipErrorInvalidValue;
        total_row_tiles += L.row_tiles;
    }
    MfmaParams P{};
    P.ep = QmmEpilogue{nullptr, 0};
    P.w = (const uint8_t*)tiled[0];
    P.ws = (const uint8_t*)workspace;
    P.y = ys[0];
    P.m = (int)m;
    P.n = (int)L0.n;
    P.k_units = (int)L0.k_units;
    P.k_groups = (int)L0.k_groups;
    P.slots = L0.slots;
    P.row_tiles = (int)L0.row_tiles;
    P.panel_bytes = (int)L0.panel_bytes;
    P.perm = nullptr;
    P.offsets = nullptr;
    P.tile_offsets = nullptr;
    P.n_experts = 0;
    P.stacks = 1;
    P.matrix_bytes = 0;
    P.w2 = nullptr;
    P.y2 = nullptr;
    P.double_buf = 0;
    P.window_units = (kWindowUnits / L0.s) * L0.s;
    const int padded_units = (int)(L0.k_groups * L0.s);
    if (P.window_units > padded_units) P.window_units = padded_units;
    // the one-shot forms with one window: one wave per panel of a row-tile, up to four tiles of rows
    if (m > 64 || L0.k_units > P.window_units || L0.k_groups > kMaxWaves || total_row_tiles >= 8 * (int64_t)n_cus)
        return hipErrorNotSupported;
    const int n_tiles = (int)((m + 15) / 16);
    P.n_tiles = n_tiles;
    P.nwk = (int)L0.k_groups;
    const int nwr_max = kMaxWaves / P.nwk;
    // as few workgroups as CUs where the waves allow it (q|k|v of the 8B shapes, 384 row-tiles: 7.3 us as
    // 192 workgroups of two row-tiles, 7.5 - 7.7 as 384 of one)
    const int64_t want = (total_row_tiles + n_cus - 1) / n_cus;
    P.nwr = (int)(want < 1 ? 1 : (want > nwr_max ? nwr_max : want));
    P.wave_magic = (65536 + P.nwk - 1) / P.nwk;
    P.n_weights = n_weights;
    int64_t groups = 0;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        groups += (L.row_tiles + P.nwr - 1) / P.nwr;
        P.rtg_end[i] = (int)groups;
        P.nv[i] = (int)L.n;
        P.row_tiles_v[i] = (int)L.row_tiles;
        P.wv[i] = (const uint8_t*)tiled[i];
        P.yv[i] = ys[i];
    }
    P.rt_groups = (int)groups;
    const int waves = P.nwk * P.nwr;
    // (every tile of rows with workgroups of its own: the single-stage forms below, a longer launch)
    const bool tile_parallel = tile_parallel_applies(n_tiles);
    const unsigned grid = tile_parallel ? (unsigned)(((groups + 7) / 8) * 8 * n_tiles) : (unsigned)groups;
    if (n_tiles > 1 && !tile_parallel) {
        // several tiles of rows against a resident panel (the form of the single-weight call at these m)
        const size_t window_bytes = (size_t)P.window_units * unit_bytes(L0.dtype), red_bytes = (size_t)waves * 256 * 4;
        P.double_buf = 2 * window_bytes + red_bytes <= 160 * 1024;
        const size_t lds = (P.double_buf ? 2 : 1) * window_bytes + red_bytes;
        if (lds > 160 * 1024) return hipErrorNotSupported;
        const bool prepared = L0.dtype == QMM_Q4_K && full_panels(L0);
        const void* fn = prepared               ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, false, 4>)
                         : L0.dtype == QMM_Q4_K ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, false>)
                         : L0.dtype == QMM_Q6_K ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q6_K, false>)
                                                : reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q8_0, false>);
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
        }
        if (prepared) launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, false, false, false, 4>, (unsigned)groups, 64 * waves, lds, stream, P);
        else if (L0.dtype == QMM_Q4_K) launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, false>, (unsigned)groups, 64 * waves, lds, stream, P);
        else if (L0.dtype == QMM_Q6_K) launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q6_K, false>, (unsigned)groups, 64 * waves, lds, stream, P);
        else launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q8_0, false>, (unsigned)groups, 64 * waves, lds, stream, P);
        return hipGetLastError();
    }
    if (direct_form_applies(L0.dtype, 1, P.nwr, true)) {
        if (full_panels(L0)) launch_mfma(gemv_mfma_direct_q4k_kernel<false, 4>, grid, 64 * waves, (size_t)waves * 256 * 4, stream, P);
        else launch_mfma(gemv_mfma_direct_q4k_kernel<false>, grid, 64 * waves, (size_t)waves * 256 * 4, stream, P);
        return hipGetLastError();
    }
    const size_t lds = std::max((size_t)P.window_units * unit_bytes(L0.dtype), (size_t)waves * 256 * 4);
    if (lds > 160 * 1024) return hipErrorNotSupported;
    const bool full = L0.dtype == QMM_Q4_K && full_panels(L0) && straight_line_fits(groups * (tile_parallel ? n_tiles : 1), waves, n_cus);
    const void* fn = full                   ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, false, 4>)
                     : L0.dtype == QMM_Q4_K ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q4_K, true>)
                     : L0.dtype == QMM_Q6_K ? reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q6_K, true>)
                                            : reinterpret_cast<const void*>(&gemv_mfma_oneshot_kernel<QMM_Q8_0, true>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    if (full)
        launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, true, false, false, 4>, grid, 64 * waves, lds, stream, P);
    else if (L0.dtype == QMM_Q4_K)
        launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q4_K, true>, grid, 64 * waves, lds, stream, P);
    else if (L0.dtype == QMM_Q6_K)
        launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q6_K, true>, grid, 64 * waves, lds, stream, P);
    else
        launch_mfma(gemv_mfma_oneshot_kernel<QMM_Q8_0, true>, grid, 64 * waves, lds, stream, P);
    return hipGetLastError();
}
