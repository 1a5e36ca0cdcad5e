// Device building blocks of the decode kernels (single-row dot4 form): 16-lane reductions, the
// activation quantizers, the LDS view of the quantized activations, panel loads and the per-panel
// block dot products.  Shared by the per-call kernels (qmm_gemv.hip) and the chained kernel
// (qmm_chain.hip); everything lives in an unnamed namespace, one copy per including file.
#ifndef IZWI_QMM_GEMV_BLOCKS_H
#define IZWI_QMM_GEMV_BLOCKS_H

#include <hip/hip_runtime.h>

#include <cstddef>

#include "qmm_internal.h"

namespace {

constexpr int kMaxWaves = 12;
constexpr int kXUnitStride = 272; // 256 B of int8 + 16 B pad (bank rotation between units)
constexpr uint32_t kNib = 0x0f0f0f0fu;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// ---- 16-lane (one DPP row) reductions -----------------------------------------
constexpr int kDppXor1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int kDppRor4 = 0x124; // row_ror:4
constexpr int kDppRor8 = 0x128; // row_ror:8

template <int CTRL>
__device__ __forceinline__ int dpp(int v) {
    return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false);
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, __int_as_float(dpp<kDppXor1>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp<kDppXor2>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp<kDppRor4>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp<kDppRor8>(__float_as_int(v))));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(dpp<kDppXor1>(__float_as_int(v)));
    v += __int_as_float(dpp<kDppXor2>(__float_as_int(v)));
    v += __int_as_float(dpp<kDppRor4>(__float_as_int(v)));
    v += __int_as_float(dpp<kDppRor8>(__float_as_int(v)));
    return v;
}
__device__ __forceinline__ int row16_min(int v) {
    v = min(v, dpp<kDppXor1>(v));
    v = min(v, dpp<kDppXor2>(v));
    v = min(v, dpp<kDppRor4>(v));
    v = min(v, dpp<kDppRor8>(v));
    return v;
}

// ---- activation quantizers (16 lanes cooperate on 256 values) ---------------

// BlockQ8K::from_float on one 256-value block spread over a 16-lane group
// (lane j holds values 16j..16j+15).  Returns this lane's 16 quants packed in
// four dwords, the block scale and the sum of this lane's 16 quants (bsums[j]).
__device__ __forceinline__ void quantize_q8k_lane(const float (&v)[16], int j, uint32_t (&q)[4],
                                                  float& d, int& sum16) {
    // the lane's first value of largest magnitude (strictly greater: an equal later one does not
    // replace it; a NaN never wins, as with fmaxf), with its sign
    float best = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) best = fabsf(v[i]) > fabsf(best) ? v[i] : best;
    const float amax = row16_max(fabsf(best));
    // the reference keeps the FIRST value of the block whose magnitude equals the maximum: the
    // lowest lane that holds it (key = lane << 1 | sign, smallest key over the block wins)
    int key = fabsf(best) == amax ? (j << 1) | (int)(__float_as_uint(best) >> 31) : 0x7fffffff;
    key = row16_min(key);
    sum16 = 0;
    if (amax == 0.0f) {
        d = 0.0f;
        q[0] = q[1] = q[2] = q[3] = 0;
        return;
    }
    const float mx = (key & 1) ? -amax : amax;
    const float iscale = __fdiv_rn(-128.0f, mx);
    d = __fdiv_rn(1.0f, iscale);
#pragma unroll
    for (int w = 0; w < 4; w++) {
        int qi[4];
#pragma unroll
        for (int b = 0; b < 4; b++) qi[b] = qmm_round_clamp_i8(__fmul_rn(iscale, v[4 * w + b]));
        q[w] = qmm_pack_i8x4(qi[0], qi[1], qi[2], qi[3]);
        sum16 = __builtin_amdgcn_sdot4((int)q[w], 0x01010101, sum16, false);
    }
}

// BlockQ8_0::from_float on a 32-value block held by a lane pair (16 values per
// lane).  Returns the packed quants and the block scale after its f16 rounding.
__device__ __forceinline__ void quantize_q80_lane(const float (&v)[16], uint32_t (&q)[4],
                                                  float& d_f16, uint16_t& d_bits) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, __int_as_float(dpp<kDppXor1>(__float_as_int(amax))));
    float d = __fdiv_rn(amax, 127.0f);
    float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    d_bits = qmm_f32_to_f16_bits(d);
    d_f16 = qmm_f16_bits_to_f32(d_bits);
#pragma unroll
    for (int w = 0; w < 4; w++) {
        int qi[4];
#pragma unroll
        for (int b = 0; b < 4; b++) qi[b] = qmm_round_clamp_i8(__fmul_rn(v[4 * w + b], id));
        q[w] = qmm_pack_i8x4(qi[0], qi[1], qi[2], qi[3]);
    }
}

// Sixteen consecutive activations of one row as four 16 B loads.  k is a
// multiple of 32, so a 16-value run is either inside the row or entirely past
// its end.  The loads are unconditional (out-of-range lanes read the start of
// `safe` instead) so that the issuing code stays one basic block and the waits
// on these loads can be counted separately from the weight loads behind them;
// x16_finish applies the range check to the values.
// XB: the activations are bf16 (two 16 B loads per run, widened to f32 exactly) instead of f32.
template <bool XB = false>
__device__ __forceinline__ void x16_issue(const void* __restrict__ src, const void* __restrict__ safe,
                                          bool in_range, float4 (&f)[4]) {
    const float4* p = reinterpret_cast<const float4*>(in_range ? src : safe);
#pragma unroll
    for (int i = 0; i < (XB ? 2 : 4); i++) f[i] = p[i];
}
// WHOLE: the caller knows the run is in range (it uses the values only then): no selects.
template <bool XB = false, bool WHOLE = false>
__device__ __forceinline__ void x16_finish(const float4 (&f)[4], bool in_range, float (&v)[16]) {
    if (WHOLE) in_range = true;
    if (XB) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t w[4] = {__float_as_uint(f[i].x), __float_as_uint(f[i].y), __float_as_uint(f[i].z),
                                   __float_as_uint(f[i].w)};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                v[8 * i + 2 * c] = in_range ? __uint_as_float(w[c] << 16) : 0.0f;
                v[8 * i + 2 * c + 1] = in_range ? __uint_as_float(w[c] & 0xffff0000u) : 0.0f;
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[4 * i] = in_range ? f[i].x : 0.0f;
        v[4 * i + 1] = in_range ? f[i].y : 0.0f;
        v[4 * i + 2] = in_range ? f[i].z : 0.0f;
        v[4 * i + 3] = in_range ? f[i].w : 0.0f;
    }
}

// Workgroup barrier that orders LDS traffic only: the compiler's own barrier
// also waits for every outstanding global load of the wave, which would
// serialize the weight panel behind the activation quantizer.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- LDS view ---------------------------------------------------------------
template <int QT>
struct XLds {
    uint8_t* xq;  // [MT][k_units][kXUnitStride]
    float* xd;    // Q4_K, Q6_K: [MT][k_units]   Q8_0: [MT][k_units][8]
    int* xbs;     // Q4_K: [MT][k_units][8] sums of 32   Q6_K: [MT][k_units][16] sums of 16   Q8_0: unused
    float* red;   // [2][waves][MT][16]
};
// block scales and partial sums kept per quantized unit of x
template <int QT>
constexpr int kXdPerItem = QT == QMM_Q8_0 ? 8 : 1;
template <int QT>
constexpr int kXbsPerItem = QT == QMM_Q4_K ? 8 : (QT == QMM_Q6_K ? 16 : 0);

template <int QT, int MT>
__host__ __device__ inline size_t lds_bytes(int64_t k_units, int waves) {
    size_t b = (size_t)MT * k_units * kXUnitStride;
    b += (size_t)MT * k_units * kXdPerItem<QT> * sizeof(float);
    b += (size_t)MT * k_units * kXbsPerItem<QT> * sizeof(int);
    b = (b + 15) & ~(size_t)15;
    b += (size_t)2 * waves * MT * 16 * sizeof(float);
    return b;
}

template <int QT, int MT>
__device__ inline XLds<QT> carve(uint8_t* base, int64_t k_units) {
    XLds<QT> l;
    l.xq = base;
    size_t b = (size_t)MT * k_units * kXUnitStride;
    l.xd = reinterpret_cast<float*>(base + b);
    b += (size_t)MT * k_units * kXdPerItem<QT> * sizeof(float);
    l.xbs = reinterpret_cast<int*>(base + b);
    b += (size_t)MT * k_units * kXbsPerItem<QT> * sizeof(int);
    b = (b + 15) & ~(size_t)15;
    l.red = reinterpret_cast<float*>(base + b);
    return l;
}

// One 16-lane group quantizes one (row, 256-value unit) item of x into LDS.
// Item i of a pass is unit i / MT of row m0 + i % MT; rows >= m are zero.
// With `perm` the row is x[perm[row] / x_div] (expert-grouped pairs).
struct XSource {
    const void* x; // f32 or bf16 rows
    const int32_t* perm;
    int x_div;
    int m0, m, k;
    int k_units;
};

template <int MT, bool XB = false>
__device__ __forceinline__ bool x_item_issue(const XSource& s, int item, bool item_ok, float4 (&f)[4]) {
    const int j = threadIdx.x & 15;
    const int mi = item % MT, unit = item / MT;
    const bool row_ok = item_ok && s.m0 + mi < s.m;
    int64_t xr = s.m0 + mi;
    if (s.perm != nullptr) xr = row_ok ? s.perm[s.m0 + mi] / s.x_div : 0;
    const int64_t k0 = (int64_t)unit * 256 + 16 * j;
    const bool in_range = row_ok && k0 + 16 <= s.k;
    if (XB) x16_issue<true>(static_cast<const uint16_t*>(s.x) + xr * s.k + k0, s.x, in_range, f);
    else x16_issue<false>(static_cast<const float*>(s.x) + xr * s.k + k0, s.x, in_range, f);
    return in_range;
}

template <int QT, int MT>
__device__ __forceinline__ void x_item_quantize(const XLds<QT>& l, int k_units, int item,
                                                const float (&v)[16]) {
    const int j = threadIdx.x & 15;
    const int slot = (item % MT) * k_units + item / MT; // [mi][unit]
    uint32_t q[4];
    if (QT == QMM_Q4_K) {
        float d;
        int s16;
        quantize_q8k_lane(v, j, q, d, s16);
        int s32 = s16 + dpp<kDppXor1>(s16);
        if ((j & 1) == 0) l.xbs[slot * 8 + (j >> 1)] = s32;
        if (j == 0) l.xd[slot] = d;
    } else if (QT == QMM_Q6_K) {
        float d;
        int s16;
        quantize_q8k_lane(v, j, q, d, s16);
        l.xbs[slot * 16 + j] = s16;
        if (j == 0) l.xd[slot] = d;
    } else {
        float d;
        uint16_t bits;
        quantize_q80_lane(v, q, d, bits);
        if ((j & 1) == 0) l.xd[slot * 8 + (j >> 1)] = d;
    }
    *reinterpret_cast<uint4*>(l.xq + (size_t)slot * kXUnitStride + 16 * j) =
        make_uint4(q[0], q[1], q[2], q[3]);
}

// ---- activations quantized ahead of the kernel ("x blocks") ---------------------------------
// What the quantizer above leaves in LDS per (row, unit), kept in device memory for rows that many
// workgroups need (the tokens of an expert-grouped launch: every workgroup of a segment would
// quantize the same rows again): three arrays over slot = row * k_units + unit, strides as in LDS.
struct XBlocks {
    uint8_t* xq; // [rows * k_units][kXUnitStride]
    float* xd;   // [rows * k_units][kXdPerItem]
    int* xbs;    // [rows * k_units][kXbsPerItem]
};
__host__ __device__ inline size_t x_blocks_part_bytes(size_t n) { return (n + 255) & ~(size_t)255; }
// (the largest per-slot sizes of the three block types: one buffer layout for all of them)
__host__ __device__ inline size_t x_blocks_bytes(int64_t rows, int64_t k_units) {
    const size_t slots = (size_t)rows * (size_t)k_units;
    return x_blocks_part_bytes(slots * kXUnitStride) + x_blocks_part_bytes(slots * 8 * sizeof(float)) +
           x_blocks_part_bytes(slots * 16 * sizeof(int));
}
__host__ __device__ inline XBlocks x_blocks_carve(void* base, int64_t rows, int64_t k_units) {
    const size_t slots = (size_t)rows * (size_t)k_units;
    uint8_t* b = static_cast<uint8_t*>(base);
    XBlocks xb;
    xb.xq = b;
    xb.xd = reinterpret_cast<float*>(b + x_blocks_part_bytes(slots * kXUnitStride));
    xb.xbs = reinterpret_cast<int*>(b + x_blocks_part_bytes(slots * kXUnitStride) + x_blocks_part_bytes(slots * 8 * sizeof(float)));
    return xb;
}

// One wave quantizes row `row` of x [rows, k] (f32) into its x blocks: its four 16-lane groups take
// the units in turn, with the quantizer of the kernels (the same values as quantizing in the kernel).
// Two steps, so that the caller can put other work between the loads of the first two units of
// every group (k <= 2048: all of the row) and their use.
struct XRowLoads {
    float4 f[2][4];
    bool in_range[2];
};
__device__ __forceinline__ void x_row_issue(const float* __restrict__ x, int64_t row, int k, int k_units, XRowLoads& ld) {
    const int lane = threadIdx.x & 63, j = lane & 15;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int unit = (lane >> 4) + 4 * i;
        const int k0 = unit * 256 + 16 * j;
        ld.in_range[i] = unit < k_units && k0 + 16 <= k;
        x16_issue<false>(x + row * k + k0, x, ld.in_range[i], ld.f[i]);
    }
}
template <int QT>
__device__ __forceinline__ void x_row_to_blocks(const float* __restrict__ x, int64_t row, int k, int k_units,
                                                const XBlocks& xb, const XRowLoads& ld) {
    const int lane = threadIdx.x & 63, j = lane & 15;
    XLds<QT> g;
    g.xq = xb.xq + (size_t)row * k_units * kXUnitStride;
    g.xd = xb.xd + (size_t)row * k_units * kXdPerItem<QT>;
    g.xbs = xb.xbs + (size_t)row * k_units * kXbsPerItem<QT>;
    g.red = nullptr;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int unit = (lane >> 4) + 4 * i;
        if (unit < k_units) { // uniform for the 16-lane group
            float v[16];
            x16_finish<false>(ld.f[i], ld.in_range[i], v);
            x_item_quantize<QT, 1>(g, k_units, unit, v);
        }
    }
    for (int unit = (lane >> 4) + 8; unit < k_units; unit += 4) {
        const int k0 = unit * 256 + 16 * j;
        const bool in_range = k0 + 16 <= k;
        float4 f[4];
        float v[16];
        x16_issue<false>(x + row * k + k0, x, in_range, f);
        x16_finish<false>(f, in_range, v);
        x_item_quantize<QT, 1>(g, k_units, unit, v);
    }
}

// A 16-lane group copies the x blocks of (source row, unit) into LDS slot `dst_slot`; zeros for a
// row that does not exist (what the quantizer makes of a zero row).
template <int QT>
__device__ __forceinline__ void x_blocks_to_lds(const XLds<QT>& l, int dst_slot, const XBlocks& xb, int64_t src_slot,
                                                bool row_ok) {
    const int j = threadIdx.x & 15;
    const int64_t s = row_ok ? src_slot : 0;
    uint4 q = *reinterpret_cast<const uint4*>(xb.xq + (size_t)s * kXUnitStride + 16 * j);
    float d = j < kXdPerItem<QT> ? xb.xd[s * kXdPerItem<QT> + j] : 0.0f;
    int bs = 0;
    if (kXbsPerItem<QT> > 0) bs = j < kXbsPerItem<QT> ? xb.xbs[s * (kXbsPerItem<QT> > 0 ? kXbsPerItem<QT> : 1) + j] : 0;
    if (!row_ok) q = make_uint4(0, 0, 0, 0), d = 0.0f, bs = 0;
    *reinterpret_cast<uint4*>(l.xq + (size_t)dst_slot * kXUnitStride + 16 * j) = q;
    if (j < kXdPerItem<QT>) l.xd[dst_slot * kXdPerItem<QT> + j] = d;
    if (kXbsPerItem<QT> > 0 && j < kXbsPerItem<QT>) l.xbs[dst_slot * (kXbsPerItem<QT> > 0 ? kXbsPerItem<QT> : 1) + j] = bs;
}

// ---- panel registers ----------------------------------------------------------
template <int QT>
struct Panel {
    static constexpr int QC = QT == QMM_Q4_K ? 8 : (QT == QMM_Q6_K ? 13 : 16);
    u32x4 hdr;
    u32x4 q[QC];
};

// Unconditional loads (see x16_issue): a lane without a slot reads lane 0's
// data and the caller clears its header, which zeroes every scale and with
// them the lane's contribution.
template <int QT>
__device__ __forceinline__ void load_panel(Panel<QT>& p, const uint8_t* __restrict__ base,
                                           int slots, int lane, bool active) {
    const u32x4* src = reinterpret_cast<const u32x4*>(base) + (active ? lane : 0);
    p.hdr = __builtin_nontemporal_load(src);
#pragma unroll
    for (int c = 0; c < Panel<QT>::QC; c++)
        p.q[c] = __builtin_nontemporal_load(src + (size_t)(1 + c) * slots);
}
template <int QT>
__device__ __forceinline__ void mask_panel(Panel<QT>& p, bool active) {
    p.hdr.x = active ? p.hdr.x : 0u;
    p.hdr.y = active ? p.hdr.y : 0u;
    p.hdr.z = active ? p.hdr.z : 0u;
    p.hdr.w = active ? p.hdr.w : 0u;
}

__device__ __forceinline__ int dot16(const u32x4& a, const uint4& b, int acc) {
    acc = dot4(a.x, b.x, acc);
    acc = dot4(a.y, b.y, acc);
    acc = dot4(a.z, b.z, acc);
    acc = dot4(a.w, b.w, acc);
    return acc;
}

// acc[mi] += dot(weight unit held in p, quantized x unit `unit` of row mi)
template <int QT, int MT>
__device__ __forceinline__ void multiply_panel(const Panel<QT>& p, const XLds<QT>& l, int unit,
                                               int k_units, float (&acc)[MT]) {
    if (QT == QMM_Q4_K) {
        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
        qmm_unpack_q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        int isum[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) isum[mi] = 0;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // 64 elements: low nibbles are sub-block 2g, high nibbles sub-block 2g+1
            const u32x4 lo0 = p.q[2 * g] & kNib, lo1 = p.q[2 * g + 1] & kNib;
            const u32x4 hi0 = (p.q[2 * g] >> 4) & kNib, hi1 = (p.q[2 * g + 1] >> 4) & kNib;
            const int sc0 = (int)qmm_byte_of(sc_lo, sc_hi, 2 * g);
            const int sc1 = (int)qmm_byte_of(sc_lo, sc_hi, 2 * g + 1);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const uint4* xq = reinterpret_cast<const uint4*>(
                    l.xq + (size_t)(mi * k_units + unit) * kXUnitStride);
                int dlo = dot16(lo0, xq[4 * g], 0);
                dlo = dot16(lo1, xq[4 * g + 1], dlo);
                int dhi = dot16(hi0, xq[4 * g + 2], 0);
                dhi = dot16(hi1, xq[4 * g + 3], dhi);
                isum[mi] += __mul24(sc0, dlo) + __mul24(sc1, dhi); // |dot| < 2^17, scale < 64
            }
        }
        const float d = qmm_f16_bits_to_f32((uint16_t)(p.hdr.x & 0xffffu));
        const float dmin = qmm_f16_bits_to_f32((uint16_t)(p.hdr.x >> 16));
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const int item = mi * k_units + unit;
            const int4* bs = reinterpret_cast<const int4*>(l.xbs + item * 8);
            const int4 b0 = bs[0], b1 = bs[1];
            // 24-bit multiplies: mins < 64, |sub-block sums| <= 32 * 128
            int msum = __mul24((int)qmm_byte_of(mn_lo, mn_hi, 0), b0.x) + __mul24((int)qmm_byte_of(mn_lo, mn_hi, 1), b0.y) +
                       __mul24((int)qmm_byte_of(mn_lo, mn_hi, 2), b0.z) + __mul24((int)qmm_byte_of(mn_lo, mn_hi, 3), b0.w) +
                       __mul24((int)qmm_byte_of(mn_lo, mn_hi, 4), b1.x) + __mul24((int)qmm_byte_of(mn_lo, mn_hi, 5), b1.y) +
                       __mul24((int)qmm_byte_of(mn_lo, mn_hi, 6), b1.z) + __mul24((int)qmm_byte_of(mn_lo, mn_hi, 7), b1.w);
            const float dx = l.xd[item];
            acc[mi] += (d * dx) * (float)isum[mi] - (dmin * dx) * (float)msum;
        }
    } else if (QT == QMM_Q6_K) {
        // q[0..7] = ql, q[8..11] = qh, q[12].x = d; hdr = 16 signed scales, scale j for the
        // elements 16 j .. 16 j + 15.  Element 128 h + 32 g + e (e < 32) is
        // nibble(g >> 1) of ql[64 h + 32 (g & 1) + e] | bits 2g, 2g+1 of qh[32 h + e], minus 32:
        // the 32 is taken off through the sums of x (dot - 32 * sum of the 16 quants of x).
        const uint32_t hw[4] = {p.hdr.x, p.hdr.y, p.hdr.z, p.hdr.w};
        constexpr uint32_t kTwo = 0x03030303u;
        int isum[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) isum[mi] = 0;
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int lb = 0; lb < 2; lb++) {
                const u32x4 a = p.q[4 * h + lb], b = p.q[4 * h + 2 + lb], hh = p.q[8 + 2 * h + lb];
                u32x4 v[4];
                v[0] = (a & kNib) | ((hh & kTwo) << 4);
                v[1] = (b & kNib) | (((hh >> 2) & kTwo) << 4);
                v[2] = ((a >> 4) & kNib) | (((hh >> 4) & kTwo) << 4);
                v[3] = ((b >> 4) & kNib) | (((hh >> 6) & kTwo) << 4);
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int j = 8 * h + 2 * g + lb; // scale index = 16-element group of the unit
                    const int sc = (int)(int8_t)((hw[j >> 2] >> (8 * (j & 3))) & 0xffu);
#pragma unroll
                    for (int mi = 0; mi < MT; mi++) {
                        const int item = mi * k_units + unit;
                        const uint4* xq = reinterpret_cast<const uint4*>(l.xq + (size_t)item * kXUnitStride);
                        const int dot = dot16(v[g], xq[j], 0) - 32 * l.xbs[item * 16 + j];
                        isum[mi] += __mul24(sc, dot); // |dot| < 2^18, |scale| <= 128
                    }
                }
            }
        }
        const float d = qmm_f16_bits_to_f32((uint16_t)(p.q[12].x & 0xffffu));
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] += (d * l.xd[mi * k_units + unit]) * (float)isum[mi];
    } else {
        const uint32_t hw[4] = {p.hdr.x, p.hdr.y, p.hdr.z, p.hdr.w};
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const float dw = qmm_f16_bits_to_f32((uint16_t)((hw[b >> 1] >> (16 * (b & 1))) & 0xffffu));
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const int item = mi * k_units + unit;
                const uint4* xq = reinterpret_cast<const uint4*>(l.xq + (size_t)item * kXUnitStride);
                int sumi = dot16(p.q[2 * b], xq[2 * b], 0);
                sumi = dot16(p.q[2 * b + 1], xq[2 * b + 1], sumi);
                acc[mi] += ((float)sumi * dw) * l.xd[item * 8 + b];
            }
        }
    }
}

} // namespace

#endif // IZWI_QMM_GEMV_BLOCKS_H
