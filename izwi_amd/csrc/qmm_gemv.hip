// Decode kernel: fused activation-quantize + block dot products, M = 1..64.
//
// The arithmetic is candle-core's CPU `matmul` (quantize each activation row to
// the weight type's dot type, integer block dots, f32 scaling); only the f32
// summation order differs.  The work is bounded by streaming the weight bytes
// from HBM once:
//   * a wavefront reads a panel (16 rows x S units of 256 k-elements) as one
//     16 B/lane coalesced load for the headers plus 8 (Q4_K) or 16 (Q8_0) for
//     the quants; lane (u, r) owns unit u of row r, so no weight byte is
//     shuffled between lanes and all nibble / int8 products run on
//     v_dot4_i32_i8 (0.6 VALU lane-ops per weight element);
//   * the next panel is loaded into a second register set while the current
//     one is being multiplied;
//   * the workgroup quantizes the activations once into LDS; lanes of one
//     16-row group read the same LDS words (broadcast), the unit stride is
//     padded by 16 B so the S groups hit different banks;
//   * the S partial sums of a row are combined with two cross-lane steps, the
//     k-split between waves through LDS.
#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

constexpr int kWgThreads = 256;
constexpr int kWaves = 4;
constexpr int kXUnitStride = 272; // 256 B of int8 + 16 B pad (bank rotation between units)
constexpr uint32_t kNib = 0x0f0f0f0fu;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// ---- activation quantizers (16 lanes cooperate on 256 values) ---------------

// BlockQ8K::from_float on one 256-value block spread over a 16-lane group
// (lane j holds values 16j..16j+15).  Returns this lane's 16 quants packed in
// four dwords, the block scale and the sum of this lane's 16 quants (bsums[j]).
__device__ __forceinline__ void quantize_q8k_lane(const float (&v)[16], uint32_t (&q)[4], float& d,
                                                  int& sum16) {
    float amax = 0.0f, mx = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float a = fabsf(v[i]);
        if (amax < a) {
            amax = a;
            mx = v[i];
        }
    }
    // first occurrence of the largest |x| over the group: the lower lane wins ties
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        float oa = __shfl_xor(amax, off, 16);
        float om = __shfl_xor(mx, off, 16);
        bool self_is_lower = (threadIdx.x & off) == 0;
        float lo_a = self_is_lower ? amax : oa, lo_m = self_is_lower ? mx : om;
        float hi_a = self_is_lower ? oa : amax, hi_m = self_is_lower ? om : mx;
        bool take_hi = lo_a < hi_a;
        amax = take_hi ? hi_a : lo_a;
        mx = take_hi ? hi_m : lo_m;
    }
    sum16 = 0;
    if (amax == 0.0f) {
        d = 0.0f;
        q[0] = q[1] = q[2] = q[3] = 0;
        return;
    }
    float iscale = __fdiv_rn(-128.0f, mx);
    d = __fdiv_rn(1.0f, iscale);
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t packed = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            float r = roundf(__fmul_rn(iscale, v[4 * w + b]));
            int qi = (int)fminf(r, 127.0f);
            qi = max(qi, -128);
            sum16 += qi;
            packed |= ((uint32_t)qi & 0xffu) << (8 * b);
        }
        q[w] = packed;
    }
}

// BlockQ8_0::from_float on a 32-value block held by a lane pair (16 values per
// lane).  Returns the packed quants and the block scale after its f16 rounding.
__device__ __forceinline__ void quantize_q80_lane(const float (&v)[16], uint32_t (&q)[4],
                                                  float& d_f16, uint16_t& d_bits) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 16));
    float d = __fdiv_rn(amax, 127.0f);
    float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    d_bits = qmm_f32_to_f16_bits(d);
    d_f16 = qmm_f16_bits_to_f32(d_bits);
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t packed = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            float r = roundf(__fmul_rn(v[4 * w + b], id));
            int qi = (int)fminf(fmaxf(r, -128.0f), 127.0f);
            packed |= ((uint32_t)qi & 0xffu) << (8 * b);
        }
        q[w] = packed;
    }
}

__device__ __forceinline__ void load16(const float* __restrict__ row, int64_t k0, int64_t k,
                                       bool row_ok, float (&v)[16]) {
    if (row_ok && k0 + 16 <= k) {
        const float4* p = reinterpret_cast<const float4*>(row + k0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 f = p[i];
            v[4 * i] = f.x;
            v[4 * i + 1] = f.y;
            v[4 * i + 2] = f.z;
            v[4 * i + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = (row_ok && k0 + i < k) ? row[k0 + i] : 0.0f;
    }
}

// ---- LDS view ---------------------------------------------------------------
template <int QT>
struct XLds {
    uint8_t* xq;  // [MT][k_units][kXUnitStride]
    float* xd;    // Q4_K: [MT][k_units]      Q8_0: [MT][k_units][8]
    int* xbs;     // Q4_K: [MT][k_units][8]   Q8_0: unused
    float* red;   // [2][kWaves][G][MT][16]
};

template <int QT, int MT, int G>
__host__ __device__ inline size_t lds_bytes(int64_t k_units) {
    size_t b = (size_t)MT * k_units * kXUnitStride;
    b += (size_t)MT * k_units * (QT == QMM_Q4_K ? 1 : 8) * sizeof(float);
    if (QT == QMM_Q4_K) b += (size_t)MT * k_units * 8 * sizeof(int);
    b += 2 * kWaves * G * MT * 16 * sizeof(float);
    return (b + 15) & ~(size_t)15;
}

template <int QT, int MT, int G>
__device__ inline XLds<QT> carve(uint8_t* base, int64_t k_units) {
    XLds<QT> l;
    l.xq = base;
    base += (size_t)MT * k_units * kXUnitStride;
    l.xd = reinterpret_cast<float*>(base);
    base += (size_t)MT * k_units * (QT == QMM_Q4_K ? 1 : 8) * sizeof(float);
    l.xbs = reinterpret_cast<int*>(base);
    if (QT == QMM_Q4_K) base += (size_t)MT * k_units * 8 * sizeof(int);
    l.red = reinterpret_cast<float*>(base);
    return l;
}

// Quantizes rows m0..m0+MT of x into LDS (rows >= m are zero).  With `perm`
// the i-th row is x[perm[i] / x_div] (expert-grouped pairs).
template <int QT, int MT>
__device__ inline void quantize_rows_to_lds(const XLds<QT>& l, const float* __restrict__ x,
                                            const int32_t* __restrict__ perm, int x_div,
                                            int64_t m0, int64_t m, int64_t k, int k_units) {
    const int group = threadIdx.x >> 4; // 16 groups of 16 lanes
    const int j = threadIdx.x & 15;
    const int items = MT * k_units;
    for (int item = group; item < items; item += kWgThreads / 16) {
        int mi = item / k_units;
        int unit = item - mi * k_units;
        float v[16];
        const bool row_ok = m0 + mi < m;
        int64_t xr = m0 + mi;
        if (perm != nullptr) xr = row_ok ? perm[m0 + mi] / x_div : 0;
        load16(x + xr * k, (int64_t)unit * 256 + 16 * j, k, row_ok, v);
        uint32_t q[4];
        uint8_t* dst = l.xq + (size_t)item * kXUnitStride + 16 * j;
        if (QT == QMM_Q4_K) {
            float d;
            int s16;
            quantize_q8k_lane(v, q, d, s16);
            int s32 = s16 + __shfl_xor(s16, 1, 16);
            if ((j & 1) == 0) l.xbs[item * 8 + (j >> 1)] = s32;
            if (j == 0) l.xd[item] = d;
        } else {
            float d;
            uint16_t bits;
            quantize_q80_lane(v, q, d, bits);
            if ((j & 1) == 0) l.xd[item * 8 + (j >> 1)] = d;
        }
        *reinterpret_cast<uint4*>(dst) = make_uint4(q[0], q[1], q[2], q[3]);
    }
}

// ---- panel registers ----------------------------------------------------------
template <int QT>
struct Panel {
    static constexpr int QC = QT == QMM_Q4_K ? 8 : 16;
    u32x4 hdr;
    u32x4 q[QC];
};

template <int QT>
__device__ __forceinline__ void load_panel(Panel<QT>& p, const uint8_t* __restrict__ base,
                                           int slots, int lane, bool active) {
    if (active) {
        const u32x4* src = reinterpret_cast<const u32x4*>(base) + lane;
        p.hdr = __builtin_nontemporal_load(src);
#pragma unroll
        for (int c = 0; c < Panel<QT>::QC; c++)
            p.q[c] = __builtin_nontemporal_load(src + (size_t)(1 + c) * slots);
    } else {
        p.hdr = u32x4{0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < Panel<QT>::QC; c++) p.q[c] = u32x4{0, 0, 0, 0};
    }
}

__device__ __forceinline__ int dot16(const u32x4& a, const uint4& b, int acc) {
    acc = dot4(a.x, b.x, acc);
    acc = dot4(a.y, b.y, acc);
    acc = dot4(a.z, b.z, acc);
    acc = dot4(a.w, b.w, acc);
    return acc;
}

__device__ __forceinline__ u32x4 lo_nibbles(const u32x4& v) { return v & kNib; }
__device__ __forceinline__ u32x4 hi_nibbles(const u32x4& v) { return (v >> 4) & kNib; }

// acc[mi] += dot(weight unit held in p, quantized x unit `unit` of row mi)
template <int QT, int MT>
__device__ __forceinline__ void multiply_panel(const Panel<QT>& p, const XLds<QT>& l, int unit,
                                               int k_units, float (&acc)[MT]) {
    if (QT == QMM_Q4_K) {
        const float d = qmm_f16_bits_to_f32((uint16_t)(p.hdr.x & 0xffffu));
        const float dmin = qmm_f16_bits_to_f32((uint16_t)(p.hdr.x >> 16));
        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
        qmm_unpack_q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        u32x4 lo[8], hi[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            lo[c] = lo_nibbles(p.q[c]);
            hi[c] = hi_nibbles(p.q[c]);
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const int item = mi * k_units + unit;
            const uint4* xq = reinterpret_cast<const uint4*>(l.xq + (size_t)item * kXUnitStride);
            int isum = 0;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                int dlo = dot16(lo[2 * g], xq[4 * g], 0);
                dlo = dot16(lo[2 * g + 1], xq[4 * g + 1], dlo);
                int dhi = dot16(hi[2 * g], xq[4 * g + 2], 0);
                dhi = dot16(hi[2 * g + 1], xq[4 * g + 3], dhi);
                isum += (int)qmm_byte_of(sc_lo, sc_hi, 2 * g) * dlo;
                isum += (int)qmm_byte_of(sc_lo, sc_hi, 2 * g + 1) * dhi;
            }
            const int4* bs = reinterpret_cast<const int4*>(l.xbs + item * 8);
            int4 b0 = bs[0], b1 = bs[1];
            int msum = (int)qmm_byte_of(mn_lo, mn_hi, 0) * b0.x + (int)qmm_byte_of(mn_lo, mn_hi, 1) * b0.y +
                       (int)qmm_byte_of(mn_lo, mn_hi, 2) * b0.z + (int)qmm_byte_of(mn_lo, mn_hi, 3) * b0.w +
                       (int)qmm_byte_of(mn_lo, mn_hi, 4) * b1.x + (int)qmm_byte_of(mn_lo, mn_hi, 5) * b1.y +
                       (int)qmm_byte_of(mn_lo, mn_hi, 6) * b1.z + (int)qmm_byte_of(mn_lo, mn_hi, 7) * b1.w;
            const float dx = l.xd[item];
            acc[mi] += (d * dx) * (float)isum - (dmin * dx) * (float)msum;
        }
    } else {
        const uint32_t hw[4] = {p.hdr.x, p.hdr.y, p.hdr.z, p.hdr.w};
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const int item = mi * k_units + unit;
            const uint4* xq = reinterpret_cast<const uint4*>(l.xq + (size_t)item * kXUnitStride);
            const float4* xd = reinterpret_cast<const float4*>(l.xd + item * 8);
            const float4 xd0 = xd[0], xd1 = xd[1];
            const float dxs[8] = {xd0.x, xd0.y, xd0.z, xd0.w, xd1.x, xd1.y, xd1.z, xd1.w};
#pragma unroll
            for (int b = 0; b < 8; b++) {
                int sumi = dot16(p.q[2 * b], xq[2 * b], 0);
                sumi = dot16(p.q[2 * b + 1], xq[2 * b + 1], sumi);
                float dw = qmm_f16_bits_to_f32((uint16_t)((hw[b >> 1] >> (16 * (b & 1))) & 0xffffu));
                acc[mi] += ((float)sumi * dw) * dxs[b];
            }
        }
    }
}

struct GemvParams {
    const uint8_t* w;  // tiled matrix (expert 0 of a stack)
    const uint8_t* w2; // gated form only: the second stack ("up"), same layout as w
    const float* x;    // [m, k]            (grouped: [tokens, k] or [pairs, k])
    float* y;          // [m, n]            (grouped: [pairs, n])
    int64_t m, n, k;
    int k_units, k_groups, s, slots;
    int64_t row_tiles, panel_bytes, matrix_bytes;
    int nwk; // waves splitting k (1, 2 or 4); 4 / nwk row-tiles are processed side by side
    // grouped (expert) mode when perm != nullptr: blockIdx.y is a segment of up
    // to 4 sorted pairs that share one expert
    const int32_t* perm;
    const int32_t* offsets;     // [n_experts + 1]
    const int32_t* seg_offsets; // [n_experts + 1], segments of 4 pairs per expert
    int n_experts;
    int x_div; // x row of pair p is p / x_div
};

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// MT rows per pass; GATED: two weight stacks share x and the result is
// silu(w x) * (w2 x) (the expert MLP's gate/up pair).
template <int QT, int MT, bool GATED>
__global__ __launch_bounds__(kWgThreads) void gemv_kernel(GemvParams P) {
    constexpr int G = GATED ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const XLds<QT> l = carve<QT, MT, G>(smem, P.k_units);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwk = P.nwk, nwr = kWaves / nwk;
    const int wk = wave % nwk, wr = wave / nwk;
    const int kpw = (P.k_groups + nwk - 1) / nwk; // k-steps per row-tile for every wave
    const int64_t rt_groups = (P.row_tiles + nwr - 1) / nwr;
    const int64_t n_it =
        blockIdx.x < rt_groups ? (rt_groups - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int64_t total = n_it * kpw;
    const bool lane_active = lane < P.slots;
    const int us = lane >> 4;

    // rows this block works on
    const bool grouped = P.perm != nullptr;
    int64_t m_begin = 0, m_end = P.m;
    const uint8_t* wbase = P.w;
    const uint8_t* wbase2 = P.w2;
    if (grouped) {
        const int seg = blockIdx.y;
        if (seg >= P.seg_offsets[P.n_experts]) return; // uniform for the block
        int lo = 0, hi = P.n_experts; // last e with seg_offsets[e] <= seg
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (P.seg_offsets[mid] <= seg) lo = mid;
            else hi = mid;
        }
        m_begin = P.offsets[lo] + (int64_t)(seg - P.seg_offsets[lo]) * 4;
        m_end = min((int64_t)P.offsets[lo + 1], m_begin + 4);
        wbase += (int64_t)lo * P.matrix_bytes;
        if (GATED) wbase2 += (int64_t)lo * P.matrix_bytes;
    }

    auto item_panel = [&](int64_t i, int64_t& rt, int& kg) -> bool {
        int64_t it = i / kpw;
        kg = (int)(i - it * kpw) * nwk + wk;
        rt = (it * gridDim.x + blockIdx.x) * nwr + wr;
        return i < total && rt < P.row_tiles && kg < P.k_groups;
    };
    auto fetch = [&](Panel<QT> (&p)[G], int64_t i) {
        int64_t rt;
        int kg;
        bool ok = item_panel(i, rt, kg);
        int64_t off = ok ? (rt * P.k_groups + kg) * P.panel_bytes : 0;
        load_panel<QT>(p[0], wbase + off, P.slots, lane, ok && lane_active);
        if (GATED) load_panel<QT>(p[G - 1], wbase2 + off, P.slots, lane, ok && lane_active);
    };

    for (int64_t m0 = m_begin; m0 < m_end; m0 += MT) {
        Panel<QT> pa[G], pb[G];
        fetch(pa, 0); // weight loads fly while the activations are quantized
        if (m0 != m_begin) __syncthreads();
        quantize_rows_to_lds<QT, MT>(l, P.x, P.perm, P.x_div, m0, m_end, P.k, P.k_units);
        __syncthreads();

        float acc[G][MT];
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int mi = 0; mi < MT; mi++) acc[g][mi] = 0.0f;
        int red_buf = 0;

        auto step = [&](Panel<QT> (&cur)[G], Panel<QT> (&nxt)[G], int64_t i) {
            fetch(nxt, i + 1);
            int64_t rt;
            int kg;
            item_panel(i, rt, kg);
            int unit = min(kg * P.s + us, P.k_units - 1);
#pragma unroll
            for (int g = 0; g < G; g++) multiply_panel<QT, MT>(cur[g], l, unit, P.k_units, acc[g]);
            if ((i + 1) % kpw == 0) { // row-tile finished
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int mi = 0; mi < MT; mi++) {
                        acc[g][mi] += __shfl_xor(acc[g][mi], 16);
                        acc[g][mi] += __shfl_xor(acc[g][mi], 32);
                    }
                if (nwk == 1) {
                    int64_t row = rt * 16 + lane;
                    if (lane < 16 && rt < P.row_tiles && row < P.n) {
#pragma unroll
                        for (int mi = 0; mi < MT; mi++) {
                            if (m0 + mi < m_end) {
                                int64_t yr = grouped ? P.perm[m0 + mi] : m0 + mi;
                                float v = GATED ? silu(acc[0][mi]) * acc[G - 1][mi] : acc[0][mi];
                                P.y[yr * P.n + row] = v;
                            }
                        }
                    }
                } else {
                    float* red = l.red + red_buf * (kWaves * G * MT * 16);
                    if (lane < 16) {
#pragma unroll
                        for (int g = 0; g < G; g++)
#pragma unroll
                            for (int mi = 0; mi < MT; mi++)
                                red[((wave * G + g) * MT + mi) * 16 + lane] = acc[g][mi];
                    }
                    __syncthreads();
                    if (wk == 0 && lane < 16 * MT) {
                        int mi = lane >> 4, r = lane & 15;
                        float sum[G];
#pragma unroll
                        for (int g = 0; g < G; g++) {
                            sum[g] = 0.0f;
                            for (int w2 = 0; w2 < nwk; w2++)
                                sum[g] += red[(((wr * nwk + w2) * G + g) * MT + mi) * 16 + r];
                        }
                        int64_t row = rt * 16 + r;
                        if (rt < P.row_tiles && row < P.n && m0 + mi < m_end) {
                            int64_t yr = grouped ? P.perm[m0 + mi] : m0 + mi;
                            P.y[yr * P.n + row] = GATED ? silu(sum[0]) * sum[G - 1] : sum[0];
                        }
                    }
                    red_buf ^= 1;
                }
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int mi = 0; mi < MT; mi++) acc[g][mi] = 0.0f;
            }
        };

        int64_t i = 0;
        for (; i + 1 < total; i += 2) {
            step(pa, pb, i);
            step(pb, pa, i + 1);
        }
        if (i < total) step(pa, pb, i);
    }
}

template <int QT, int MT, bool GATED>
hipError_t launch_mt(const GemvParams& P, int n_cus, int grid_y, hipStream_t stream) {
    size_t lds = lds_bytes<QT, MT, GATED ? 2 : 1>(P.k_units);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(
            reinterpret_cast<const void*>(&gemv_kernel<QT, MT, GATED>),
            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    const int nwr = kWaves / P.nwk;
    int64_t rt_groups = (P.row_tiles + nwr - 1) / nwr;
    int64_t cap = (int64_t)n_cus * 8;
    if (grid_y > 1) cap = cap / grid_y > 64 ? cap / grid_y : 64;
    int64_t grid = rt_groups < cap ? rt_groups : cap;
    if (grid < 1) grid = 1;
    gemv_kernel<QT, MT, GATED>
        <<<dim3((unsigned)grid, (unsigned)grid_y), dim3(kWgThreads), lds, stream>>>(P);
    return hipGetLastError();
}

template <int QT>
hipError_t launch_plain(GemvParams P, int n_cus, hipStream_t stream) {
    // the widest row tile whose quantized activations fit comfortably in LDS
    int mt = P.m >= 3 ? 4 : (P.m == 2 ? 2 : 1);
    if (mt == 4 && lds_bytes<QT, 4, 1>(P.k_units) > 64 * 1024) mt = 2;
    if (mt == 2 && lds_bytes<QT, 2, 1>(P.k_units) > 64 * 1024) mt = 1;
    if (mt == 4) return launch_mt<QT, 4, false>(P, n_cus, 1, stream);
    if (mt == 2) return launch_mt<QT, 2, false>(P, n_cus, 1, stream);
    return launch_mt<QT, 1, false>(P, n_cus, 1, stream);
}

GemvParams make_params(const QmmLayout& L, const void* tiled, const float* x, int64_t m, float* y) {
    GemvParams P;
    P.w = (const uint8_t*)tiled;
    P.w2 = nullptr;
    P.x = x;
    P.y = y;
    P.m = m;
    P.n = L.n;
    P.k = L.k;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.s = L.s;
    P.slots = L.slots;
    P.row_tiles = L.row_tiles;
    P.panel_bytes = L.panel_bytes;
    P.matrix_bytes = L.matrix_bytes;
    int nwk = 1;
    if (L.row_tiles < 4096) {
        if (L.k_groups >= 4) nwk = 4;
        else if (L.k_groups >= 2) nwk = 2;
    }
    P.nwk = nwk;
    P.perm = nullptr;
    P.offsets = nullptr;
    P.seg_offsets = nullptr;
    P.n_experts = 0;
    P.x_div = 1;
    return P;
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
    load16(x + mi * k, unit * 256 + 16 * j, k, true, v);
    uint32_t q[4];
    if (QT == QMM_Q4_K) {
        float d;
        int s16;
        quantize_q8k_lane(v, q, d, s16);
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
                           float* y, int n_cus, hipStream_t stream) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    GemvParams P = make_params(L, tiled, x, m, y);
    return L.dtype == QMM_Q4_K ? launch_plain<QMM_Q4_K>(P, n_cus, stream)
                               : launch_plain<QMM_Q8_0>(P, n_cus, stream);
}

hipError_t qmm_launch_gemv_grouped(const QmmLayout& L, const void* tiled, const void* tiled2,
                                   const float* x, int x_div, float* y, const int32_t* perm,
                                   const int32_t* offsets, const int32_t* seg_offsets,
                                   int n_experts, int64_t max_segments, int n_cus,
                                   hipStream_t stream) {
    if (max_segments <= 0 || L.n == 0) return hipSuccess;
    if (max_segments > 65535) return hipErrorInvalidValue;
    GemvParams P = make_params(L, tiled, x, 0, y);
    P.w2 = (const uint8_t*)tiled2;
    P.perm = perm;
    P.offsets = offsets;
    P.seg_offsets = seg_offsets;
    P.n_experts = n_experts;
    P.x_div = x_div;
    // many small matrices: keep the k-split inside a workgroup
    P.nwk = L.k_groups >= 4 ? 4 : (L.k_groups >= 2 ? 2 : 1);
    const bool gated = tiled2 != nullptr;
    if (L.dtype == QMM_Q4_K)
        return gated ? launch_mt<QMM_Q4_K, 4, true>(P, n_cus, (int)max_segments, stream)
                     : launch_mt<QMM_Q4_K, 4, false>(P, n_cus, (int)max_segments, stream);
    return gated ? launch_mt<QMM_Q8_0, 4, true>(P, n_cus, (int)max_segments, stream)
                 : launch_mt<QMM_Q8_0, 4, false>(P, n_cus, (int)max_segments, stream);
}

hipError_t qmm_launch_quantize_activations(int weight_dtype, const float* x, int64_t m, int64_t k,
                                           void* out_blocks, hipStream_t stream) {
    int64_t k_units = (k + 255) / 256;
    int64_t threads = m * k_units * 16;
    if (threads == 0) return hipSuccess;
    unsigned grid = (unsigned)((threads + 255) / 256);
    if (weight_dtype == QMM_Q4_K)
        quantize_export_kernel<QMM_Q4_K>
            <<<grid, 256, 0, stream>>>(x, m, k, k_units, (uint8_t*)out_blocks);
    else
        quantize_export_kernel<QMM_Q8_0>
            <<<grid, 256, 0, stream>>>(x, m, k, k_units, (uint8_t*)out_blocks);
    return hipGetLastError();
}
