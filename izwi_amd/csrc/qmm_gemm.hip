// Prefill kernel: y[m, n] = x[m, k] * dequant(W)[n, k]^T with bf16 MFMA.
//
// A workgroup (4 waves, 2 x 2) owns a BM x BN output tile (256 x 256 when the
// problem fills the chip with such tiles, smaller tiles otherwise); each wave
// a (BM/2) x (BN/2) sub-tile held in v_mfma_f32_32x32x16_bf16 accumulators.
// Per 64-wide k step the workgroup
//   * copies the BM x 64 bf16 activation tile to LDS,
//   * reads the matching 64 k-elements of BN weight rows straight from the
//     panel layout (header + nibble / int8 chunks), dequantizes them in
//     registers and writes bf16 to LDS,
//   * runs 4 k16 steps of MFMAs per wave, operands read from LDS as one
//     16-byte load per lane (row stride padded to 144 B: conflict free).
// LDS holds two such stages: while the MFMAs of step i run out of one, the
// tile of step i+1 (loaded to registers during step i-1) is dequantized into
// the other and the global loads of step i+2 are issued, with one barrier per
// step.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include <type_traits>
#include <utility>

#include "qmm_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kRowStride = 144; // bytes per LDS tile row: 64 bf16 + 16 B pad
#ifndef QMM_GEMM_VALU_PER_MFMA
#define QMM_GEMM_VALU_PER_MFMA 4
#endif

struct GemmParams {
    const uint8_t* w;
    const uint16_t* x; // bf16 [m, k]
    void* y;
    int64_t m, n, k;
    int64_t n_begin, n_end; // output columns (weight rows) of this launch, n_begin a multiple of 256
    int k_units, k_groups, s, slots;
    int64_t row_tiles, panel_bytes;
    int out_bf16;
    int tiles_m, tiles_n;
    // split-k form (blockIdx.y = slice): slice s covers units [s * slice_units, ..) of 256
    // k-elements and writes its f32 tile to partial[s][m][n]; a second kernel adds the slices
    // in order
    int slice_units;
    // 0x0f0f0f0f, passed as data: with the constant in the code the compiler folds mask and
    // byte select into one bit-field extract per weight, followed by a convert; with an unknown
    // mask it emits one AND per four weights and v_cvt_f32_ubyteN for each
    uint32_t nibble_mask;
    float* partial;
    const void* residual; // of y's type, added to the sums before they are stored (may alias y)
    // several weights of equal k and type on the same activations in one launch (pipelined tiles
    // only): column tile t of the grid belongs to weight i with tn_end[i - 1] <= t < tn_end[i];
    // w / y / n / n_end / row_tiles / partial above are replaced by the member's at kernel entry
    int n_weights; // 0 or 1: a single weight
    int tn_end[QMM_MAX_GROUP];
    const uint8_t* wv[QMM_MAX_GROUP];
    void* yv[QMM_MAX_GROUP];
    int64_t nv[QMM_MAX_GROUP], row_tiles_v[QMM_MAX_GROUP];
    float* partial_v[QMM_MAX_GROUP];
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {(__bf16)a, (__bf16)b}; // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(uint32_t, v);
}

// byte N of v as float (v_cvt_f32_ubyteN)
template <int N>
__device__ __forceinline__ float ubyte_f32(uint32_t v) {
    return (float)((v >> (8 * N)) & 0xffu);
}

// Quant chunks a thread holds for its share of one weight row and k step.
template <int QT, int TPR>
struct WRegs {
    static constexpr int NC = (QT == QMM_Q4_K ? 2 : 4) / TPR;
    u32x4 hdr;
    u32x4 q[NC];
    // Q6_K only (two threads per row): the 32 bytes of high bit pairs and the chunk with d
    u32x4 qh[2];
    u32x4 dch;
};

// Weight row `row`, k step kt (64 elements), part `part` of TPR: header + chunks.
template <int QT, int TPR>
__device__ __forceinline__ void load_w(WRegs<QT, TPR>& r, const GemmParams& P, int64_t row, int kt,
                                       int part) {
    constexpr int NC = WRegs<QT, TPR>::NC;
    const int unit = kt >> 2, sub = kt & 3;
    // branch-free: out-of-range rows / units read a valid address and are zeroed by a select
    // when the tile is written to LDS, so the k loop stays one basic block and loads, LDS
    // traffic and MFMAs can interleave
    const bool ok = (row >> 4) < P.row_tiles && unit < P.k_units;
    const int64_t rt = ok ? (row >> 4) : 0;
    const int u = ok ? unit : 0;
    const int kg = u / P.s, us = u - kg * P.s;
    const int slot = us * 16 + (int)(row & 15);
    const u32x4* base =
        reinterpret_cast<const u32x4*>(P.w + (rt * P.k_groups + kg) * P.panel_bytes) + slot;
    // (the select itself happens in store_w: applying it here would make every load wait)
    r.hdr = base[0];
    if (QT == QMM_Q6_K) {
        // the 64 elements of step `sub` are one nibble (sub & 1) of the 64 ql bytes of half
        // sub >> 1 and one bit pair of its 32 qh bytes; byte e of the 64 pairs with qh byte e % 32
        static_assert(QT != QMM_Q6_K || TPR == 2, "Q6_K tiles use two threads per weight row");
        const int h = sub >> 1;
#pragma unroll
        for (int c = 0; c < NC; c++) r.q[c] = base[(size_t)(1 + 4 * h + part * NC + c) * P.slots];
        r.qh[0] = base[(size_t)(9 + 2 * h) * P.slots];
        r.qh[1] = base[(size_t)(10 + 2 * h) * P.slots];
        r.dch = base[(size_t)13 * P.slots];
        return;
    }
#pragma unroll
    for (int c = 0; c < NC; c++) r.q[c] = base[(size_t)(1 + sub * NC * TPR + part * NC + c) * P.slots];
}

// Dequantizes the thread's share of the 64 k-elements to bf16 and writes it to the LDS row.
template <int QT, int TPR>
__device__ __forceinline__ void store_w(const WRegs<QT, TPR>& r, int kt, int part, bool ok,
                                        uint8_t* lds_row) {
    constexpr int NC = WRegs<QT, TPR>::NC;
    // This kernel's results are compared within a tolerance (bf16 operands), so the
    // dequantization may use fused multiply-adds and per-byte converts:
    // 1 convert + 1 fma + half a pack per weight.
    if (QT == QMM_Q4_K) {
        const int g = kt & 3;
        // a row or unit outside the matrix gets zero scales: every weight becomes 0, no branch
        const float d = ok ? qmm_f16_bits_to_f32((uint16_t)(r.hdr.x & 0xffffu)) : 0.0f;
        const float dmin = ok ? qmm_f16_bits_to_f32((uint16_t)(r.hdr.x >> 16)) : 0.0f;
        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
        qmm_unpack_q4k_scales(r.hdr.y, r.hdr.z, r.hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        const float d1 = d * (float)qmm_byte_of(sc_lo, sc_hi, 2 * g);
        const float m1 = -(dmin * (float)qmm_byte_of(mn_lo, mn_hi, 2 * g));
        const float d2 = d * (float)qmm_byte_of(sc_lo, sc_hi, 2 * g + 1);
        const float m2 = -(dmin * (float)qmm_byte_of(mn_lo, mn_hi, 2 * g + 1));
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int h = part * NC + c; // which 16-byte half of the 32 nibble bytes
            uint32_t lo[8], hi[8];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t vl = r.q[c][j] & 0x0f0f0f0fu, vh = (r.q[c][j] >> 4) & 0x0f0f0f0fu;
                lo[2 * j] = pack_bf16(__builtin_fmaf(d1, ubyte_f32<0>(vl), m1),
                                      __builtin_fmaf(d1, ubyte_f32<1>(vl), m1));
                lo[2 * j + 1] = pack_bf16(__builtin_fmaf(d1, ubyte_f32<2>(vl), m1),
                                          __builtin_fmaf(d1, ubyte_f32<3>(vl), m1));
                hi[2 * j] = pack_bf16(__builtin_fmaf(d2, ubyte_f32<0>(vh), m2),
                                      __builtin_fmaf(d2, ubyte_f32<1>(vh), m2));
                hi[2 * j + 1] = pack_bf16(__builtin_fmaf(d2, ubyte_f32<2>(vh), m2),
                                          __builtin_fmaf(d2, ubyte_f32<3>(vh), m2));
            }
            // low nibbles: k 16h .. 16h+15, high nibbles: k 32 + 16h ..
            uint4* dl = reinterpret_cast<uint4*>(lds_row + 32 * h);
            uint4* dh = reinterpret_cast<uint4*>(lds_row + 64 + 32 * h);
            dl[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            dl[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
            dh[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            dh[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        }
    } else if (QT == QMM_Q6_K) {
        // part p holds the elements 32 p .. 32 p + 31 of the step: nibble s1 of its two ql chunks,
        // bit pair 4 s1 + 2 p of the 32 qh bytes; the 16-element groups 4 sub + 2 p, + 1 carry
        // the scales.  w = d * scale * (q - 32) as one fma per weight.
        const int sub = kt & 3, s1 = sub & 1;
        const float d = ok ? qmm_f16_bits_to_f32((uint16_t)(r.dch.x & 0xffffu)) : 0.0f;
        const uint32_t hw[4] = {r.hdr.x, r.hdr.y, r.hdr.z, r.hdr.w};
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int j = 4 * sub + 2 * part + c;
            const float ds = d * (float)(int8_t)((hw[j >> 2] >> (8 * (j & 3))) & 0xffu);
            const float bias = -32.0f * ds;
            uint32_t o[8];
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t nib = (r.q[c][w] >> (4 * s1)) & 0x0f0f0f0fu;
                const uint32_t two = (r.qh[c][w] >> (4 * s1 + 2 * part)) & 0x03030303u;
                const uint32_t q6 = nib | (two << 4);
                o[2 * w] = pack_bf16(__builtin_fmaf(ds, ubyte_f32<0>(q6), bias),
                                     __builtin_fmaf(ds, ubyte_f32<1>(q6), bias));
                o[2 * w + 1] = pack_bf16(__builtin_fmaf(ds, ubyte_f32<2>(q6), bias),
                                         __builtin_fmaf(ds, ubyte_f32<3>(q6), bias));
            }
            uint4* dst = reinterpret_cast<uint4*>(lds_row + 64 * part + 32 * c);
            dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
            dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
        }
    } else {
        const int b0 = (kt & 3) * 2; // first of the two 32-element blocks of this k step
        const uint32_t hw[4] = {r.hdr.x, r.hdr.y, r.hdr.z, r.hdr.w};
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int cc = part * NC + c; // chunk 0..3 of the step: block cc / 2, half cc % 2
            const int b = b0 + (cc >> 1);
            const float d =
                ok ? qmm_f16_bits_to_f32((uint16_t)((hw[b >> 1] >> (16 * (b & 1))) & 0xffffu)) : 0.0f;
            const float bias = -128.0f * d; // int8 q as unsigned byte u = q + 128: q * d = u * d - 128 d
            uint32_t o[8];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t u = r.q[c][j] ^ 0x80808080u;
                o[2 * j] = pack_bf16(__builtin_fmaf(d, ubyte_f32<0>(u), bias),
                                     __builtin_fmaf(d, ubyte_f32<1>(u), bias));
                o[2 * j + 1] = pack_bf16(__builtin_fmaf(d, ubyte_f32<2>(u), bias),
                                         __builtin_fmaf(d, ubyte_f32<3>(u), bias));
            }
            uint4* dst = reinterpret_cast<uint4*>(lds_row + 32 * cc);
            dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
            dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
        }
    }
}

template <int QT, int BM, int BN>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmParams P) {
    constexpr int MT = BM / 64, NT = BN / 64; // 32x32 MFMA tiles per wave in m and n
    constexpr int XC = BM / 32;               // 16-byte activation chunks per thread and k step
    constexpr int TPR = kThreads / BN;        // threads sharing one weight row
    constexpr int kStage = (BM + BN) * kRowStride;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // consecutive workgroups walk down m inside one weight column block, so the
    // weight rows they share stay in L2 while all of m is swept
    const int tm = blockIdx.x % P.tiles_m;
    const int tn = blockIdx.x / P.tiles_m;
    const int64_t m0 = (int64_t)tm * BM, n0 = P.n_begin + (int64_t)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_steps = P.k_units * 4;
    const int w_row = tid % BN, w_part = tid / BN;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // activation tile: BM rows x 8 chunks of 16 B; thread t copies chunks t + 256 i
    u32x4 xr[XC];
    WRegs<QT, TPR> wr;
    // rows past m read row m-1 (their results are never stored); k is a multiple of 32, so a
    // 16-byte chunk is entirely inside or outside [0, k): outside chunks become zeros
    auto load_x = [&](int kt) {
#pragma unroll
        for (int i = 0; i < XC; i++) {
            const int c = tid + kThreads * i;
            const int row = c >> 3, kc = c & 7;
            const int64_t gm = min(m0 + row, P.m - 1);
            const int64_t gk = (int64_t)kt * BK + kc * 8;
            xr[i] = *reinterpret_cast<const u32x4*>(P.x + gm * P.k + (gk < P.k ? gk : 0));
        }
    };
    auto store_tile = [&](int kt, uint8_t* stage) {
#pragma unroll
        for (int i = 0; i < XC; i++) {
            const int c = tid + kThreads * i;
            const int row = c >> 3, kc = c & 7;
            const bool ok = (int64_t)kt * BK + kc * 8 < P.k;
            *reinterpret_cast<u32x4*>(stage + row * kRowStride + kc * 16) = ok ? xr[i] : u32x4{0, 0, 0, 0};
        }
        const bool w_ok = ((n0 + w_row) >> 4) < P.row_tiles && (kt >> 2) < P.k_units;
        store_w<QT, TPR>(wr, kt, w_part, w_ok, stage + (BM + w_row) * kRowStride);
    };
    auto load_tile = [&](int kt) {
        load_x(kt);
        load_w<QT, TPR>(wr, P, n0 + w_row, kt, w_part);
    };

    load_tile(0);
    store_tile(0, smem);
    if (k_steps > 1) load_tile(1);
    __syncthreads();

    // One k step: MFMAs out of `cur`; with FEED, the next step's tile (in registers since the
    // previous step) is dequantized into `next` and the loads of the step after are issued.
    // No branch inside, so the whole step is one basic block and the scheduler is free to
    // interleave LDS traffic, dequantization and global loads with the MFMAs.
    auto k_step = [&](int kt, const uint8_t* cur, uint8_t* next, auto feed) {
        constexpr bool FEED = decltype(feed)::value;
        const uint8_t* xs = cur;
        const uint8_t* ws = cur + BM * kRowStride;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int koff = kk * 32 + (lane >> 5) * 16; // bytes inside the tile row
            bf16x8 a[MT], b[NT];
#pragma unroll
            for (int i = 0; i < MT; i++)
                a[i] = *reinterpret_cast<const bf16x8*>(
                    xs + (wm * (BM / 2) + i * 32 + (lane & 31)) * kRowStride + koff);
#pragma unroll
            for (int j = 0; j < NT; j++)
                b[j] = *reinterpret_cast<const bf16x8*>(
                    ws + (wn * (BN / 2) + j * 32 + (lane & 31)) * kRowStride + koff);
#pragma unroll
            for (int i = 0; i < MT; i++)
#pragma unroll
                for (int j = 0; j < NT; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            if (FEED && kk == 0) {
                store_tile(kt + 1, next);
                load_tile(kt + 2); // past the end this reads a valid address and yields zeros
            }
        }
#ifdef QMM_GEMM_SCHED
        if (FEED) {
#pragma unroll
            for (int i = 0; i < MT * NT * 4; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, QMM_GEMM_SCHED, 0); // VALU
                if (i % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
                if (i % 4 == 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // DS write
                if (i % 5 == 3) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
            }
        }
#endif
        __syncthreads();
    };
    for (int kt = 0; kt + 1 < k_steps; kt++)
        k_step(kt, smem + (kt & 1) * kStage, smem + ((kt + 1) & 1) * kStage, std::true_type{});
    k_step(k_steps - 1, smem + ((k_steps - 1) & 1) * kStage, nullptr, std::false_type{});

    // D[i][j]: lane holds column j = lane % 32 and rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < MT; i++) {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const int64_t gn = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
            if (gn >= P.n_end) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t gm = m0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm >= P.m) continue;
                qmm_store(P.y, QmmEpilogue{P.residual, P.out_bf16}, gm * P.n + gn, acc[i][j][r]);
            }
        }
    }
}

// ---- software-pipelined variant (BN = 256: one weight row per thread) ----------------
// With one wave per SIMD nothing hides a wave's own non-matrix work, so the next tile's
// staging (dequantization, LDS writes, global loads) is cut into slices and one slice
// is placed after every group of four MFMAs; scheduling fences keep the slices there.
// The MFMA pipe then drains its queue while the VALU / LDS / memory slices issue.
template <int N, class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
}

// Pipelined 256-column tile.  The k loop runs over units of 256 k-elements with the four
// 64-wide steps of a unit unrolled, so that the sub-block index, the LDS stage and the
// chunk offsets inside the panel are compile-time constants; whatever depends on the
// step otherwise (unit offset inside the panel row, activation column) is uniform and
// stays in scalar registers, the per-lane part of every address is a 32-bit offset
// computed once.  XTAIL: k is not a multiple of 64 (Q8_0 only), activation chunks at or
// past k are zeroed on their way to LDS.
template <int QT, int BM, int BN, bool XTAIL, int NW = 4>
__global__ __launch_bounds__(64 * NW) void gemm_pipe_kernel(GemmParams P_in) {
    GemmParams P = P_in;
    int tn_local = (int)(blockIdx.x / P_in.tiles_m);
    if (P_in.n_weights > 1) { // a projection group: this workgroup's member (uniform)
        int i = 0;
        while (i + 1 < P_in.n_weights && tn_local >= P_in.tn_end[i]) i++;
        tn_local -= i ? P_in.tn_end[i - 1] : 0;
        P.w = P_in.wv[i];
        P.y = P_in.yv[i];
        P.n = P.n_end = P_in.nv[i];
        P.row_tiles = P_in.row_tiles_v[i];
        P.partial = P_in.partial ? P_in.partial_v[i] : nullptr;
    }
    // NW waves as a (NW / 2) x 2 grid of wave tiles; with eight waves two share a SIMD, each with
    // half the accumulators, and one issues while the other waits
    constexpr int THREADS = 64 * NW, WM = NW / 2;
    constexpr int MT = BM / WM / 32, NT = BN / 64;       // 32 x 32 accumulator tiles per wave
    constexpr int XC = BM * 8 / THREADS;                 // 16-byte activation chunks per thread and k step
    constexpr int TPR = THREADS / BN;                    // threads that share a weight row: 1, 2 or 4
    constexpr bool Q6 = QT == QMM_Q6_K;
    static_assert(!Q6 || TPR == 2 || TPR == 4, "Q6_K is staged by two or four threads per weight row");
    constexpr int NCR = QT == QMM_Q4_K ? 2 : 4;          // 16-byte quant chunks per row and k step
    // Q6_K: a half unit (two k steps) shares its 64 bytes of low nibbles and 32 bytes of bit pairs.
    // A thread takes 16 of the 32 byte positions (the half `lh` = part & 1) in both 32-element groups
    // of a step (two parts per row) or in one of them (four parts): NQL dwords of nibbles, NQH of
    // bit pairs, held for both steps
    constexpr int NGG = 4 / TPR, NQL = 4 * NGG, NQH = 4;
    constexpr int ND = Q6 ? NQL + NQH : 4 * NCR / TPR;   // the thread's run of quant dwords: 2 .. 16
    constexpr int NC = Q6 ? NGG : ND >= 4 ? ND / 4 : 1; // loads per thread and k step (16 bytes; 8 if ND = 2)
    constexpr int NP = 16 / TPR;                         // pieces of four weights per thread and k step
    constexpr int GPK = MT * NT / 4; // groups of four MFMAs per k16 step
    constexpr int NG = 4 * GPK;      // groups per k step: 16 (BM = 256) or 8 (BM = 128)
    constexpr int kStage = (BM + BN) * kRowStride;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tm = blockIdx.x % P.tiles_m;
    const int tn = tn_local;
    const int64_t m0 = (int64_t)tm * BM, n0 = P.n_begin + (int64_t)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int u0 = P.partial ? (int)blockIdx.y * P.slice_units : 0;             // first unit of this workgroup
    const int u1 = P.partial ? min(P.k_units, u0 + P.slice_units) : P.k_units;  // one past its last
    const int last_step = P.k_units * 4 - 1;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // ---- staging state: tile kt+1 sits in xr / wr while step kt runs
    // activation chunks in flight: tile kt+1 (written to LDS during step kt) and, where the
    // register file allows, tile kt+2 behind it, so that a chunk is requested XD k steps
    // before it is needed
    constexpr int XD = BN == 128 ? 2 : 1;
    u32x4 xr[XD][XC];
    u32x4 w_hdr;      // header of the unit fetched last (Q6_K: its 16 signed scales)
    uint32_t w_d = 0; // Q6_K: the dword with d of that unit
    // quant dwords of tile kt+1 (being dequantized) and tile kt+2 (in flight), by parity of the k step
    // (Q6_K: of the half unit; low nibbles first, bit pairs behind them)
    uint32_t wq[2][ND];
    // activations: uniform tile base + uniform column + per-lane (row, chunk) offset
    const uint8_t* x_tile = reinterpret_cast<const uint8_t*>(P.x) + m0 * P.k * 2;
    uint32_t x_off[XC];
    int x_lds[XC];
#pragma unroll
    for (int i = 0; i < XC; i++) {
        const int c = tid + THREADS * i;
        const int row = c >> 3, kc = c & 7;
        x_off[i] = (uint32_t)((min(m0 + row, P.m - 1) - m0) * P.k * 2 + kc * 16);
        x_lds[i] = row * kRowStride + kc * 16;
    }
    // weights: thread t stages part t / BN of row n0 + t % BN (the lanes of a wave write 64
    // different rows of the padded LDS tile: no bank conflicts, and the part is wave-uniform);
    // rows past the matrix read the last row-tile (their output columns are never stored)
    const int w_row = tid % BN, w_part = tid / BN;
    const int64_t rt0 = n0 >> 4;
    const int64_t rowtile_bytes = (int64_t)P.k_groups * P.panel_bytes;
    const uint8_t* w_tile = P.w + rt0 * rowtile_bytes;
    const uint32_t slot_bytes = (uint32_t)P.slots * 16u;
    const uint32_t w_off =
        (uint32_t)((min(rt0 + (w_row >> 4), P.row_tiles - 1) - rt0) * rowtile_bytes) + (uint32_t)(w_row & 15) * 16u;
    // part p holds dwords p ND .. p ND + ND - 1 of the row's quant dwords of a step (Q4_K: 8
    // dwords of nibbles, dword D = elements 4 D .. (low) and 32 + 4 D .. (high); Q8_0: 16 dwords of
    // int8): its first chunk (and, for half a chunk, the offset inside it) and its LDS position
    const int w_d0 = Q6 ? 0 : w_part * ND;
    const uint32_t w_off_q = w_off + (uint32_t)(w_d0 / 4) * slot_bytes + (uint32_t)(w_d0 % 4) * 4u;
    // Q6_K: element 32 gg + l of the k step with nibble `nib` of half unit h is nibble `nib` of
    // ql[64 h + 32 gg + l] with bit pair 2 nib + gg of qh[32 h + l]; its 16-element group is
    // 4 (2 h + nib) + 2 gg + l / 16.  Part p: l = 16 lh .., lh = p & 1; gg = 0 and 1 (two parts)
    // or p / 2 (four parts)
    const int q6_lh = w_part & 1, q6_gg = TPR == 4 ? w_part >> 1 : 0;
    const uint32_t w_off_ql = w_off + (uint32_t)(2 * q6_gg + q6_lh) * slot_bytes;
    const uint32_t w_off_qh = w_off + (uint32_t)q6_lh * slot_bytes;
    const int q6_pair_shift = 2 * q6_gg;
    const int q6_scale_shift = 8 * (2 * q6_gg + q6_lh); // of the step's four scale bytes
    const int w_lds = (BM + w_row) * kRowStride + (Q6 ? 32 * w_part : w_d0 * 8);
    // load cursor: the unit whose chunks are fetched next (clamped to the last unit)
    int cur_us = u0 < P.k_units ? u0 % P.s : 0;
    uint32_t cur_kg_off = (uint32_t)((u0 < P.k_units ? u0 / P.s : 0) * P.panel_bytes);
    int cur_unit = min(u0, P.k_units - 1);
    auto advance_cursor = [&]() {
        if (cur_unit + 1 < P.k_units) {
            cur_unit++;
            cur_us++;
            if (cur_us == P.s) cur_us = 0, cur_kg_off += (uint32_t)P.panel_bytes;
        }
    };

    auto x_load = [&](int kt, int buf, int i) {
        if (XTAIL) {
            // chunks at or past k read chunk 0 of the row; x_write turns them into zeros
            const bool ok = (int64_t)kt * BK + (tid & 7) * 8 < P.k;
            xr[buf][i] = *reinterpret_cast<const u32x4*>(x_tile + (ok ? (int64_t)kt * (BK * 2) : -(int64_t)((tid & 7) * 16)) + x_off[i]);
        } else {
            xr[buf][i] = *reinterpret_cast<const u32x4*>(x_tile + (size_t)min(kt, last_step) * (BK * 2) + x_off[i]);
        }
    };
    auto x_write = [&](int kt, int buf, int i, uint8_t* stage) {
        if (XTAIL) {
            const bool ok = (int64_t)kt * BK + (tid & 7) * 8 < P.k;
            *reinterpret_cast<u32x4*>(stage + x_lds[i]) = ok ? xr[buf][i] : u32x4{0, 0, 0, 0};
        } else {
            *reinterpret_cast<u32x4*>(stage + x_lds[i]) = xr[buf][i];
        }
    };
    auto w_load_hdr = [&]() {
        w_hdr = *reinterpret_cast<const u32x4*>(w_tile + (cur_kg_off + (uint32_t)cur_us * 256u) + w_off);
        if constexpr (Q6)
            w_d = *reinterpret_cast<const uint32_t*>(w_tile + (cur_kg_off + (uint32_t)cur_us * 256u + 13u * slot_bytes) + w_off);
    };
    // Q6_K: the low nibbles of the thread's group c (HI = 0) or its bit pairs (HI = 1, c = 0) of half
    // unit HALF of the cursor's unit
    auto w_load_q6 = [&](auto HALF, auto HI, int c) {
        constexpr int half = decltype(HALF)::value, hi = decltype(HI)::value;
        const uint8_t* src = w_tile +
                             (cur_kg_off + (uint32_t)cur_us * 256u + (uint32_t)(hi ? 9 + 2 * half : 1 + 4 * half + 2 * c) * slot_bytes) +
                             (hi ? w_off_qh : w_off_ql);
        const u32x4 v = *reinterpret_cast<const u32x4*>(src);
        constexpr int o = hi ? NQL : 0;
        wq[half][o + 4 * c] = v.x, wq[half][o + 4 * c + 1] = v.y, wq[half][o + 4 * c + 2] = v.z, wq[half][o + 4 * c + 3] = v.w;
    };
    auto w_load_q = [&](int sub, int c) {
        const uint8_t* src =
            w_tile + (cur_kg_off + (uint32_t)cur_us * 256u + (uint32_t)(1 + sub * NCR + c) * slot_bytes) + w_off_q;
        if constexpr (ND >= 4) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(src);
            wq[sub & 1][4 * c] = v.x, wq[sub & 1][4 * c + 1] = v.y, wq[sub & 1][4 * c + 2] = v.z, wq[sub & 1][4 * c + 3] = v.w;
        } else {
            const uint2 v = *reinterpret_cast<const uint2*>(src);
            wq[sub & 1][0] = v.x, wq[sub & 1][1] = v.y;
        }
    };
    // header of the unit being staged, unpacked once per unit
    float hd = 0, hdmin = 0;                            // Q4_K: d, dmin
    uint32_t sc_lo = 0, sc_hi = 0, mn_lo = 0, mn_hi = 0; // Q4_K: 8 scale bytes, 8 min bytes; Q8_0: 8 f16 scales
    auto w_unpack = [&]() {
        if (QT == QMM_Q4_K) {
            hd = qmm_f16_bits_to_f32((uint16_t)(w_hdr.x & 0xffffu));
            hdmin = -qmm_f16_bits_to_f32((uint16_t)(w_hdr.x >> 16));
            qmm_unpack_q4k_scales(w_hdr.y, w_hdr.z, w_hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        } else if (Q6) {
            hd = qmm_f16_bits_to_f32((uint16_t)(w_d & 0xffffu));
            sc_lo = w_hdr.x, sc_hi = w_hdr.y, mn_lo = w_hdr.z, mn_hi = w_hdr.w; // scales 4 sub .. 4 sub + 3 in dword sub
        } else {
            sc_lo = w_hdr.x, sc_hi = w_hdr.y, mn_lo = w_hdr.z, mn_hi = w_hdr.w;
        }
    };
    // scales of the tile being staged
    float sa = 0, ba = 0, sb = 0, bb = 0; // Q4_K: (d1, -m1, d2, -m2); Q8_0: (dA, -128 dA, dB, -128 dB)
    float sw = 0, bw = 0;                 // Q8_0, two threads per row: the scale of this thread's block
    auto w_scales = [&](auto SUB) {
        constexpr int g = decltype(SUB)::value;
        if (QT == QMM_Q4_K) {
            const uint32_t sc = g < 2 ? sc_lo : sc_hi, mn = g < 2 ? mn_lo : mn_hi;
            sa = hd * ubyte_f32<(2 * g) & 3>(sc);
            ba = hdmin * ubyte_f32<(2 * g) & 3>(mn);
            sb = hd * ubyte_f32<(2 * g + 1) & 3>(sc);
            bb = hdmin * ubyte_f32<(2 * g + 1) & 3>(mn);
        } else if (Q6) {
            // the thread's 16-element group(s) of the step: w = d scale (q - 32)
            const uint32_t four = g == 0 ? sc_lo : g == 1 ? sc_hi : g == 2 ? mn_lo : mn_hi;
            sa = hd * (float)(int8_t)(four >> q6_scale_shift);
            ba = -32.0f * sa;
            if (TPR == 2) { // the same byte positions of the step's second 32-element group
                sb = hd * (float)(int8_t)(four >> (q6_scale_shift + 16));
                bb = -32.0f * sb;
            }
        } else {
            const uint32_t pair = g == 0 ? sc_lo : g == 1 ? sc_hi : g == 2 ? mn_lo : mn_hi; // blocks 2g, 2g + 1
            sa = qmm_f16_bits_to_f32((uint16_t)(pair & 0xffffu));
            sb = qmm_f16_bits_to_f32((uint16_t)(pair >> 16));
            ba = -128.0f * sa;
            bb = -128.0f * sb;
            sw = (w_d0 / 8) ? sb : sa; // the thread's dwords lie in one block of 8 dwords
            bw = -128.0f * sw;
        }
    };
    const uint32_t nibble_mask = P.nibble_mask;
    uint32_t stash[4]; // finished bf16 pairs waiting for their 16-byte LDS write
    // piece H of NP of the tile with sub-block parity PAR: four of the thread's weights (Q4_K: the
    // low or the high nibbles of one dword; Q8_0: one dword), converted and, every other piece,
    // written as 16 bytes
    auto w_piece = [&](auto NSUB, auto HH, uint8_t* stage) {
        constexpr int par = decltype(NSUB)::value & 1, h = decltype(HH)::value;
        uint8_t* row = stage + w_lds;
        if constexpr (Q6) {
            // dword h % 4 of the thread's 16 byte positions in its group h / 4: four elements
            constexpr int half = decltype(NSUB)::value >> 1, nib = par, gi = h / 4, dw = h % 4;
            const uint32_t v = wq[half][h], vh = wq[half][NQL + dw];
            const uint32_t q4 = (nib ? v >> 4 : v) & nibble_mask;
            const uint32_t two = (vh >> (4 * nib + 2 * gi + q6_pair_shift)) & 0x03030303u;
            const uint32_t q6 = q4 | (two << 4);
            const float sc = gi ? sb : sa, bi = gi ? bb : ba;
            constexpr int o = (h % 2) * 2;
            stash[o] = pack_bf16(__builtin_fmaf(sc, ubyte_f32<0>(q6), bi), __builtin_fmaf(sc, ubyte_f32<1>(q6), bi));
            stash[o + 1] = pack_bf16(__builtin_fmaf(sc, ubyte_f32<2>(q6), bi), __builtin_fmaf(sc, ubyte_f32<3>(q6), bi));
            if (h % 2) *reinterpret_cast<uint4*>(row + 64 * gi + 16 * (dw / 2)) = make_uint4(stash[0], stash[1], stash[2], stash[3]);
        } else if constexpr (QT == QMM_Q4_K) {
            // the thread's dword pair pp: low nibbles of both dwords, then high nibbles of both
            constexpr int pp = h / 4, hi = (h % 4) / 2;
            const uint32_t v = wq[par][2 * pp + (h % 2)];
            const uint32_t q4 = (hi ? v >> 4 : v) & nibble_mask;
            const float sc = hi ? sb : sa, bi = hi ? bb : ba;
            constexpr int o = (h % 2) * 2;
            stash[o] = pack_bf16(__builtin_fmaf(sc, ubyte_f32<0>(q4), bi), __builtin_fmaf(sc, ubyte_f32<1>(q4), bi));
            stash[o + 1] = pack_bf16(__builtin_fmaf(sc, ubyte_f32<2>(q4), bi), __builtin_fmaf(sc, ubyte_f32<3>(q4), bi));
            if (h % 2) // low nibbles: k 8 (d0 / 2 + pp) .., high nibbles: 32 elements further
                *reinterpret_cast<uint4*>(row + 64 * hi + 16 * pp) = make_uint4(stash[0], stash[1], stash[2], stash[3]);
        } else {
            // the thread's dword h: block (d0 + h) / 8 of the step
            float d, bias;
            if (TPR == 1) d = (h >> 3) ? sb : sa, bias = (h >> 3) ? bb : ba;
            else d = sw, bias = bw;
            const uint32_t u = wq[par][h] ^ 0x80808080u;
            constexpr int o = (h % 2) * 2;
            stash[o] = pack_bf16(__builtin_fmaf(d, ubyte_f32<0>(u), bias), __builtin_fmaf(d, ubyte_f32<1>(u), bias));
            stash[o + 1] = pack_bf16(__builtin_fmaf(d, ubyte_f32<2>(u), bias), __builtin_fmaf(d, ubyte_f32<3>(u), bias));
            if (h % 2) *reinterpret_cast<uint4*>(row + 16 * (h / 2)) = make_uint4(stash[0], stash[1], stash[2], stash[3]);
        }
    };

    // Operand fragments of one k16 step, two sets: the MFMAs of step kk read set kk & 1 while
    // the other set is filled.  A group of four MFMAs uses one row fragment and all column
    // fragments, so the column fragments are fetched first.
    bf16x8 fa[2][MT], fb[2][NT];
    const int frag_x = (wm * (BM / WM) + (lane & 31)) * kRowStride + (lane >> 5) * 16;
    const int frag_w = (BM + wn * (BN / 2) + (lane & 31)) * kRowStride + (lane >> 5) * 16;
    // part gi of GPK: read while group gi runs, used from group gi of the next k16 step on
    auto read_frags = [&](const uint8_t* stage, int kk, int set, auto PART) {
        constexpr int part = decltype(PART)::value;
        constexpr int jb = GPK == 1 ? 0 : NT == 4 ? (part < GPK / 2 ? part * 2 * NT / GPK : NT) : (part == 0 ? 0 : NT);
        constexpr int je = GPK == 1 ? NT : NT == 4 ? (part < GPK / 2 ? (part + 1) * 2 * NT / GPK : NT) : NT;
        constexpr int ib = GPK == 1 ? 0 : NT == 4 ? (part < GPK / 2 ? 0 : (part - GPK / 2) * 2 * MT / GPK) : (part == 0 ? 0 : MT / 2);
        constexpr int ie = GPK == 1 ? MT : NT == 4 ? (part < GPK / 2 ? 0 : (part - GPK / 2 + 1) * 2 * MT / GPK) : (part == 0 ? MT / 2 : MT);
#pragma unroll
        for (int j = jb; j < je; j++)
            fb[set][j] = *reinterpret_cast<const bf16x8*>(stage + frag_w + j * 32 * kRowStride + kk * 32);
#pragma unroll
        for (int i = ib; i < ie; i++)
            fa[set][i] = *reinterpret_cast<const bf16x8*>(stage + frag_x + i * 32 * kRowStride + kk * 32);
    };

    // One k step: MFMAs out of stage SUB & 1; between them tile kt+1 goes from registers to the
    // other stage (first three quarters of the step), tile kt+2 is fetched, and after the
    // step's only barrier, which follows the last fragment reads of this stage and the last
    // writes to the other one, the first fragments of step kt+1 are read while the last quarter
    // of the MFMAs runs.  Steps past the workgroup's last one stage and fetch the (clamped) last
    // tile again: nobody uses it.
    auto k_step = [&](int unit, auto SUB) {
        constexpr int sub = decltype(SUB)::value;
        constexpr int nsub = (sub + 1) & 3, lsub = (sub + 2) & 3; // sub-block staged / fetched meanwhile
        const int kt = unit * 4 + sub;
        const uint8_t* cur = smem + (sub & 1) * kStage;
        uint8_t* next = smem + ((sub + 1) & 1) * kStage;
        static_for<4>([&](auto KK) {
            constexpr int kk = decltype(KK)::value;
            static_for<GPK>([&](auto GI) {
                constexpr int gi = decltype(GI)::value;
                constexpr int g = kk * GPK + gi;
                // the operands of the next k16 step (of the next k step in the last quarter)
                read_frags(kk < 3 ? cur : next, (kk + 1) & 3, (kk + 1) & 1, GI);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int t = gi * 4 + q, i = t / NT, j = t % NT;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
                }
                // group g's share of staging tile kt+1 (the thread's NP weight pieces and XC
                // activation chunks over the first 3 NG / 4 groups) and of fetching tile kt+2
                constexpr int NGS = 3 * NG / 4;
                constexpr int p0 = (NP * g + NGS - 1) / NGS, p1 = g < NGS ? (NP * (g + 1) + NGS - 1) / NGS : p0;
                constexpr int c0 = (XC * g + NGS - 1) / NGS, c1 = g < NGS ? (XC * (g + 1) + NGS - 1) / NGS : c0;
                constexpr int l0 = g == 0 ? 0 : (XC * (g - 1) + NGS - 1) / NGS, l1 = g == 0 ? 0 : c0; // chunks written a group ago
                if (g == 0) {
                    if (sub == 3) w_unpack(); // tile kt+1 opens the next unit: its header arrived a step ago
                    w_scales(std::integral_constant<int, nsub>{});
                }
                static_for<p1 - p0>([&](auto PI) {
                    w_piece(std::integral_constant<int, nsub>{},
                            std::integral_constant<int, (p0 + decltype(PI)::value) % NP>{}, next);
                });
                constexpr int xbuf = (sub + 1) % XD; // registers of tile kt+1, refilled with tile kt+1+XD
#pragma unroll
                for (int i = c0; i < c1; i++) x_write(kt + 1, xbuf, i, next);
#pragma unroll
                for (int i = l0; i < (g <= NGS ? l1 : l0); i++) x_load(kt + 1 + XD, xbuf, i);
                // Q6_K fetches by half units, a step earlier: step 1 requests the low nibbles of the
                // next unit's first half, step 2 its bit pairs, step 3 the low nibbles of the second
                // half and step 0 (of that unit) its bit pairs; each half is complete one step before
                // its first tile is dequantized
                if (g == 1 && sub == (Q6 ? 1 : 2)) advance_cursor();
                if (g == 1 && sub == 2) w_load_hdr();
                if (g >= 2 && g < 2 + NC) {
                    if constexpr (!Q6) w_load_q(lsub, g - 2);
                    else if constexpr (sub % 2 == 1 || g == 2)
                        w_load_q6(std::integral_constant<int, (sub == 0 || sub == 3) ? 1 : 0>{},
                                  std::integral_constant<int, (sub % 2 == 0) ? 1 : 0>{}, g - 2);
                }
                // inside the group: one MFMA, then its share of the other instructions, so
                // the matrix pipe is fed while they issue
                constexpr int valu = (Q6 ? 4 : 3) * (p1 - p0) + (g == 0 ? 4 : 1);
                constexpr int reads = GPK == 1 ? NT + MT : NT == 4 ? (gi < GPK / 2 ? 2 * NT / GPK : 2 * MT / GPK) : (gi == 0 ? NT + MT / 2 : MT / 2);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, valu, 0);
                    if (q == 0) __builtin_amdgcn_sched_group_barrier(0x100, (reads + 1) / 2, 0);
                    if (q == 1) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
                    if (q == 2) __builtin_amdgcn_sched_group_barrier(0x100, reads / 2, 0);
                    if (q == 3) __builtin_amdgcn_sched_group_barrier(0x200, 3, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if (kk == 2) {
                // this stage's fragments are all in registers, the other stage is complete
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
        });
    };

    if (u0 < u1) {
        // ---- prologue: tile (u0, 0) -> stage 0, tile (u0, 1) -> registers
#pragma unroll
        for (int i = 0; i < XC; i++) x_load(u0 * 4, 0, i);
        w_load_hdr();
#pragma unroll
        for (int c = 0; c < NC; c++) {
            if constexpr (Q6) {
                w_load_q6(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, c);
                if (c == 0) w_load_q6(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, 0);
            } else {
                w_load_q(0, c);
            }
        }
#pragma unroll
        for (int i = 0; i < XC; i++) x_write(u0 * 4, 0, i, smem);
        w_unpack();
        w_scales(std::integral_constant<int, 0>{});
        static_for<NP>([&](auto HH) { w_piece(std::integral_constant<int, 0>{}, HH, smem); });
#pragma unroll
        for (int d = 1; d <= XD; d++)
#pragma unroll
            for (int i = 0; i < XC; i++) x_load(u0 * 4 + d, d % XD, i);
#pragma unroll
        for (int c = 0; c < NC; c++) {
            if constexpr (Q6) w_load_q6(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, c);
            else w_load_q(1, c);
        }
        __syncthreads();
        static_for<GPK>([&](auto PART) { read_frags(smem, 0, 0, PART); });

        for (int unit = u0; unit < u1; unit++) static_for<4>([&](auto SUB) { k_step(unit, SUB); });
    }

    // a split-k slice stores f32 into its own [m, n] plane of the workspace
    float* out_f32 = P.partial ? P.partial + (int64_t)blockIdx.y * P.m * P.n : reinterpret_cast<float*>(P.y);
#pragma unroll
    for (int i = 0; i < MT; i++) {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const int64_t gn = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
            if (gn >= P.n_end) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t gm = m0 + wm * (BM / WM) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm >= P.m) continue;
                if (P.partial) out_f32[gm * P.n + gn] = acc[i][j][r]; // a slice: the second kernel finishes
                else qmm_store(P.y, QmmEpilogue{P.residual, P.out_bf16}, gm * P.n + gn, acc[i][j][r]);
            }
        }
    }
}

// out[i] = sum over slices (in order) of partial[s][i], as f32 or bf16; i runs over the
// columns [n_begin, n_end) of all rows
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, int slices, int64_t m, int64_t n,
                                     int64_t n_begin, int64_t n_end, void* y, int out_bf16, const void* residual) {
    const int64_t width = n_end - n_begin;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= m * width) return;
    const int64_t row = idx / width, col = n_begin + (idx - row * width);
    float sum = 0.0f;
    for (int s = 0; s < slices; s++) sum += partial[((int64_t)s * m + row) * n + col];
    qmm_store(y, QmmEpilogue{residual, out_bf16}, row * n + col, sum);
}

__global__ void f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out,
                                   int64_t count) {
    int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 4 <= count) {
        float4 f = *reinterpret_cast<const float4*>(x + i);
        uint2 o;
        o.x = pack_bf16(f.x, f.y);
        o.y = pack_bf16(f.z, f.w);
        *reinterpret_cast<uint2*>(out + i) = o;
    } else {
        for (; i < count; i++) out[i] = qmm_f32_to_bf16_bits(x[i]);
    }
}

__global__ void epilogue_kernel(const float* __restrict__ t, const void* residual, void* y, int y_bf16,
                                int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) qmm_store(y, QmmEpilogue{residual, y_bf16}, i, t[i]);
}

__global__ void bf16_to_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) out[i] = qmm_bf16_bits_to_f32(x[i]);
}

template <int QT, int BM, int BN, int NW = 4>
hipError_t launch_tile(GemmParams P, int slices, hipStream_t stream) {
    P.tiles_m = (int)((P.m + BM - 1) / BM);
    P.tiles_n = (int)((P.n_end - P.n_begin + BN - 1) / BN);
    if (P.n_weights > 1) { // a projection group: the members' column tiles one after the other
        int64_t t = 0;
        for (int i = 0; i < P.n_weights; i++) P.tn_end[i] = (int)(t += (P.nv[i] + BN - 1) / BN);
        P.tiles_n = (int)t;
    }
    const int64_t grid = (int64_t)P.tiles_m * P.tiles_n;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    const size_t lds = (size_t)2 * (BM + BN) * kRowStride;
    const bool x_tail = QT == QMM_Q8_0 && (P.k & 63) != 0; // the K-quant types have k a multiple of 256
    // Q6_K is pipelined with eight waves only (two or four threads per weight row)
    constexpr bool kPipe = (BM == 256 || BN == 256) && (QT != QMM_Q6_K || NW == 8);
    const void* fn;
    if constexpr (kPipe)
        fn = x_tail ? reinterpret_cast<const void*>(&gemm_pipe_kernel<QT, BM, BN, QT == QMM_Q8_0, NW>)
                    : reinterpret_cast<const void*>(&gemm_pipe_kernel<QT, BM, BN, false, NW>);
    else fn = reinterpret_cast<const void*>(&gemm_kernel<QT, BM, BN>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    if constexpr (kPipe) {
        float* partial = P.partial;
        if (slices > 1) P.slice_units = (P.k_units + slices - 1) / slices;
        else P.partial = nullptr;
        const dim3 grid2((unsigned)grid, (unsigned)slices);
        if (x_tail) gemm_pipe_kernel<QT, BM, BN, QT == QMM_Q8_0, NW><<<grid2, dim3(64 * NW), lds, stream>>>(P);
        else gemm_pipe_kernel<QT, BM, BN, false, NW><<<grid2, dim3(64 * NW), lds, stream>>>(P);
        if (slices > 1 && P.n_weights > 1) {
            for (int i = 0; i < P.n_weights; i++) {
                const int64_t count = P.m * P.nv[i];
                splitk_reduce_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
                    P.partial_v[i], slices, P.m, P.nv[i], 0, P.nv[i], P.yv[i], P.out_bf16, nullptr);
            }
        } else if (slices > 1) {
            const int64_t count = P.m * (P.n_end - P.n_begin);
            splitk_reduce_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
                partial, slices, P.m, P.n, P.n_begin, P.n_end, P.y, P.out_bf16, P.residual);
        }
    } else {
        gemm_kernel<QT, BM, BN><<<dim3((unsigned)grid), dim3(kThreads), lds, stream>>>(P);
    }
    return hipGetLastError();
}

// How a [m, n] x k product is cut into launches.  Big tiles reuse each LDS byte most, but
// the grid runs in rounds of one workgroup per CU and a partly filled last round idles
// CUs; a product with few tiles can be split along k (each slice writes an f32 tile, a
// second kernel adds the slices in order).  Costs are in k steps of a 256 x 256 tile
// (relative tile efficiencies measured on the 8B shapes).
struct GemmPlan {
    int bm, bn;          // tile of the only / the second launch
    int slices;          // split along k (BN == 256 tiles only)
    int64_t full_cols;   // > 0: first a launch of 256 x 256 tiles over this many 256-column strips
};

// IZWI_QMM_GEMM_TILE="bm,bn,slices" (tuning aid) replaces the plan: bm, bn in {128, 256}.
bool forced_plan(GemmPlan& plan) {
    static const GemmPlan forced = [] {
        GemmPlan p{0, 0, 1, 0};
        const char* e = getenv("IZWI_QMM_GEMM_TILE");
        if (e && sscanf(e, "%d,%d,%d", &p.bm, &p.bn, &p.slices) >= 2) {
            const bool ok = (p.bm == 128 || p.bm == 256) && (p.bn == 128 || p.bn == 256) && p.slices >= 1 && p.slices <= 8;
            if (!ok || (p.bm == 128 && p.bn == 128)) p.slices = 1;
            if (!ok) p.bm = p.bn = 0;
        }
        return p;
    }();
    if (forced.bm == 0) return false;
    plan = forced;
    return true;
}

GemmPlan plan_gemm(int64_t m, int64_t n, int k_steps, int n_cus, bool group = false) {
    // relative rate of a half-size tile (256 x 128 dequantizes half as many weights per MFMA
    // as 128 x 256 and is used whenever there are more than 128 rows) and of a quarter-size one
    const double kQ128 = m > 128 ? 0.76 : 0.68, kQ64 = 0.4;
    const int hm = m > 128 ? 256 : 128, hn = m > 128 ? 128 : 256; // the half-size tile
    {
        GemmPlan forced;
        if (forced_plan(forced)) {
            while (forced.slices > 1 && k_steps / 4 < forced.slices) forced.slices /= 2;
            return forced;
        }
    }
    auto tiles = [&](int bm, int bn, int64_t cols) { return ((m + bm - 1) / bm) * ((cols + bn - 1) / bn); };
    auto rounds = [&](int64_t t) { return (double)((t + n_cus - 1) / n_cus); };
    GemmPlan best{256, 256, 1, 0};
    double best_cost = rounds(tiles(256, 256, n)) * k_steps;
    auto consider = [&](GemmPlan p, double cost) {
        if (cost < 0.97 * best_cost) best = p, best_cost = cost;
    };
    consider({hm, hn, 1, 0}, rounds(tiles(hm, hn, n)) * k_steps * 0.5 / kQ128);
    // (a projection group runs on the pipelined tiles only, in one launch)
    if (!group) consider({128, 128, 1, 0}, rounds(tiles(128, 128, n)) * k_steps * 0.25 / kQ64);
    // whole rounds of 256 x 256 tiles first, the remaining columns as half-size tiles
    const int64_t tiles_m256 = (m + 255) / 256, cols256 = (n + 255) / 256;
    const int64_t full_cols = (tiles_m256 * cols256 / n_cus) * n_cus / tiles_m256;
    if (!group && full_cols > 0 && full_cols < cols256)
        consider({hm, hn, 1, full_cols},
                 (double)(tiles_m256 * full_cols / n_cus) * k_steps +
                     rounds(tiles(hm, hn, n - full_cols * 256)) * k_steps * 0.5 / kQ128);
    // split along k: the slices' f32 tiles are written and read once more (about 4 TB/s,
    // a 256 x 256 k step takes about 1.5 us)
    for (int slices = 2; slices <= 8; slices *= 2) {
        if (k_steps / slices < 8) break;
        const double reduce_cost = 2.0 * slices * (double)m * (double)n * 4.0 / 4e12 * 1e6 / 1.5 + 2.0;
        const double steps = 4.0 * (double)((k_steps / 4 + slices - 1) / slices); // slices are whole units
        consider({256, 256, slices, 0}, rounds(tiles(256, 256, n) * slices) * steps + reduce_cost);
        consider({hm, hn, slices, 0}, rounds(tiles(hm, hn, n) * slices) * steps * 0.5 / kQ128 + reduce_cost);
    }
    return best;
}

template <int QT>
hipError_t launch_qt(const GemmParams& P0, int n_cus, hipStream_t stream) {
    const GemmPlan plan = plan_gemm(P0.m, P0.n, P0.k_units * 4, n_cus);
    GemmParams P = P0;
    P.n_begin = 0;
    P.n_end = P0.n;
    if (plan.slices > 1 && P0.partial == nullptr) return hipErrorInvalidValue;
    if (plan.full_cols > 0) {
        P.n_end = plan.full_cols * 256;
        hipError_t e = launch_tile<QT, 256, 256, 8>(P, 1, stream);
        if (e != hipSuccess) return e;
        P.n_begin = P.n_end;
        P.n_end = P0.n;
    }
    if (plan.bm == 256 && plan.bn == 256) return launch_tile<QT, 256, 256, 8>(P, plan.slices, stream);
    if (plan.bm == 256) return launch_tile<QT, 256, 128, 8>(P, plan.slices, stream);
    if constexpr (QT != QMM_Q6_K) { // the plan picks this tile for m <= 128 only, where Q6_K does not come here
        if (plan.bn == 256) return launch_tile<QT, 128, 256>(P, plan.slices, stream);
    }
    return launch_tile<QT, 128, 128>(P, 1, stream);
}

// n of the single matrix a group is planned as: the members' columns, each rounded up to whole
// 256-column strips
int64_t group_columns(const QmmLayout* const* layouts, int n_weights) {
    int64_t n = 0;
    for (int i = 0; i < n_weights; i++) n += (layouts[i]->n + 255) / 256 * 256;
    return n;
}

template <int QT>
hipError_t launch_group_qt(GemmParams P, int64_t n_planned, int n_cus, hipStream_t stream) {
    const GemmPlan plan = plan_gemm(P.m, n_planned, P.k_units * 4, n_cus, true);
    if (plan.slices > 1) {
        if (P.partial == nullptr) return hipErrorInvalidValue;
        float* base = P.partial;
        for (int i = 0; i < P.n_weights; i++) {
            P.partial_v[i] = base;
            base += (size_t)plan.slices * (size_t)P.m * (size_t)P.nv[i];
        }
    }
    if (plan.bm == 256 && plan.bn == 256) return launch_tile<QT, 256, 256, 8>(P, plan.slices, stream);
    if (plan.bm == 256 && plan.bn == 128) return launch_tile<QT, 256, 128, 8>(P, plan.slices, stream);
    return hipErrorNotSupported;
}

} // namespace

// a group takes the plane form when every member can
static bool group_plane_applies(const QmmLayout* const* layouts, int n_weights, int64_t m) {
    for (int i = 0; i < n_weights; i++)
        if (!qmm_gemm_plane_applies(*layouts[i], m) || layouts[i]->k != layouts[0]->k) return false;
    return n_weights >= 1;
}

size_t qmm_gemm_group_workspace_bytes(const QmmLayout* const* layouts, int n_weights, int64_t m, int n_cus) {
    if (m <= 128 || n_weights < 2) return 0;
    if (group_plane_applies(layouts, n_weights, m)) {
        size_t total = 0;
        for (int i = 0; i < n_weights; i++) total += qmm_gemm_plane_bytes(*layouts[i]);
        return total;
    }
    const GemmPlan plan = plan_gemm(m, group_columns(layouts, n_weights), (int)layouts[0]->k_units * 4, n_cus > 0 ? n_cus : 1, true);
    if (plan.slices <= 1) return 0;
    size_t total = 0;
    for (int i = 0; i < n_weights; i++) total += (size_t)plan.slices * (size_t)m * (size_t)layouts[i]->n * sizeof(float);
    return total;
}

hipError_t qmm_launch_gemm_bf16_multi(const QmmLayout* const* layouts, const void* const* tiled, int n_weights,
                                      const uint16_t* x_bf16, int64_t m, void* const* ys, int out_bf16,
                                      void* workspace, int n_cus, hipStream_t stream) {
    if (n_weights < 2 || n_weights > QMM_MAX_GROUP) return hipErrorInvalidValue;
    if (m <= 128) return hipErrorNotSupported; // the plain tile kernels: one call per weight
    if (n_cus <= 0) n_cus = 1;
    if (group_plane_applies(layouts, n_weights, m)) {
        if (workspace == nullptr) return hipErrorInvalidValue;
        return qmm_launch_gemm_plane(layouts, tiled, n_weights, x_bf16, m, ys, out_bf16, workspace, n_cus, stream);
    }
    const QmmLayout& L0 = *layouts[0];
    GemmParams P;
    P.w = (const uint8_t*)tiled[0];
    P.x = x_bf16;
    P.y = ys[0];
    P.m = m;
    P.n = L0.n;
    P.n_begin = 0;
    P.n_end = L0.n;
    P.k = L0.k;
    P.k_units = (int)L0.k_units;
    P.k_groups = (int)L0.k_groups;
    P.s = L0.s;
    P.slots = L0.slots;
    P.row_tiles = L0.row_tiles;
    P.panel_bytes = L0.panel_bytes;
    P.out_bf16 = out_bf16;
    P.tiles_m = P.tiles_n = 0;
    P.slice_units = 0;
    P.nibble_mask = 0x0f0f0f0fu;
    P.partial = (float*)workspace;
    P.residual = nullptr;
    P.n_weights = n_weights;
    for (int i = 0; i < n_weights; i++) {
        const QmmLayout& L = *layouts[i];
        if (L.dtype != L0.dtype || L.k != L0.k || L.n_stacked != 1 || L.n == 0) return hipErrorInvalidValue;
        P.wv[i] = (const uint8_t*)tiled[i];
        P.yv[i] = ys[i];
        P.nv[i] = L.n;
        P.row_tiles_v[i] = L.row_tiles;
        P.partial_v[i] = nullptr;
        P.tn_end[i] = 0;
    }
    const int64_t n_planned = group_columns(layouts, n_weights);
    if (L0.dtype == QMM_Q6_K) return launch_group_qt<QMM_Q6_K>(P, n_planned, n_cus, stream);
    return L0.dtype == QMM_Q4_K ? launch_group_qt<QMM_Q4_K>(P, n_planned, n_cus, stream)
                                : launch_group_qt<QMM_Q8_0>(P, n_planned, n_cus, stream);
}

size_t qmm_gemm_workspace_bytes(const QmmLayout& L, int64_t m, int n_cus) {
    if (m <= 0 || L.n == 0 || (L.dtype == QMM_Q6_K && m <= 128)) return 0;
    if (qmm_gemm_plane_applies(L, m)) return qmm_gemm_plane_bytes(L);
    const GemmPlan plan = plan_gemm(m, L.n, (int)L.k_units * 4, n_cus > 0 ? n_cus : 1);
    return plan.slices > 1 ? (size_t)plan.slices * (size_t)m * (size_t)L.n * sizeof(float) : 0;
}

hipError_t qmm_launch_gemm_bf16(const QmmLayout& L, const void* tiled, const uint16_t* x_bf16,
                                int64_t m, void* y, int out_bf16, void* workspace, int n_cus,
                                hipStream_t stream, const void* residual) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    if (n_cus <= 0) n_cus = 1;
    if (qmm_gemm_plane_applies(L, m)) {
        if (workspace == nullptr) return hipErrorInvalidValue;
        const QmmLayout* lp = &L;
        return qmm_launch_gemm_plane(&lp, &tiled, 1, x_bf16, m, &y, out_bf16, workspace, n_cus, stream, residual);
    }
    GemmParams P;
    P.w = (const uint8_t*)tiled;
    P.x = x_bf16;
    P.y = y;
    P.m = m;
    P.n = L.n;
    P.n_begin = 0;
    P.n_end = L.n;
    P.k = L.k;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.s = L.s;
    P.slots = L.slots;
    P.row_tiles = L.row_tiles;
    P.panel_bytes = L.panel_bytes;
    P.out_bf16 = out_bf16;
    P.tiles_m = P.tiles_n = 0;
    P.slice_units = 0;
    P.nibble_mask = 0x0f0f0f0fu;
    P.partial = (float*)workspace;
    P.residual = residual;
    P.n_weights = 0;
    if (L.dtype == QMM_Q6_K) {
        // more than 128 rows: the pipelined tiles; up to 128 the plain tile kernel, half-height
        // tiles when full ones would leave CUs idle
        static const bool plain_only = getenv("IZWI_QMM_Q6K_PLAIN_TILES") != nullptr; // comparison aid
        if (m > 128 && !plain_only) return launch_qt<QMM_Q6_K>(P, n_cus, stream);
        const int64_t t128 = ((m + 127) / 128) * ((L.n + 127) / 128);
        if (t128 < (int64_t)n_cus && m > 64) return launch_tile<QMM_Q6_K, 64, 128>(P, 1, stream);
        return launch_tile<QMM_Q6_K, 128, 128>(P, 1, stream);
    }
    return L.dtype == QMM_Q4_K ? launch_qt<QMM_Q4_K>(P, n_cus, stream)
                               : launch_qt<QMM_Q8_0>(P, n_cus, stream);
}

hipError_t qmm_launch_f32_to_bf16(const float* x, uint16_t* out, int64_t count,
                                  hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    int64_t threads = (count + 3) / 4;
    f32_to_bf16_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, stream>>>(x, out, count);
    return hipGetLastError();
}

hipError_t qmm_launch_epilogue(const float* t, const void* residual, void* y, int y_bf16, int64_t count,
                               hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    if ((count + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    epilogue_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(t, residual, y, y_bf16, count);
    return hipGetLastError();
}

hipError_t qmm_launch_bf16_to_f32(const uint16_t* x, float* out, int64_t count, hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    if ((count + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    bf16_to_f32_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(x, out, count);
    return hipGetLastError();
}
