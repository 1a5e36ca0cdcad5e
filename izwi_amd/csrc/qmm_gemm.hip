// Prefill kernel: y[m, n] = x[m, k] * dequant(W)[n, k]^T with bf16 MFMA.
//
// A workgroup (4 waves, 2 x 2) owns a 256 x 256 output tile; each wave a
// 128 x 128 sub-tile held as 4 x 4 v_mfma_f32_32x32x16_bf16 accumulators
// (256 f32 registers).  Per 64-wide k step the workgroup
//   * copies the 256 x 64 bf16 activation tile to LDS,
//   * reads the matching 64 k-elements of 256 weight rows straight from the
//     panel layout (header + two nibble chunks for Q4_K, header + four int8
//     chunks for Q8_0), dequantizes them in registers and writes bf16 to LDS,
//   * runs 4 k16 steps of 16 MFMAs per wave, operands read from LDS as one
//     16-byte load per lane (row stride padded to 144 B: conflict free).
// Global loads of the next k step are issued before the MFMAs of the current
// one, so HBM/L2 latency hides behind the matrix work.
#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kRowStride = 144; // bytes per LDS tile row: 64 bf16 + 16 B pad

struct GemmParams {
    const uint8_t* w;
    const uint16_t* x; // bf16 [m, k]
    void* y;
    int64_t m, n, k;
    int k_units, k_groups, s, slots;
    int64_t row_tiles, panel_bytes;
    int out_bf16;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    return (uint32_t)qmm_f32_to_bf16_bits(a) | ((uint32_t)qmm_f32_to_bf16_bits(b) << 16);
}

template <int QT>
struct WRegs {
    static constexpr int NC = QT == QMM_Q4_K ? 2 : 4;
    u32x4 hdr;
    u32x4 q[NC];
};

// Weight row `row` (global), k step kt (64 elements): header + its quant chunks.
template <int QT>
__device__ __forceinline__ void load_w(WRegs<QT>& r, const GemmParams& P, int64_t row, int kt) {
    const int unit = kt >> 2, part = kt & 3;
    const int64_t rt = row >> 4;
    if (rt >= P.row_tiles || unit >= P.k_units) {
        r.hdr = u32x4{0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < WRegs<QT>::NC; c++) r.q[c] = u32x4{0, 0, 0, 0};
        return;
    }
    const int kg = unit / P.s, us = unit - kg * P.s;
    const int slot = us * 16 + (int)(row & 15);
    const u32x4* base =
        reinterpret_cast<const u32x4*>(P.w + (rt * P.k_groups + kg) * P.panel_bytes) + slot;
    r.hdr = base[0];
#pragma unroll
    for (int c = 0; c < WRegs<QT>::NC; c++)
        r.q[c] = base[(size_t)(1 + part * WRegs<QT>::NC + c) * P.slots];
}

// Dequantizes the 64 k-elements held in r to bf16 and writes one LDS tile row.
template <int QT>
__device__ __forceinline__ void store_w(const WRegs<QT>& r, int kt, uint8_t* lds_row) {
    uint32_t out[32];
    if (QT == QMM_Q4_K) {
        const int g = kt & 3;
        const float d = qmm_f16_bits_to_f32((uint16_t)(r.hdr.x & 0xffffu));
        const float dmin = qmm_f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
        qmm_unpack_q4k_scales(r.hdr.y, r.hdr.z, r.hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
        const float d1 = d * (float)qmm_byte_of(sc_lo, sc_hi, 2 * g);
        const float m1 = dmin * (float)qmm_byte_of(mn_lo, mn_hi, 2 * g);
        const float d2 = d * (float)qmm_byte_of(sc_lo, sc_hi, 2 * g + 1);
        const float m2 = dmin * (float)qmm_byte_of(mn_lo, mn_hi, 2 * g + 1);
#pragma unroll
        for (int c = 0; c < 2; c++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint32_t v = r.q[c][j];
                float lo[4], hi[4];
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    uint32_t byte = (v >> (8 * b)) & 0xffu;
                    lo[b] = d1 * (float)(byte & 0xF) - m1;
                    hi[b] = d2 * (float)(byte >> 4) - m2;
                }
                // low nibbles: k 16c + 4j .., high nibbles: k 32 + 16c + 4j ..
                out[8 * c + 2 * j] = pack_bf16(lo[0], lo[1]);
                out[8 * c + 2 * j + 1] = pack_bf16(lo[2], lo[3]);
                out[16 + 8 * c + 2 * j] = pack_bf16(hi[0], hi[1]);
                out[16 + 8 * c + 2 * j + 1] = pack_bf16(hi[2], hi[3]);
            }
        }
    } else {
        const int b0 = (kt & 3) * 2; // first of the two 32-element blocks
        const uint32_t hw[4] = {r.hdr.x, r.hdr.y, r.hdr.z, r.hdr.w};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int b = b0 + (c >> 1);
            const float d = qmm_f16_bits_to_f32((uint16_t)((hw[b >> 1] >> (16 * (b & 1))) & 0xffffu));
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint32_t v = r.q[c][j];
                float f[4];
#pragma unroll
                for (int i = 0; i < 4; i++) f[i] = (float)(int8_t)((v >> (8 * i)) & 0xffu) * d;
                out[8 * c + 2 * j] = pack_bf16(f[0], f[1]);
                out[8 * c + 2 * j + 1] = pack_bf16(f[2], f[3]);
            }
        }
    }
    uint4* dst = reinterpret_cast<uint4*>(lds_row);
#pragma unroll
    for (int i = 0; i < 8; i++)
        dst[i] = make_uint4(out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]);
}

template <int QT>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmParams P) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* xs = smem;
    uint8_t* ws = smem + BM * kRowStride;

    // consecutive workgroups walk down m inside one weight column block, so the
    // 256 weight rows they share stay in L2 while all of m is swept
    const int tm = blockIdx.x % P.tiles_m;
    const int tn = blockIdx.x / P.tiles_m;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_steps = P.k_units * 4;

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // activation tile: 256 rows x 8 chunks of 16 B; thread t copies chunks t + 256 i
    u32x4 xr[8];
    WRegs<QT> wr;
    auto load_x = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int c = tid + kThreads * i;
            int row = c >> 3, kc = c & 7;
            int64_t gm = m0 + row, gk = (int64_t)kt * BK + kc * 8;
            if (gm < P.m && gk + 8 <= P.k) {
                xr[i] = *reinterpret_cast<const u32x4*>(P.x + gm * P.k + gk);
            } else {
                union {
                    u32x4 v;
                    uint16_t h[8];
                } u;
                u.v = u32x4{0, 0, 0, 0};
                if (gm < P.m)
                    for (int e = 0; e < 8; e++)
                        if (gk + e < P.k) u.h[e] = P.x[gm * P.k + gk + e];
                xr[i] = u.v;
            }
        }
    };
    auto store_x = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int c = tid + kThreads * i;
            int row = c >> 3, kc = c & 7;
            *reinterpret_cast<u32x4*>(xs + row * kRowStride + kc * 16) = xr[i];
        }
    };

    load_x(0);
    load_w<QT>(wr, P, n0 + tid, 0);

    for (int kt = 0; kt < k_steps; kt++) {
        store_x();
        store_w<QT>(wr, kt, ws + tid * kRowStride);
        __syncthreads();
        if (kt + 1 < k_steps) {
            load_x(kt + 1);
            load_w<QT>(wr, P, n0 + tid, kt + 1);
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int koff = kk * 32 + (lane >> 5) * 16; // bytes inside the tile row
            bf16x8 a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                a[i] = *reinterpret_cast<const bf16x8*>(
                    xs + (wm * 128 + i * 32 + (lane & 31)) * kRowStride + koff);
                b[i] = *reinterpret_cast<const bf16x8*>(
                    ws + (wn * 128 + i * 32 + (lane & 31)) * kRowStride + koff);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // D[i][j]: lane holds column j = lane % 32 and rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t gn = n0 + wn * 128 + j * 32 + (lane & 31);
            if (gn >= P.n) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t gm = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm >= P.m) continue;
                if (P.out_bf16)
                    reinterpret_cast<uint16_t*>(P.y)[gm * P.n + gn] = qmm_f32_to_bf16_bits(acc[i][j][r]);
                else
                    reinterpret_cast<float*>(P.y)[gm * P.n + gn] = acc[i][j][r];
            }
        }
    }
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

} // namespace

hipError_t qmm_launch_gemm_bf16(const QmmLayout& L, const void* tiled, const uint16_t* x_bf16,
                                int64_t m, void* y, int out_bf16, int n_cus, hipStream_t stream) {
    (void)n_cus;
    if (m <= 0 || L.n == 0) return hipSuccess;
    GemmParams P;
    P.w = (const uint8_t*)tiled;
    P.x = x_bf16;
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
    P.out_bf16 = out_bf16;
    P.tiles_m = (int)((m + BM - 1) / BM);
    P.tiles_n = (int)((L.n + BN - 1) / BN);
    int64_t grid = (int64_t)P.tiles_m * P.tiles_n;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    const size_t lds = (size_t)(BM + BN) * kRowStride;
    const void* fn = L.dtype == QMM_Q4_K ? reinterpret_cast<const void*>(&gemm_kernel<QMM_Q4_K>)
                                         : reinterpret_cast<const void*>(&gemm_kernel<QMM_Q8_0>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    if (L.dtype == QMM_Q4_K)
        gemm_kernel<QMM_Q4_K><<<dim3((unsigned)grid), dim3(kThreads), lds, stream>>>(P);
    else
        gemm_kernel<QMM_Q8_0><<<dim3((unsigned)grid), dim3(kThreads), lds, stream>>>(P);
    return hipGetLastError();
}

hipError_t qmm_launch_f32_to_bf16(const float* x, uint16_t* out, int64_t count,
                                  hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    int64_t threads = (count + 3) / 4;
    f32_to_bf16_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, stream>>>(x, out, count);
    return hipGetLastError();
}
