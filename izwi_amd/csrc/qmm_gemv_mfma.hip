// Batched decode kernel (M = 3..64): the same arithmetic as the M <= 2 kernel
// (candle-core's integer block dots on Q8-quantized activations), with the
// int8 products on v_mfma_i32_16x16x32_i8 so that the cost per weight byte does
// not grow with M.
//
// Two launches:
//  1. the activations are quantized ONCE into a workspace laid out exactly as
//     the MFMA A operand wants them (16 rows per tile: [unit][sub-block]
//     [octet][row][8 B]), so the matmul workgroups copy it to LDS verbatim;
//  2. each wave streams weight panels (16 rows x S units) as in the M <= 2
//     kernel.  A panel lane holds one (row, unit); the MFMA B operand wants
//     (row, 8-element octet) per lane, so the quants are transposed between
//     the four 16-lane rows in registers (v_permlane32_swap + v_permlane16_swap,
//     two swaps per dword).  One MFMA per 32-element sub-block: D[m][row] are
//     the block dots of 16 activation rows at once; the 6-bit sub-block scales
//     are applied on integers (v_mad_i32_i24), the Q4_K min term comes from a
//     second chained MFMA whose B operand is the min replicated over the octet
//     (min * sum of activation quants, accumulated over the 8 sub-blocks).
#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

constexpr int kMaxWaves = 12;
constexpr int kChunkUnits = 16;       // units of x held in LDS at a time (64 KiB of int8)
constexpr int kUnitBytes = 4096;      // [8 sub-blocks][4 octets][16 rows][8 B]
constexpr uint32_t kNib = 0x0f0f0f0fu;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppRor4 = 0x124, kDppRor8 = 0x128;
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
__device__ __forceinline__ int row16_min(int v) {
    v = min(v, dpp<kDppXor1>(v));
    v = min(v, dpp<kDppXor2>(v));
    v = min(v, dpp<kDppRor4>(v));
    v = min(v, dpp<kDppRor8>(v));
    return v;
}

// workspace geometry for one call
struct XWs {
    int k_units;
    int n_tiles; // ceil(m / 16)
    __host__ __device__ size_t xq_bytes() const { return (size_t)n_tiles * k_units * kUnitBytes; }
    // side information per unit, in floats.  Q4_K: 16 row scales, then per row the
    // eight sub-block sums of the quants split into two int8 planes (sum = 128 * hi + lo).
    // Q8_0: one scale per (block, row).
    __host__ __device__ static int xd_per_unit(int qt) { return qt == QMM_Q4_K ? 16 + 64 : 128; }
    __host__ __device__ size_t xd_floats(int qt) const {
        return (size_t)n_tiles * k_units * xd_per_unit(qt);
    }
};

// ---- launch 1: activation quantizer into the MFMA layout --------------------
// One 16-lane group per (row, unit); lane j holds elements 16j..16j+15, i.e.
// sub-block j / 2, octets 2 (j % 2) and 2 (j % 2) + 1.
template <int QT>
__global__ void quantize_ws_kernel(const float* __restrict__ x, int m, int k, XWs ws,
                                   uint8_t* __restrict__ xq, float* __restrict__ xd) {
    const int group = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int j = threadIdx.x & 15;
    const int rows = ws.n_tiles * 16;
    if (group >= rows * ws.k_units) return; // whole 16-lane groups leave together
    const int row = group / ws.k_units, unit = group - row * ws.k_units;
    const int tile = row >> 4, mr = row & 15;
    float v[16];
    const int k0 = unit * 256 + 16 * j;
    if (row < m && k0 + 16 <= k) {
        const float4* p = reinterpret_cast<const float4*>(x + (int64_t)row * k + k0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 f = p[i];
            v[4 * i] = f.x, v[4 * i + 1] = f.y, v[4 * i + 2] = f.z, v[4 * i + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = (row < m && k0 + i < k) ? x[(int64_t)row * k + k0 + i] : 0.0f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(v[i]));
    float scale_mul; // quant = round(v * scale_mul)
    const int64_t tu = (int64_t)tile * ws.k_units + unit;
    if (QT == QMM_Q4_K) {
        // BlockQ8K::from_float: iscale = -128 / (first value of largest magnitude)
        amax = row16_max(amax);
        int key = 0x7fffffff;
#pragma unroll
        for (int i = 15; i >= 0; i--)
            if (fabsf(v[i]) == amax) key = ((16 * j + i) << 1) | (v[i] < 0.0f ? 1 : 0);
        key = row16_min(key);
        float d = 0.0f;
        scale_mul = 0.0f;
        if (amax != 0.0f) {
            scale_mul = __fdiv_rn(-128.0f, (key & 1) ? -amax : amax);
            d = __fdiv_rn(1.0f, scale_mul);
        }
        if (j == 0) xd[tu * 80 + mr] = d;
    } else {
        // BlockQ8_0::from_float on the lane pair's 32 values
        amax = fmaxf(amax, __int_as_float(dpp<kDppXor1>(__float_as_int(amax))));
        const float d = __fdiv_rn(amax, 127.0f);
        scale_mul = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        if ((j & 1) == 0) xd[(tu * 8 + (j >> 1)) * 16 + mr] = qmm_f16_bits_to_f32(qmm_f32_to_f16_bits(d));
    }
    uint32_t q[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t packed = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            // both reference quantizers compute scale * value in f32 and round half away
            float r = roundf(QT == QMM_Q4_K ? __fmul_rn(scale_mul, v[4 * w + b]) : __fmul_rn(v[4 * w + b], scale_mul));
            int qi = (int)fminf(fmaxf(r, -128.0f), 127.0f);
            packed |= ((uint32_t)qi & 0xffu) << (8 * b);
        }
        q[w] = packed;
    }
    const int s = j >> 1, oct = 2 * (j & 1);
    if (QT == QMM_Q4_K) {
        int s16 = __builtin_amdgcn_sdot4((int)q[0], 0x01010101, 0, false);
        s16 = __builtin_amdgcn_sdot4((int)q[1], 0x01010101, s16, false);
        s16 = __builtin_amdgcn_sdot4((int)q[2], 0x01010101, s16, false);
        s16 = __builtin_amdgcn_sdot4((int)q[3], 0x01010101, s16, false);
        const int bsum = s16 + dpp<kDppXor1>(s16); // the sub-block's 32 quants
        if ((j & 1) == 0) {
            uint8_t* side = reinterpret_cast<uint8_t*>(xd + tu * 80 + 16) + mr * 16;
            side[s] = (uint8_t)(bsum & 127);
            side[8 + s] = (uint8_t)(bsum >> 7);
        }
    }
    uint8_t* dst = xq + ((tu * 8 + s) * 4 + oct) * 128 + mr * 8;
    *reinterpret_cast<uint2*>(dst) = make_uint2(q[0], q[1]);
    *reinterpret_cast<uint2*>(dst + 128) = make_uint2(q[2], q[3]);
}

// ---- launch 2 ------------------------------------------------------------------
struct MfmaParams {
    const uint8_t* w;
    const uint8_t* xq;
    const float* xd;
    float* y;
    int m, n, k;
    int k_units, k_groups, s, slots;
    int row_tiles, panel_bytes;
    int nwk, nwr, wave_magic;
    int chunk_units; // multiple of s, <= kChunkUnits
    int n_tiles;
};

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

template <int QT>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_mfma_kernel(MfmaParams P) {
    constexpr int QC = QT == QMM_Q4_K ? 8 : 16;
    constexpr int XD_PER_UNIT = QT == QMM_Q4_K ? 80 : 128; // floats of side information per unit
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* lds_xq = smem;                                                        // chunk_units * 4096
    float* lds_xd = reinterpret_cast<float*>(smem + (size_t)P.chunk_units * kUnitBytes); // chunk_units * XD_PER_UNIT
    float* lds_red = lds_xd + P.chunk_units * XD_PER_UNIT;                         // waves * 256

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wr = (wave * P.wave_magic) >> 16;
    const int wk = wave - wr * P.nwk;
    const int j = lane & 15, grp = lane >> 4;
    const int rt = blockIdx.x * P.nwr + wr;
    const bool rt_ok = rt < P.row_tiles;
    const bool lane_active = lane < P.slots;

    auto load_panel = [&](int kg, u32x4 (&hdr)[4], u32x4 (&q)[QC]) {
        const bool ok = rt_ok && lane_active;
        const u32x4* base =
            reinterpret_cast<const u32x4*>(P.w + (int64_t)(rt * P.k_groups + kg) * P.panel_bytes);
#pragma unroll
        for (int c = 0; c < QC; c++)
            q[c] = ok ? __builtin_nontemporal_load(base + (size_t)(1 + c) * P.slots + lane)
                      : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 4; u++) hdr[u] = (rt_ok && u < P.s) ? base[u * 16 + j] : u32x4{0, 0, 0, 0};
    };

    for (int tile = 0; tile < P.n_tiles; tile++) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int cu0 = 0; cu0 < P.k_units; cu0 += P.chunk_units) {
            const int cu_n = min(P.chunk_units, P.k_units - cu0);
            const int kg0 = cu0 / P.s, kg1 = (cu0 + cu_n + P.s - 1) / P.s;
            // A workgroup barrier also waits for the calling wave's outstanding loads, so
            // everything this chunk needs is requested before the one barrier that follows:
            // first the activations (global -> LDS without passing through registers, each
            // wave moving 1 KiB pieces, 16 B per lane), then the wave's first weight panel
            // (this lane's (row j, unit grp) header + quants, and the headers of all units
            // of row j).
            if (tile != 0 || cu0 != 0) __syncthreads(); // every wave is done reading the previous chunk
            {
                const u32x4* src = reinterpret_cast<const u32x4*>(
                    P.xq + ((size_t)tile * P.k_units + cu0) * kUnitBytes);
                const int pieces = cu_n * (kUnitBytes / 1024);
                const int waves = blockDim.x >> 6;
                for (int c = wave; c < pieces; c += waves)
                    __builtin_amdgcn_global_load_lds(
                        (const __attribute__((address_space(1))) void*)(src + c * 64 + lane),
                        (__attribute__((address_space(3))) void*)(lds_xq + c * 1024), 16, 0, 0);
            }
            u32x4 hdr[4];
            u32x4 q[QC];
            bool have_panel = false;
            if (kg0 + wk < kg1) {
                load_panel(kg0 + wk, hdr, q);
                have_panel = true;
            }
            {
                const float* sd = P.xd + ((size_t)tile * P.k_units + cu0) * XD_PER_UNIT;
                for (int i = threadIdx.x; i < cu_n * XD_PER_UNIT; i += blockDim.x) lds_xd[i] = sd[i];
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the LDS-direct loads have landed
            }
            __syncthreads();
            for (int kg = kg0 + wk; kg < kg1; kg += P.nwk) {
                if (!have_panel) load_panel(kg, hdr, q);
                have_panel = false;
                // ---- (row, unit) per lane -> (row, octet) per lane, for each unit u in register slot u
#pragma unroll
                for (int b = 0; b < QC / 2; b++) {
                    uint32_t a0 = q[2 * b].x, a1 = q[2 * b].z, a2 = q[2 * b + 1].x, a3 = q[2 * b + 1].z;
                    uint32_t b0 = q[2 * b].y, b1 = q[2 * b].w, b2 = q[2 * b + 1].y, b3 = q[2 * b + 1].w;
                    transpose_rows(a0, a1, a2, a3);
                    transpose_rows(b0, b1, b2, b3);
                    q[2 * b] = u32x4{a0, b0, a1, b1};
                    q[2 * b + 1] = u32x4{a2, b2, a3, b3};
                }
                // after the transpose, unit u of group b sits in dwords (x,y) / (z,w) of q[2b] / q[2b+1]:
                //   u = 0: q[2b].xy   u = 1: q[2b].zw   u = 2: q[2b+1].xy   u = 3: q[2b+1].zw
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int unit = kg * P.s + u;
                    if (u >= P.s || unit >= P.k_units) continue; // uniform
                    const int lu = unit - cu0;
                    const uint8_t* xu = lds_xq + (size_t)lu * kUnitBytes + grp * 128 + j * 8;
                    if (QT == QMM_Q4_K) {
                        uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
                        qmm_unpack_q4k_scales(hdr[u].y, hdr[u].z, hdr[u].w, sc_lo, sc_hi, mn_lo, mn_hi);
                        // all eight block-dot MFMAs (and the two of the min term) are issued
                        // back to back; their results are consumed afterwards, so the matrix
                        // pipe's latency is paid once per unit, not once per sub-block
                        i32x4 dd[8];
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            const u32x4 qq = q[2 * g + (u >> 1)];
                            const uint32_t w0 = (u & 1) ? qq.z : qq.x, w1 = (u & 1) ? qq.w : qq.y;
                            const long a_lo = *reinterpret_cast<const long*>(xu + (2 * g) * 512);
                            const long a_hi = *reinterpret_cast<const long*>(xu + (2 * g + 1) * 512);
                            dd[2 * g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(
                                a_lo, pack64(w0 & kNib, w1 & kNib), i32x4{0, 0, 0, 0}, 0, 0, 0);
                            dd[2 * g + 1] = __builtin_amdgcn_mfma_i32_16x16x32_i8(
                                a_hi, pack64((w0 >> 4) & kNib, (w1 >> 4) & kNib), i32x4{0, 0, 0, 0}, 0, 0, 0);
                        }
                        const float d = qmm_f16_bits_to_f32((uint16_t)(hdr[u].x & 0xffffu));
                        const float dmin = qmm_f16_bits_to_f32((uint16_t)(hdr[u].x >> 16));
                        // min term: sum_s min_s * bsum_s as two MFMAs over k = sub-block index; only
                        // the first 16-lane row carries data (k slots 0..7), the rest multiply zeros
                        const uint8_t* side = reinterpret_cast<const uint8_t*>(lds_xd + lu * 80 + 16) + j * 16;
                        const long bs_lo = grp == 0 ? *reinterpret_cast<const long*>(side) : 0L;
                        const long bs_hi = grp == 0 ? *reinterpret_cast<const long*>(side + 8) : 0L;
                        const long bmn = pack64(mn_lo, mn_hi);
                        const i32x4 m_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_lo, bmn, i32x4{0, 0, 0, 0}, 0, 0, 0);
                        const i32x4 m_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(bs_hi, bmn, i32x4{0, 0, 0, 0}, 0, 0, 0);
                        const float4 dx = *reinterpret_cast<const float4*>(lds_xd + lu * 80 + grp * 4);
                        const float dxs[4] = {dx.x, dx.y, dx.z, dx.w};
                        int isum[4] = {0, 0, 0, 0};
#pragma unroll
                        for (int s8 = 0; s8 < 8; s8++) {
                            const int sc = (int)qmm_byte_of(sc_lo, sc_hi, s8);
#pragma unroll
                            for (int r = 0; r < 4; r++) isum[r] += __mul24(sc, dd[s8][r]); // |dd| < 2^17, sc < 64
                        }
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const int msum = m_lo[r] + (m_hi[r] << 7);
                            acc[r] += (d * dxs[r]) * (float)isum[r] - (dmin * dxs[r]) * (float)msum;
                        }
                    } else {
                        const uint32_t hw[4] = {hdr[u].x, hdr[u].y, hdr[u].z, hdr[u].w};
#pragma unroll
                        for (int b = 0; b < 8; b++) {
                            const u32x4 qq = q[2 * b + (u >> 1)];
                            const uint32_t w0 = (u & 1) ? qq.z : qq.x, w1 = (u & 1) ? qq.w : qq.y;
                            const long a = *reinterpret_cast<const long*>(xu + b * 512);
                            i32x4 dd = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, pack64(w0, w1), i32x4{0, 0, 0, 0}, 0, 0, 0);
                            const float dw = qmm_f16_bits_to_f32((uint16_t)((hw[b >> 1] >> (16 * (b & 1))) & 0xffffu));
                            const float4 dx = *reinterpret_cast<const float4*>(lds_xd + (lu * 8 + b) * 16 + grp * 4);
                            acc[0] += ((float)dd[0] * dw) * dx.x;
                            acc[1] += ((float)dd[1] * dw) * dx.y;
                            acc[2] += ((float)dd[2] * dw) * dx.z;
                            acc[3] += ((float)dd[3] * dw) * dx.w;
                        }
                    }
                }
            }
        }
        // ---- combine the waves that split k, write y[tile*16 + 4*grp + r][rt*16 + j]
        const int row = rt * 16 + j;
        if (P.nwk == 1) {
            if (rt_ok && row < P.n) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int mm = tile * 16 + grp * 4 + r;
                    if (mm < P.m) P.y[(int64_t)mm * P.n + row] = acc[r];
                }
            }
        } else {
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 4; r++) lds_red[(wave * 4 + r) * 64 + lane] = acc[r];
            __syncthreads();
            if (wk == 0 && rt_ok && row < P.n) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float sum = 0.0f;
                    for (int w2 = 0; w2 < P.nwk; w2++) sum += lds_red[((wr * P.nwk + w2) * 4 + r) * 64 + lane];
                    const int mm = tile * 16 + grp * 4 + r;
                    if (mm < P.m) P.y[(int64_t)mm * P.n + row] = sum;
                }
            }
        }
    }
}

} // namespace

size_t qmm_gemv_mfma_workspace_bytes(const QmmLayout& L, int64_t m) {
    XWs ws{(int)L.k_units, (int)((m + 15) / 16)};
    return ws.xq_bytes() + ws.xd_floats(L.dtype) * sizeof(float);
}

hipError_t qmm_launch_gemv_mfma(const QmmLayout& L, const void* tiled, const float* x, int64_t m,
                                float* y, void* workspace, int n_cus, hipStream_t stream) {
    if (m <= 0 || L.n == 0) return hipSuccess;
    if (L.n > 0x3fffffff || L.k > 0x3fffffff || m > 0x3fffffff ||
        L.row_tiles * L.k_groups > 0x7fffffff)
        return hipErrorInvalidValue;
    XWs ws{(int)L.k_units, (int)((m + 15) / 16)};
    uint8_t* xq = (uint8_t*)workspace;
    float* xd = (float*)(xq + ws.xq_bytes());
    {
        int64_t threads = (int64_t)ws.n_tiles * 16 * ws.k_units * 16;
        unsigned grid = (unsigned)((threads + 255) / 256);
        if (L.dtype == QMM_Q4_K)
            quantize_ws_kernel<QMM_Q4_K><<<grid, 256, 0, stream>>>(x, (int)m, (int)L.k, ws, xq, xd);
        else
            quantize_ws_kernel<QMM_Q8_0><<<grid, 256, 0, stream>>>(x, (int)m, (int)L.k, ws, xq, xd);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    MfmaParams P;
    P.w = (const uint8_t*)tiled;
    P.xq = xq;
    P.xd = xd;
    P.y = y;
    P.m = (int)m;
    P.n = (int)L.n;
    P.k = (int)L.k;
    P.k_units = (int)L.k_units;
    P.k_groups = (int)L.k_groups;
    P.s = L.s;
    P.slots = L.slots;
    P.row_tiles = (int)L.row_tiles;
    P.panel_bytes = (int)L.panel_bytes;
    P.n_tiles = ws.n_tiles;
    P.chunk_units = (kChunkUnits / L.s) * L.s;
    if (P.chunk_units > P.k_units) P.chunk_units = ((P.k_units + L.s - 1) / L.s) * L.s;
    // waves along k inside a chunk, row-tiles side by side to amortize the LDS copy of x
    int chunk_groups = P.chunk_units / L.s;
    int nwk = chunk_groups < 4 ? chunk_groups : 4;
    int nwr_max = kMaxWaves / nwk;
    int64_t want = L.row_tiles / (n_cus > 0 ? n_cus : 1);
    int nwr = (int)(want < 1 ? 1 : (want > nwr_max ? nwr_max : want));
    P.nwk = nwk;
    P.nwr = nwr;
    P.wave_magic = (65536 + nwk - 1) / nwk;
    const int waves = nwk * nwr;
    const int xd_per_unit = XWs::xd_per_unit(L.dtype);
    size_t lds = (size_t)P.chunk_units * kUnitBytes + (size_t)P.chunk_units * xd_per_unit * 4 +
                 (size_t)waves * 256 * 4;
    const void* fn = L.dtype == QMM_Q4_K ? reinterpret_cast<const void*>(&gemv_mfma_kernel<QMM_Q4_K>)
                                         : reinterpret_cast<const void*>(&gemv_mfma_kernel<QMM_Q8_0>);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    unsigned grid = (unsigned)((L.row_tiles + nwr - 1) / nwr);
    if (L.dtype == QMM_Q4_K)
        gemv_mfma_kernel<QMM_Q4_K><<<grid, 64 * waves, lds, stream>>>(P);
    else
        gemv_mfma_kernel<QMM_Q8_0><<<grid, 64 * waves, lds, stream>>>(P);
    return hipGetLastError();
}
