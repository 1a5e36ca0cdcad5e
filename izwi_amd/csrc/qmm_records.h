// The activation records of the batched decode kernels: layout of a unit record (256 k-values x 16
// rows, quantized to the weight type's dot type and laid out as the int8 matrix-core operand wants
// them) and the 16-lane quantizer that writes one row's share of a record.  Shared by the kernels
// that consume records (qmm_gemv_mfma.hip) and the producers that emit them directly (RMSNorm and
// silu * up in decode_ops.hip); unnamed namespace, one copy per including file.
#ifndef IZWI_QMM_RECORDS_H
#define IZWI_QMM_RECORDS_H

#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

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


template <int QT>
struct Unit {
    // [4 sub-block pairs][4 octets][16 rows][16 B]: the 8 quants of (sub-block 2b, octet, row), then
    // those of sub-block 2b + 1 - one 16-byte load per lane (lane = 16 * octet + row) brings both
    // matrix-core operands of a pair
    static constexpr int kQuant = 4096;
    // Q4_K: 16 row scales (f32), then per row the eight sub-block sums of the quants split
    // into two int8 planes (sum = 128 * hi + lo): 64 + 16 * 16 bytes.
    // Q8_0: one f32 scale per (block, row): 8 * 16 * 4 bytes.
    // Q6_K: the record of Q4_K (the same Q8_K quantization; the sub-block sums go unused).
    static constexpr int kSide = QT == QMM_Q8_0 ? 512 : 320;
    static constexpr int kBytes = kQuant + kSide;
};

// A row record holds what ONE row contributes to a unit record, in 16-byte pieces that a copy can
// place into the unit record of any tile the row belongs to: the sixteen chunks (sub-block pair b,
// octet o) at 16 (4 b + o), then the side data of the row - Q4_K / Q6_K: the sixteen sum bytes at 256
// and the scale at 272; Q8_0: the eight block scales at 256.
constexpr int kRowUnitBytes = 288;

// ---- launch 1: activation quantizer into the unit records -------------------
// One 16-lane group per (row, unit); lane j holds elements 16j..16j+15 of the
// unit in v, i.e. sub-block j / 2, octets 2 (j % 2) and 2 (j % 2) + 1.  `mr` is
// the row inside the 16-row tile whose record starts at `rec`; with ROW, `rec` is
// the row's own record of the unit (see kRowUnitBytes) and `mr` is unused.
template <int QT, bool ROW = false>
__device__ __forceinline__ void quantize_into_record(const float (&v)[16], int j, int mr, uint8_t* rec) {
    // the lane's first value of largest magnitude (strictly greater: an equal later one does not
    // replace it; a NaN never wins, as with fmaxf), with its sign
    float best = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) best = fabsf(v[i]) > fabsf(best) ? v[i] : best;
    float amax = fabsf(best);
    float scale_mul; // quant = round(v * scale_mul)
    float* side = reinterpret_cast<float*>(rec + (ROW ? 256 : Unit<QT>::kQuant));
    if (QT == QMM_Q4_K) {
        // BlockQ8K::from_float: iscale = -128 / (first value of largest magnitude): the lowest lane
        // that holds the block's maximum decides the sign
        amax = row16_max(amax);
        int key = fabsf(best) == amax ? (j << 1) | (int)(__float_as_uint(best) >> 31) : 0x7fffffff;
        key = row16_min(key);
        float d = 0.0f;
        scale_mul = 0.0f;
        if (amax != 0.0f) {
            scale_mul = __fdiv_rn(-128.0f, (key & 1) ? -amax : amax);
            d = __fdiv_rn(1.0f, scale_mul);
        }
        if (j == 0) side[ROW ? 4 : mr] = d;
    } else {
        // BlockQ8_0::from_float on the lane pair's 32 values
        amax = fmaxf(amax, __int_as_float(dpp<kDppXor1>(__float_as_int(amax))));
        const float d = __fdiv_rn(amax, 127.0f);
        scale_mul = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
        if ((j & 1) == 0) side[ROW ? (j >> 1) : (j >> 1) * 16 + mr] = qmm_f16_bits_to_f32(qmm_f32_to_f16_bits(d));
    }
    uint32_t q[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        int qi[4];
#pragma unroll
        for (int b = 0; b < 4; b++) // both reference quantizers compute scale * value in f32 and round half away
            qi[b] = qmm_round_clamp_i8(QT == QMM_Q4_K ? __fmul_rn(scale_mul, v[4 * w + b]) : __fmul_rn(v[4 * w + b], scale_mul));
        q[w] = qmm_pack_i8x4(qi[0], qi[1], qi[2], qi[3]);
    }
    const int s = j >> 1, oct = 2 * (j & 1);
    if (QT == QMM_Q4_K) {
        int s16 = __builtin_amdgcn_sdot4((int)q[0], 0x01010101, 0, false);
        s16 = __builtin_amdgcn_sdot4((int)q[1], 0x01010101, s16, false);
        s16 = __builtin_amdgcn_sdot4((int)q[2], 0x01010101, s16, false);
        s16 = __builtin_amdgcn_sdot4((int)q[3], 0x01010101, s16, false);
        const int bsum = s16 + dpp<kDppXor1>(s16); // the sub-block's 32 quants
        if ((j & 1) == 0) {
            uint8_t* planes = ROW ? reinterpret_cast<uint8_t*>(side) : reinterpret_cast<uint8_t*>(side + 16) + mr * 16;
            planes[s] = (uint8_t)(bsum & 127);
            planes[8 + s] = (uint8_t)(bsum >> 7);
        }
    }
    uint8_t* dst = ROW ? rec + ((s >> 1) * 4 + oct) * 16 + (s & 1) * 8
                       : rec + (s >> 1) * 1024 + (oct * 16 + mr) * 16 + (s & 1) * 8;
    *reinterpret_cast<uint2*>(dst) = make_uint2(q[0], q[1]);
    *reinterpret_cast<uint2*>(dst + (ROW ? 16 : 256)) = make_uint2(q[2], q[3]);
}

} // namespace

#endif // IZWI_QMM_RECORDS_H
