// Layout conversion (GGUF blocks <-> panel tiles) and bit-exact dequantization.
// All three are load-time / diagnostic operations bounded by HBM bandwidth;
// none is on the per-token path.
#include <hip/hip_runtime.h>

#include "qmm_internal.h"

namespace {

struct Piece {
    int64_t e, row, unit;
    int piece;  // 0 = header, 1 + c = quant chunk c
    bool valid; // false: padding (row >= n or unit >= k_units)
};

// Decodes the index of a 16-byte piece of the tiled buffer.
__device__ inline Piece decode_piece(const QmmLayout& L, int64_t idx) {
    const int64_t pieces_per_panel = (int64_t)L.slots * (1 + L.qc);
    int64_t panel = idx / pieces_per_panel;
    int64_t in_panel = idx - panel * pieces_per_panel;
    Piece p;
    p.piece = (int)(in_panel / L.slots);
    int slot = (int)(in_panel - (int64_t)p.piece * L.slots);
    int64_t kg = panel % L.k_groups;
    int64_t rt_all = panel / L.k_groups;
    p.e = rt_all / L.row_tiles;
    int64_t rt = rt_all - p.e * L.row_tiles;
    p.row = rt * QMM_PANEL_ROWS + (slot & 15);
    p.unit = kg * L.s + (slot >> 4);
    p.valid = p.row < L.n && p.unit < L.k_units;
    return p;
}

// Byte offset of a 16-byte piece of (e, row, unit) inside the tiled buffer.
__device__ inline int64_t piece_offset(const QmmLayout& L, int64_t e, int64_t row, int64_t unit,
                                       int piece) {
    int64_t rt = row / QMM_PANEL_ROWS, r = row % QMM_PANEL_ROWS;
    int64_t kg = unit / L.s, us = unit % L.s;
    int64_t panel = (e * L.row_tiles + rt) * L.k_groups + kg;
    return panel * L.panel_bytes + ((int64_t)piece * L.slots + us * 16 + r) * 16;
}

__global__ void repack_q4k_kernel(QmmLayout L, const uint8_t* __restrict__ src,
                                  uint8_t* __restrict__ dst, int64_t n_pieces) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_pieces) return;
    Piece p = decode_piece(L, idx);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (p.valid) {
        int64_t blk = (p.e * L.n + p.row) * L.k_units + p.unit;
        v = *reinterpret_cast<const uint4*>(src + blk * 144 + 16 * p.piece);
    }
    *reinterpret_cast<uint4*>(dst + idx * 16) = v;
}

__global__ void repack_q80_kernel(QmmLayout L, const uint8_t* __restrict__ src,
                                  uint8_t* __restrict__ dst, int64_t n_pieces) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_pieces) return;
    Piece p = decode_piece(L, idx);
    const int64_t blocks_per_row = L.k / 32;
    union {
        uint4 v;
        uint16_t h[8];
    } u;
    u.v = make_uint4(0, 0, 0, 0);
    if (p.valid) {
        int64_t row_blk = (p.e * L.n + p.row) * blocks_per_row;
        if (p.piece == 0) {
            for (int b = 0; b < 8; b++) {
                int64_t kb = p.unit * 8 + b;
                if (kb < blocks_per_row)
                    u.h[b] = *reinterpret_cast<const uint16_t*>(src + (row_blk + kb) * 34);
            }
        } else {
            int c = p.piece - 1;
            int64_t kb = p.unit * 8 + (c >> 1);
            if (kb < blocks_per_row) {
                const uint16_t* s =
                    reinterpret_cast<const uint16_t*>(src + (row_blk + kb) * 34 + 2 + 16 * (c & 1));
                for (int i = 0; i < 8; i++) u.h[i] = s[i];
            }
        }
    }
    *reinterpret_cast<uint4*>(dst + idx * 16) = u.v;
}

__global__ void unpack_q4k_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                  uint8_t* __restrict__ dst, int64_t n_chunks) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // 16-byte chunk of native bytes
    if (idx >= n_chunks) return;
    int64_t blk = idx / 9;
    int piece = (int)(idx - blk * 9);
    int64_t unit = blk % L.k_units;
    int64_t row_all = blk / L.k_units;
    int64_t e = row_all / L.n, row = row_all % L.n;
    *reinterpret_cast<uint4*>(dst + idx * 16) =
        *reinterpret_cast<const uint4*>(tiled + piece_offset(L, e, row, unit, piece));
}

__global__ void unpack_q80_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                  uint8_t* __restrict__ dst, int64_t n_blocks) {
    int64_t blk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // native 34-byte block
    if (blk >= n_blocks) return;
    const int64_t blocks_per_row = L.k / 32;
    int64_t kb = blk % blocks_per_row;
    int64_t row_all = blk / blocks_per_row;
    int64_t e = row_all / L.n, row = row_all % L.n;
    int64_t unit = kb / 8;
    int b = (int)(kb % 8);
    uint16_t* out = reinterpret_cast<uint16_t*>(dst + blk * 34);
    out[0] = reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, e, row, unit, 0))[b];
    for (int h = 0; h < 2; h++) {
        const uint16_t* s =
            reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, e, row, unit, 1 + 2 * b + h));
        for (int i = 0; i < 8; i++) out[1 + 8 * h + i] = s[i];
    }
}

// One thread per 16-byte quant chunk; f32 products are rounded after each
// operation (__fmul_rn / __fsub_rn never contract into an FMA).
__global__ void dequant_q4k_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                   float* __restrict__ out, int64_t n_chunks) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_chunks) return;
    int c = (int)(idx & 7);
    int64_t blk = idx >> 3;
    int64_t unit = blk % L.k_units;
    int64_t row_all = blk / L.k_units;
    int64_t e = row_all / L.n, row = row_all % L.n;
    uint4 hdr = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, e, row, unit, 0));
    uint4 qv = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, e, row, unit, 1 + c));
    float d = qmm_f16_bits_to_f32((uint16_t)(hdr.x & 0xffffu));
    float dmin = qmm_f16_bits_to_f32((uint16_t)(hdr.x >> 16));
    uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
    qmm_unpack_q4k_scales(hdr.y, hdr.z, hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
    int g = c >> 1, h = c & 1;
    int s0 = 2 * g, s1 = 2 * g + 1;
    float d1 = __fmul_rn(d, (float)qmm_byte_of(sc_lo, sc_hi, s0));
    float m1 = __fmul_rn(dmin, (float)qmm_byte_of(mn_lo, mn_hi, s0));
    float d2 = __fmul_rn(d, (float)qmm_byte_of(sc_lo, sc_hi, s1));
    float m2 = __fmul_rn(dmin, (float)qmm_byte_of(mn_lo, mn_hi, s1));
    float* o = out + row_all * L.k + unit * 256 + 64 * g + 16 * h;
    uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            uint32_t byte = (w[j] >> (8 * b)) & 0xffu;
            o[4 * j + b] = __fsub_rn(__fmul_rn(d1, (float)(byte & 0xF)), m1);
            o[32 + 4 * j + b] = __fsub_rn(__fmul_rn(d2, (float)(byte >> 4)), m2);
        }
    }
}

__global__ void dequant_q80_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                   float* __restrict__ out, int64_t n_chunks) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // 16-byte half block
    if (idx >= n_chunks) return;
    const int64_t blocks_per_row = L.k / 32;
    int h = (int)(idx & 1);
    int64_t blk = idx >> 1;
    int64_t kb = blk % blocks_per_row;
    int64_t row_all = blk / blocks_per_row;
    int64_t e = row_all / L.n, row = row_all % L.n;
    int64_t unit = kb / 8;
    int b = (int)(kb % 8);
    uint16_t dbits = reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, e, row, unit, 0))[b];
    float d = qmm_f16_bits_to_f32(dbits);
    uint4 qv = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, e, row, unit, 1 + 2 * b + h));
    float* o = out + row_all * L.k + kb * 32 + 16 * h;
    uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
            o[4 * j + i] = __fmul_rn((float)(int8_t)((w[j] >> (8 * i)) & 0xffu), d);
}

// Q6_K block: ql[128] | qh[64] | scales[16] | d (f16) at bytes 0, 128, 192, 208.  The 210-byte
// block is only 2-byte aligned, so the pieces are gathered as 16-bit words.
// Tiled pieces: 0 = scales, 1..8 = ql, 9..12 = qh, 13 = d followed by zeros.
__device__ inline int q6k_piece_src(int piece) {
    return piece == 0 ? 192 : (piece <= 8 ? 16 * (piece - 1) : (piece <= 12 ? 128 + 16 * (piece - 9) : 208));
}

__global__ void repack_q6k_kernel(QmmLayout L, const uint8_t* __restrict__ src,
                                  uint8_t* __restrict__ dst, int64_t n_pieces) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_pieces) return;
    Piece p = decode_piece(L, idx);
    union {
        uint4 v;
        uint16_t h[8];
    } u;
    u.v = make_uint4(0, 0, 0, 0);
    if (p.valid) {
        int64_t blk = (p.e * L.n + p.row) * L.k_units + p.unit;
        const uint16_t* s = reinterpret_cast<const uint16_t*>(src + blk * 210 + q6k_piece_src(p.piece));
        if (p.piece == 13) u.h[0] = s[0];
        else
            for (int i = 0; i < 8; i++) u.h[i] = s[i];
    }
    *reinterpret_cast<uint4*>(dst + idx * 16) = u.v;
}

__global__ void unpack_q6k_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                  uint8_t* __restrict__ dst, int64_t n_items) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // (block, piece)
    if (idx >= n_items) return;
    int64_t blk = idx / 14;
    int piece = (int)(idx - blk * 14);
    int64_t unit = blk % L.k_units;
    int64_t row_all = blk / L.k_units;
    int64_t e = row_all / L.n, row = row_all % L.n;
    const uint16_t* s = reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, e, row, unit, piece));
    uint16_t* out = reinterpret_cast<uint16_t*>(dst + blk * 210 + q6k_piece_src(piece));
    if (piece == 13) out[0] = s[0];
    else
        for (int i = 0; i < 8; i++) out[i] = s[i];
}

// One thread per (block, half of 128, l < 32): the elements l, l + 32, l + 64, l + 96 of the
// half, d * scale * (q - 32) evaluated left to right with a rounding after each product.
__global__ void dequant_q6k_tiled_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                         float* __restrict__ out, int64_t n_items) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_items) return;
    const int l = (int)(idx & 31), half = (int)(idx >> 5) & 1, is = l >> 4;
    int64_t blk = idx >> 6;
    int64_t unit = blk % L.k_units;
    int64_t row_all = blk / L.k_units;
    int64_t e = row_all / L.n, row = row_all % L.n;
    const int8_t* sc = reinterpret_cast<const int8_t*>(tiled + piece_offset(L, e, row, unit, 0)) + 8 * half;
    const uint8_t qa = tiled[piece_offset(L, e, row, unit, 1 + 4 * half + (l >> 4)) + (l & 15)];      // ql[64 half + l]
    const uint8_t qb = tiled[piece_offset(L, e, row, unit, 1 + 4 * half + 2 + (l >> 4)) + (l & 15)];  // ql[64 half + 32 + l]
    const uint8_t qh = tiled[piece_offset(L, e, row, unit, 9 + 2 * half + (l >> 4)) + (l & 15)];
    const float d = qmm_f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, e, row, unit, 13)));
    const int q1 = (int)((qa & 0xF) | ((qh & 3) << 4)) - 32;
    const int q2 = (int)((qb & 0xF) | (((qh >> 2) & 3) << 4)) - 32;
    const int q3 = (int)((qa >> 4) | (((qh >> 4) & 3) << 4)) - 32;
    const int q4 = (int)((qb >> 4) | (((qh >> 6) & 3) << 4)) - 32;
    float* y = out + row_all * L.k + unit * 256 + 128 * half;
    y[l] = __fmul_rn(__fmul_rn(d, (float)sc[is]), (float)q1);
    y[l + 32] = __fmul_rn(__fmul_rn(d, (float)sc[is + 2]), (float)q2);
    y[l + 64] = __fmul_rn(__fmul_rn(d, (float)sc[is + 4]), (float)q3);
    y[l + 96] = __fmul_rn(__fmul_rn(d, (float)sc[is + 6]), (float)q4);
}

// ---- selected rows of the dequantized matrix (the embedding lookup) -----------------------------
// out[i, :] = row rows[i] of the first matrix, the arithmetic of the kernels above value for value,
// stored as f32 or rounded to bf16 (nearest even, what a cast of the f32 table gives).  A row id
// outside [0, n) gives a row of zeros.
__device__ __forceinline__ void store_row_value(void* out, int out_bf16, int64_t i, float v) {
    if (out_bf16) reinterpret_cast<uint16_t*>(out)[i] = qmm_f32_to_bf16_bits(v);
    else reinterpret_cast<float*>(out)[i] = v;
}

__global__ void dequant_rows_q4k_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                        const int32_t* __restrict__ rows, void* __restrict__ out, int out_bf16,
                                        int64_t n_chunks) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_chunks) return;
    int c = (int)(idx & 7);
    int64_t blk = idx >> 3;
    int64_t unit = blk % L.k_units, ri = blk / L.k_units;
    const int64_t row = rows[ri];
    const bool ok = row >= 0 && row < L.n;
    const int64_t r = ok ? row : 0;
    uint4 hdr = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, 0, r, unit, 0));
    uint4 qv = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, 0, r, unit, 1 + c));
    float d = qmm_f16_bits_to_f32((uint16_t)(hdr.x & 0xffffu));
    float dmin = qmm_f16_bits_to_f32((uint16_t)(hdr.x >> 16));
    uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
    qmm_unpack_q4k_scales(hdr.y, hdr.z, hdr.w, sc_lo, sc_hi, mn_lo, mn_hi);
    int g = c >> 1, h = c & 1;
    int s0 = 2 * g, s1 = 2 * g + 1;
    float d1 = __fmul_rn(d, (float)qmm_byte_of(sc_lo, sc_hi, s0));
    float m1 = __fmul_rn(dmin, (float)qmm_byte_of(mn_lo, mn_hi, s0));
    float d2 = __fmul_rn(d, (float)qmm_byte_of(sc_lo, sc_hi, s1));
    float m2 = __fmul_rn(dmin, (float)qmm_byte_of(mn_lo, mn_hi, s1));
    const int64_t o = ri * L.k + unit * 256 + 64 * g + 16 * h;
    uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            uint32_t byte = (w[j] >> (8 * b)) & 0xffu;
            store_row_value(out, out_bf16, o + 4 * j + b, ok ? __fsub_rn(__fmul_rn(d1, (float)(byte & 0xF)), m1) : 0.0f);
            store_row_value(out, out_bf16, o + 32 + 4 * j + b, ok ? __fsub_rn(__fmul_rn(d2, (float)(byte >> 4)), m2) : 0.0f);
        }
    }
}

__global__ void dequant_rows_q80_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                        const int32_t* __restrict__ rows, void* __restrict__ out, int out_bf16,
                                        int64_t n_chunks) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // 16-byte half block
    if (idx >= n_chunks) return;
    const int64_t blocks_per_row = L.k / 32;
    int h = (int)(idx & 1);
    int64_t blk = idx >> 1;
    int64_t kb = blk % blocks_per_row, ri = blk / blocks_per_row;
    const int64_t row = rows[ri];
    const bool ok = row >= 0 && row < L.n;
    const int64_t r = ok ? row : 0;
    int64_t unit = kb / 8;
    int b = (int)(kb % 8);
    uint16_t dbits = reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, 0, r, unit, 0))[b];
    float d = qmm_f16_bits_to_f32(dbits);
    uint4 qv = *reinterpret_cast<const uint4*>(tiled + piece_offset(L, 0, r, unit, 1 + 2 * b + h));
    const int64_t o = ri * L.k + kb * 32 + 16 * h;
    uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
            store_row_value(out, out_bf16, o + 4 * j + i, ok ? __fmul_rn((float)(int8_t)((w[j] >> (8 * i)) & 0xffu), d) : 0.0f);
}

__global__ void dequant_rows_q6k_kernel(QmmLayout L, const uint8_t* __restrict__ tiled,
                                        const int32_t* __restrict__ rows, void* __restrict__ out, int out_bf16,
                                        int64_t n_items) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_items) return;
    const int l = (int)(idx & 31), half = (int)(idx >> 5) & 1, is = l >> 4;
    int64_t blk = idx >> 6;
    int64_t unit = blk % L.k_units, ri = blk / L.k_units;
    const int64_t row = rows[ri];
    const bool ok = row >= 0 && row < L.n;
    const int64_t r = ok ? row : 0;
    const int8_t* sc = reinterpret_cast<const int8_t*>(tiled + piece_offset(L, 0, r, unit, 0)) + 8 * half;
    const uint8_t qa = tiled[piece_offset(L, 0, r, unit, 1 + 4 * half + (l >> 4)) + (l & 15)];
    const uint8_t qb = tiled[piece_offset(L, 0, r, unit, 1 + 4 * half + 2 + (l >> 4)) + (l & 15)];
    const uint8_t qh = tiled[piece_offset(L, 0, r, unit, 9 + 2 * half + (l >> 4)) + (l & 15)];
    const float d = qmm_f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(tiled + piece_offset(L, 0, r, unit, 13)));
    const int q1 = (int)((qa & 0xF) | ((qh & 3) << 4)) - 32;
    const int q2 = (int)((qb & 0xF) | (((qh >> 2) & 3) << 4)) - 32;
    const int q3 = (int)((qa >> 4) | (((qh >> 4) & 3) << 4)) - 32;
    const int q4 = (int)((qb >> 4) | (((qh >> 6) & 3) << 4)) - 32;
    const int64_t y = ri * L.k + unit * 256 + 128 * half;
    store_row_value(out, out_bf16, y + l, ok ? __fmul_rn(__fmul_rn(d, (float)sc[is]), (float)q1) : 0.0f);
    store_row_value(out, out_bf16, y + l + 32, ok ? __fmul_rn(__fmul_rn(d, (float)sc[is + 2]), (float)q2) : 0.0f);
    store_row_value(out, out_bf16, y + l + 64, ok ? __fmul_rn(__fmul_rn(d, (float)sc[is + 4]), (float)q3) : 0.0f);
    store_row_value(out, out_bf16, y + l + 96, ok ? __fmul_rn(__fmul_rn(d, (float)sc[is + 6]), (float)q4) : 0.0f);
}

inline unsigned grid_for(int64_t n, int block) { return (unsigned)((n + block - 1) / block); }

} // namespace

hipError_t qmm_launch_repack(const QmmLayout& L, const void* native, void* tiled,
                             hipStream_t stream) {
    int64_t n_pieces = L.n_stacked * L.matrix_bytes / 16;
    if (n_pieces == 0) return hipSuccess;
    if (L.dtype == QMM_Q4_K)
        repack_q4k_kernel<<<grid_for(n_pieces, 256), 256, 0, stream>>>(
            L, (const uint8_t*)native, (uint8_t*)tiled, n_pieces);
    else if (L.dtype == QMM_Q6_K)
        repack_q6k_kernel<<<grid_for(n_pieces, 256), 256, 0, stream>>>(
            L, (const uint8_t*)native, (uint8_t*)tiled, n_pieces);
    else
        repack_q80_kernel<<<grid_for(n_pieces, 256), 256, 0, stream>>>(
            L, (const uint8_t*)native, (uint8_t*)tiled, n_pieces);
    return hipGetLastError();
}

hipError_t qmm_launch_unpack(const QmmLayout& L, const void* tiled, void* native,
                             hipStream_t stream) {
    if (L.dtype == QMM_Q4_K) {
        int64_t n_chunks = L.n_stacked * L.n * L.k_units * 9;
        if (n_chunks == 0) return hipSuccess;
        unpack_q4k_kernel<<<grid_for(n_chunks, 256), 256, 0, stream>>>(
            L, (const uint8_t*)tiled, (uint8_t*)native, n_chunks);
    } else if (L.dtype == QMM_Q6_K) {
        int64_t n_items = L.n_stacked * L.n * L.k_units * 14;
        if (n_items == 0) return hipSuccess;
        unpack_q6k_kernel<<<grid_for(n_items, 256), 256, 0, stream>>>(
            L, (const uint8_t*)tiled, (uint8_t*)native, n_items);
    } else {
        int64_t n_blocks = L.n_stacked * L.n * (L.k / 32);
        if (n_blocks == 0) return hipSuccess;
        unpack_q80_kernel<<<grid_for(n_blocks, 256), 256, 0, stream>>>(
            L, (const uint8_t*)tiled, (uint8_t*)native, n_blocks);
    }
    return hipGetLastError();
}

hipError_t qmm_launch_dequant(const QmmLayout& L, const void* tiled, float* out,
                              hipStream_t stream) {
    if (L.dtype == QMM_Q4_K) {
        int64_t n_chunks = L.n_stacked * L.n * L.k_units * 8;
        if (n_chunks == 0) return hipSuccess;
        dequant_q4k_kernel<<<grid_for(n_chunks, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled,
                                                                        out, n_chunks);
    } else if (L.dtype == QMM_Q6_K) {
        int64_t n_items = L.n_stacked * L.n * L.k_units * 64;
        if (n_items == 0) return hipSuccess;
        dequant_q6k_tiled_kernel<<<grid_for(n_items, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled,
                                                                              out, n_items);
    } else {
        int64_t n_chunks = L.n_stacked * L.n * (L.k / 32) * 2;
        if (n_chunks == 0) return hipSuccess;
        dequant_q80_kernel<<<grid_for(n_chunks, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled,
                                                                        out, n_chunks);
    }
    return hipGetLastError();
}

hipError_t qmm_launch_dequant_rows(const QmmLayout& L, const void* tiled, const int32_t* rows, int64_t n_rows,
                                   void* out, int out_bf16, hipStream_t stream) {
    if (n_rows <= 0 || L.k == 0) return hipSuccess;
    if (L.dtype == QMM_Q4_K) {
        const int64_t n_chunks = n_rows * L.k_units * 8;
        dequant_rows_q4k_kernel<<<grid_for(n_chunks, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled, rows, out,
                                                                             out_bf16, n_chunks);
    } else if (L.dtype == QMM_Q6_K) {
        const int64_t n_items = n_rows * L.k_units * 64;
        dequant_rows_q6k_kernel<<<grid_for(n_items, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled, rows, out,
                                                                            out_bf16, n_items);
    } else {
        const int64_t n_chunks = n_rows * (L.k / 32) * 2;
        dequant_rows_q80_kernel<<<grid_for(n_chunks, 256), 256, 0, stream>>>(L, (const uint8_t*)tiled, rows, out,
                                                                             out_bf16, n_chunks);
    }
    return hipGetLastError();
}

// ---- QTensor::quantize for Q4_K: f32 rows -> GGUF block bytes -----------------------------------
// candle-core k_quants.rs `BlockQ4K::from_float` with utils.rs `make_qkx1_quants(15, 5, ..)`: a
// thread owns one sub-block of 32 values and runs the search exactly as the scalar code does (the
// same f32 operations in the same order: the sums over the 32 values are sequential), the eight
// threads of a block share their scale and min through wave shuffles, and the quants of the block
// pass through LDS on their way into the nibble-pair layout.  Load-time work, not a hot path.
namespace {
__device__ __forceinline__ int nearest_int_f(float v) { return (int)roundf(v); } // half away from zero

__global__ __launch_bounds__(256) void quantize_q4k_weights_kernel(const float* __restrict__ x, int64_t n_blocks,
                                                                   uint8_t* __restrict__ out) {
    __shared__ uint8_t l_sh[32][256];
    const int64_t sub = (int64_t)blockIdx.x * 256 + threadIdx.x; // sub-block of 32 values
    const int64_t blk = sub >> 3;
    const int j = (int)(threadIdx.x & 7), bl = (int)(threadIdx.x >> 3);
    const bool live = blk < n_blocks;
    float v[32];
#pragma unroll
    for (int i = 0; i < 32; i++) v[i] = live ? x[sub * 32 + i] : 0.0f;
    // make_qkx1_quants(nmax = 15, ntry = 5)
    float scale = 0.0f, neg_min = 0.0f;
    {
        uint8_t l[32];
#pragma unroll
        for (int i = 0; i < 32; i++) l[i] = 0;
        float mn = v[0], mx = v[0];
#pragma unroll
        for (int i = 1; i < 32; i++) {
            if (v[i] < mn) mn = v[i];
            if (v[i] > mx) mx = v[i];
        }
        if (mx != mn) {
            if (mn > 0.0f) mn = 0.0f;
            float iscale = 15.0f / (mx - mn);
            scale = 1.0f / iscale;
            for (int t = 0; t < 5; t++) {
                float sumlx = 0.0f;
                int suml2 = 0;
                bool did_change = false;
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    int li = nearest_int_f(iscale * (v[i] - mn));
                    li = li < 0 ? 0 : (li > 15 ? 15 : li);
                    if ((uint8_t)li != l[i]) l[i] = (uint8_t)li, did_change = true;
                    sumlx += (v[i] - mn) * (float)li;
                    suml2 += li * li;
                }
                scale = sumlx / (float)suml2;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 32; i++) sum += v[i] - scale * (float)l[i];
                mn = sum / 32.0f;
                if (mn > 0.0f) mn = 0.0f;
                iscale = 1.0f / scale;
                if (!did_change) break;
            }
            neg_min = -mn;
        }
    }
    // the block's largest scale and min (the eight threads of a block are neighbours in a wave)
    // (the scalar code starts both maxima at +0.0 and replaces them on `>`: a min of -0.0 stays +0.0)
    float max_scale = scale > 0.0f ? scale : 0.0f, max_min = neg_min > 0.0f ? neg_min : 0.0f;
#pragma unroll
    for (int d = 1; d < 8; d <<= 1) {
        const float os = __shfl_xor(max_scale, d), om = __shfl_xor(max_min, d);
        max_scale = os > max_scale ? os : max_scale;
        max_min = om > max_min ? om : max_min;
    }
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    int ls = nearest_int_f(inv_scale * scale), lm = nearest_int_f(inv_min * neg_min);
    ls = ls > 63 ? 63 : ls;
    lm = lm > 63 ? 63 : lm;
    const uint16_t d_bits = qmm_f32_to_f16_bits(max_scale / 63.0f), dmin_bits = qmm_f32_to_f16_bits(max_min / 63.0f);
    // quants against the block's rounded scales (what get_scale_min_k4 returns is ls, lm again)
    const float d = qmm_f16_bits_to_f32(d_bits) * (float)ls;
    if (d != 0.0f) {
        const float dm = qmm_f16_bits_to_f32(dmin_bits) * (float)lm;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            int lv = nearest_int_f((v[i] + dm) / d);
            l_sh[bl][32 * j + i] = (uint8_t)(lv < 0 ? 0 : (lv > 15 ? 15 : lv));
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) l_sh[bl][32 * j + i] = 0;
    }
    // the 12 scale bytes: sub-blocks 0..3 hold their six bits whole, 4..7 split them
    int ls_all[8], lm_all[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {
        ls_all[q] = __shfl(ls, (int)((threadIdx.x & 63) & ~7) + q);
        lm_all[q] = __shfl(lm, (int)((threadIdx.x & 63) & ~7) + q);
    }
    __syncthreads();
    if (!live) return;
    uint8_t* b = out + blk * 144;
    if (j == 0) {
        uint8_t sc[12];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            sc[q] = (uint8_t)(ls_all[q] | ((ls_all[q + 4] >> 4) << 6));
            sc[q + 4] = (uint8_t)(lm_all[q] | ((lm_all[q + 4] >> 4) << 6));
            sc[q + 8] = (uint8_t)((ls_all[q + 4] & 0xF) | ((lm_all[q + 4] & 0xF) << 4));
        }
        b[0] = (uint8_t)(d_bits & 0xff), b[1] = (uint8_t)(d_bits >> 8);
        b[2] = (uint8_t)(dmin_bits & 0xff), b[3] = (uint8_t)(dmin_bits >> 8);
#pragma unroll
        for (int q = 0; q < 12; q++) b[4 + q] = sc[q];
    }
    // qs: byte (c * 32 + i) = l[64 c + i] | l[64 c + 32 + i] << 4; thread j packs bytes 16 j .. 16 j + 15
#pragma unroll
    for (int q = 0; q < 16; q++) {
        const int byte = 16 * j + q, c = byte >> 5, i = byte & 31;
        b[16 + byte] = (uint8_t)(l_sh[bl][64 * c + i] | (l_sh[bl][64 * c + 32 + i] << 4));
    }
}
} // namespace

hipError_t qmm_launch_quantize_q4k_weights(const float* x, int64_t n_blocks, void* out, hipStream_t stream) {
    if (n_blocks <= 0) return hipSuccess;
    const int64_t wgs = (n_blocks * 8 + 255) / 256;
    if (wgs > 0x7fffffff) return hipErrorInvalidValue;
    quantize_q4k_weights_kernel<<<(unsigned)wgs, 256, 0, stream>>>(x, n_blocks, (uint8_t*)out);
    return hipGetLastError();
}
