// Device-resident weight layout shared by host and kernels.
//
// GGUF stores a [n, k] weight as rows of consecutive blocks.  Q8_0's 34-byte
// block is only 2-byte aligned and Q4_K's 144-byte block interleaves a header
// with nibbles, so neither allows one contiguous 1 KiB wavefront load of
// 16 bytes per lane.  weight_create therefore re-tiles the bytes (no byte is
// added, dropped or changed except zero padding of ragged edges):
//
//   unit   = 256 consecutive k-elements of one row
//            Q4_K: one block   = 16 B header (d, dmin, 12 scale bytes) + 8 x 16 B of nibbles
//            Q8_0: eight blocks = 16 B header (8 f16 scales)           + 16 x 16 B of int8
//            Q6_K: one block   = 16 B header (16 int8 scales) + 8 x 16 B of low nibbles (ql)
//                                + 4 x 16 B of high bit pairs (qh) + 16 B holding d (f16) and
//                                14 zero bytes: 224 B for the block's 210
//   panel  = 16 rows x S units (S = 1..4), slot = unit_in_panel * 16 + row_in_panel
//            bytes: [slots x 16 B headers][QC x (slots x 16 B quant chunks)]
//            so that lane `slot` of a wavefront reads its header and its c-th
//            quant chunk with one fully coalesced 16 B/lane load each.
//   order  = panels of one row-tile (16 rows) are consecutive along k, row-tiles
//            consecutive along n, experts (stacked handles) outermost.
#pragma once
#include <stdint.h>

#define QMM_Q8_0 8
#define QMM_Q4_K 12
#define QMM_Q6_K 14

#define QMM_UNIT_ELEMS 256
#define QMM_PANEL_ROWS 16

struct QmmLayout {
    int dtype;           // QMM_Q8_0 / QMM_Q4_K / QMM_Q6_K
    int s;               // units per panel along k (1..4)
    int qc;              // 16-byte chunks per unit after the header: 8 (Q4_K), 16 (Q8_0), 13 (Q6_K)
    int slots;           // 16 * s
    int64_t n, k;        // logical shape of one matrix
    int64_t n_stacked;   // matrices in the handle
    int64_t k_units;     // ceil(k / 256)
    int64_t row_tiles;   // ceil(n / 16)
    int64_t k_groups;    // ceil(k_units / s): panels per row-tile
    int64_t panel_bytes; // slots * 16 * (1 + qc)
    int64_t matrix_bytes; // row_tiles * k_groups * panel_bytes
};

static inline int qmm_block_elems(int dtype) { return dtype == QMM_Q8_0 ? 32 : 256; }
static inline int qmm_block_bytes(int dtype) { return dtype == QMM_Q8_0 ? 34 : (dtype == QMM_Q6_K ? 210 : 144); }

static inline QmmLayout qmm_make_layout(int dtype, int64_t n_stacked, int64_t n, int64_t k) {
    QmmLayout L;
    L.dtype = dtype;
    L.n = n;
    L.k = k;
    L.n_stacked = n_stacked;
    L.k_units = (k + QMM_UNIT_ELEMS - 1) / QMM_UNIT_ELEMS;
    L.row_tiles = (n + QMM_PANEL_ROWS - 1) / QMM_PANEL_ROWS;
    int s = 4;
    if (L.k_units % 4 == 0) s = 4;
    else if (L.k_units % 3 == 0) s = 3;
    else if (L.k_units % 2 == 0) s = 2;
    else if (L.k_units == 1) s = 1;
    L.s = s;
    L.qc = dtype == QMM_Q8_0 ? 16 : (dtype == QMM_Q6_K ? 13 : 8);
    L.slots = 16 * s;
    L.k_groups = (L.k_units + s - 1) / s;
    L.panel_bytes = (int64_t)L.slots * 16 * (1 + L.qc);
    L.matrix_bytes = L.row_tiles * L.k_groups * L.panel_bytes;
    return L;
}
