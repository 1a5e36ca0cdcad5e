/*
 * CPU oracle for the quantized linear-layer path (TEST INFRASTRUCTURE ONLY).
 *
 * This file is a plain-C restatement of the scalar CPU algorithm of the
 * third-party crate candle-core 0.10.2 (pinned by the reference's
 * Cargo.lock:722-725), which holds all of the arithmetic behind the
 * reference's `QMatMul::forward` call sites
 * (crates/izwi-core/src/models/architectures/qwen3/core.rs:712,812,884).
 * The crate's source is not shipped with the reference, so every function
 * below restates the crate's published algorithm (module `quantized`,
 * files k_quants.rs / utils.rs / mod.rs) and is pinned by the checks listed
 * beside it in tests/test_oracle_*.py.  Nothing in the product library may
 * link, import or call this file: only tests/, the smoke check and the
 * `cpu_baseline` leg of bench.py use it, as the checker / timed baseline.
 *
 * Pin status (what independent evidence fixes each function):
 *   f16 <-> f32 conversion ......... exhaustive against numpy.float16
 *   dequantize_row_q8_0 / q4_k ..... hand-built blocks + numpy restatement
 *   quantize_row_q8_0 .............. invariants (|w-w^| <= d/2, max|q|=127) and
 *                                    the reference test's case (core.rs:3099-3142)
 *   quantize_row_q8_k .............. invariants (q = -128 at the extreme, bsums)
 *   quantize_row_q4_k, make_qkx1_quants
 *                                    closed-form vectors (tests/golden/q4k_quantizer_cases.json,
 *                                    worked out in exact rational arithmetic by the generator
 *                                    beside it): sub-blocks on an exact 16-level grid must come
 *                                    back as (step, -min) and whole blocks byte for byte, an
 *                                    all-positive block (min clamps to 0), a constant sub-block,
 *                                    a three-pass and a five-pass (cut-off) refinement, a
 *                                    round-half-away tie; plus invariants on random data
 *   vec_dot_q8_0_q8_0 / q4_k_q8_k .. integer brute force + f64 bound + the
 *                                    reference test's known answers
 *   dequantize_row_q6_k ............ hand-built block with all 256 closed-form values +
 *                                    numpy restatement of the public block format
 *   vec_dot_q6_k_q8_k .............. integer brute force from the numpy restatement of the
 *                                    block format + f64 bound; the reference's tests hold no
 *                                    Q6_K vector, so both Q6_K functions stay "parity
 *                                    unpinned" against the crate's own bytes
 *   moe_* .......................... no counterpart in the reference (it has no
 *                                    MoE code); defined by the build's config and
 *                                    pinned by brute force (numpy stable argsort; the
 *                                    forward, also with a down stack of its own block
 *                                    type, by the per-pair composition of qmatmul).
 *
 * Compile with -ffp-contract=off: every f32 expression below is meant to round
 * after each operation, as the Rust original does.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK8_0 32
#define QK_K 256

typedef struct {
    uint16_t d; /* f16 bits */
    int8_t qs[QK8_0];
} __attribute__((packed)) block_q8_0; /* 34 bytes */

typedef struct {
    uint16_t d;    /* f16 bits, super-block scale for quantized scales */
    uint16_t dmin; /* f16 bits, super-block scale for quantized mins */
    uint8_t scales[12];
    uint8_t qs[QK_K / 2];
} __attribute__((packed)) block_q4_k; /* 144 bytes */

typedef struct {
    float d;
    int8_t qs[QK_K];
    int16_t bsums[QK_K / 16];
} __attribute__((packed)) block_q8_k; /* 292 bytes */

typedef struct {
    uint8_t ql[QK_K / 2];     /* low 4 bits of the 6-bit quants */
    uint8_t qh[QK_K / 4];     /* high 2 bits */
    int8_t scales[QK_K / 16]; /* one 8-bit scale per 16 elements */
    uint16_t d;               /* f16 bits, super-block scale */
} __attribute__((packed)) block_q6_k; /* 210 bytes */

_Static_assert(sizeof(block_q6_k) == 210, "Q6_K block is 210 bytes");
_Static_assert(sizeof(block_q8_0) == 34, "Q8_0 block is 34 bytes");
_Static_assert(sizeof(block_q4_k) == 144, "Q4_K block is 144 bytes");
_Static_assert(sizeof(block_q8_k) == 292, "Q8_K block is 292 bytes");

/* ------------------------------------------------------------------ f16 -- */
/* half 2.7.1 `f16::to_f32` / `f16::from_f32` (Cargo.lock:2931-2934): IEEE
 * binary16, conversion from f32 rounds to nearest even, NaN stays NaN. */
float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oracle_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) { /* inf / nan */
        uint32_t nan_bit = man ? 0x200u : 0;
        return (uint16_t)(sign | 0x7c00u | nan_bit | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
    if (e <= 0) {                                  /* subnormal or zero */
        if (e < -10) return (uint16_t)sign;        /* too small, rounds to 0 */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t round_bit = 1u << (shift - 1);
        if ((man & round_bit) && ((man & (3u * round_bit - 1u)) != 0)) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = sign | ((uint32_t)e << 10) | (man >> 13);
    uint32_t round_bit = 0x1000u;
    if ((man & round_bit) && ((man & (3u * round_bit - 1u)) != 0)) half++; /* may carry into exp */
    return (uint16_t)half;
}

/* Rust `f32::round`: half away from zero == C roundf. */
static inline int32_t nearest_int(float v) { return (int32_t)roundf(v); }

/* -------------------------------------------------------------- Q8_0 ----- */
/* candle-core k_quants.rs, `impl GgmlType for BlockQ8_0 :: to_float`. */
void oracle_dequantize_row_q8_0(const block_q8_0* x, float* y, int64_t k) {
    int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float d = oracle_f16_to_f32(x[i].d);
        for (int j = 0; j < QK8_0; j++) y[i * QK8_0 + j] = (float)x[i].qs[j] * d;
    }
}

/* candle-core k_quants.rs, `BlockQ8_0::from_float`. */
void oracle_quantize_row_q8_0(const float* x, block_q8_0* y, int64_t k) {
    int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        const float* xs = x + i * QK8_0;
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) {
            float a = fabsf(xs[j]);
            if (a > amax) amax = a;
        }
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        y[i].d = oracle_f32_to_f16(d);
        for (int j = 0; j < QK8_0; j++) {
            float v = roundf(xs[j] * id);
            /* Rust `as i8` saturates */
            if (v > 127.0f) v = 127.0f;
            if (v < -128.0f) v = -128.0f;
            y[i].qs[j] = (int8_t)v;
        }
    }
}

/* candle-core k_quants.rs, `BlockQ8_0::vec_dot_unopt` (the scalar path that a
 * default x86 release build of the reference runs: no target-cpu flags are set
 * anywhere in the reference's build files). */
float oracle_vec_dot_q8_0_q8_0(int64_t k, const block_q8_0* w, const block_q8_0* a) {
    int64_t nb = k / QK8_0;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sumi = 0;
        for (int j = 0; j < QK8_0; j++) sumi += (int32_t)w[i].qs[j] * (int32_t)a[i].qs[j];
        sumf += (float)sumi * oracle_f16_to_f32(w[i].d) * oracle_f16_to_f32(a[i].d);
    }
    return sumf;
}

/* -------------------------------------------------------------- Q4_K ----- */
/* candle-core utils.rs `get_scale_min_k4`. */
static inline void get_scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

void oracle_get_scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
    get_scale_min_k4(j, q, d, m);
}

/* candle-core k_quants.rs, `BlockQ4K::to_float`. */
void oracle_dequantize_row_q4_k(const block_q4_k* x, float* y, int64_t k) {
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        float d = oracle_f16_to_f32(x[i].d);
        float min = oracle_f16_to_f32(x[i].dmin);
        const uint8_t* q = x[i].qs;
        int is = 0;
        float* yo = y + i * QK_K;
        for (int j = 0; j < QK_K; j += 64) {
            uint8_t sc, m;
            get_scale_min_k4(is, x[i].scales, &sc, &m);
            float d1 = d * (float)sc;
            float m1 = min * (float)m;
            get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            float d2 = d * (float)sc;
            float m2 = min * (float)m;
            for (int l = 0; l < 32; l++) *yo++ = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) *yo++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* candle-core k_quants.rs, `BlockQ6K::to_float` (ggml `dequantize_row_q6_K`): per half of 128
 * elements, byte l of ql / qh carries elements l, l+32 (low nibbles of ql[l], ql[l+32]) and l+64,
 * l+96 (high nibbles); y = d * scale * (q - 32), evaluated left to right. */
void oracle_dequantize_row_q6_k(const block_q6_k* x, float* y, int64_t k) {
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float d = oracle_f16_to_f32(x[i].d);
        for (int n = 0; n < QK_K; n += 128) {
            const int idx = n / 128;
            float* yo = y + i * QK_K + n;
            const int8_t* sc = x[i].scales + 8 * idx;
            const uint8_t* ql = x[i].ql + 64 * idx;
            const uint8_t* qh = x[i].qh + 32 * idx;
            for (int l = 0; l < 32; l++) {
                const int is = l / 16;
                const int8_t q1 = (int8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32;
                const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                const int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                yo[l] = d * (float)sc[is] * (float)q1;
                yo[l + 32] = d * (float)sc[is + 2] * (float)q2;
                yo[l + 64] = d * (float)sc[is + 4] * (float)q3;
                yo[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
}

/* candle-core utils.rs `make_qkx1_quants(nmax, ntry, x)` -> (scale, -min). */
static void make_qkx1_quants(int nmax, int ntry, const float* x, int n, float* out_scale,
                             float* out_min) {
    uint8_t l[32];
    memset(l, 0, sizeof l);
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
    }
    if (max == min) {
        *out_scale = 0.0f;
        *out_min = 0.0f;
        return;
    }
    if (min > 0.0f) min = 0.0f;
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int32_t suml2 = 0;
        int did_change = 0;
        for (int i = 0; i < n; i++) {
            int32_t li = nearest_int(iscale * (x[i] - min));
            if (li < 0) li = 0;
            if (li > nmax) li = nmax;
            if ((uint8_t)li != l[i]) {
                l[i] = (uint8_t)li;
                did_change = 1;
            }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.0f;
        for (int i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        min = sum / (float)n;
        if (min > 0.0f) min = 0.0f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *out_scale = scale;
    *out_min = -min;
}

/* The sub-block search on its own, for the closed-form vectors of tests/golden. */
void oracle_make_qkx1_quants(int nmax, int ntry, const float* x, int n, float* out_scale,
                             float* out_neg_min) {
    make_qkx1_quants(nmax, ntry, x, n, out_scale, out_neg_min);
}

/* candle-core k_quants.rs, `BlockQ4K::from_float`.  Only used to MAKE weights. */
void oracle_quantize_row_q4_k(const float* x, block_q4_k* y, int64_t k) {
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float* xb = x + i * QK_K;
        block_q4_k* b = &y[i];
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) make_qkx1_quants(15, 5, xb + 32 * j, 32, &scales[j], &mins[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        memset(b->scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            int32_t lsi = nearest_int(inv_scale * scales[j]);
            int32_t lmi = nearest_int(inv_min * mins[j]);
            if (lsi > 63) lsi = 63;
            if (lmi > 63) lmi = 63;
            uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
            if (j < 4) {
                b->scales[j] = ls;
                b->scales[j + 4] = lm;
            } else {
                b->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                b->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                b->scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        b->d = oracle_f32_to_f16(max_scale / 63.0f);
        b->dmin = oracle_f32_to_f16(max_min / 63.0f);
        uint8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, b->scales, &sc, &m);
            float d = oracle_f16_to_f32(b->d) * (float)sc;
            if (d != 0.0f) {
                float dm = oracle_f16_to_f32(b->dmin) * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = nearest_int((xb[32 * j + ii] + dm) / d);
                    if (lv < 0) lv = 0;
                    if (lv > 15) lv = 15;
                    l[32 * j + ii] = (uint8_t)lv;
                }
            }
        }
        for (int j = 0; j < QK_K; j += 64)
            for (int lv = 0; lv < 32; lv++)
                b->qs[(j / 64) * 32 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 4));
    }
}

/* candle-core k_quants.rs, `BlockQ8K::from_float`. */
void oracle_quantize_row_q8_k(const float* x, block_q8_k* y, int64_t k) {
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float* xs = x + i * QK_K;
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            float a = fabsf(xs[j]);
            if (amax < a) {
                amax = a;
                max = xs[j];
            }
        }
        if (amax == 0.0f) {
            /* the crate zeroes d and qs; bsums keep the zeros the block was
             * created with (`zeros()` in `matmul`) */
            y[i].d = 0.0f;
            memset(y[i].qs, 0, QK_K);
            memset(y[i].bsums, 0, sizeof y[i].bsums);
            continue;
        }
        float iscale = -128.0f / max;
        for (int j = 0; j < QK_K; j++) {
            float v = roundf(iscale * xs[j]);
            if (v > 127.0f) v = 127.0f;
            if (v < -128.0f) v = -128.0f; /* Rust `as i8` saturates */
            y[i].qs[j] = (int8_t)v;
        }
        for (int j = 0; j < QK_K / 16; j++) {
            int32_t sum = 0;
            for (int ii = 0; ii < 16; ii++) sum += y[i].qs[j * 16 + ii];
            y[i].bsums[j] = (int16_t)sum;
        }
        y[i].d = 1.0f / iscale;
    }
}

/* candle-core k_quants.rs, `BlockQ4K::vec_dot_unopt` (scalar path). */
float oracle_vec_dot_q4_k_q8_k(int64_t k, const block_q4_k* w, const block_q8_k* a) {
    const uint32_t KMASK1 = 0x3f3f3f3fu, KMASK2 = 0x0f0f0f0fu, KMASK3 = 0x03030303u;
    int64_t nb = k / QK_K;
    uint32_t utmp[4];
    uint8_t scales[8], mins[8];
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8];
    int32_t aux32[8];
    memset(sums, 0, sizeof sums);
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t* q4 = w[i].qs;
        const int8_t* q8 = a[i].qs;
        memset(aux32, 0, sizeof aux32);
        int8_t* ap = aux8;
        for (int j = 0; j < QK_K / 64; j++) {
            for (int l = 0; l < 32; l++) ap[l] = (int8_t)(q4[l] & 0xF);
            ap += 32;
            for (int l = 0; l < 32; l++) ap[l] = (int8_t)(q4[l] >> 4);
            ap += 32;
            q4 += 32;
        }
        memcpy(utmp, w[i].scales, 12);
        utmp[3] = ((utmp[2] >> 4) & KMASK2) | (((utmp[1] >> 6) & KMASK3) << 4);
        uint32_t uaux = utmp[1] & KMASK1;
        utmp[1] = (utmp[2] & KMASK2) | (((utmp[0] >> 6) & KMASK3) << 4);
        utmp[2] = uaux;
        utmp[0] &= KMASK1;
        memcpy(scales, &utmp[0], 8);
        memcpy(mins, &utmp[2], 8);
        int32_t sumi = 0;
        for (int j = 0; j < QK_K / 16; j++) sumi += (int32_t)a[i].bsums[j] * (int32_t)mins[j / 2];
        const int8_t* av = aux8;
        for (int j = 0; j < 8; j++) {
            int32_t scale = scales[j];
            for (int r = 0; r < 4; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)av[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                av += 8;
            }
        }
        float d = oracle_f16_to_f32(w[i].d) * a[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        float dmin = oracle_f16_to_f32(w[i].dmin) * a[i].d;
        sumf -= dmin * (float)sumi;
    }
    float tail = 0.0f;
    for (int l = 0; l < 8; l++) tail += sums[l];
    return sumf + tail;
}

/* candle-core k_quants.rs, `BlockQ6K::vec_dot_unopt` (ggml `ggml_vec_dot_q6_K_q8_K`, scalar
 * path): the 256 six-bit quants are expanded to int8 (q - 32), each group of 16 is multiplied
 * with the Q8_K quants into eight running lanes weighted by the group's int8 scale, the lanes are
 * scaled by d_w * d_x per block and summed at the end.  The lane sums are integers below 2^24,
 * so holding them in int32 or in f32 gives the same values. */
float oracle_vec_dot_q6_k_q8_k(int64_t k, const block_q6_k* w, const block_q8_k* a) {
    int64_t nb = k / QK_K;
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8];
    int32_t aux32[8];
    memset(sums, 0, sizeof sums);
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t* q4 = w[i].ql;
        const uint8_t* qh = w[i].qh;
        const int8_t* q8 = a[i].qs;
        memset(aux32, 0, sizeof aux32);
        int8_t* ap = aux8;
        for (int j = 0; j < QK_K; j += 128) {
            for (int l = 0; l < 32; l++) {
                ap[l] = (int8_t)((int)((q4[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
                ap[l + 32] = (int8_t)((int)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
                ap[l + 64] = (int8_t)((int)((q4[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                ap[l + 96] = (int8_t)((int)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            }
            ap += 128;
            q4 += 64;
            qh += 32;
        }
        const int8_t* av = aux8;
        for (int j = 0; j < QK_K / 16; j++) {
            const int32_t scale = w[i].scales[j];
            for (int r = 0; r < 2; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)av[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                av += 8;
            }
        }
        float d = oracle_f16_to_f32(w[i].d) * a[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    }
    float total = 0.0f;
    for (int l = 0; l < 8; l++) total += sums[l];
    return total;
}

/* ------------------------------------------------------------ matmul ----- */
/* GGML dtype ids as the reference sees them (GgmlDType in candle-core mod.rs). */
#define GGML_Q8_0 8
#define GGML_Q4_K 12
#define GGML_Q6_K 14 /* no quantizer here: tests build Q6_K blocks directly */

int64_t oracle_storage_bytes(int dtype, int64_t rows, int64_t cols) {
    int64_t elems = rows * cols;
    if (dtype == GGML_Q8_0) return elems % QK8_0 ? -1 : elems / QK8_0 * 34;
    if (dtype == GGML_Q4_K) return elems % QK_K ? -1 : elems / QK_K * 144;
    if (dtype == GGML_Q6_K) return elems % QK_K ? -1 : elems / QK_K * 210;
    return -1;
}

/* candle-core k_quants.rs `matmul::<T>((m,k,n), lhs, rhs_t, dst)`: every lhs row
 * is quantized to T::VecDotType first, then rows are visited sequentially and
 * output columns in parallel (rayon there, OpenMP here), re-streaming the
 * weights once per row.  Returns 0, or -1 on a shape the crate rejects. */
int oracle_qmatmul(int dtype, int64_t m, int64_t k, int64_t n, const float* lhs, const void* rhs_t,
                   float* dst) {
    if (dtype == GGML_Q8_0) {
        if (k % QK8_0) return -1;
        int64_t kb = k / QK8_0;
        block_q8_0* lb = (block_q8_0*)malloc((size_t)(m * kb) * sizeof(block_q8_0));
        for (int64_t r = 0; r < m; r++) oracle_quantize_row_q8_0(lhs + r * k, lb + r * kb, k);
        const block_q8_0* w = (const block_q8_0*)rhs_t;
        for (int64_t r = 0; r < m; r++) {
#pragma omp parallel for schedule(static)
            for (int64_t c = 0; c < n; c++)
                dst[r * n + c] = oracle_vec_dot_q8_0_q8_0(k, w + c * kb, lb + r * kb);
        }
        free(lb);
        return 0;
    }
    if (dtype == GGML_Q4_K) {
        if (k % QK_K) return -1;
        int64_t kb = k / QK_K;
        block_q8_k* lb = (block_q8_k*)calloc((size_t)(m * kb), sizeof(block_q8_k));
        for (int64_t r = 0; r < m; r++) oracle_quantize_row_q8_k(lhs + r * k, lb + r * kb, k);
        const block_q4_k* w = (const block_q4_k*)rhs_t;
        for (int64_t r = 0; r < m; r++) {
#pragma omp parallel for schedule(static)
            for (int64_t c = 0; c < n; c++)
                dst[r * n + c] = oracle_vec_dot_q4_k_q8_k(k, w + c * kb, lb + r * kb);
        }
        free(lb);
        return 0;
    }
    if (dtype == GGML_Q6_K) {
        if (k % QK_K) return -1;
        int64_t kb = k / QK_K;
        block_q8_k* lb = (block_q8_k*)calloc((size_t)(m * kb), sizeof(block_q8_k));
        for (int64_t r = 0; r < m; r++) oracle_quantize_row_q8_k(lhs + r * k, lb + r * kb, k);
        const block_q6_k* w = (const block_q6_k*)rhs_t;
        for (int64_t r = 0; r < m; r++) {
#pragma omp parallel for schedule(static)
            for (int64_t c = 0; c < n; c++)
                dst[r * n + c] = oracle_vec_dot_q6_k_q8_k(k, w + c * kb, lb + r * kb);
        }
        free(lb);
        return 0;
    }
    return -1;
}

/* `QTensor::quantize` / `QTensor::dequantize` over a [rows, cols] matrix. */
int oracle_quantize(int dtype, int64_t rows, int64_t cols, const float* src, void* dst) {
    if (dtype == GGML_Q8_0) {
        if (cols % QK8_0) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; r++)
            oracle_quantize_row_q8_0(src + r * cols, (block_q8_0*)dst + r * (cols / QK8_0), cols);
        return 0;
    }
    if (dtype == GGML_Q4_K) {
        if (cols % QK_K) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; r++)
            oracle_quantize_row_q4_k(src + r * cols, (block_q4_k*)dst + r * (cols / QK_K), cols);
        return 0;
    }
    return -1;
}

int oracle_dequantize(int dtype, int64_t rows, int64_t cols, const void* src, float* dst) {
    if (dtype == GGML_Q8_0) {
        if (cols % QK8_0) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; r++)
            oracle_dequantize_row_q8_0((const block_q8_0*)src + r * (cols / QK8_0), dst + r * cols,
                                       cols);
        return 0;
    }
    if (dtype == GGML_Q4_K) {
        if (cols % QK_K) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; r++)
            oracle_dequantize_row_q4_k((const block_q4_k*)src + r * (cols / QK_K), dst + r * cols,
                                       cols);
        return 0;
    }
    if (dtype == GGML_Q6_K) {
        if (cols % QK_K) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; r++)
            oracle_dequantize_row_q6_k((const block_q6_k*)src + r * (cols / QK_K), dst + r * cols,
                                       cols);
        return 0;
    }
    return -1;
}

/* Activation-side quantization exposed for bit-exact checks of the device's
 * own activation quantizer: `T::VecDotType::from_float` per row. */
int oracle_quantize_activations(int weight_dtype, int64_t m, int64_t k, const float* x, void* out) {
    if (weight_dtype == GGML_Q8_0) {
        if (k % QK8_0) return -1;
        for (int64_t r = 0; r < m; r++)
            oracle_quantize_row_q8_0(x + r * k, (block_q8_0*)out + r * (k / QK8_0), k);
        return 0;
    }
    if (weight_dtype == GGML_Q4_K || weight_dtype == GGML_Q6_K) { /* both dot types are Q8_K */
        if (k % QK_K) return -1;
        memset(out, 0, (size_t)(m * (k / QK_K)) * sizeof(block_q8_k));
        for (int64_t r = 0; r < m; r++)
            oracle_quantize_row_q8_k(x + r * k, (block_q8_k*)out + r * (k / QK_K), k);
        return 0;
    }
    return -1;
}

/* --------------------------------------------------------------- MoE ----- */
/* The reference has no MoE code (no `moe|expert|router` anywhere in crates/);
 * these functions DEFINE the expert-grouped form for this build:
 *   route : per token, the top_k largest logits (ties -> lower expert index),
 *           slots in descending-logit order; weights = exp(l - lmax) over the
 *           selected slots, renormalised to sum 1 (== renormalised softmax).
 *   sort  : stable counting sort of the T*top_k (token,slot) pairs by expert.
 *   forward: per pair, h = silu(Wg x) * (Wu x), y = Wd h with QMatMul semantics
 *           (each matmul re-quantizes its input), out[t] = sum_s w[t,s]*y[t,s]
 *           accumulated in slot order. */
void oracle_moe_route(const float* logits, int64_t T, int E, int top_k, int32_t* ids, float* wts) {
    uint8_t* taken = (uint8_t*)malloc((size_t)E);
    for (int64_t t = 0; t < T; t++) {
        const float* l = logits + t * E;
        memset(taken, 0, (size_t)E);
        for (int s = 0; s < top_k; s++) {
            int best = -1;
            for (int e = 0; e < E; e++) {
                if (taken[e]) continue;
                if (best < 0 || l[e] > l[best]) best = e; /* strict > keeps the lower index */
            }
            taken[best] = 1;
            ids[t * top_k + s] = best;
        }
        float lmax = l[ids[t * top_k]];
        float denom = 0.0f;
        for (int s = 0; s < top_k; s++) {
            float p = expf(l[ids[t * top_k + s]] - lmax);
            wts[t * top_k + s] = p;
            denom += p;
        }
        for (int s = 0; s < top_k; s++) wts[t * top_k + s] = wts[t * top_k + s] / denom;
    }
    free(taken);
}

void oracle_moe_sort(const int32_t* ids, int64_t T, int top_k, int E, int32_t* perm,
                     int32_t* offsets) {
    int64_t P = T * top_k;
    memset(offsets, 0, (size_t)(E + 1) * sizeof(int32_t));
    for (int64_t p = 0; p < P; p++) offsets[ids[p] + 1]++;
    for (int e = 0; e < E; e++) offsets[e + 1] += offsets[e];
    int32_t* cur = (int32_t*)malloc((size_t)E * sizeof(int32_t));
    memcpy(cur, offsets, (size_t)E * sizeof(int32_t));
    for (int64_t p = 0; p < P; p++) perm[cur[ids[p]]++] = (int32_t)p;
    free(cur);
}

static inline float silu_f32(float v) { return v / (1.0f + expf(-v)); }

/* gate/up: [E][inter][hidden] blocks, down: [E][hidden][inter] blocks. */
static int moe_forward_impl(int dtype, int down_dtype, int64_t T, int E, int top_k, int64_t hidden, int64_t inter,
                            const float* x, const int32_t* ids, const float* wts, const void* gate,
                            const void* up, const void* down, float* out) {
    int64_t gu_bytes = oracle_storage_bytes(dtype, inter, hidden);
    int64_t dn_bytes = oracle_storage_bytes(down_dtype, hidden, inter);
    if (gu_bytes < 0 || dn_bytes < 0) return -1;
    float* g = (float*)malloc((size_t)inter * sizeof(float));
    float* u = (float*)malloc((size_t)inter * sizeof(float));
    float* y = (float*)malloc((size_t)hidden * sizeof(float));
    for (int64_t t = 0; t < T; t++) {
        float* o = out + t * hidden;
        for (int64_t c = 0; c < hidden; c++) o[c] = 0.0f;
        for (int s = 0; s < top_k; s++) {
            int e = ids[t * top_k + s];
            float w = wts[t * top_k + s];
            oracle_qmatmul(dtype, 1, hidden, inter, x + t * hidden,
                           (const uint8_t*)gate + (size_t)e * gu_bytes, g);
            oracle_qmatmul(dtype, 1, hidden, inter, x + t * hidden,
                           (const uint8_t*)up + (size_t)e * gu_bytes, u);
            for (int64_t c = 0; c < inter; c++) g[c] = silu_f32(g[c]) * u[c];
            oracle_qmatmul(down_dtype, 1, inter, hidden, g, (const uint8_t*)down + (size_t)e * dn_bytes,
                           y);
            for (int64_t c = 0; c < hidden; c++) o[c] += w * y[c];
        }
    }
    free(g);
    free(u);
    free(y);
    return 0;
}

int oracle_moe_forward(int dtype, int64_t T, int E, int top_k, int64_t hidden, int64_t inter,
                       const float* x, const int32_t* ids, const float* wts, const void* gate,
                       const void* up, const void* down, float* out) {
    return moe_forward_impl(dtype, dtype, T, E, top_k, hidden, inter, x, ids, wts, gate, up, down, out);
}

/* The same with the down stack in a type of its own (a Q4_K_M file keeps ffn_down_exps of some
 * layers in Q6_K beside Q4_K gate / up stacks): each product is the reference's QMatMul::forward
 * for its tensor's type. */
int oracle_moe_forward_mixed(int gate_up_dtype, int down_dtype, int64_t T, int E, int top_k, int64_t hidden,
                             int64_t inter, const float* x, const int32_t* ids, const float* wts,
                             const void* gate, const void* up, const void* down, float* out) {
    return moe_forward_impl(gate_up_dtype, down_dtype, T, E, top_k, hidden, inter, x, ids, wts, gate, up, down, out);
}

/* ------------------------------------------------------- seeded inputs --- */
/* Counter-based generator: value i of stream `seed` depends on (seed, i) only,
 * so any slice can be produced in parallel and on any machine.  splitmix64
 * finaliser -> two 24-bit uniforms -> Box-Muller. */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

void oracle_fill_normal(uint64_t seed, int64_t offset, int64_t count, float mean, float std,
                        float* out) {
    uint64_t key = splitmix64(seed);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; i++) {
        uint64_t r = splitmix64(key ^ (uint64_t)(offset + i) * 0xd1342543de82ef95ull);
        float u1 = ((float)(r >> 40) + 1.0f) * (1.0f / 16777216.0f); /* (0,1] */
        float u2 = (float)((r >> 16) & 0xffffffu) * (1.0f / 16777216.0f);
        float radius = sqrtf(-2.0f * logf(u1));
        out[i] = mean + std * radius * cosf(6.28318530717958647692f * u2);
    }
}
