"""Writes q4k_quantizer_cases.json: vectors that pin `BlockQ4K::from_float` and its scale search
`make_qkx1_quants(nmax = 15, ntry = 5)` (candle-core 0.10.2, k_quants.rs / utils.rs; the crate is
not in the reference's tree and cannot be run here, so the vectors come from what the published
algorithm's mathematics fixes, worked out below in exact rational arithmetic, with no code of
the oracle or of the library involved).

The algorithm, per 32-value sub-block: min <- min(min x, 0), iscale <- 15 / (max x - min); then up
to five passes of { l_i <- clamp(round_half_away(iscale (x_i - min)), 0, 15);
scale <- sum (x_i - min) l_i / sum l_i^2;  min <- min(mean(x_i - scale l_i), 0);  iscale <- 1 / scale;
stop after a pass that changed no l_i }; result (scale, -min), or (0, 0) when max x = min x.
Per 256-value block: the eight (scale_j, min_j) are coded on six bits against the block's largest
(ls_j = round(63 scale_j / max scale), d = f16(max scale / 63), likewise lm_j, dmin), and every
value is coded again as q = clamp(round((x + dmin lm_j) / (d ls_j)), 0, 15) with d, dmin as stored.

Cases (each one fails for a plausible wrong restatement, named beside it):

* grid sub-blocks: x_i = min + s l_i with l covering 0..15, s and min on a binary grid, so every
  product and sum is exact in f32: pass 0 recovers l, the least-squares scale is s exactly, the mean
  residual is min exactly, pass 1 changes nothing.  A block of eight such sub-blocks whose s_j, -min_j
  are integer multiples c_j, e_j of max/63 must come back as d = max s / 63, dmin = max(-min) / 63,
  six-bit codes c_j, e_j and quants l: wrong packing of the twelve scale bytes, wrong nibble
  order, a sign error on min, all show in the bytes.
* all-positive sub-block (no value 0, no l = 0): min clamps to 0, the grid starts at 0.  Without the
  clamp the grid would start at min x and every quant would differ.
* constant sub-block: (0, 0), quants 0, whatever the constant is.
* three-pass sub-block {15, 0, 30 x 1.375}: the code of 15 goes 15 -> 14 -> 13 while the scale
  goes 266.25/255 -> 251.25/226 -> 236.25/199 (trace below).  No refinement, or fewer than three
  passes, gives another scale and another six-bit code.
* cut-off sub-block: the fifth pass still changes a code; the search stops there (ntry = 5) with
  scale 1.11958 where one more pass would give 1.12433.
* tie sub-block {15, 0, 30 x 2.5}: round half away from zero codes 2.5 as 3 (ggml's ties-to-even
  trick gives 2) and the scale follows: 450/495 after pass 0 against 375/345.

Run:  python tests/golden/make_q4k_quantizer_vectors.py
"""
import json
import os
from fractions import Fraction as F

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
TIE_MARGIN = F(1, 200)   # every rounding decision of a case is at least this far from a tie


def round_half_away(v):
    """(integer, distance of v from the nearest tie)."""
    a = abs(v)
    whole = a.numerator // a.denominator
    frac = a - whole
    r = whole + (1 if frac >= F(1, 2) else 0)
    return (r if v >= 0 else -r), abs(frac - F(1, 2))


def scale_search(x, allow_ties=False, ntry=5):
    """The sub-block search in exact arithmetic.  Returns (scale, -min, codes per pass)."""
    n, nmax = len(x), 15
    lo, hi = min(x), max(x)
    if lo == hi:
        return F(0), F(0), []
    lo = min(lo, F(0))
    iscale = F(nmax) / (hi - lo)
    codes = [0] * n
    trace = []
    for _ in range(ntry):
        changed = False
        sumlx, suml2 = F(0), 0
        for i, v in enumerate(x):
            li, margin = round_half_away(iscale * (v - lo))
            assert allow_ties or margin == F(1, 2) or margin >= TIE_MARGIN, (v, margin)
            li = max(0, min(nmax, li))
            if li != codes[i]:
                codes[i], changed = li, True
            sumlx += (v - lo) * li
            suml2 += li * li
        scale = sumlx / suml2
        lo = min(sum(v - scale * li for v, li in zip(x, codes)) / n, F(0))
        iscale = 1 / scale
        trace.append(list(codes))
        if not changed:
            break
    return scale, -lo, trace


def f16(v):
    """Fraction -> value of the nearest binary16 (numpy rounds to nearest even), as a Fraction."""
    h = np.float16(float(v))
    return F(float(h)), int(h.view(np.uint16))


def pack_scales(ls, lm):
    """The twelve scale bytes of the public Q4_K block format: codes 0..3 in the low six bits of
    bytes 0..3 (scales) and 4..7 (mins), codes 4..7 as low nibbles of bytes 8..11 with their top
    two bits in bits 6..7 of bytes 0..3 (scales) and 4..7 (mins)."""
    out = [0] * 12
    for j in range(4):
        out[j] = ls[j] | ((ls[j + 4] >> 4) << 6)
        out[j + 4] = lm[j] | ((lm[j + 4] >> 4) << 6)
        out[j + 8] = (ls[j + 4] & 15) | ((lm[j + 4] & 15) << 4)
    return bytes(out)


def encode_block(x, allow_ties_in=()):
    """`from_float` on 256 exact values -> (144 bytes, per-sub-block (scale, -min))."""
    subs = [scale_search(x[32 * j:32 * j + 32], allow_ties=j in allow_ties_in)[:2] for j in range(8)]
    max_scale = max(s for s, _ in subs)
    max_min = max(m for _, m in subs)
    ls, lm = [], []
    for s, m in subs:
        a, ma = round_half_away(63 * s / max_scale) if max_scale else (0, F(1, 2))
        b, mb = round_half_away(63 * m / max_min) if max_min else (0, F(1, 2))
        assert (ma == F(1, 2) or ma >= TIE_MARGIN) and (mb == F(1, 2) or mb >= TIE_MARGIN)
        ls.append(min(63, a))
        lm.append(min(63, b))
    d, d_bits = f16(max_scale / 63)
    dmin, dmin_bits = f16(max_min / 63)
    q = [0] * 256
    for j in range(8):
        dd = d * ls[j]
        if dd == 0:
            continue
        for i in range(32):
            v, margin = round_half_away((x[32 * j + i] + dmin * lm[j]) / dd)
            assert margin == F(1, 2) or margin >= TIE_MARGIN, (j, i, margin)
            q[32 * j + i] = max(0, min(15, v))
    qs = bytes(q[64 * g + l] | (q[64 * g + 32 + l] << 4) for g in range(4) for l in range(32))
    head = np.array([d_bits, dmin_bits], dtype="<u2").tobytes()
    return head + pack_scales(ls, lm) + qs, subs, ls, lm, q


def codes_pattern(seed, lowest=0):
    """32 codes covering lowest..15 (so that min and max of the sub-block are the grid's ends)."""
    rng = np.random.default_rng(seed)
    base = list(range(lowest, 16))
    extra = list(rng.integers(lowest, 16, size=32 - len(base)))
    out = np.array(base + extra)
    rng.shuffle(out)
    return [int(v) for v in out]


def grid_sub(c, e, u, v, seed, lowest=0):
    """x_i = -e v + c u l_i."""
    return [-e * v + c * u * l for l in codes_pattern(seed, lowest)]


THREE_PASS = [F(15), F(0)] + [F(11, 8)] * 30
# found by a random search over multiples of 1/8: a code still moves in the fifth pass
FIVE_PASS_CUTOFF = [F(15), F(-1), F(57, 4)] + [F(13, 8)] * 18 + [F(25, 4)] * 5 + [F(6)] * 6
TIE = [F(15), F(0)] + [F(5, 2)] * 30


def sub_block_cases():
    u = F(1, 1024)
    cases = []

    def add(name, x, exact, allow_ties=False, **extra):
        s, m, trace = scale_search(x, allow_ties=allow_ties)
        cases.append({"name": name, "x": [float(t) for t in x], "scale": float(s), "neg_min": float(m),
                      "scale_num_den": [float(s.numerator), float(s.denominator)],
                      # exact: every f32 operation of the search is exact up to the final division, so
                      # the f32 result is float32(num) / float32(den) bit for bit; otherwise the f32
                      # sums round on the way and the result agrees to a few ulp
                      "exact_in_f32": exact, "passes": len(trace), **extra})
        return s, m, trace

    s, m, _ = add("grid_c7_e13", grid_sub(7, 13, u, 2 * u, 1), True)
    assert (s, m) == (7 * u, 26 * u)
    s, m, _ = add("grid_c63_e0", grid_sub(63, 0, u, 2 * u, 2), True)
    assert (s, m) == (63 * u, 0)
    s, m, _ = add("all_positive_min_clamps_to_zero", grid_sub(5, 0, u, 2 * u, 3, lowest=3), True)
    assert (s, m) == (5 * u, 0)
    s, m, _ = add("constant_nonzero", [F(1, 8)] * 32, True)
    assert (s, m) == (0, 0)
    # trace of the code of the value 15, and the scale after each pass (30 values 1.375 keep code 1):
    #   pass 0: iscale 1           -> 15;  scale (225 + 41.25) / (225 + 30) = 266.25 / 255 = 1.04412
    #   pass 1: 15 / 1.04412 = 14.37 -> 14; scale (210 + 41.25) / (196 + 30) = 251.25 / 226 = 1.11173
    #   pass 2: 15 / 1.11173 = 13.49 -> 13; scale (195 + 41.25) / (169 + 30) = 236.25 / 199 = 1.18719
    #   pass 3: 15 / 1.18719 = 12.63 -> 13; nothing changed, same scale, stop.  mean residual > 0 -> min 0
    s, m, trace = add("three_passes", THREE_PASS, True)
    assert [t[0] for t in trace] == [15, 14, 13, 13] and all(t[2] == 1 for t in trace)
    assert (s, m) == (F(23625, 19900), 0)
    # the fifth pass still changes a code (14.25: 14 -> 13), so a longer search would run a sixth pass
    # and work out scale and min once more: five passes end at 1.11958, six at 1.12433
    s, m, trace = add("five_pass_cutoff", FIVE_PASS_CUTOFF, False)
    s6, m6, trace6 = scale_search(FIVE_PASS_CUTOFF, ntry=12)
    assert len(trace) == 5 and trace[4] != trace[3] and len(trace6) == 6 and abs(s6 - s) > F(1, 250)
    # 2.5 -> 3 (half away from zero): pass 0 scale (225 + 30 * 7.5) / (225 + 270) = 450 / 495, mean
    # residual (15 - 15 * 10/11 + 30 * (2.5 - 30/11)) / 32 = -15/88; pass 1 changes no code, but
    # scale and min are worked out once more with the new min before the search stops
    s, m, trace = add("tie_rounds_away_from_zero", TIE, False, allow_ties=True)
    assert [t[2] for t in trace] == [3, 3] and len(trace) == 2
    lo = F(-15, 88)
    s1 = ((15 - lo) * 15 + 30 * (F(5, 2) - lo) * 3) / 495
    m1 = ((0 - 0) + (15 - 15 * s1) + 30 * (F(5, 2) - 3 * s1)) / 32
    assert (s, m) == (s1, -m1)
    return cases


def block_cases():
    u, v = F(1, 1024), F(1, 512)
    out = []

    def add(name, x, want=None, allow_ties_in=()):
        raw, subs, ls, lm, q = encode_block(x, allow_ties_in)
        if want is not None:
            assert (ls, lm) == want, (ls, lm)
        out.append({"name": name, "x": [float(t) for t in x], "block_hex": raw.hex(),
                    "scale_codes": ls, "min_codes": lm, "quants": q})
        return raw, subs, ls, lm, q

    # (1) multiples of max / 63 with the maximum 63: d = u, dmin = v, codes = the multiples, quants = l
    c = [63, 1, 7, 32, 21, 40, 63, 5]
    e = [0, 63, 13, 1, 33, 47, 20, 62]
    x = sum((grid_sub(c[j], e[j], u, v, 10 + j) for j in range(8)), [])
    raw, _, _, _, q = add("grid_multiples_of_max_over_63", x, (c, e))
    assert raw[:4] == np.array([float(u), float(v)], dtype="<f2").tobytes()
    assert q == sum((codes_pattern(10 + j) for j in range(8)), [])
    # (2) maximum multiples 21 and 9: codes 3 c_j and 7 e_j; d = f16(u / 3), dmin = f16(v / 7) round
    c = [21, 1, 7, 14, 21, 2, 9, 5]
    e = [0, 9, 3, 1, 4, 7, 2, 6]
    x = sum((grid_sub(c[j], e[j], u, v, 20 + j) for j in range(8)), [])
    _, _, _, _, q = add("grid_maximum_below_63", x, ([3 * t for t in c], [7 * t for t in e]))
    assert q == sum((codes_pattern(20 + j) for j in range(8)), [])
    # (3) no value below 3 s_j anywhere: every min clamps to 0, dmin = 0, all min codes 0
    c = [63, 9, 18, 27, 36, 45, 54, 3]
    x = sum((grid_sub(c[j], 0, u, v, 30 + j, lowest=3) for j in range(8)), [])
    raw, _, _, _, q = add("all_positive_block", x, (c, [0] * 8))
    assert raw[2:4] == b"\0\0" and q == sum((codes_pattern(30 + j, lowest=3) for j in range(8)), [])
    # (4) the three-pass, tie, all-positive and constant sub-blocks between grid sub-blocks that
    # hold the block's largest scale (63 / 16) and largest min (63 / 32): codes by 16 x and 32 x
    big_u, big_v = F(1, 16), F(1, 32)
    x = (grid_sub(63, 10, big_u, big_v, 40) + THREE_PASS + grid_sub(4, 63, big_u, big_v, 41) + TIE
         + grid_sub(16, 0, big_u, big_v, 42, lowest=3) + [F(1, 8)] * 32
         + grid_sub(30, 31, big_u, big_v, 43) + grid_sub(1, 1, big_u, big_v, 44))
    _, subs, ls, lm, _ = add("mixed_block", x, allow_ties_in=(3,))
    # 16 * 236.25 / 199 = 18.99 -> 19 (one pass: 16.7 -> 17, two: 17.8 -> 18); tie sub-block 15.1 -> 15, 9.25 -> 9
    assert ls == [63, 19, 4, 15, 16, 0, 30, 1] and lm == [10, 0, 63, 9, 0, 0, 31, 1]
    return out


if __name__ == "__main__":
    rec = {"nmax": 15, "ntry": 5, "sub_blocks": sub_block_cases(), "blocks": block_cases()}
    path = os.path.join(HERE, "q4k_quantizer_cases.json")
    with open(path, "w") as f:
        json.dump(rec, f, indent=1)
    print("wrote", path, len(rec["sub_blocks"]), "sub-block cases,", len(rec["blocks"]), "block cases")
