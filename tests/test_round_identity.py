"""CPU check of the arithmetic identity the GPU activation quantizers rely on: for a float v,
trunc(v + copysign(0.5 - 2^-25, v)) (one f32 addition, round to nearest even) equals the reference
quantizers' round-half-away-from-zero (Rust `f32::round`, candle-core k_quants.rs `from_float` of
BlockQ8_0 / BlockQ8K).  Every float from 0.25 up to 512 (the quantizers' products stay within
+-128 before the clamp), every float below 0.25 on a stride, the halves' neighbours by name."""
import numpy as np

HALF_BELOW = np.frombuffer(np.uint32(0x3EFFFFFF).tobytes(), dtype=np.float32)[0]


def _check(bits):
    x = bits.view(np.float32)
    got = np.trunc(x + HALF_BELOW).astype(np.float64)
    want = np.floor(x.astype(np.float64) + 0.5)  # exact in f64; half away from zero for x >= 0
    return int((got != want).sum())


def test_constant_is_the_float_below_one_half():
    assert HALF_BELOW == np.nextafter(np.float32(0.5), np.float32(0.0))


def test_add_and_truncate_is_round_half_away_for_every_float_in_range():
    lo, hi = 0x3E800000, 0x44000000  # 0.25 .. 512.0
    step = 1 << 25
    for start in range(lo, hi, step):
        assert _check(np.arange(start, min(start + step, hi), dtype=np.uint32)) == 0
    assert _check(np.arange(0, lo, 61, dtype=np.uint32)) == 0  # zero, subnormals, small normals


def test_named_neighbours_of_the_halves():
    for base in (0.0, 1.0, 2.0, 63.0, 126.0, 127.0):
        h = np.float32(base + 0.5)
        for v, want in ((h, base + 1), (np.nextafter(h, np.float32(0)), base), (np.nextafter(h, np.float32(1e9)), base + 1)):
            for sign in (1.0, -1.0):
                x = np.float32(sign) * v
                got = np.trunc(x + np.copysign(HALF_BELOW, x))
                assert got == sign * want, (x, got)
