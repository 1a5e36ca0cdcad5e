"""Pins the oracle's codecs (f16, Q8_0, Q4_K, Q8_K) without the reference's
third-party arithmetic: closed forms, hand-built blocks, invariants and an
independent numpy restatement (tests/np_ref.py)."""
import numpy as np
import pytest

import np_ref

Q8_0, Q4_K = 8, 12


def test_block_sizes_match_quantized_storage_bytes_rule(oracle):
    # qwen3/core.rs:891-909: bytes = rows*cols / block_size * type_size, else error
    assert oracle.storage_bytes(Q8_0, 3072, 1024) == 3_342_336
    assert oracle.storage_bytes(Q4_K, 4096, 4096) == 9_437_184
    assert oracle.storage_bytes(Q4_K, 151936, 4096) == 350_060_544
    assert oracle.storage_bytes(Q8_0, 1, 31) == -1
    assert oracle.storage_bytes(Q4_K, 3, 100) == -1


def test_f16_to_f32_exhaustive_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_round_to_nearest_even_against_numpy(oracle):
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
        # exact ties and the neighbourhoods of every f16 value
        (np.arange(1, 0x7c00, 7, dtype=np.uint16).view(np.float16).astype(np.float32)
         + np.arange(1, 0x7c01, 7, dtype=np.uint16).view(np.float16).astype(np.float32)) / 2,
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  2.9802326e-8, 6.1e-5, 6.097e-5, np.inf, -np.inf], dtype=np.float32),
    ]).astype(np.float32)
    want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_q8_0_dequant_hand_block(oracle):
    # d = 0.5 (f16 0x3800), qs = -128..-97 ; d = max f16 ; d = smallest subnormal
    blk = bytearray()
    blk += bytes([0x00, 0x38]) + bytes((np.arange(32) - 128).astype(np.int8).view(np.uint8))
    blk += bytes([0xff, 0x7b]) + bytes(np.full(32, 127, np.int8).view(np.uint8))
    blk += bytes([0x01, 0x00]) + bytes((np.arange(32) - 16).astype(np.int8).view(np.uint8))
    y = oracle.dequantize(Q8_0, np.frombuffer(bytes(blk), np.uint8), 1, 96)
    assert np.array_equal(y[0, :32], (np.arange(32) - 128) * 0.5)
    assert np.array_equal(y[0, 32:64], np.full(32, 127 * 65504.0, np.float32))
    assert np.array_equal(y[0, 64:], ((np.arange(32) - 16) * 2.0 ** -24).astype(np.float32))


def q4k_hand_block():
    # d = 1.0, dmin = 0.5, scales encode sc = [1,2,3,4,17,34,51,63], m = [0,5,10,15,20,40,60,63]
    scales = bytes([0x41, 0x82, 0xC3, 0xC4, 0x40, 0x85, 0xCA, 0xCF, 0x41, 0x82, 0xC3, 0xFF])
    return bytes([0x00, 0x3C, 0x00, 0x38]) + scales + bytes(range(128))


def test_q4_k_scale_unpack_both_branches(oracle):
    import ctypes as C
    s = np.frombuffer(q4k_hand_block()[4:16], np.uint8).copy()
    got_sc, got_m = [], []
    for j in range(8):
        d, m = C.c_uint8(), C.c_uint8()
        oracle.lib().oracle_get_scale_min_k4(j, s.ctypes.data, C.addressof(d), C.addressof(m))
        got_sc.append(d.value)
        got_m.append(m.value)
    assert got_sc == [1, 2, 3, 4, 17, 34, 51, 63]
    assert got_m == [0, 5, 10, 15, 20, 40, 60, 63]


def test_q4_k_dequant_hand_block(oracle):
    y = oracle.dequantize(Q4_K, np.frombuffer(q4k_hand_block(), np.uint8), 1, 256)[0]
    want = {0: 0, 1: 1, 15: 15, 31: 15, 32: -2.5, 63: -0.5, 64: -5, 79: 40, 96: 0.5, 127: 4.5,
            128: -10, 160: 116, 191: 150, 192: -30, 224: 346.5, 255: 409.5}
    for i, v in want.items():
        assert y[i] == np.float32(v), (i, y[i], v)
    assert float(y.astype(np.float64).sum()) == 32224.0
    # closed form for every element: sc*q - 0.5*m, element order low nibbles then high per 64-group
    sc = [1, 2, 3, 4, 17, 34, 51, 63]
    mn = [0, 5, 10, 15, 20, 40, 60, 63]
    for g in range(4):
        for l in range(32):
            b = 32 * g + l
            assert y[64 * g + l] == sc[2 * g] * (b & 15) - 0.5 * mn[2 * g]
            assert y[64 * g + 32 + l] == sc[2 * g + 1] * (b >> 4) - 0.5 * mn[2 * g + 1]


def test_q4_k_dequant_random_bytes_against_numpy(oracle):
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, size=(4096, 144), dtype=np.uint8)
    # keep d/dmin finite: clear the f16 exponent's top bit
    raw[:, 1] &= 0x3F
    raw[:, 3] &= 0x3F
    got = oracle.dequantize(Q4_K, raw.reshape(-1), 64, 64 * 256)
    want = np_ref.dequant_q4_k(raw.reshape(-1), 64, 64 * 256)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # d*sc*q is an 11-bit x 6-bit x 4-bit product, exact in f32, so the only
    # rounding is the final subtraction: the exact value rounded once must agree
    d, dmin, sc, mn, q = np_ref.q4_k_fields(raw.reshape(-1))
    d1 = d[:, None].astype(np.float64) * sc
    m1 = dmin[:, None].astype(np.float64) * mn
    exact = (d1[:, :, None] * q - m1[:, :, None]).astype(np.float32).reshape(64, -1)
    assert np.array_equal(exact.view(np.uint32), got.view(np.uint32))


def test_q8_0_dequant_random_bytes_against_numpy(oracle):
    rng = np.random.default_rng(4)
    raw = rng.integers(0, 256, size=(8192, 34), dtype=np.uint8)
    raw[:, 1] &= 0x7B  # finite scales
    got = oracle.dequantize(Q8_0, raw.reshape(-1), 32, 8192)
    want = np_ref.dequant_q8_0(raw.reshape(-1), 32, 8192)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q8_0_quantize_invariants(oracle):
    w = oracle.randn(11, (64, 1024), std=0.02)
    w[3, 64:96] = 0.0  # an all-zero block
    blocks = oracle.quantize(Q8_0, w)
    d, q = np_ref.q8_0_fields(blocks)
    wb = w.reshape(-1, 32)
    amax_pos = np.abs(wb).argmax(axis=1)
    nz = np.abs(wb).max(axis=1) > 0
    assert np.all(np.abs(q[np.arange(q.shape[0]), amax_pos])[nz] == 127)
    assert np.all(d[~nz] == 0) and np.all(q[~nz] == 0)
    # scale is f16(amax/127) and |w - w^| <= d_f32/2 (+ f16 rounding of d on 127 steps)
    assert np.array_equal(d, (np.abs(wb).max(axis=1) / np.float32(127)).astype(np.float16).astype(np.float32))
    back = oracle.dequantize(Q8_0, blocks, 64, 1024).reshape(-1, 32)
    bound = d[:, None] * 0.5 + 127 * d[:, None] * 2.0 ** -11 + 1e-12
    assert np.all(np.abs(back - wb) <= bound)
    # quantizing again is idempotent on the dequantized values' quants
    d2, q2 = np_ref.quant_act_q8_0(w)
    assert np.array_equal(q2, q) and np.array_equal(d2, d)


def test_q4_k_quantize_invariants(oracle):
    w = oracle.randn(12, (32, 2048), std=0.02)
    w[5, 256:512] = 0.125  # constant super-block: max == min in every sub-block
    blocks = oracle.quantize(Q4_K, w)
    d, dmin, sc, mn, q = np_ref.q4_k_fields(blocks)
    assert q.max() <= 15 and sc.max() <= 63 and mn.max() <= 63
    assert np.all(dmin >= 0) and np.all(d >= 0)
    blk = 5 * 8 + 1
    assert np.all(sc[blk] == 0) and np.all(mn[blk] == 0) and np.all(q[blk] == 0)
    back = oracle.dequantize(Q4_K, blocks, 32, 2048)
    err = np.abs(back - w)
    err[5, 256:512] = 0
    # 4-bit grid over each sub-block's range: error below ~ range/15
    sub = w.reshape(-1, 32)
    rng_ = (sub.max(axis=1) - np.minimum(sub.min(axis=1), 0)).reshape(32, 64)
    assert np.all(err.reshape(32, 64, 32) <= rng_[:, :, None] / 15 * 1.01 + 1e-6)
    rel = np.sqrt((err ** 2).mean() / (w ** 2).mean())
    assert rel < 0.1


def test_q8_k_activation_quantization_against_numpy(oracle):
    x = oracle.randn(21, (8, 1024))
    x[2, 256:512] = 0.0
    x[4, 5] = -7.5   # the extreme (either sign) maps to -128 ...
    x[4, 9] = 7.5    # ... and a later element of opposite sign and equal size to +128 -> 127
    x[6, 300] = 9.25
    raw = oracle.quantize_activations(Q4_K, x).reshape(-1, 292)
    d = raw[:, :4].copy().view(np.float32).reshape(-1)
    q = raw[:, 4:260].copy().view(np.int8)
    bs = raw[:, 260:].copy().view(np.int16)
    d_np, q_np = np_ref.quant_act_q8_k(x)
    assert np.array_equal(d.view(np.uint32), d_np.view(np.uint32))
    assert np.array_equal(q, q_np)
    assert np.array_equal(bs, q.reshape(-1, 16, 16).astype(np.int32).sum(axis=2))
    blk = 2 * 4 + 1
    assert d[blk] == 0 and not q[blk].any() and not bs[blk].any()
    assert q[4 * 4 + 0, 5] == -128 and q[4 * 4 + 0, 9] == 127 and q[6 * 4 + 1, 300 - 256] == -128


def test_q8_0_activation_quantization_against_numpy(oracle):
    x = oracle.randn(22, (4, 512))
    raw = oracle.quantize_activations(Q8_0, x)
    d, q = np_ref.q8_0_fields(raw)
    d_np, q_np = np_ref.quant_act_q8_0(x)
    assert np.array_equal(d, d_np) and np.array_equal(q, q_np)


def test_generator_is_counter_based_and_normal(oracle):
    a = oracle.randn(5, (1 << 16,))
    b = oracle.randn(5, (1 << 15,), offset=1 << 15)
    assert np.array_equal(a[1 << 15:], b)
    assert abs(float(a.mean())) < 0.02 and abs(float(a.std()) - 1.0) < 0.02
    assert not np.array_equal(a, oracle.randn(6, (1 << 16,)))
    assert np.isfinite(a).all()


def test_quantize_rejects_bad_last_dim(oracle):
    with pytest.raises(ValueError):
        oracle.quantize(Q4_K, np.zeros((2, 128), np.float32))
    with pytest.raises(ValueError):
        oracle.quantize(Q8_0, np.zeros((2, 48), np.float32))
