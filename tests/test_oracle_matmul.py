"""Pins the oracle's quantized matmul: the reference's own test case
(qwen3/core.rs:3099-3142), integer brute force, an f64 bound and the
row-independence / concatenation properties the reference relies on."""
import numpy as np
import pytest

import np_ref

Q8_0, Q4_K, Q6_K = 8, 12, 14


def reference_packed_case():
    # qwen3/core.rs:3104-3124
    w1 = ((np.arange(64, dtype=np.float32) - 31.0) / 8.0).reshape(2, 32)
    w2 = ((15.0 - np.arange(32, dtype=np.float32)) / 7.0).reshape(1, 32)
    x = ((np.arange(32, dtype=np.float32) + 1.0) / 16.0).reshape(1, 32)
    return w1, w2, x


def test_reference_packed_qmatmul_case(oracle):
    w1, w2, x = reference_packed_case()
    q1, q2 = oracle.quantize(Q8_0, w1), oracle.quantize(Q8_0, w2)
    packed = np.concatenate([q1, q2])  # packed_qmatmul_from_qtensors: byte concatenation
    y_packed = oracle.qmatmul(Q8_0, x, packed, 3)
    y_sep = np.concatenate([oracle.qmatmul(Q8_0, x, q1, 2), oracle.qmatmul(Q8_0, x, q2, 1)], axis=1)
    # the reference asserts 1e-5 closeness; row independence makes it exact here
    assert np.array_equal(y_packed, y_sep)
    # block fields: f16 scale bits and quants worked out by hand for this input
    d1, _ = np_ref.q8_0_fields(q1)
    d2, _ = np_ref.q8_0_fields(q2)
    bits = lambda d: int(np.float32(d).astype(np.float16).view(np.uint16))
    assert [bits(d1[0]), bits(d1[1]), bits(d2[0])] == [10192, 10248, 9372]
    xa = oracle.quantize_activations(Q8_0, x)
    dx, qx = np_ref.q8_0_fields(xa)
    assert bits(dx[0]) == 9224
    assert qx[0, 0] == 4 and qx[0, 1] == 8 and qx[0, 31] == 127
    # known answers of the quantized product (exact-math products: -42.625, 89.375, -26.714286)
    want = np.array([-42.692207, 89.229607, -26.613434], dtype=np.float32)
    assert np.allclose(y_packed[0], want, rtol=0, atol=2e-6)
    exact = np.concatenate([w1, w2]) @ x[0]
    assert np.allclose(y_packed[0], exact, rtol=5e-3)


@pytest.mark.parametrize("dtype,k", [(Q8_0, 256), (Q8_0, 1024), (Q4_K, 256), (Q4_K, 1024), (Q4_K, 768)])
def test_matmul_equals_integer_brute_force(oracle, dtype, k):
    n, m = 48, 3
    w = oracle.randn(100 + k + dtype, (n, k), std=0.02)
    x = oracle.randn(200 + k + dtype, (m, k))
    blocks = oracle.quantize(dtype, w)
    y = oracle.qmatmul(dtype, x, blocks, n)
    want = np_ref.qmatmul_int(dtype, x, blocks, n)
    scale = np.abs(want).max()
    # same integers, same scales; only f32 accumulation order/rounding separates them
    assert np.abs(y - want).max() <= 2e-6 * scale
    # and the quantized product stays near the dense product of the dequantized weights
    dense = x.astype(np.float64) @ oracle.dequantize(dtype, blocks, n, k).astype(np.float64).T
    assert np.abs(y - dense).max() <= 1e-2 * np.abs(dense).max()


def test_q4_k_min_term_sign_and_scale(oracle):
    # a weight block with q == 0 everywhere leaves only the -dmin*m*sum(x) term
    scales = bytes([0x41, 0x82, 0xC3, 0xC4, 0x40, 0x85, 0xCA, 0xCF, 0x41, 0x82, 0xC3, 0xFF])
    blk = bytes([0x00, 0x3C, 0x00, 0x38]) + scales + bytes(128)
    mins = [0, 5, 10, 15, 20, 40, 60, 63]
    x = np.zeros((1, 256), np.float32)
    x[0, :] = 1.0  # quantizes to -128 each with d = -1/128 -> exact
    y = oracle.qmatmul(Q4_K, x, np.frombuffer(blk, np.uint8), 1)
    assert y[0, 0] == -0.5 * 32 * sum(mins)
    # one nibble set: adds d*sc*q*x for that element only
    qs = bytearray(128)
    qs[32 + 7] = 0x90  # high nibble of byte 39 -> element 64+32+7, sub-block 3 (sc = 4), q = 9
    blk2 = bytes([0x00, 0x3C, 0x00, 0x38]) + scales + bytes(qs)
    y2 = oracle.qmatmul(Q4_K, x, np.frombuffer(blk2, np.uint8), 1)
    assert y2[0, 0] == y[0, 0] + 4 * 9


@pytest.mark.parametrize("k", [256, 768, 1024])
def test_q6_k_matmul_equals_integer_brute_force(oracle, k):
    """The reference's tests hold no Q6_K vector: the oracle's vec_dot is held to the integer dot
    products of an independent numpy reading of the public block format (random block bytes, so
    every quant, bit pair and signed scale occurs) and to the dense product of the dequantized
    weights."""
    n, m = 40, 3
    blocks = np_ref.random_q6_k_blocks(500 + k, n, k)
    x = oracle.randn(600 + k, (m, k))
    y = oracle.qmatmul(Q6_K, x, blocks, n)
    want = np_ref.qmatmul_int(Q6_K, x, blocks, n)
    assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max()
    dense = x.astype(np.float64) @ oracle.dequantize(Q6_K, blocks, n, k).astype(np.float64).T
    assert np.abs(y - dense).max() <= 1e-2 * np.abs(dense).max()
    # activations of a Q6_K weight are Q8_K blocks, the same bytes as for Q4_K
    assert np.array_equal(oracle.quantize_activations(Q6_K, x), oracle.quantize_activations(Q4_K, x))


def test_q6_k_closed_form_single_elements(oracle):
    """One block, d = 1, x = 1 everywhere (quantizes to -128 with d_x = -1/128, exact): y is the sum of
    scale_j * (q - 32) over the block, worked out by hand for a few byte patterns."""
    x = np.ones((1, 256), np.float32)

    def block(ql=None, qh=None, scales=None):
        b = bytearray(210)
        b[0:128] = ql if ql is not None else bytes(128)
        b[128:192] = qh if qh is not None else bytes(64)
        b[192:208] = bytes((s & 0xFF) for s in (scales if scales is not None else [1] * 16))
        b[208:210] = bytes([0x00, 0x3C])  # f16 1.0
        return np.frombuffer(bytes(b), np.uint8)

    # all quants zero: every element is -32, scales all 1 -> -32 * 256
    assert oracle.qmatmul(Q6_K, x, block(), 1)[0, 0] == -32.0 * 256
    # scales j = j - 8 (signed): sum_j (j - 8) * 16 * (-32)
    sc = [j - 8 for j in range(16)]
    assert oracle.qmatmul(Q6_K, x, block(scales=sc), 1)[0, 0] == -32.0 * 16 * sum(sc)
    # high nibble of ql[32 + 5] = 0xA: element 96 + 5 of the first half (group 6), scale 3 there
    ql = bytearray(128)
    ql[37] = 0xA0
    sc = [1] * 16
    sc[6] = 3
    base = -32.0 * 16 * sum(sc)
    assert oracle.qmatmul(Q6_K, x, block(ql=bytes(ql), scales=sc), 1)[0, 0] == base + 3 * 10
    # bits 4, 5 of qh[32 + 20] = 0b10: element 128 + 64 + 20 (group 8 + 5), adds 2 << 4 = 32
    qh = bytearray(64)
    qh[52] = 0x20
    sc = [1] * 16
    sc[13] = -7
    base = -32.0 * 16 * sum(sc)
    assert oracle.qmatmul(Q6_K, x, block(qh=bytes(qh), scales=sc), 1)[0, 0] == base + (-7) * 32
    # and the dequantized block says the same about that element
    w = oracle.dequantize(Q6_K, block(qh=bytes(qh), scales=sc), 1, 256)[0]
    assert w[128 + 64 + 20] == 0.0 and w[128 + 64 + 21] == -7 * -32.0


def test_rows_are_independent_and_m_loops(oracle):
    n, k = 40, 512
    blocks = oracle.quantize(Q4_K, oracle.randn(1, (n, k), std=0.02))
    x = oracle.randn(2, (5, k))
    y = oracle.qmatmul(Q4_K, x, blocks, n)
    for r in range(5):
        assert np.array_equal(y[r:r + 1], oracle.qmatmul(Q4_K, x[r:r + 1], blocks, n))
    # a row subset of the weight gives the same columns
    sub = blocks.reshape(n, -1)[8:24].reshape(-1)
    assert np.array_equal(oracle.qmatmul(Q4_K, x, sub, 16), y[:, 8:24])


def test_zero_activation_row_gives_zero(oracle):
    blocks = oracle.quantize(Q4_K, oracle.randn(3, (16, 256), std=0.02))
    y = oracle.qmatmul(Q4_K, np.zeros((1, 256), np.float32), blocks, 16)
    assert not y.any()
    blocks8 = oracle.quantize(Q8_0, oracle.randn(3, (16, 256), std=0.02))
    assert not oracle.qmatmul(Q8_0, np.zeros((2, 256), np.float32), blocks8, 16).any()
