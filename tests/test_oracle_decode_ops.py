"""Pins the oracle of the decode-step neighbours (RMSNorm, q/k norm, RoPE, single-token GQA
attention): the input vectors of the reference's own tests (kernels/metal.rs:2917-3290) with
expected values from the closed-form definitions in f64, within the 1e-5 those tests use, and an
independent numpy restatement on random inputs."""
import numpy as np
import pytest

TOL = 1e-5  # the reference's f32 tolerance (metal.rs:2956, 3058, 3147, 3275)


def np_rms_norm(x, w, eps):
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w.astype(np.float64)


def np_rope(x, cos, sin):
    """candle_nn::rotary_emb::rope on [b, s, h, d] (the reference's test transposes to [b, h, s, d] and
    back): the halves of the last dimension rotate against each other, position = index along s."""
    x = x.astype(np.float64)
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c = cos.astype(np.float64)[None, :, None, :]
    s = sin.astype(np.float64)[None, :, None, :]
    return np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c], axis=-1)


def np_attention(q, k, v, kv_len, scale):
    heads, d = q.shape[1], q.shape[3]
    kv_heads = k.shape[1]
    out = np.zeros((1, heads, 1, d))
    for h in range(heads):
        kh = h // (heads // kv_heads)
        kk = k[0, kh, :kv_len].astype(np.float64)
        vv = v[0, kh, :kv_len].astype(np.float64)
        s = kk @ q[0, h, 0].astype(np.float64) * scale
        p = np.exp(s - s.max())
        out[0, h, 0] = (p / p.sum()) @ vv
    return out


REF_X3 = np.array([0.2, -0.4, 0.6, 0.8, -1.0, 1.2, -1.4, 1.6, 1.8, -2.0, 2.2, -2.4], np.float32)
REF_W = np.array([1.0, 1.1, 0.9, 0.8], np.float32)


def test_rms_norm_reference_case(oracle):
    # metal.rs:2921-2937
    x = REF_X3.reshape(1, 3, 4)
    got = oracle.rms_norm(x, REF_W, 1e-6)
    assert np.abs(got - np_rms_norm(x, REF_W, 1e-6)).max() <= TOL
    # first row by hand: mean square = (0.04 + 0.16 + 0.36 + 0.64) / 4 = 0.3
    assert np.allclose(got[0, 0], x[0, 0] / np.sqrt(0.3 + 1e-6) * REF_W, atol=TOL)


def test_qk_rms_norm_reference_case(oracle):
    # metal.rs:3203-3226: q [1, 1, 2, 4], k [1, 1, 1, 4], separate weights concatenated
    q = REF_X3[:8].reshape(1, 1, 2, 4)
    k = np.array([0.3, -0.5, 0.7, -0.9], np.float32).reshape(1, 1, 1, 4)
    kw = np.array([0.7, 1.2, 0.6, 1.3], np.float32)
    qo, ko = oracle.qk_rms_norm(q, k, np.concatenate([REF_W, kw]), 1e-6)
    assert np.abs(qo - np_rms_norm(q, REF_W, 1e-6)).max() <= TOL
    assert np.abs(ko - np_rms_norm(k, kw, 1e-6)).max() <= TOL


def test_rope_pair_reference_case(oracle):
    # metal.rs:2970-2999: q [1, 2, 2, 4], k [1, 2, 1, 4], cos / sin [2, 2]
    q = np.array([0.2, -0.4, 0.6, 0.8, -1.0, 1.2, -1.4, 1.6, 1.8, -2.0, 2.2, -2.4, -2.6, 2.8, -3.0, 3.2],
                 np.float32).reshape(1, 2, 2, 4)
    k = np.array([0.3, -0.5, 0.7, -0.9, 1.1, -1.3, 1.5, -1.7], np.float32).reshape(1, 2, 1, 4)
    cos = np.array([0.9, 0.8, 0.7, 0.6], np.float32).reshape(2, 2)
    sin = np.array([0.1, 0.2, 0.3, 0.4], np.float32).reshape(2, 2)
    qo, ko = oracle.rope_pair_bshd(q, k, np.concatenate([cos, sin], axis=1))
    assert np.abs(qo - np_rope(q, cos, sin)).max() <= TOL
    assert np.abs(ko - np_rope(k, cos, sin)).max() <= TOL
    # one value by hand: q[0, 1, 0] = (-1.4 ...)? position 1, head 0 is row 2: [1.8, -2.0, 2.2, -2.4]
    assert abs(qo[0, 1, 0, 0] - (1.8 * 0.7 - 2.2 * 0.3)) <= TOL
    assert abs(qo[0, 1, 0, 3] - (-2.0 * 0.4 + -2.4 * 0.6)) <= TOL


def test_decode_gqa_attention_reference_case_and_padded_cache(oracle):
    # metal.rs:3079-3110 and 3153-3181: two heads on one kv head, three positions; then the same
    # with a cache of capacity five whose tail must be ignored
    q = REF_X3[:8].reshape(1, 2, 1, 4)
    k = np.array([0.3, -0.5, 0.7, -0.9, 1.1, -1.3, 1.5, -1.7, 1.9, -2.1, 2.3, -2.5], np.float32).reshape(1, 1, 3, 4)
    v = np.array([-0.2, 0.4, -0.6, 0.8, 1.0, -1.2, 1.4, -1.6, -1.8, 2.0, -2.2, 2.4], np.float32).reshape(1, 1, 3, 4)
    want = np_attention(q, k, v, 3, 0.5)
    assert np.abs(oracle.decode_gqa_attention(q, k, v, 3, 0.5) - want).max() <= TOL
    k_pad = np.concatenate([k, np.array([90, 91, 92, 93, -90, -91, -92, -93], np.float32).reshape(1, 1, 2, 4)], axis=2)
    v_pad = np.concatenate([v, np.array([80, 81, 82, 83, -80, -81, -82, -83], np.float32).reshape(1, 1, 2, 4)], axis=2)
    assert np.abs(oracle.decode_gqa_attention(q, k_pad, v_pad, 3, 0.5) - want).max() <= TOL
    with pytest.raises(ValueError):
        oracle.decode_gqa_attention(q, k_pad, v_pad, 6, 0.5)  # kv_len beyond the capacity


@pytest.mark.parametrize("rows,hidden", [(1, 4096), (5, 1024), (3, 128), (2, 100)])
def test_rms_norm_random(oracle, rows, hidden):
    x = oracle.randn(rows + hidden, (rows, hidden))
    w = oracle.randn(7, (hidden,), mean=1.0, std=0.1)
    want = np_rms_norm(x, w, 1e-6)
    assert np.abs(oracle.rms_norm(x, w, 1e-6) - want).max() <= 1e-5 * np.abs(want).max()


def test_rope_and_attention_random_qwen3_shapes(oracle):
    b, s, hq, hk, d = 2, 3, 32, 8, 128
    q, k = oracle.randn(1, (b, s, hq, d)), oracle.randn(2, (b, s, hk, d))
    ang = oracle.randn(3, (s, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    qo, ko = oracle.rope_pair_bshd(q, k, np.concatenate([cos, sin], axis=1))
    assert np.abs(qo - np_rope(q, cos, sin)).max() <= 1e-5 and np.abs(ko - np_rope(k, cos, sin)).max() <= 1e-5
    # rotation keeps the norm of every (d, d + half) pair
    assert np.allclose((qo ** 2).sum(-1), (q ** 2).sum(-1), rtol=1e-5)
    kv_len, cap = 300, 320
    q1 = oracle.randn(4, (1, hq, 1, d))
    kc, vc = oracle.randn(5, (1, hk, cap, d)), oracle.randn(6, (1, hk, cap, d))
    got = oracle.decode_gqa_attention(q1, kc, vc, kv_len, d ** -0.5)
    assert np.abs(got - np_attention(q1, kc, vc, kv_len, d ** -0.5)).max() <= 1e-5
    # one position: the output is that position's value row, whatever the scores
    one = oracle.decode_gqa_attention(q1, kc, vc, 1, 1.0)
    assert np.allclose(one[0, :, 0], np.repeat(vc[0, :, 0], hq // hk, axis=0), atol=1e-6)


def test_argmax_first_index_of_the_maximum(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 1000)).astype(np.float32)
    x[1, 17] = x[1, 900] = 9.0          # a tie: the first wins
    x[2, :] = -np.inf                   # every value equal
    x[3, 5] = np.nan                    # NaN is never the maximum
    x[3, 6] = 50.0
    got = oracle.argmax(x)
    want = np.argmax(np.where(np.isnan(x), -np.inf, x), axis=1)
    assert np.array_equal(got, want) and got[1] == 17 and got[2] == 0 and got[3] == 6
