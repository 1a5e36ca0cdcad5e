"""GPU parity of the decode-step neighbours (pytest -m gpu): the HIP kernels behind the
reference's fused-kernel hooks against the CPU oracle, through the C ABI.  Tolerance: the
reference's own 1e-5 for f32 (kernels/metal.rs:2956), absolute on its O(1) test vectors and
relative to max|y| on the model-sized inputs."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def close(got, want, tol=TOL):
    want = np.asarray(want, dtype=np.float64)
    return float(np.abs(got.cpu().numpy() - want).max()) <= tol * max(1.0, float(np.abs(want).max()))


REF_X3 = np.array([0.2, -0.4, 0.6, 0.8, -1.0, 1.2, -1.4, 1.6, 1.8, -2.0, 2.2, -2.4], np.float32)
REF_W = np.array([1.0, 1.1, 0.9, 0.8], np.float32)


def test_reference_test_vectors(qa, oracle):
    """The four cases of the reference's own tests (metal.rs:2917-3290)."""
    x = REF_X3.reshape(1, 3, 4)
    assert close(qa.try_fused_rms_norm(dev(x), dev(REF_W), 1e-6), oracle.rms_norm(x, REF_W, 1e-6))
    q = REF_X3[:8].reshape(1, 1, 2, 4)
    k = np.array([0.3, -0.5, 0.7, -0.9], np.float32).reshape(1, 1, 1, 4)
    qkw = np.concatenate([REF_W, np.array([0.7, 1.2, 0.6, 1.3], np.float32)])
    qo, ko = qa.try_fused_qk_rms_norm(dev(q), dev(k), dev(qkw), 1e-6)
    wq, wk = oracle.qk_rms_norm(q, k, qkw, 1e-6)
    assert close(qo, wq) and close(ko, wk) and qo.shape == (1, 1, 2, 4) and ko.shape == (1, 1, 1, 4)
    q = np.array([0.2, -0.4, 0.6, 0.8, -1.0, 1.2, -1.4, 1.6, 1.8, -2.0, 2.2, -2.4, -2.6, 2.8, -3.0, 3.2],
                 np.float32).reshape(1, 2, 2, 4)
    k = np.array([0.3, -0.5, 0.7, -0.9, 1.1, -1.3, 1.5, -1.7], np.float32).reshape(1, 2, 1, 4)
    cs = np.array([[0.9, 0.8, 0.1, 0.2], [0.7, 0.6, 0.3, 0.4]], np.float32)
    qo, ko = qa.try_fused_rope_pair_bshd(dev(q), dev(k), dev(cs))
    wq, wk = oracle.rope_pair_bshd(q, k, cs)
    assert close(qo, wq) and close(ko, wk)
    # attention: head_dim 4 is below what the kernel is built for -> the hook declines (None), as the
    # reference's does off Metal; the same case at head_dim 64 (zero-padded) is computed
    q4 = REF_X3[:8].reshape(1, 2, 1, 4)
    k4 = np.array([0.3, -0.5, 0.7, -0.9, 1.1, -1.3, 1.5, -1.7, 1.9, -2.1, 2.3, -2.5], np.float32).reshape(1, 1, 3, 4)
    v4 = np.array([-0.2, 0.4, -0.6, 0.8, 1.0, -1.2, 1.4, -1.6, -1.8, 2.0, -2.2, 2.4], np.float32).reshape(1, 1, 3, 4)
    assert qa.try_fused_decode_gqa_attention(dev(q4), dev(k4), dev(v4), 2, 1, 4, 0.5) is None
    pad = lambda a: np.concatenate([a, np.zeros(a.shape[:-1] + (60,), np.float32)], axis=-1)  # noqa: E731
    want = oracle.decode_gqa_attention(q4, k4, v4, 3, 0.5)
    got = qa.try_fused_decode_gqa_attention(dev(pad(q4)), dev(pad(k4)), dev(pad(v4)), 2, 1, 64, 0.5)
    assert close(got[..., :4], want) and not got[..., 4:].any()
    # cache with capacity 5 whose tail must be ignored (metal.rs:3153-3181)
    k5 = np.concatenate([k4, np.array([90, 91, 92, 93, -90, -91, -92, -93], np.float32).reshape(1, 1, 2, 4)], axis=2)
    v5 = np.concatenate([v4, np.array([80, 81, 82, 83, -80, -81, -82, -83], np.float32).reshape(1, 1, 2, 4)], axis=2)
    got = qa.try_fused_decode_gqa_attention_with_kv_len(dev(pad(q4)), dev(pad(k5)), dev(pad(v5)), 2, 1, 64, 3, 0.5)
    assert close(got[..., :4], want)


@pytest.mark.parametrize("rows,hidden", [(1, 4096), (16, 4096), (64, 4096), (3, 1024), (5, 100), (2, 6), (1, 12288),
                                         (2, 20000), (7, 5120)])
def test_rms_norm_shapes(qa, oracle, rows, hidden):
    _say(f"rms_norm rows={rows} hidden={hidden}")
    x = oracle.randn(rows + hidden, (rows, hidden))
    w = oracle.randn(3, (hidden,), mean=1.0, std=0.1)
    xd = dev(x)
    got = qa.try_fused_rms_norm(xd, dev(w), 1e-6)
    assert close(got, oracle.rms_norm(x, w, 1e-6))
    # a view that is not 16-byte aligned takes the scalar path: same values within rounding
    if hidden > 8:
        flat = torch.zeros(rows * hidden + 1, device="cuda")
        flat[1:] = xd.reshape(-1)
        assert close(qa.try_fused_rms_norm(flat[1:].view(rows, hidden), dev(w), 1e-6), oracle.rms_norm(x, w, 1e-6))


def test_rms_norm_in_place_through_the_c_abi(qa, oracle):
    from izwi_amd import capi
    x = oracle.randn(1, (4, 4096))
    w = oracle.randn(2, (4096,), mean=1.0, std=0.1)
    buf, wd = dev(x), dev(w)
    assert capi.lib().izwi_rms_norm_f32(buf.data_ptr(), wd.data_ptr(), 4, 4096, 1e-6, buf.data_ptr(), capi.DEVICE, None) == 0
    assert close(buf, oracle.rms_norm(x, w, 1e-6))
    # host pointers
    out = np.empty_like(x)
    assert capi.lib().izwi_rms_norm_f32(x.ctypes.data, w.ctypes.data, 4, 4096, 1e-6, out.ctypes.data, capi.HOST, None) == 0
    assert np.abs(out - oracle.rms_norm(x, w, 1e-6)).max() <= 1e-5 * np.abs(out).max()
    assert capi.lib().izwi_rms_norm_f32(buf.data_ptr(), wd.data_ptr(), 4, 0, 1e-6, buf.data_ptr(), capi.DEVICE, None) == -1
    assert capi.lib().izwi_rms_norm_f32(buf.data_ptr(), wd.data_ptr(), 0, 4096, 1e-6, buf.data_ptr(), capi.DEVICE, None) == 0


@pytest.mark.parametrize("b,hq,hk,d", [(1, 32, 8, 128), (4, 32, 8, 128), (1, 16, 8, 64), (2, 5, 1, 256), (1, 3, 2, 20)])
def test_qk_rms_norm_shapes(qa, oracle, b, hq, hk, d):
    q, k = oracle.randn(1, (b, 1, hq, d)), oracle.randn(2, (b, 1, hk, d))
    w = oracle.randn(3, (2 * d,), mean=1.0, std=0.2)
    qo, ko = qa.try_fused_qk_rms_norm(dev(q), dev(k), dev(w), 1e-6)
    wq, wk = oracle.qk_rms_norm(q, k, w, 1e-6)
    assert close(qo, wq) and close(ko, wk)
    # the pair equals two plain norms with the two halves of the weight
    assert torch.equal(qo, qa.try_fused_rms_norm(dev(q), dev(w[:d]), 1e-6))
    assert torch.equal(ko, qa.try_fused_rms_norm(dev(k), dev(w[d:]), 1e-6))


@pytest.mark.parametrize("b,s,hq,hk,d", [(1, 1, 32, 8, 128), (2, 7, 32, 8, 128), (1, 300, 16, 2, 64), (3, 2, 1, 1, 2)])
def test_rope_pair_shapes(qa, oracle, b, s, hq, hk, d):
    q, k = oracle.randn(1, (b, s, hq, d)), oracle.randn(2, (b, s, hk, d))
    ang = oracle.randn(3, (s, d // 2)) * 3.0
    cs = np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)
    qo, ko = qa.try_fused_rope_pair_bshd(dev(q), dev(k), dev(cs))
    wq, wk = oracle.rope_pair_bshd(q, k, cs)
    assert close(qo, wq) and close(ko, wk)
    # a rotation keeps the length of every head vector
    assert torch.allclose((qo ** 2).sum(-1), (dev(q) ** 2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("heads,kv_heads,d,kv_len,cap", [
    (32, 8, 128, 1, 1), (32, 8, 128, 17, 64), (32, 8, 128, 300, 512), (32, 8, 128, 2048, 2048),
    (32, 8, 128, 5000, 8192), (16, 8, 128, 777, 1000), (8, 8, 128, 100, 100), (24, 4, 128, 129, 200),
    (14, 2, 64, 333, 400), (16, 16, 64, 64, 64), (8, 2, 256, 500, 512), (3, 3, 256, 65, 65)])
def test_decode_gqa_attention_shapes(qa, oracle, heads, kv_heads, d, kv_len, cap):
    _say(f"attention heads={heads} kv_heads={kv_heads} d={d} kv_len={kv_len} cap={cap}")
    q = oracle.randn(1, (1, heads, 1, d))
    k, v = oracle.randn(2, (1, kv_heads, cap, d)), oracle.randn(3, (1, kv_heads, cap, d))
    k[:, :, kv_len:] = 1e4  # whatever sits past kv_len must not count
    v[:, :, kv_len:] = -1e4
    scale = d ** -0.5
    got = qa.try_fused_decode_gqa_attention_with_kv_len(dev(q), dev(k), dev(v), heads, kv_heads, d, kv_len, scale)
    want = oracle.decode_gqa_attention(q, k, v, kv_len, scale)
    assert got.shape == (1, heads, 1, d)
    assert close(got, want)
    if kv_len == cap:
        assert torch.equal(got, qa.try_fused_decode_gqa_attention(dev(q), dev(k), dev(v), heads, kv_heads, d, scale))


def test_decode_gqa_attention_long_cache_and_peaked_scores(qa, oracle):
    """40960 positions (the longest context of the 8B model) split over many workgroups; and scores
    spread over +-60 so that the running-maximum rescaling does all the work."""
    heads, kv_heads, d, kv_len = 32, 8, 128, 40960
    q = oracle.randn(1, (1, heads, 1, d))
    k, v = oracle.randn(2, (1, kv_heads, kv_len, d)), oracle.randn(3, (1, kv_heads, kv_len, d))
    got = qa.try_fused_decode_gqa_attention(dev(q), dev(k), dev(v), heads, kv_heads, d, d ** -0.5)
    assert close(got, oracle.decode_gqa_attention(q, k, v, kv_len, d ** -0.5))
    kv_len = 3000
    k2 = k[:, :, :kv_len].copy() * 4.0
    got = qa.try_fused_decode_gqa_attention(dev(q), dev(k2), dev(v[:, :, :kv_len]), heads, kv_heads, d, 0.5)
    want = oracle.decode_gqa_attention(q, k2, v[:, :, :kv_len], kv_len, 0.5)
    assert close(got, want, 2e-5)


def test_hooks_decline_what_the_reference_declines(qa, oracle):
    x = dev(oracle.randn(1, (2, 8)))
    w = dev(oracle.randn(2, (8,)))
    assert qa.try_fused_rms_norm(x.cpu(), w.cpu(), 1e-6) is None                 # not on the GPU
    assert qa.try_fused_rms_norm(x.bfloat16(), w.bfloat16(), 1e-6) is None       # the hooks take f32 and f16 only
    assert qa.try_fused_rms_norm(x.half(), w, 1e-6) is None                      # mixed types
    assert qa.try_fused_rms_norm(x.t(), w[:2], 1e-6) is None                     # not contiguous
    assert qa.try_fused_rms_norm(x, w[:4], 1e-6) is None                         # weight shape
    q = dev(oracle.randn(3, (1, 2, 4, 8)))
    assert qa.try_fused_qk_rms_norm(q, q, dev(oracle.randn(4, (16,))), 1e-6) is None   # seq != 1
    assert qa.try_fused_rope_pair_bshd(q, q, dev(oracle.randn(5, (2, 6)))) is None      # cos_sin shape
    q1 = dev(oracle.randn(6, (1, 4, 1, 64)))
    kv = dev(oracle.randn(7, (1, 2, 10, 64)))
    assert qa.try_fused_decode_gqa_attention_with_kv_len(q1, kv, kv, 4, 2, 64, 11, 1.0) is None  # kv_len > capacity
    assert qa.try_fused_decode_gqa_attention(q1, kv, kv, 4, 3, 64, 1.0) is None                   # heads % kv_heads
    from izwi_amd import capi
    L = capi.lib()
    out = torch.empty_like(q1)
    assert L.izwi_decode_gqa_attention_f32(q1.data_ptr(), kv.data_ptr(), kv.data_ptr(), 4, 2, 48, 10, 10, C.c_float(1.0),
                                           out.data_ptr(), capi.DEVICE, None) == -2
    assert L.izwi_decode_gqa_attention_f32(q1.data_ptr(), kv.data_ptr(), kv.data_ptr(), 4, 2, 64, 0, 10, C.c_float(1.0),
                                           out.data_ptr(), capi.DEVICE, None) == -1


@pytest.mark.parametrize("heads,kv_heads,d", [(32, 8, 128), (16, 8, 64), (4, 2, 256), (3, 1, 20), (2, 2, 512)])
def test_qk_norm_rope_append_equals_the_separate_hooks(qa, oracle, heads, kv_heads, d):
    """The one-launch form of q/k norm + rotary + cache append against the oracle's composition and the
    library's own separate calls; positions other than `pos` of the caches stay untouched."""
    cap, pos = 9, 5
    q, k, v = oracle.randn(1, (heads * d,)), oracle.randn(2, (kv_heads * d,)), oracle.randn(3, (kv_heads * d,))
    w = oracle.randn(4, (2 * d,), mean=1.0, std=0.2)
    ang = oracle.randn(5, (d // 2,)) * 3.0
    cs = np.concatenate([np.cos(ang), np.sin(ang)]).astype(np.float32).reshape(1, d)
    kc0, vc0 = oracle.randn(6, (1, kv_heads, cap, d)), oracle.randn(7, (1, kv_heads, cap, d))
    kc, vc = dev(kc0), dev(vc0)
    q_rot = qa.qk_norm_rope_append(dev(q), dev(k), dev(v), dev(w), dev(cs), kc, vc, pos, 1e-6)
    qn, kn = oracle.qk_rms_norm(q.reshape(1, 1, heads, d), k.reshape(1, 1, kv_heads, d), w, 1e-6)
    qr, kr = oracle.rope_pair_bshd(qn, kn, cs)
    assert q_rot.shape == (1, heads, 1, d) and close(q_rot.view(1, 1, heads, d), qr)
    want_k, want_v = kc0.copy(), vc0.copy()
    want_k[0, :, pos], want_v[0, :, pos] = kr.reshape(kv_heads, d), v.reshape(kv_heads, d)
    assert close(kc, want_k) and torch.equal(vc, dev(want_v))
    assert torch.equal(kc[0, :, :pos], dev(kc0)[0, :, :pos]) and torch.equal(kc[0, :, pos + 1:], dev(kc0)[0, :, pos + 1:])
    if True:
        q2, k2 = qa.try_fused_qk_rms_norm(dev(q).view(1, 1, heads, d), dev(k).view(1, 1, kv_heads, d), dev(w), 1e-6)
        q2, k2 = qa.try_fused_rope_pair_bshd(q2, k2, dev(cs))
        assert torch.allclose(q_rot.view(1, 1, heads, d), q2, rtol=2e-6, atol=1e-6)
        assert torch.allclose(kc[0, :, pos], k2.view(kv_heads, d), rtol=2e-6, atol=1e-6)
    from izwi_amd import capi
    L = capi.lib()
    assert L.izwi_qk_norm_rope_append_f32(kc.data_ptr(), kc.data_ptr(), kc.data_ptr(), kc.data_ptr(), kc.data_ptr(), heads,
                                          kv_heads, d, 1e-6, kc.data_ptr(), kc.data_ptr(), vc.data_ptr(), cap, cap, None) == -1


@pytest.mark.parametrize("heads,kv_heads,d,pos,cap", [
    (32, 8, 128, 0, 4), (32, 8, 128, 5, 9), (32, 8, 128, 300, 512), (32, 8, 128, 4095, 4096), (32, 8, 128, 1000, 1001),
    (8, 8, 64, 77, 100), (6, 3, 256, 130, 200), (4, 4, 128, 64, 65),
])
def test_decode_attention_step_equals_prep_then_attention(qa, oracle, heads, kv_heads, d, pos, cap):
    """The one-call form (q/k norm, rotary and cache append inside the attention launch) against the two
    calls it replaces, bit for bit (output and caches), and against the oracle's composition."""
    print(f"attention step heads={heads} kv={kv_heads} d={d} pos={pos} cap={cap}", flush=True)
    q, k, v = oracle.randn(1, (heads * d,)), oracle.randn(2, (kv_heads * d,)), oracle.randn(3, (kv_heads * d,))
    w = oracle.randn(4, (2 * d,), mean=1.0, std=0.2)
    ang = oracle.randn(5, (d // 2,)) * 3.0
    cs = np.concatenate([np.cos(ang), np.sin(ang)]).astype(np.float32).reshape(1, d)
    kc0, vc0 = oracle.randn(6, (1, kv_heads, cap, d)), oracle.randn(7, (1, kv_heads, cap, d))
    kc_a, vc_a, kc_b, vc_b = dev(kc0), dev(vc0), dev(kc0), dev(vc0)
    scale = d ** -0.5
    q_rot = qa.qk_norm_rope_append(dev(q), dev(k), dev(v), dev(w), dev(cs), kc_a, vc_a, pos, 1e-6)
    want = qa.try_fused_decode_gqa_attention_with_kv_len(q_rot, kc_a, vc_a, heads, kv_heads, d, pos + 1, scale)
    got = qa.decode_attention_step(dev(q), dev(k), dev(v), dev(w), dev(cs), kc_b, vc_b, pos, 1e-6, scale)
    assert got.shape == (1, heads, 1, d)
    assert torch.equal(got, want) and torch.equal(kc_b, kc_a) and torch.equal(vc_b, vc_a)
    if pos <= 300:
        qn, kn = oracle.qk_rms_norm(q.reshape(1, 1, heads, d), k.reshape(1, 1, kv_heads, d), w, 1e-6)
        qr, kr = oracle.rope_pair_bshd(qn, kn, cs)
        kc0[0, :, pos], vc0[0, :, pos] = kr.reshape(kv_heads, d), v.reshape(kv_heads, d)
        assert close(got, oracle.decode_gqa_attention(qr.reshape(1, heads, 1, d), kc0, vc0, pos + 1, scale))
    from izwi_amd import capi
    p = kc_b.data_ptr()
    assert capi.lib().izwi_decode_attention_step_f32(p, p, p, p, p, heads, kv_heads, d, 1e-6, p, p, cap, cap, scale, p, None) == -1


@pytest.mark.parametrize("rows,n", [(1, 151936), (4, 151936), (3, 1000), (2, 7), (1, 1), (5, 4097), (3, 20000), (2, 16385)])
def test_argmax_on_device(qa, oracle, rows, n):
    x = oracle.randn(rows + n, (rows, n))
    if n > 20:
        x[0, 17] = x[0, n - 3] = 9.0     # tie: first index
        x[-1, :] = -np.inf
        x[-1, 5] = np.nan
    got = qa.argmax(dev(x))
    assert got.dtype == torch.int32 and tuple(got.shape) == (rows,)
    assert np.array_equal(got.cpu().numpy().astype(np.uint32), oracle.argmax(x))
    # after the LM head: greedy token = argmax of the projection's output, no logits to the host
    from izwi_amd import capi
    out = np.empty(rows, np.uint32)
    assert capi.lib().izwi_argmax_f32(x.ctypes.data, rows, n, out.ctypes.data, capi.HOST, None) == 0
    assert np.array_equal(out, oracle.argmax(x))
    assert capi.lib().izwi_argmax_f32(x.ctypes.data, rows, 0, out.ctypes.data, capi.HOST, None) == -1


F16_TOL = 2.0 ** -10  # one rounding to f16 of an f32 result; the reference allows 5e-3 (metal.rs:2956)


def half(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float16)).cuda()


def close16(got, want_f32):
    """got (f16 tensor) against the f32 oracle result rounded to f16: equal up to the last f16 bit of the sums."""
    want = np.asarray(want_f32, dtype=np.float32).astype(np.float16).astype(np.float64)
    g = got.float().cpu().numpy().astype(np.float64)
    return got.dtype == torch.float16 and float(np.abs(g - want).max()) <= F16_TOL * max(1.0, float(np.abs(want).max()))


def test_f16_arm_reference_vectors_and_model_shapes(qa, oracle):
    """The hooks' F16 arm: the reference's test vectors (its tests run both dtypes, metal.rs:2920, 2969, 3076,
    3202) and Qwen3 shapes; the oracle is the f32 oracle on the widened inputs, rounded once."""
    w16 = lambda a: np.asarray(a, np.float16).astype(np.float32)  # noqa: E731  (the values the kernel sees)
    x = w16(REF_X3.reshape(1, 3, 4))
    assert close16(qa.try_fused_rms_norm(half(x), half(REF_W), 1e-6), oracle.rms_norm(x, w16(REF_W), 1e-6))
    for rows, hidden in ((1, 4096), (5, 1000), (3, 36)):
        xx, ww = w16(oracle.randn(1, (rows, hidden))), w16(oracle.randn(2, (hidden,), mean=1.0, std=0.1))
        assert close16(qa.try_fused_rms_norm(half(xx), half(ww), 1e-6), oracle.rms_norm(xx, ww, 1e-6))
    q, k = w16(oracle.randn(3, (2, 1, 32, 128))), w16(oracle.randn(4, (2, 1, 8, 128)))
    qkw = w16(oracle.randn(5, (256,), mean=1.0, std=0.2))
    qo, ko = qa.try_fused_qk_rms_norm(half(q), half(k), half(qkw), 1e-6)
    wq, wk = oracle.qk_rms_norm(q, k, qkw, 1e-6)
    assert close16(qo, wq) and close16(ko, wk)
    q, k = w16(oracle.randn(6, (2, 5, 32, 128))), w16(oracle.randn(7, (2, 5, 8, 128)))
    ang = oracle.randn(8, (5, 64)) * 3.0
    cs = w16(np.concatenate([np.cos(ang), np.sin(ang)], axis=1))
    qo, ko = qa.try_fused_rope_pair_bshd(half(q), half(k), half(cs))
    wq, wk = oracle.rope_pair_bshd(q, k, cs)
    assert close16(qo, wq) and close16(ko, wk)


@pytest.mark.parametrize("heads,kv_heads,d,kv_len,cap", [(32, 8, 128, 1, 4), (32, 8, 128, 300, 512), (32, 8, 128, 5000, 5000),
                                                         (14, 2, 64, 333, 400), (8, 2, 256, 500, 512), (16, 8, 128, 40960, 40960)])
def test_f16_attention(qa, oracle, heads, kv_heads, d, kv_len, cap):
    q = oracle.randn(1, (1, heads, 1, d)).astype(np.float16).astype(np.float32)
    k = oracle.randn(2, (1, kv_heads, cap, d)).astype(np.float16).astype(np.float32)
    v = oracle.randn(3, (1, kv_heads, cap, d)).astype(np.float16).astype(np.float32)
    k[:, :, kv_len:], v[:, :, kv_len:] = 1e4, -1e4
    got = qa.try_fused_decode_gqa_attention_with_kv_len(half(q), half(k), half(v), heads, kv_heads, d, kv_len, d ** -0.5)
    assert got.shape == (1, heads, 1, d)
    assert close16(got, oracle.decode_gqa_attention(q, k, v, kv_len, d ** -0.5))
