"""One Qwen3 decoder layer at one token, composed from the library's calls (izwi_amd/qwen3_layer.py),
against the same composition of the CPU oracle's functions (pytest -m gpu)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q4_K = 12


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


def silu(v):
    return v / (1.0 + np.exp(-v))


@pytest.mark.parametrize("fuse_prep,fuse_norm,fuse_step", [(True, True, True), (False, False, False), (True, False, False),
                                                           (True, True, False)])
@pytest.mark.parametrize("hidden,heads,kv_heads,d,inter,steps", [(1024, 8, 2, 128, 3072, 5), (512, 8, 8, 64, 1024, 3)])
def test_decode_layer_matches_the_oracle_composition(qa, oracle, hidden, heads, kv_heads, d, inter, steps, fuse_prep, fuse_norm,
                                                     fuse_step):
    from izwi_amd.qwen3_layer import Qwen3DecodeLayer
    shapes = {"q": (heads * d, hidden), "k": (kv_heads * d, hidden), "v": (kv_heads * d, hidden),
              "o": (hidden, heads * d), "gate": (inter, hidden), "up": (inter, hidden), "down": (hidden, inter)}
    blocks = {n: oracle.quantize(Q4_K, oracle.randn(10 + i, s, std=0.03)) for i, (n, s) in enumerate(shapes.items())}
    mm = {n: qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks[n], shapes[n])) for n in shapes}
    w_in = oracle.randn(30, (hidden,), mean=1.0, std=0.1)
    w_post = oracle.randn(31, (hidden,), mean=1.0, std=0.1)
    qk_w = oracle.randn(32, (2 * d,), mean=1.0, std=0.1)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    layer = Qwen3DecodeLayer(dev(w_in), dev(w_post), mm["q"], mm["k"], mm["v"], dev(qk_w), mm["o"], mm["gate"],
                             mm["up"], mm["down"], heads, kv_heads, d, 1e-6, fuse_prep=fuse_prep, fuse_norm=fuse_norm,
                             fuse_step=fuse_step)
    cap = 16
    kc_d, vc_d = torch.zeros(1, kv_heads, cap, d, device="cuda"), torch.zeros(1, kv_heads, cap, d, device="cuda")
    kc, vc = np.zeros((1, kv_heads, cap, d), np.float32), np.zeros((1, kv_heads, cap, d), np.float32)
    qm = lambda n, x: oracle.qmatmul(Q4_K, x, blocks[n], shapes[n][0])  # noqa: E731
    for pos in range(steps):
        x = oracle.randn(100 + pos, (1, hidden))
        ang = (pos * (10000.0 ** (-np.arange(d // 2) / (d // 2)))).astype(np.float32)
        cos_sin = np.concatenate([np.cos(ang), np.sin(ang)]).astype(np.float32).reshape(1, d)
        got = layer.forward(dev(x), dev(cos_sin), kc_d, vc_d, pos).cpu().numpy()
        # the same steps with the oracle's functions
        normed = oracle.rms_norm(x, w_in, 1e-6)
        q, k, v = qm("q", normed), qm("k", normed), qm("v", normed)
        q4, k4 = oracle.qk_rms_norm(q.reshape(1, 1, heads, d), k.reshape(1, 1, kv_heads, d), qk_w, 1e-6)
        q4, k4 = oracle.rope_pair_bshd(q4, k4, cos_sin)
        kc[0, :, pos], vc[0, :, pos] = k4.reshape(kv_heads, d), v.reshape(kv_heads, d)
        attn = oracle.decode_gqa_attention(q4.reshape(1, heads, 1, d), kc, vc, pos + 1, d ** -0.5)
        x1 = x + qm("o", attn.reshape(1, heads * d))
        normed = oracle.rms_norm(x1, w_post, 1e-6)
        hid = (silu(qm("gate", normed)) * qm("up", normed)).astype(np.float32)
        want = x1 + qm("down", hid)
        assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max(), pos
        assert np.abs(kc_d.cpu().numpy() - kc).max() <= 1e-4 * np.abs(kc).max()
