"""The library's calls under HIP graph capture: a decode-layer token (projections with folded norms and
residuals, the attention step, argmax) is captured once and replayed several times with new inputs
and a growing cache position written into the captured buffers between replays; every replay must
equal the same calls run eagerly.  (Serving loops capture the step; the calls must neither allocate
nor memset inside the capture once their scratch is warm.)"""
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


def test_decode_layer_step_replays_equal_eager(qa, oracle):
    from izwi_amd.qwen3_layer import Qwen3DecodeLayer
    hidden, heads, kv_heads, d, inter, vocab = 1024, 8, 2, 128, 2048, 20000
    shapes = {"q": (heads * d, hidden), "k": (kv_heads * d, hidden), "v": (kv_heads * d, hidden), "o": (hidden, heads * d),
              "gate": (inter, hidden), "up": (inter, hidden), "down": (hidden, inter), "head": (vocab, hidden)}
    mm = {n: qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(
        qa.GgmlDType.Q4K, oracle.quantize(Q4_K, oracle.randn(40 + i, s, std=0.03)), s)) for i, (n, s) in enumerate(shapes.items())}
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    w_in, w_post, w_fin = (dev(oracle.randn(60 + i, (hidden,), mean=1.0, std=0.1)) for i in range(3))
    qk_w = dev(oracle.randn(63, (2 * d,), mean=1.0, std=0.1))
    layer = Qwen3DecodeLayer(w_in, w_post, mm["q"], mm["k"], mm["v"], qk_w, mm["o"], mm["gate"], mm["up"], mm["down"],
                             heads, kv_heads, d, 1e-6)
    cap, pos = 64, 40  # one captured position: the cache row it writes is overwritten by every replay
    kc0, vc0 = dev(oracle.randn(70, (1, kv_heads, cap, d))), dev(oracle.randn(71, (1, kv_heads, cap, d)))
    x, cos_sin = torch.zeros(1, hidden, device="cuda"), torch.zeros(1, d, device="cuda")
    kc, vc = kc0.clone(), vc0.clone()

    def step():
        y = layer.forward(x, cos_sin, kc, vc, pos)
        return y, qa.argmax(mm["head"].forward_normed(y, w_fin, 1e-6))

    def new_inputs(i):
        x.copy_(dev(oracle.randn(80 + i, (1, hidden))))
        ang = ((pos + i) * (10000.0 ** (-np.arange(d // 2) / (d // 2)))).astype(np.float32)
        cos_sin.copy_(dev(np.concatenate([np.cos(ang), np.sin(ang)]).reshape(1, d)))

    new_inputs(0)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        step()  # the stream's scratch buffer and lazy module loads happen outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            y_g, tok_g = step()
    torch.cuda.synchronize()
    for i in range(1, 5):
        new_inputs(i)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_y, got_tok, got_k = y_g.clone(), tok_g.clone(), kc[0, :, pos].clone()
        # the same calls eagerly, on the same inputs (other work and synchronizations between replays)
        kc_e, vc_e = kc0.clone(), vc0.clone()
        want_y = layer.forward(x, cos_sin, kc_e, vc_e, pos)
        want_tok = qa.argmax(mm["head"].forward_normed(want_y, w_fin, 1e-6))
        torch.cuda.synchronize()
        assert torch.equal(got_y, want_y), i
        assert torch.equal(got_tok, want_tok), i
        assert torch.equal(got_k, kc_e[0, :, pos]), i
