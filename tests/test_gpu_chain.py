"""Chained decode (izwi_qmm_chain_*, pytest -m gpu): a list of dependent projection steps as one
launch, bit-identical to the same steps issued as separate izwi_qmm_forward_group_f32 calls, and its
bounded waits (a wait that gives up is reported, every workgroup still exits)."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12


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


def weight(qa, oracle, dtype, n, k, seed, blocks_out=None):
    blocks = oracle.quantize(dtype, oracle.randn(seed, (n, k), std=0.02))
    if blocks_out is not None:
        blocks_out.append(blocks)
    return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))


def layer_steps(qa, oracle, dtype, hidden, q_out, kv_out, inter, layers, seed):
    """The projections of `layers` decoder layers wired so that data really flows from step to step:
    q|k|v reads the hidden state, o reads q's output, gate|up reads o's, down reads gate's, the next
    layer reads down's (attention and activation left out: they are not projections)."""
    f = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    x0 = torch.from_numpy(oracle.randn(seed, (hidden,))).cuda()
    steps, x = [], x0
    for li in range(layers):
        s = seed + 10 * li
        q, k, v = (weight(qa, oracle, dtype, n, hidden, s + i) for i, n in enumerate((q_out, kv_out, kv_out)))
        o = weight(qa, oracle, dtype, hidden, q_out, s + 3)
        g, u = (weight(qa, oracle, dtype, inter, hidden, s + 4 + i) for i in range(2))
        d = weight(qa, oracle, dtype, hidden, inter, s + 6)
        yq, yk, yv, yo, yg, yu, yd = f(q_out), f(kv_out), f(kv_out), f(hidden), f(inter), f(inter), f(hidden)
        steps += [([q, k, v], x, [yq, yk, yv]), ([o], yq, [yo]), ([g, u], yo, [yg, yu]), ([d], yg, [yd])]
        x = yd
    return x0, steps


def run_separately(qa, steps):
    for projections, x, ys in steps:
        outs = qa.forward_group(projections, x.view(1, -1))
        for y, o in zip(ys, outs):
            y.copy_(o.view(-1))
    torch.cuda.synchronize()
    return [[y.clone() for y in ys] for _, _, ys in steps]


@pytest.mark.parametrize("dtype,hidden,q_out,kv_out,inter,layers", [
    (Q4_K, 4096, 4096, 1024, 12288, 3),      # Qwen3-8B shapes
    (Q8_0, 1024, 2048, 1024, 3072, 4),       # Qwen3-0.6B shapes
    (Q4_K, 1024, 1280, 256, 2816, 2)])       # ragged: row tiles that do not fill the grid, 11 panels per row tile
def test_chain_equals_separate_calls(qa, oracle, dtype, hidden, q_out, kv_out, inter, layers):
    _say(f"chain dtype={dtype} hidden={hidden} layers={layers}")
    x0, steps = layer_steps(qa, oracle, dtype, hidden, q_out, kv_out, inter, layers, 3000)
    want = run_separately(qa, steps)
    for _, _, ys in steps:
        for y in ys:
            y.fill_(float("nan"))
    chain = qa.DecodeChain(steps)
    for rep in range(3):            # the counters are left at zero by every run
        chain.run()
        chain.status()
        for si, (_, _, ys) in enumerate(steps):
            for y, w in zip(ys, want[si]):
                assert torch.equal(y, w), (rep, si)
        for _, _, ys in steps:
            for y in ys:
                y.fill_(float("nan"))
    # the oracle on the first step: the chain computes the reference's product
    blocks = []
    w = weight(qa, oracle, dtype, 64, hidden, 3999, blocks)
    y = torch.zeros(64, device="cuda")
    c2 = qa.DecodeChain([([w], x0, [y])])
    c2.run()
    c2.status()
    ref = oracle.qmatmul(dtype, x0.cpu().numpy().reshape(1, -1), blocks[0], 64)[0]
    assert float(np.abs(y.cpu().numpy() - ref).max() / np.abs(ref).max()) < 1e-4


def test_chain_q6_k_random_blocks(qa, oracle):
    """Q6_K weights (the oracle has no Q6_K quantizer: random block bytes with a finite scale), 3 units per
    panel at k = 768."""
    import np_ref
    def w6(n, k, seed):
        return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(14), np_ref.random_q6_k_blocks(seed, n, k), (n, k)))
    f = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    x0 = torch.from_numpy(oracle.randn(3400, (2048,))).cuda()
    a, b, c = w6(768, 2048, 1), w6(512, 2048, 2), w6(2048, 768, 3)
    ya, yb, yc = f(768), f(512), f(2048)
    steps = [([a, b], x0, [ya, yb]), ([c], ya, [yc]), ([a], yc, [f(768)])]
    want = run_separately(qa, steps)
    chain = qa.DecodeChain(steps)
    for _, _, ys in steps:
        for y in ys:
            y.fill_(float("nan"))
    chain.run()
    chain.status()
    for si, (_, _, ys) in enumerate(steps):
        for y, w in zip(ys, want[si]):
            assert torch.equal(y, w), si


def test_chain_in_a_graph_and_with_a_tall_matrix(qa, oracle):
    hidden = 4096
    x0, steps = layer_steps(qa, oracle, Q4_K, hidden, 4096, 1024, 12288, 1, 3100)
    head = weight(qa, oracle, Q4_K, 40000, hidden, 3190)      # many rounds of row tiles per workgroup
    logits = torch.zeros(40000, device="cuda")
    steps.append(([head], steps[-1][2][0], [logits]))
    want = run_separately(qa, steps)
    chain = qa.DecodeChain(steps)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        chain.run()
        s.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            chain.run()
        for rep in range(4):
            for _, _, ys in steps:
                for y in ys:
                    y.fill_(float("nan"))
            g.replay()
            chain.status()
            for si, (_, _, ys) in enumerate(steps):
                for y, w in zip(ys, want[si]):
                    assert torch.equal(y, w), (rep, si)


def test_a_wait_that_gives_up_is_reported_and_the_chain_recovers(qa, oracle):
    from izwi_amd import capi
    x0, steps = layer_steps(qa, oracle, Q4_K, 1024, 1024, 256, 3072, 2, 3200)
    want = run_separately(qa, steps)
    chain = qa.DecodeChain(steps)
    chain.set_spin_limit(0)            # a step whose predecessor is not yet complete gives up at its first poll
    chain.run()
    with pytest.raises(capi.QmmError, match="gave up"):
        chain.status()                 # every workgroup exited; the error word is reported and cleared
    chain.set_spin_limit(1 << 21)
    for rep in range(2):
        chain.run()
        chain.status()
        for si, (_, _, ys) in enumerate(steps):
            for y, w in zip(ys, want[si]):
                assert torch.equal(y, w), (rep, si)


def test_chain_argument_errors(qa, oracle):
    from izwi_amd import capi
    w4 = weight(qa, oracle, Q4_K, 64, 1024, 3300)
    w8 = weight(qa, oracle, Q8_0, 64, 1024, 3301)
    wk = weight(qa, oracle, Q4_K, 64, 2048, 3302)
    x = torch.zeros(1024, device="cuda")
    y = [torch.zeros(64, device="cuda") for _ in range(2)]
    with pytest.raises(capi.QmmError, match="one block type"):
        qa.DecodeChain([([w4], x, y[:1]), ([w8], x, y[1:])])
    with pytest.raises(capi.QmmError, match="input mismatch"):
        arr = (capi.ChainStep * 1)()
        arr[0].n_weights = 2
        arr[0].x = x.data_ptr()
        arr[0].weights[0], arr[0].weights[1] = w4.qtensor._h, wk.qtensor._h
        arr[0].ys[0], arr[0].ys[1] = y[0].data_ptr(), y[1].data_ptr()
        import ctypes as C
        h = C.c_void_p()
        capi.check(capi.lib().izwi_qmm_chain_create(arr, 1, C.byref(h)))
    big = weight(qa, oracle, Q4_K, 16, 16384, 3303)            # 16 panels per row tile: no chained form
    with pytest.raises(capi.QmmError, match="no chained form"):
        qa.DecodeChain([([big], torch.zeros(16384, device="cuda"), [torch.zeros(16, device="cuda")])])
    tall = weight(qa, oracle, Q8_0, 70000, 256, 3304)          # the per-call kernel splits a very tall matrix otherwise
    with pytest.raises(capi.QmmError, match="no chained form"):
        qa.DecodeChain([([tall], torch.zeros(256, device="cuda"), [torch.zeros(70000, device="cuda")])])
