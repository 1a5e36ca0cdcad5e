"""GPU tests of the host-pointer form of the entry points (pytest -m gpu): the literal shape of the
reference's CPU call, `QMatMul::forward` on tensors in host memory
(crates/izwi-core/src/models/architectures/qwen3/core.rs:791-831).  The library stages such calls
through pooled pinned buffers (inputs copied to the device, outputs stored by the kernels into
pinned memory); the results have to be the device-pointer results bit for bit, whatever the sizes
of the calls before (the pool reuses and grows its buffers), beyond the pooled size (pageable
copies) and from several host threads at once."""
import threading

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import izwi_amd
    return izwi_amd


def _weight(qa, dtype, n, k, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.02
    return qa.QMatMul.from_qtensor(qa.QTensor.quantize(w.cuda(), qa.GgmlDType(dtype)))


def _x(m, k, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(m, k, generator=g)


# (dtype, n, k, m): one row, a few rows (matrix-core kernels, activation records in scratch), more than 64
# rows (bf16 tiles), an output beyond the pooled size (600 x 4096 f32 = 9.8 MB), ragged n
CASES = [(12, 4096, 1024, 1), (8, 1000, 512, 1), (12, 4096, 1024, 8), (8, 2048, 768, 5), (8, 3072, 1024, 33),
         (12, 1024, 4096, 100), (12, 4096, 1024, 600), (12, 40, 256, 3)]


def test_host_calls_equal_device_calls_in_any_order(qa):
    """Every case twice, in an order that makes the pool shrink and grow between calls."""
    mats = {c: _weight(qa, c[0], c[1], c[2], 100 + i) for i, c in enumerate(CASES)}
    order = list(range(len(CASES))) + [6, 0, 7, 3, 6, 1, 5, 2, 4]
    for step, i in enumerate(order):
        dtype, n, k, m = CASES[i]
        print(f"host forward step={step} dtype={dtype} n={n} k={k} m={m}", flush=True)
        x = _x(m, k, 7 * step + 1)
        want = mats[CASES[i]].forward(x.cuda())
        got = mats[CASES[i]].forward(x)
        assert not got.is_cuda
        assert torch.equal(got, want.cpu())


def test_host_bf16_fused_and_group_calls_equal_device_calls(qa):
    mm = _weight(qa, 12, 2048, 1024, 5)
    for m in (1, 16, 130):
        print(f"host bf16 m={m}", flush=True)
        x = _x(m, 1024, m).to(torch.bfloat16)
        assert torch.equal(mm.forward(x), mm.forward(x.cuda()).cpu())
        xf = _x(m, 1024, 50 + m)
        res = _x(m, 2048, 90 + m)
        assert torch.equal(mm.forward_fused(xf, residual=res), mm.forward_fused(xf.cuda(), residual=res.cuda()).cpu())
    parts = [_weight(qa, 12, n, 1024, 20 + n) for n in (2048, 512, 512)]
    for m in (1, 4):
        x = _x(m, 1024, 70 + m)
        got = qa.forward_group(parts, x)
        want = qa.forward_group(parts, x.cuda())
        for g, w in zip(got, want):
            assert torch.equal(g, w.cpu())


def test_host_dequantize_and_data_round_trip(qa):
    """Outputs of 64 KB (pooled) and 16 MB (beyond the pooled size)."""
    for n, k in ((64, 256), (4096, 1024)):
        w = torch.randn(n, k) * 0.02
        qt = qa.QTensor.quantize(w.cuda(), qa.GgmlDType(12))
        dev = qt.dequantize("cuda")
        host = qt.dequantize("cpu")
        assert torch.equal(host, dev.cpu())
        again = qa.QTensor.from_blocks(qa.GgmlDType(12), qt.data(), (n, k))
        assert np.array_equal(again.data(), qt.data())


def test_host_moe_calls_equal_device_calls(qa):
    e, top_k, hidden, inter = 16, 4, 512, 256
    g = torch.Generator(device="cpu").manual_seed(3)
    stack = lambda rows, cols: qa.QTensor.quantize((torch.randn(e * rows, cols, generator=g) * 0.05).cuda(), qa.GgmlDType(12))
    gate, up, down = stack(inter, hidden), stack(inter, hidden), stack(hidden, inter)
    def stacked(qt, rows, cols):
        return qa.QTensor.from_blocks(qa.GgmlDType(12), qt.data(), (e, rows, cols))

    experts = qa.MoeExperts(stacked(gate, inter, hidden), stacked(up, inter, hidden), stacked(down, hidden, inter))
    for t in (1, 7, 40, 200):
        print(f"host moe t={t}", flush=True)
        logits = torch.randn(t, e, generator=g)
        x = torch.randn(t, hidden, generator=g)
        ids_d, w_d = qa.moe_route(logits.cuda(), top_k)
        ids_h, w_h = qa.moe_route(logits, top_k)
        assert torch.equal(ids_h, ids_d.cpu()) and torch.equal(w_h, w_d.cpu())
        perm_d, off_d = qa.moe_sort(ids_d, e)
        perm_h, off_h = qa.moe_sort(ids_h, e)
        assert torch.equal(perm_h, perm_d.cpu()) and torch.equal(off_h, off_d.cpu())
        want = experts.forward(x.cuda(), ids_d, w_d, perm_d, off_d)
        assert torch.equal(experts.forward(x, ids_h, w_h, perm_h, off_h), want.cpu())
        out_d, i_d, ww_d = experts.layer(logits.cuda(), x.cuda(), top_k, return_routing=True)
        out_h, i_h, ww_h = experts.layer(logits, x, top_k, return_routing=True)
        assert torch.equal(out_h, out_d.cpu()) and torch.equal(i_h, i_d.cpu()) and torch.equal(ww_h, ww_d.cpu())


def test_host_calls_from_four_threads(qa):
    """The reference calls forward from parallel worker threads (engine/executor/dispatch.rs:150-204): four
    threads, one shared handle, host pointers, every thread its own sizes."""
    mm = _weight(qa, 12, 3072, 1024, 9)
    ms = (1, 5, 16, 70)
    xs = [_x(m, 1024, 200 + m) for m in ms]
    want = [mm.forward(x.cuda()).cpu() for x in xs]
    errors = []

    def work(i):
        try:
            for _ in range(20):
                if not torch.equal(mm.forward(xs[i]), want[i]):
                    errors.append(f"thread {i}: result differs")
                    return
        except Exception as exc:  # noqa: BLE001
            errors.append(f"thread {i}: {exc!r}")

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
