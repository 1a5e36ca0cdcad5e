"""GPU tests (pytest -m gpu) of the plane form of the prefill product: the weights dequantized once
per call into a bf16 plane, then a plain bf16 matrix-core loop (izwi_qmm_set_prefill_form).

Same bf16 operands and f32 accumulation as the in-LDS form, so the two agree to the last bits of
the f32 sums (bf16 outputs: within one bf16 step); against the CPU oracle the bar is the path's 1e-2."""
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


@pytest.fixture()
def plane(qa):
    before = qa.get_prefill_form()
    qa.set_prefill_form(1)
    yield
    qa.set_prefill_form(before)


def rel_err(y, want):
    return float(np.abs(y.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


def make_weight(oracle, dtype, n, k, seed):
    return oracle.quantize(dtype, oracle.randn(seed, (n, k), std=0.02))


def test_form_switch_round_trip(qa):
    before = qa.get_prefill_form()
    for form in (0, 1, -1):
        qa.set_prefill_form(form)
        assert qa.get_prefill_form() == form
    with pytest.raises(qa.QmmError):
        qa.set_prefill_form(7)
    qa.set_prefill_form(before)


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m,n,k", [(512, 1024, 4096), (300, 200, 768), (129, 16, 256), (257, 520, 1024),
                                   (1000, 4096, 12288), (2048, 1024, 4096)])
def test_plane_form_against_oracle_and_in_lds_form(qa, oracle, plane, dtype, m, n, k):
    _say(f"plane dtype={dtype} m={m} n={n} k={k}")
    blocks = make_weight(oracle, dtype, n, k, 930 + n)
    xb = torch.from_numpy(oracle.randn(931 + m, (m, k))).cuda().to(torch.bfloat16)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))
    y = q.forward_bf16_to_f32(xb)
    yb = q.forward(xb)
    qa.set_prefill_form(0)
    y_lds = q.forward_bf16_to_f32(xb)
    qa.set_prefill_form(1)
    scale = float(y_lds.abs().max())
    assert float((y - y_lds).abs().max()) <= 2e-5 * scale  # f32 summation order only
    assert float((yb.float() - y).abs().max()) <= 2.0 ** -8 * scale  # one rounding to bf16
    xf = xb.float().cpu().numpy()
    if m * n * k <= 512 * 1024 * 4096:
        dense = xf.astype(np.float64) @ oracle.dequantize(dtype, blocks, n, k).astype(np.float64).T
        assert rel_err(y.cpu().numpy(), dense) < 4e-3
        if n >= 128:
            assert rel_err(y.cpu().numpy(), oracle.qmatmul(dtype, xf, blocks, n)) < 1e-2
    else:  # the oracle on a spread of weight rows
        rows = np.unique(np.random.default_rng(5).integers(0, n, 128))
        bpr = blocks.size // n
        sub = blocks.reshape(n, bpr)[rows].reshape(-1)
        want = oracle.qmatmul(dtype, xf, sub, rows.size)
        assert rel_err(y[:, torch.from_numpy(rows).cuda()].cpu().numpy(), want) < 1e-2


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m,k,ns", [(512, 4096, (4096, 1024, 1024)), (300, 768, (300, 200)), (200, 1024, (2048, 1000, 16, 512))])
def test_plane_form_projection_groups(qa, oracle, plane, dtype, m, k, ns):
    _say(f"plane group dtype={dtype} m={m} k={k} ns={ns}")
    dt = qa.GgmlDType(dtype)
    blocks = [make_weight(oracle, dtype, n, k, 940 + n + i) for i, n in enumerate(ns)]
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b, (n, k))) for b, n in zip(blocks, ns)]
    x = torch.from_numpy(oracle.randn(941 + m, (m, k))).cuda()
    xb = x.to(torch.bfloat16)
    got_f32 = qa.forward_group(parts, x)
    got_bf16 = qa.forward_group(parts, xb)
    for i, p in enumerate(parts):
        sep = p.forward_bf16_to_f32(xb)
        scale = float(sep.abs().max())
        assert float((got_f32[i] - sep).abs().max()) <= 2e-5 * scale, i
        assert float((got_bf16[i].float() - sep).abs().max()) <= 2.0 ** -7 * scale, i
    i = min((j for j, n in enumerate(ns) if n >= 128), key=lambda j: ns[j])
    want = oracle.qmatmul(dtype, xb.float().cpu().numpy(), blocks[i], ns[i])
    assert rel_err(got_bf16[i].float().cpu().numpy(), want) < 1e-2


def test_plane_form_leaves_other_shapes_to_the_in_lds_form(qa, oracle, plane):
    # k not a multiple of 64 (Q8_0) and m <= 128 have no plane form: same results as before
    blocks = make_weight(oracle, Q8_0, 256, 1056, 950)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(Q8_0), blocks, (256, 1056)))
    for m in (100, 300):
        xb = torch.from_numpy(oracle.randn(951 + m, (m, 1056))).cuda().to(torch.bfloat16)
        y = q.forward_bf16_to_f32(xb)
        qa.set_prefill_form(0)
        y0 = q.forward_bf16_to_f32(xb)
        qa.set_prefill_form(1)
        assert torch.equal(y, y0)


def test_plane_form_fused_residual_and_graph_replay(qa, oracle, plane):
    """forward_fused (bf16 in, residual added, bf16 out) on the plane form, eagerly and as replays of a
    captured graph (the scratch plane is reserved by the eager call in front of the capture)."""
    n, k, m = 1024, 4096, 384
    blocks = make_weight(oracle, Q4_K, n, k, 960)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(Q4_K), blocks, (n, k)))
    xb = torch.from_numpy(oracle.randn(961, (m, k))).cuda().to(torch.bfloat16)
    res = torch.from_numpy(oracle.randn(962, (m, n))).cuda().to(torch.bfloat16)
    want = (q.forward_bf16_to_f32(xb) + res.float()).to(torch.bfloat16)
    got = q.forward_fused(xb, residual=res, out_dtype=torch.bfloat16)
    assert float((got.float() - want.float()).abs().max()) <= 2.0 ** -7 * float(want.float().abs().max())
    out = torch.empty_like(got)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        q.forward_fused(xb, residual=res, out_dtype=torch.bfloat16, out=out)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            q.forward_fused(xb, residual=res, out_dtype=torch.bfloat16, out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, got)
