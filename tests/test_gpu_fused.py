"""GPU tests of izwi_qmm_forward_fused (pytest -m gpu): casts and residual add folded into the
projection kernels.  The sums must be those of the plain entry points bit for bit, so every case
is compared exactly with the unfused composition (plain call, then torch's add / cast)."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

import np_ref

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14


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


def make_qmatmul(qa, oracle, dtype, n, k, seed):
    if dtype == Q6_K:
        blocks = np_ref.random_q6_k_blocks(seed, n, k)
    else:
        rows = min(n, 1024)
        b = oracle.quantize(dtype, oracle.randn(seed, (rows, k), std=0.02)).reshape(rows, -1)
        blocks = np.tile(b, ((n + rows - 1) // rows, 1))[:n].reshape(-1)
    return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))


def unfused_sums(mm, x):
    """f32 sums of the plain entry points for the same activations."""
    m = x.numel() // x.shape[-1]
    if x.dtype == torch.float32:
        return mm.forward(x)
    return mm.forward(x.float()) if m <= 64 else mm.forward_bf16_to_f32(x)


def check_all_forms(qa, mm, x32, label):
    n = mm.qtensor.dims2()[0]
    m = x32.shape[0]
    res32 = torch.randn(m, n, device="cuda")
    for xdt in (torch.float32, torch.bfloat16):
        x = x32.to(xdt)
        sums = unfused_sums(mm, x)
        for ydt in (torch.float32, torch.bfloat16):
            _say(f"{label} m={m} x={xdt} y={ydt}")
            res = res32.to(ydt)
            # no residual: the plain result, cast once
            assert torch.equal(mm.forward_fused(x, out_dtype=ydt), sums.to(ydt))
            # residual: one rounding of sum + residual
            want = (sums + res.float()).to(ydt)
            assert torch.equal(mm.forward_fused(x, residual=res, out_dtype=ydt), want)
            # in place: y is the residual buffer
            buf = res.clone()
            out = mm.forward_fused(x, residual=buf, out_dtype=ydt, out=buf)
            assert out.data_ptr() == buf.data_ptr() and torch.equal(buf, want)


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0, Q6_K])
@pytest.mark.parametrize("m", [1, 2, 3, 16, 33, 64, 65, 300])
def test_fused_equals_unfused_composition(qa, oracle, dtype, m):
    n, k = 528, 1024
    mm = make_qmatmul(qa, oracle, dtype, n, k, 3 + dtype)
    x = torch.from_numpy(oracle.randn(40 + m, (m, k))).cuda()
    check_all_forms(qa, mm, x, f"fused dtype={dtype}")


@pytest.mark.parametrize("n,k,m", [(4096, 4096, 1), (4096, 12288, 2), (12288, 4096, 8), (4096, 12288, 16),
                                   (40000, 4096, 1), (40000, 4096, 5), (33000, 8448, 4), (1024, 4096, 512)])
def test_fused_8b_and_tall_shapes_q4_k(qa, oracle, n, k, m):
    """The 8B projection shapes, a matrix tall enough for the streaming form of the batched kernel
    (k inside one activation window: folded; k beyond: sums in scratch, then the epilogue kernel)
    and a prefill shape with split k."""
    mm = make_qmatmul(qa, oracle, Q4_K, n, k, n % 97)
    x = torch.from_numpy(oracle.randn(n % 89 + m, (m, k))).cuda()
    check_all_forms(qa, mm, x, f"fused n={n} k={k}")


def test_fused_against_the_oracle_and_reference_rounding(qa, oracle):
    """bf16 in, bf16 out with a residual, as the reference's layer does it (cast in, matmul, cast out,
    add): the fused call is within one bf16 rounding of that sequence and closer to the exact sum."""
    n, k, m = 1024, 4096, 2
    blocks = oracle.quantize(Q4_K, oracle.randn(1, (n, k), std=0.02))
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks, (n, k)))
    xb = torch.from_numpy(oracle.randn(2, (m, k))).cuda().to(torch.bfloat16)
    res = torch.randn(m, n, device="cuda").to(torch.bfloat16)
    sums = oracle.qmatmul(Q4_K, xb.float().cpu().numpy(), blocks, n)  # the reference's f32 product
    exact = sums.astype(np.float64) + res.float().cpu().numpy()
    reference = (torch.from_numpy(sums).cuda().to(torch.bfloat16) + res).float().cpu().numpy()  # two roundings
    got = mm.forward_fused(xb, residual=res).float().cpu().numpy()
    scale = np.abs(exact).max()
    assert np.abs(got - exact).max() <= 2.0 ** -8 * scale           # one bf16 rounding (+ 1e-4 of the sums)
    assert np.abs(got - reference).max() <= 2.0 ** -7 * scale
    assert np.abs(got - exact).mean() <= np.abs(reference - exact).mean()


def test_fused_host_memory_profile_counters_and_errors(qa, oracle):
    from izwi_amd import capi
    n, k, m = 96, 512, 3
    mm = make_qmatmul(qa, oracle, Q8_0, n, k, 9)
    x = torch.from_numpy(oracle.randn(5, (m, k)))
    res = torch.randn(m, n)
    want = mm.forward(x.cuda()) + res.cuda()
    assert torch.equal(mm.forward_fused(x, residual=res).cuda(), want)  # host pointers in, host pointer out
    L = capi.lib()
    L.izwi_qmm_profile_enable(1)
    L.izwi_qmm_profile_reset()
    xb = x.cuda().to(torch.bfloat16)
    mm.forward_fused(xb)
    mm.forward_fused(xb, out_dtype=torch.float32)
    snap = qa.profile_snapshot()
    # the ASR profile fields `izwi bench` prints (asr/mod.rs:116-147): the same counters in ms, plus the argmax
    assert L.izwi_qmm_profile_enabled() == 1
    logits = torch.from_numpy(oracle.randn(6, (2, 151936))).cuda()
    assert qa.argmax(logits).cpu().tolist() == logits.argmax(dim=-1).cpu().tolist()
    diag = qa.asr_profile_diagnostics()
    assert diag["qwen3_profile_enabled"] and diag["argmax_calls"] == 1 and diag["argmax_ms"] > 0
    assert diag["qmatmul_calls"] == 2 and diag["qmatmul_ms"] == snap["qmatmul_ns"] / 1e6
    assert diag["silu_mul_fused_calls"] == 0 and diag["lm_head_calls"] == 0
    L.izwi_qmm_profile_enable(0)
    assert L.izwi_qmm_profile_enabled() == 0
    qa.argmax(logits)
    assert qa.asr_profile_diagnostics()["argmax_calls"] == 1            # not counted while off
    assert snap["qmatmul_calls"] == 2 and snap["qmatmul_input_casts"] == 2 and snap["qmatmul_output_casts"] == 1
    assert snap["qmatmul_input_cast_ns"] == 0 and snap["qmatmul_output_cast_ns"] == 0
    y = torch.empty(m, n, device="cuda")
    xd = x.cuda()
    h = mm.qtensor._h
    assert L.izwi_qmm_forward_fused(h, xd.data_ptr(), 2, m, None, y.data_ptr(), 0, capi.DEVICE, None) == -1
    assert L.izwi_qmm_forward_fused(h, xd.data_ptr(), 0, m, None, y.data_ptr(), 7, capi.DEVICE, None) == -1
    assert L.izwi_qmm_forward_fused(h, None, 0, m, None, y.data_ptr(), 0, capi.DEVICE, None) == -1
    assert L.izwi_qmm_forward_fused(h, xd.data_ptr(), 0, 0, None, None, 0, capi.DEVICE, None) == 0  # m = 0
    with pytest.raises(capi.QmmError):
        mm.forward_fused(xd, residual=torch.zeros(m, n + 1, device="cuda"))
    with pytest.raises(capi.QmmError):
        mm.forward_fused(xd, residual=torch.zeros(m, n, device="cuda", dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0, Q6_K])
@pytest.mark.parametrize("m", [1, 2, 3, 16, 80])
def test_rms_norm_folded_into_the_projection_calls(qa, oracle, dtype, m):
    """forward_normed / forward_group(norm_weight=) / forward_silu_mul(norm_weight=) against the norm
    call followed by the plain call.  For m <= 2 the decode kernel does the norm itself (scale-invariance
    of the quantizers): results agree to f32 rounding; beyond, the library runs the two steps itself."""
    k, n1, n2 = 1024, 528, 272
    a, b = make_qmatmul(qa, oracle, dtype, n1, k, 21), make_qmatmul(qa, oracle, dtype, n2, k, 22)
    g, u = make_qmatmul(qa, oracle, dtype, n1, k, 23), make_qmatmul(qa, oracle, dtype, n1, k, 24)
    x = torch.from_numpy(oracle.randn(50 + m, (m, k)) * 3.0).cuda()
    w = torch.from_numpy(oracle.randn(7, (k,), mean=1.0, std=0.2)).cuda()
    normed = qa.try_fused_rms_norm(x, w, 1e-6)

    # Q8_0 rounds the activation blocks' scales to f16: folded, that rounding happens before the row's
    # factor is applied instead of after it, a difference of up to 2^-11 per block
    tol = 1.5e-3 if dtype == Q8_0 else 2e-4

    def near(got, want):
        return float((got - want).abs().max()) <= tol * float(want.abs().max())
    assert near(a.forward_normed(x, w, 1e-6), a.forward(normed))
    ya, yb = qa.forward_group([a, b], x, norm_weight=w, eps=1e-6)
    assert near(ya, a.forward(normed)) and near(yb, b.forward(normed))
    gu = qa.Qwen3GateUpProjection.new_separate(g, u)
    assert near(gu.forward_silu_mul(x, norm_weight=w, eps=1e-6), gu.forward_silu_mul(normed))
    # against the oracle's composition, where the library multiplies in integers as the oracle does
    # (80 rows take the prefill kernel, which has its own, wider, bound)
    xn = oracle.rms_norm(x.cpu().numpy(), w.cpu().numpy(), 1e-6)
    if dtype != Q6_K and m <= 16:
        want = oracle.qmatmul(dtype, xn, a.qtensor.data(), n1)
        got = a.forward_normed(x, w, 1e-6).cpu().numpy()
        assert np.abs(got - want).max() <= (tol + 1e-4) * np.abs(want).max()


def test_rms_norm_folded_8b_shapes_host_space_and_errors(qa, oracle):
    from izwi_amd import capi
    q = make_qmatmul(qa, oracle, Q4_K, 4096, 4096, 31)
    kk = make_qmatmul(qa, oracle, Q4_K, 1024, 4096, 32)
    v = make_qmatmul(qa, oracle, Q4_K, 1024, 4096, 33)
    x = torch.from_numpy(oracle.randn(60, (1, 4096))).cuda()
    w = torch.from_numpy(oracle.randn(8, (4096,), mean=1.0, std=0.1)).cuda()
    normed = qa.try_fused_rms_norm(x, w, 1e-6)
    for got, mm in zip(qa.forward_group([q, kk, v], x, norm_weight=w), (q, kk, v)):
        want = mm.forward(normed)
        assert float((got - want).abs().max()) <= 2e-4 * float(want.abs().max())
    head = make_qmatmul(qa, oracle, Q4_K, 40000, 4096, 34)  # tall: the looped form of the kernel
    want = head.forward(normed)
    assert float((head.forward_normed(x, w) - want).abs().max()) <= 2e-4 * float(want.abs().max())
    # host pointers: staged, same values
    got = q.forward_normed(x.cpu(), w.cpu())
    assert float((got.cuda() - q.forward(normed)).abs().max()) <= 2e-4 * float(want.abs().max())
    L = capi.lib()
    y = torch.empty(1, 4096, device="cuda")
    assert L.izwi_qmm_forward_normed_f32(q.qtensor._h, x.data_ptr(), 1, None, 1e-6, y.data_ptr(), capi.DEVICE, None) == -1
