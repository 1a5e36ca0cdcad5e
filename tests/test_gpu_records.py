"""Activation records handed over by their producers (pytest -m gpu): RMSNorm and silu(gate) * up write
the quantized activations of the batched decode kernels themselves; the projections on those records
must equal the two-launch path (quantizer launch + matrix-core kernel on f32 activations) bit for bit."""
import numpy as np
import pytest
import torch

import np_ref

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


def weight(qa, oracle, dtype, n, k, seed):
    if dtype == Q6_K:
        blocks = np_ref.random_q6_k_blocks(seed, n, k)
    else:
        blocks = oracle.quantize(dtype, oracle.randn(seed, (n, k), std=0.02))
    return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))), blocks


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m,k,ns", [(16, 4096, (4096, 1024, 1024)), (8, 4096, (12288, 12288)), (5, 1024, (2048, 1000)),
                                    (40, 2048, (512,)), (64, 12288, (4096,)), (3, 4096, (16, 48)), (5, 256, (16, 48)),
                                    (3, 256, (16, 48))])
def test_records_from_their_producers_equal_the_two_launch_path(qa, oracle, dtype, m, k, ns):
    print(f"records dtype={dtype} m={m} k={k} ns={ns}", flush=True)
    parts = [weight(qa, oracle, dtype, n, k, 5000 + n + i)[0] for i, n in enumerate(ns)]
    x = torch.from_numpy(oracle.randn(5001 + m, (m, k))).cuda()
    nw = torch.from_numpy(oracle.randn(5002, (k,), mean=1.0, std=0.1)).cuda()
    gd = qa.GgmlDType(dtype)
    # The call on x takes the batched kernels - quantizer, then the kernel that reads records - from
    # three rows on, from five where k is at most 3072 (three and four rows of a short k run on the
    # single-launch kernel: same integers, another order of the f32 sums).
    same_kernel = m >= (5 if k <= 3072 else 3)

    def check(a, b):
        if same_kernel:
            assert torch.equal(a, b)
        else:
            assert float((a - b).abs().max()) <= 2e-6 * float(b.abs().max())
    # plain quantizer: forward_group on records == forward_group on x
    want = qa.forward_group(parts, x)
    got = qa.ActivationRecords.quantize(gd, x).forward_group(parts)
    for a, b in zip(got, want):
        check(a, b)
    # RMSNorm -> records == RMSNorm, then the projections
    normed = qa.try_fused_rms_norm(x, nw, 1e-6)
    want = qa.forward_group(parts, normed)
    rec = qa.ActivationRecords.from_rms_norm(gd, x, nw, 1e-6)
    assert torch.equal(rec.data, qa.ActivationRecords.quantize(gd, normed).data)      # the records themselves
    for a, b in zip(rec.forward_group(parts), want):
        check(a, b)


def test_silu_mul_records_bit_equal_to_the_mlp_call(qa, oracle):
    """down(silu(gate x) * (up x)): the MLP with the product quantized by the producer equals
    Qwen3Mlp.forward (gate/up group call, elementwise kernel, down's own quantizer) bit for bit."""
    k, inter, m = 1024, 3072, 16
    gate, _ = weight(qa, oracle, Q4_K, inter, k, 5200)
    up, _ = weight(qa, oracle, Q4_K, inter, k, 5201)
    down, _ = weight(qa, oracle, Q4_K, k, inter, 5202)
    x = torch.from_numpy(oracle.randn(5203, (m, k))).cuda()
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up), down)
    want = mlp.forward(x)
    gd = qa.GgmlDType.Q4K
    g, u = qa.ActivationRecords.quantize(gd, x).forward_group([gate, up])
    got, = qa.ActivationRecords.from_silu_mul(gd, g, u).forward_group([down])
    assert torch.equal(got, want)


def test_q6_k_weights_read_the_q8_k_records(qa, oracle):
    k, m = 2048, 16
    a, _ = weight(qa, oracle, Q4_K, 512, k, 5300)
    b, _ = weight(qa, oracle, Q6_K, 256, k, 5301)
    x = torch.from_numpy(oracle.randn(5302, (m, k))).cuda()
    rec = qa.ActivationRecords.quantize(qa.GgmlDType.Q4K, x)
    ya, yb = rec.forward_group([a, b])
    assert torch.equal(ya, a.forward(x)) and torch.equal(yb, b.forward(x))


def test_records_argument_errors(qa, oracle):
    from izwi_amd import capi
    w, _ = weight(qa, oracle, Q4_K, 64, 1024, 5400)
    w8, _ = weight(qa, oracle, Q8_0, 64, 1024, 5401)
    x = torch.from_numpy(oracle.randn(5402, (2, 1024))).cuda()
    rec = qa.ActivationRecords.quantize(qa.GgmlDType.Q4K, torch.cat([x] * 4))
    with pytest.raises(capi.QmmError, match="dot against|given to a Q8_0 projection"):
        rec.forward_group([w, w8])
    with pytest.raises(capi.QmmError, match="3 <= m <= 64"):
        qa.ActivationRecords.quantize(qa.GgmlDType.Q4K, x).forward_group([w])
    with pytest.raises(capi.QmmError, match="multiple of 256"):
        qa.ActivationRecords.from_rms_norm(qa.GgmlDType.Q8_0, torch.zeros((4, 96), device="cuda"), torch.ones(96, device="cuda"))
    assert capi.lib().izwi_qmm_records_bytes(12, 16, 4096) == 16 * 4416 and capi.lib().izwi_qmm_records_bytes(8, 17, 256) == 2 * 4608
