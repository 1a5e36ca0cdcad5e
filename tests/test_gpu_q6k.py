"""GPU parity of the Q6_K block format (pytest -m gpu): weight bytes and dequantization bit-exact,
decode within 1e-4 and prefill within 1e-2 of the CPU oracle, through the C ABI.

Q6_K weights are built from random block bytes (the oracle has no Q6_K quantizer): every six-bit
quant, bit pair and signed scale occurs, d is a finite f16 around 1e-3."""
import sys

import numpy as np
import pytest
import torch

import np_ref

pytestmark = pytest.mark.gpu

Q4_K, Q6_K = 12, 14
DECODE_TOL = 1e-4
PREFILL_TOL = 1e-2


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


def rel_err(y, want):
    return float(np.abs(y.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


@pytest.mark.parametrize("n,k", [(16, 256), (5, 512), (33, 768), (64, 1024), (40, 1280), (128, 4096), (17, 12288)])
def test_q6_k_dequantize_and_data_bit_exact(qa, oracle, n, k):
    _say(f"q6k dequant n={n} k={k}")
    blocks = np_ref.random_q6_k_blocks(n + k, n, k)
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k))
    got = q.dequantize().cpu().numpy()
    want = oracle.dequantize(Q6_K, blocks, n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), np_ref.dequant_q6_k(blocks, n, k).view(np.uint32))
    assert np.array_equal(q.data(), blocks)
    assert qa.quantized_storage_bytes(n, k, qa.GgmlDType.Q6K) == blocks.size


def test_q6_k_hand_block_on_device(qa):
    import json
    import os
    fx = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q6k_hand_block.json")))
    blk = np.frombuffer(bytes.fromhex(fx["block_hex"]), np.uint8)
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blk, (1, 256))
    assert np.array_equal(q.dequantize().cpu().numpy().reshape(-1), np.array(fx["expected_f32"], dtype=np.float32))


def test_q6_k_activation_blocks_are_q8_k(qa, oracle):
    x = oracle.randn(5, (3, 1024))
    got = qa.quantize_activations(qa.GgmlDType.Q6K, torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(got, oracle.quantize_activations(Q6_K, x))


@pytest.mark.parametrize("n,k,m", [(1, 256, 1), (15, 256, 2), (17, 512, 3), (100, 768, 5), (250, 1280, 7),
                                   (64, 1024, 16), (130, 2048, 33), (48, 4096, 64), (31, 12288, 4)])
def test_q6_k_decode_ragged_shapes(qa, oracle, n, k, m):
    _say(f"q6k decode n={n} k={k} m={m}")
    blocks = np_ref.random_q6_k_blocks(7 * n + k + m, n, k)
    x = oracle.randn(n + k + m, (m, k))
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k)))
    y = mm.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    want = oracle.qmatmul(Q6_K, x, blocks, n)
    assert y.shape == (m, n)
    assert rel_err(y, want) <= DECODE_TOL
    # and against the integer dot products of the independent numpy reading of the format
    assert rel_err(y, np_ref.qmatmul_int(Q6_K, x, blocks, n)) <= DECODE_TOL


@pytest.mark.parametrize("n,k", [(4096, 12288), (1024, 4096), (151936 // 8, 4096)])
@pytest.mark.parametrize("m", [1, 2])
def test_q6_k_decode_8b_shapes(qa, oracle, n, k, m):
    """The tensors a Q4_K_M file of the 8B model keeps in Q6_K: ffn_down, attn_v and (an eighth
    of) the output matrix."""
    _say(f"q6k 8B n={n} k={k} m={m}")
    blocks = np_ref.random_q6_k_blocks(n + m, n, k)
    x = oracle.randn(n + k, (m, k))
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k)))
    xd = torch.from_numpy(x).cuda()
    y = mm.forward(xd)
    assert torch.equal(y, mm.forward(xd))  # repeatable bit for bit
    want = oracle.qmatmul(Q6_K, x, blocks, n)
    assert rel_err(y.cpu().numpy(), want) <= DECODE_TOL
    # scaling the activations by a power of two scales the result exactly
    assert torch.equal(mm.forward(xd * 4.0), y * 4.0)


def test_q6_k_rows_are_independent(qa, oracle):
    n, k = 96, 2048
    blocks = np_ref.random_q6_k_blocks(3, n, k)
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k)))
    x = torch.from_numpy(oracle.randn(4, (7, k))).cuda()
    y = mm.forward(x)
    for r in range(7):
        assert rel_err(mm.forward(x[r:r + 1].contiguous()).cpu().numpy(), y[r:r + 1].cpu().numpy().astype(np.float64)) <= 2e-6


# beyond 128 rows the pipelined tiles: split along k (512 x 1024 x 4096), ragged half-size tiles, one
# round of 256 x 256 tiles (2048 x 8192), and whole rounds of them followed by half-size tiles (8704
# columns); up to 128 rows the plain tile kernel
@pytest.mark.parametrize("m,n,k", [(512, 1024, 4096), (300, 200, 768), (65, 256, 1024), (129, 144, 1280), (70, 16, 256),
                                   (600, 1100, 1024), (2048, 8192, 256), (2048, 8704, 512)])
def test_q6_k_prefill_against_oracle(qa, oracle, m, n, k):
    _say(f"q6k prefill m={m} n={n} k={k}")
    blocks = np_ref.random_q6_k_blocks(m + n, n, k)
    xb = torch.from_numpy(oracle.randn(m + k, (m, k))).cuda().to(torch.bfloat16)
    xf = xb.float().cpu().numpy()
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k)))
    y = mm.forward_bf16_to_f32(xb).cpu().numpy()
    yb = mm.forward(xb)
    assert yb.dtype == torch.bfloat16
    # (a) the kernel's own arithmetic: exact bf16 activations x bf16-rounded dequantized weights
    dense = xf.astype(np.float64) @ oracle.dequantize(Q6_K, blocks, n, k).astype(np.float64).T
    assert rel_err(y, dense) < 4e-3
    assert rel_err(yb.float().cpu().numpy(), dense) < 1e-2
    # f32 activations with m > 64 take the same kernel after one conversion
    assert torch.equal(mm.forward(xb.float()), torch.from_numpy(y).cuda())
    # (b) the reference's CPU result, which also carries its int8 activation rounding (about 0.5 %
    # of the output scale): the 1e-2 bar where the output row is long enough for max|y_ref| to
    # stand above that noise's tail
    if n >= 128 and m * n * k <= 3e9:
        assert rel_err(y, oracle.qmatmul(Q6_K, xf, blocks, n)) < PREFILL_TOL


def test_q6_k_in_groups_and_mlp(qa, oracle):
    """Projection groups and gate/up pairs with Q6_K members give the results of separate calls: a
    group of one type is one launch (up to two rows) or one shared quantization (up to 64), a group of
    several types runs type by type; with the RMSNorm folded in as well."""
    k, n = 1024, 512
    b6 = np_ref.random_q6_k_blocks(1, n, k)
    b6b = np_ref.random_q6_k_blocks(3, 272, k)
    b4 = oracle.quantize(Q4_K, oracle.randn(2, (n, k), std=0.02))
    b4b = oracle.quantize(Q4_K, oracle.randn(4, (272, k), std=0.02))
    w6 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, b6, (n, k)))
    w6b = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, b6b, (272, k)))
    w4 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, b4, (n, k)))
    w4b = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, b4b, (272, k)))
    gu = qa.Qwen3GateUpProjection.new_separate(w6, w6)
    nw = torch.from_numpy(oracle.randn(9, (k,), mean=1.0, std=0.2)).cuda()
    for m in (1, 2, 5, 16, 33, 64, 80):
        x = torch.from_numpy(oracle.randn(10 + m, (m, k))).cuda()
        for group in ([w4, w6, w6], [w6, w6b, w6], [w4, w4b, w6b], [w6b, w4]):
            ys = qa.forward_group(group, x)
            for y, w in zip(ys, group):
                assert torch.equal(y, w.forward(x))
            # the norm folded in: the single-weight normed call is the yardstick (same kernel variant)
            ys = qa.forward_group(group, x, norm_weight=nw, eps=1e-6)
            for y, w in zip(ys, group):
                want = w.forward_normed(x, nw, 1e-6)
                assert float((y - want).abs().max()) <= 2e-6 * float(want.abs().max())
        g = w6.forward(x)
        assert torch.allclose(gu.forward_silu_mul(x), torch.nn.functional.silu(g) * g, rtol=1e-5, atol=1e-6)
        gn = w6.forward_normed(x, nw, 1e-6)
        assert torch.allclose(gu.forward_silu_mul(x, norm_weight=nw, eps=1e-6), torch.nn.functional.silu(gn) * gn,
                              rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("gate_up_dtype,E,hidden,inter,t,top_k", [
    (Q4_K, 8, 512, 768, 64, 4),    # the Q4_K_M case: Q4_K gate / up, Q6_K down; 32 pairs per expert: matrix-core tiles
    (Q4_K, 16, 512, 512, 6, 8),    # 3 pairs per expert: 4-row segments
    (Q4_K, 8, 1024, 256, 1, 2),    # one token
    (Q6_K, 4, 768, 512, 40, 2),    # every stack Q6_K, ragged panels
    (Q6_K, 8, 256, 512, 3, 2),
    (Q6_K, 64, 768, 256, 24, 2),   # more than 16 tokens on the segment path: token rows quantized by the routing kernel
    (Q4_K, 64, 512, 512, 30, 3),   # the same, Q4_K gate / up with a Q6_K down stack
])
def test_moe_with_q6_k_expert_stacks(qa, oracle, gate_up_dtype, E, hidden, inter, t, top_k):
    """Expert stacks in Q6_K (a Q4_K_M file keeps ffn_down_exps of some layers in it): the expert MLP
    against the oracle's composition of per-type products, and the one-call layer against the three
    calls."""
    _say(f"q6k moe gate_up={gate_up_dtype} E={E} hidden={hidden} inter={inter} t={t}")
    if gate_up_dtype == Q6_K:
        gate = np_ref.random_q6_k_blocks(311, E * inter, hidden, d_scale=2e-3)
        up = np_ref.random_q6_k_blocks(312, E * inter, hidden, d_scale=2e-3)
    else:
        gate = oracle.quantize(gate_up_dtype, oracle.randn(311, (E * inter, hidden), std=0.05))
        up = oracle.quantize(gate_up_dtype, oracle.randn(312, (E * inter, hidden), std=0.05))
    down = np_ref.random_q6_k_blocks(313, E * hidden, inter, d_scale=2e-3)
    gdt = qa.GgmlDType(gate_up_dtype)
    experts = qa.MoeExperts(qa.QTensor.from_blocks(gdt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(gdt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(qa.GgmlDType.Q6K, down, (E, hidden, inter)))
    x = oracle.randn(314, (t, hidden))
    logits = oracle.randn(315, (t, E))
    xd, ld = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    ids, wts = qa.moe_route(ld, top_k)
    perm, offsets = qa.moe_sort(ids, E)
    out = experts.forward(xd, ids, wts, perm, offsets)
    want_ids, want_wts = oracle.moe_route(logits, top_k)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    want = oracle.moe_forward(gate_up_dtype, x, want_ids, want_wts, gate, up, down, E, inter, down_dtype=Q6_K)
    assert rel_err(out.cpu().numpy(), want) < 1e-3
    assert torch.equal(experts.layer(ld, xd, top_k), out)
