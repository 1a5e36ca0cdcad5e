"""Size-independent properties of the HIP path at the full benchmark shapes (pytest -m gpu),
where the scalar oracle is too slow to check every output: exact power-of-two scaling of the
activations, invariance under a permutation of activation rows, bit-for-bit repeatability, and
agreement of the decode kernels with one another (one row alone against the same row in a
batch).  Each property follows from the arithmetic the reference defines (activation rows are
quantized one by one with a scale proportional to their largest magnitude; every output
depends on one activation row and one weight row)."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12
SHAPES = [("k", 1024, 4096), ("q", 4096, 4096), ("gate", 12288, 4096), ("down", 4096, 12288)]


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


@pytest.fixture(scope="module")
def weights(qa, oracle):
    out = {}
    for dtype in (Q4_K, Q8_0):
        for name, n, k in SHAPES:
            # 512 seeded rows repeated: the properties do not depend on the weights being distinct
            rows = oracle.quantize(dtype, oracle.randn(900 + n % 97 + dtype, (512, k), std=0.02))
            per_row = rows.size // 512
            blocks = np.tile(rows.reshape(512, per_row), (n // 512, 1)).reshape(-1)
            out[dtype, name] = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))
    return out


def _bits(t):
    return t.contiguous().view(torch.int32)


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [1, 2, 8, 16, 64])
def test_decode_scaling_permutation_repeatability(qa, oracle, weights, dtype, m):
    for name, n, k in SHAPES:
        _say(f"decode properties dtype={dtype} {name} m={m}")
        mm = weights[dtype, name]
        x = torch.from_numpy(oracle.randn(910 + m, (m, k))).cuda()
        y = mm.forward(x)
        assert torch.equal(_bits(mm.forward(x)), _bits(y))                       # repeatable bit for bit
        # x -> 4 x: the row's quantization scale grows by exactly 4, the quants stay, y -> 4 y exactly
        assert torch.equal(_bits(mm.forward(x * 4.0)), _bits(y * 4.0))
        assert torch.equal(_bits(mm.forward(x * 0.5)), _bits(y * 0.5))
        assert torch.equal(_bits(mm.forward(-x)), _bits(-y)) or dtype == Q4_K     # Q8_K's sign rule is not odd
        if m > 1:
            perm = torch.randperm(m, generator=torch.Generator().manual_seed(m)).cuda()
            assert torch.equal(_bits(mm.forward(x[perm].contiguous())), _bits(y[perm]))
            # a row alone runs another kernel (other summation order): equal within f32 rounding
            y0 = mm.forward(x[:1].contiguous())
            assert (y0 - y[:1]).abs().max().item() <= 2e-5 * y[:1].abs().max().item()


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [512, 2048])
def test_prefill_scaling_row_independence_repeatability(qa, oracle, weights, dtype, m):
    for name, n, k in SHAPES:
        _say(f"prefill properties dtype={dtype} {name} m={m}")
        mm = weights[dtype, name]
        x = torch.from_numpy(oracle.randn(920 + m, (m, k))).cuda().to(torch.bfloat16)
        y = mm.forward(x)                                                         # bf16 in, bf16 out
        assert torch.equal(mm.forward(x).view(torch.int16), y.view(torch.int16))  # also with k split over workgroups
        # power-of-two scaling is exact in bf16 products, f32 sums and the final rounding
        assert torch.equal(mm.forward(x * 2.0).view(torch.int16), (y * 2.0).view(torch.int16))
        # the first 256 rows alone: same tile arithmetic, same bits (another tiling plan may split k
        # differently, which changes the f32 summation order: within bf16 rounding then)
        y256 = mm.forward(x[:256].contiguous())
        diff = (y256.float() - y[:256].float()).abs().max().item()
        assert diff <= 2e-2 * y[:256].float().abs().max().item()
        # f32 output of the same kernel rounds to the bf16 output
        yf = mm.forward_bf16_to_f32(x)
        assert torch.equal(yf.to(torch.bfloat16).view(torch.int16), y.view(torch.int16))


@pytest.mark.parametrize("dtype", [12, 8, 14])
@pytest.mark.parametrize("k", [4096, 768, 1280, 512, 2048])
@pytest.mark.parametrize("m", [3, 16])
def test_single_stage_batched_decode_is_repeatable(qa, oracle, dtype, k, m):
    """Every single-stage instantiation of the batched decode kernel (one tile of rows, one activation
    window; Q4_K with four-unit panels in straight-line and compact form, three- and two-unit panels,
    a ragged last panel, Q8_0, Q6_K) starts its arithmetic on a counted wait for the activation window
    while the weight panel is still in flight.  A count that is one short shows as results that change
    from run to run while the chip is busy: the same call six times on a matrix of many row-tiles gives
    identical bits, and they are the oracle's sums."""
    import np_ref
    n = 8192 if k <= 2048 else 6144
    if dtype == 14:
        blocks = np_ref.random_q6_k_blocks(700 + k, n, k)
    else:
        blocks = oracle.quantize(dtype, oracle.randn(701 + k, (n, k), std=0.02))
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))
    x = torch.from_numpy(oracle.randn(702 + m, (m, k))).cuda()
    outs = [q.forward(x) for _ in range(6)]
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o.view(torch.int32), outs[0].view(torch.int32))
    rows = np.unique(np.random.default_rng(k + m).integers(0, n, 64))
    bpr = blocks.size // n
    want = oracle.qmatmul(dtype, x.cpu().numpy(), blocks.reshape(n, bpr)[rows].reshape(-1), rows.size)
    got = outs[0][:, torch.from_numpy(rows).cuda()].cpu().numpy()
    assert float(np.abs(got - want).max()) <= 1e-4 * float(np.abs(want).max())
