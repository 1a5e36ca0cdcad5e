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
