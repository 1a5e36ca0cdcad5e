"""GPU parity tests (pytest -m gpu): the HIP path, called through the C ABI,
against the CPU oracle on the same seeded inputs.

Bars: weight dequantization, weight bytes, on-chip activation quantization and
MoE indices are bit-exact; matmul outputs within max|y - y_ref| / max|y_ref|
<= 1e-2 (the tolerance the path's target states; the decode kernel, which
follows the reference's integer arithmetic, is held to 1e-4)."""
import sys

import numpy as np
import pytest
import torch

import np_ref

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12
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


def make_weight(oracle, dtype, n, k, seed):
    w = oracle.randn(seed, (n, k), std=0.02)
    return oracle.quantize(dtype, w)


# ------------------------------------------------------------------ codecs --
@pytest.mark.parametrize("dtype", [Q8_0, Q4_K])
@pytest.mark.parametrize("n,k", [(16, 256), (5, 512), (33, 768), (64, 1024), (40, 1280), (128, 4096), (17, 12288)])
def test_dequantize_and_data_bit_exact(qa, oracle, dtype, n, k):
    _say(f"dequant dtype={dtype} n={n} k={k}")
    blocks = make_weight(oracle, dtype, n, k, 1000 + n + k)
    q = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
    got = q.dequantize().cpu().numpy()
    want = oracle.dequantize(dtype, blocks, n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(q.data(), blocks)  # QTensor::data() returns the original bytes


def test_dequantize_random_bytes_and_q8_0_ragged_k(qa, oracle):
    rng = np.random.default_rng(9)
    raw = rng.integers(0, 256, size=(48 * 5, 144), dtype=np.uint8)
    raw[:, 1] &= 0x3F
    raw[:, 3] &= 0x3F
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q4K, raw.reshape(-1), (48, 1280))
    assert np.array_equal(q.dequantize().cpu().numpy().view(np.uint32),
                          np_ref.dequant_q4_k(raw.reshape(-1), 48, 1280).view(np.uint32))
    # Q8_0 only needs k % 32 == 0: 96 is not a multiple of the 256-element tile unit
    raw8 = rng.integers(0, 256, size=(20 * 3, 34), dtype=np.uint8)
    raw8[:, 1] &= 0x7B
    q8 = qa.QTensor.from_blocks(qa.GgmlDType.Q8_0, raw8.reshape(-1), (20, 96))
    assert np.array_equal(q8.dequantize().cpu().numpy().view(np.uint32),
                          np_ref.dequant_q8_0(raw8.reshape(-1), 20, 96).view(np.uint32))
    assert np.array_equal(q8.data(), raw8.reshape(-1))


def test_q4_k_hand_block_on_device(qa):
    scales = bytes([0x41, 0x82, 0xC3, 0xC4, 0x40, 0x85, 0xCA, 0xCF, 0x41, 0x82, 0xC3, 0xFF])
    blk = bytes([0x00, 0x3C, 0x00, 0x38]) + scales + bytes(range(128))
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blk, (1, 256))
    y = q.dequantize().cpu().numpy()[0]
    for i, v in {0: 0, 31: 15, 32: -2.5, 64: -5, 79: 40, 127: 4.5, 160: 116, 224: 346.5, 255: 409.5}.items():
        assert y[i] == np.float32(v)
    assert float(y.astype(np.float64).sum()) == 32224.0


@pytest.mark.parametrize("dtype", [Q8_0, Q4_K])
def test_activation_quantizer_bit_exact(qa, oracle, dtype):
    x = oracle.randn(77, (9, 2048))
    x[2, 256:512] = 0.0
    x[4, 5], x[4, 9] = -7.5, 7.5      # equal magnitudes: the first occurrence decides the sign
    x[5, 700], x[5, 600] = 8.0, -8.0
    x[6] *= 1e-3
    x[7] *= 1e4
    got = qa.quantize_activations(qa.GgmlDType(dtype), torch.from_numpy(x).cuda()).cpu().numpy()
    want = oracle.quantize_activations(dtype, x)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [Q8_0, Q4_K])
def test_activation_quantizer_rounds_halves_away_from_zero_like_the_reference(qa, oracle, dtype):
    """Blocks whose scale is exactly 1 (Q8_K: first maximum -128, Q8_0: maximum 127), so that the
    values ARE the products the quantizers round: exact halves, the floats next to a half on both
    sides, values at and beyond the clamp; once with the block maximum in front (it decides Q8_K's
    sign) and once with an equal maximum of the other sign behind it.  Bit-equal blocks from the
    single-row kernel's quantizer (the exported one), the record quantizer (through a 5-row forward
    against the oracle product) and the oracle."""
    k = 512
    top = -128.0 if dtype == Q4_K else 127.0
    below = np.nextafter(np.float32(0.5), np.float32(0.0))
    above = np.nextafter(np.float32(0.5), np.float32(1.0))
    specials = []
    for base in (0, 1, 2, 7, 63, 100, 126):
        for frac in (np.float32(0.5), below, above):
            specials += [np.float32(base) + frac, -(np.float32(base) + frac)]
    specials += [126.5, 127.49, -127.5, -127.49, 0.0, -0.0, 1e-30, -1e-30, 0.25, -0.75]
    x = np.zeros((5, k), dtype=np.float32)
    rng = np.random.default_rng(5)
    for r in range(5):
        for blk in range(k // 32):
            vals = rng.permutation(np.array(specials, dtype=np.float32))[:31]
            x[r, 32 * blk] = top
            x[r, 32 * blk + 1:32 * blk + 32] = vals
    x[1, 300] = -top  # an equal maximum of the other sign behind the first: the first still decides
    x[2, 0], x[2, 5] = 3.5, top  # the maximum not in the first lane's values
    got = qa.quantize_activations(qa.GgmlDType(dtype), torch.from_numpy(x).cuda()).cpu().numpy()
    want = oracle.quantize_activations(dtype, x)
    assert np.array_equal(got, want)
    blocks = make_weight(oracle, dtype, 64, k, 3)
    y = run_forward(qa, dtype, blocks, 64, k, x)
    ref = oracle.qmatmul(dtype, x, blocks, 64)
    assert rel_err(y, ref) < DECODE_TOL
    y1 = run_forward(qa, dtype, blocks, 64, k, x[:1])
    assert rel_err(y1, ref[:1]) < DECODE_TOL


# ------------------------------------------------------------------ decode --
def run_forward(qa, dtype, blocks, n, k, x):
    q = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
    mm = qa.QMatMul.from_qtensor(q)
    y = mm.forward(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_config1_q8_0_matvec(qa, oracle):
    # benchmark configuration 1: x [1,1024] ~ N(0,1), W [3072,1024] ~ N(0,0.02) -> Q8_0
    blocks = make_weight(oracle, Q8_0, 3072, 1024, 1)
    x = oracle.randn(2, (1, 1024))
    y = run_forward(qa, Q8_0, blocks, 3072, 1024, x)
    want = oracle.qmatmul(Q8_0, x, blocks, 3072)
    assert rel_err(y, want) < DECODE_TOL
    dense = x.astype(np.float64) @ oracle.dequantize(Q8_0, blocks, 3072, 1024).astype(np.float64).T
    assert rel_err(y, dense) < 1e-2


LAYER_06B = [("q", 2048, 1024), ("k", 1024, 1024), ("o", 1024, 2048), ("gate", 3072, 1024), ("down", 1024, 3072)]


@pytest.mark.parametrize("m", [1, 4, 16, 64])
def test_config2_q8_0_layer(qa, oracle, m):
    for i, (name, n, k) in enumerate(LAYER_06B):
        _say(f"config2 {name} m={m}")
        blocks = make_weight(oracle, Q8_0, n, k, 10 + i)
        x = oracle.randn(20 + i + m, (m, k))
        y = run_forward(qa, Q8_0, blocks, n, k, x)
        assert rel_err(y, oracle.qmatmul(Q8_0, x, blocks, n)) < DECODE_TOL, name


SHAPES_8B = [("q", 4096, 4096), ("k", 1024, 4096), ("gate", 12288, 4096), ("down", 4096, 12288)]


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [1, 8, 16])
def test_config3_8b_shapes(qa, oracle, dtype, m):
    for i, (name, n, k) in enumerate(SHAPES_8B):
        _say(f"config3 dtype={dtype} {name} m={m}")
        blocks = make_weight(oracle, dtype, n, k, 30 + i)
        x = oracle.randn(40 + i + m, (m, k))
        y = run_forward(qa, dtype, blocks, n, k, x)
        assert rel_err(y, oracle.qmatmul(dtype, x, blocks, n)) < DECODE_TOL, name


@pytest.mark.parametrize("dtype,n,k,m", [
    (Q4_K, 1000, 12288, 40),   # k past one LDS window: the register-direct form, three tiles, ragged rows
    (Q4_K, 4096, 4096, 64),    # four tiles, four-unit panels
    (Q4_K, 72, 1280, 33),      # ragged k (five units), a handful of row tiles, the last tile one row
    (Q8_0, 1024, 3072, 64),    # the down projection of config 2
    (Q8_0, 3000, 1056, 50),    # ragged k and rows
])
def test_several_tiles_of_rows_one_workgroup_each(qa, oracle, dtype, n, k, m):
    """17 .. 64 activation rows: every 16-row tile gets workgroups of its own on the single-stage kernels
    (the launch's index decodes to row-tile group and tile); each tile's rows land in their own rows of
    y and rows past m are not written."""
    _say(f"several tiles dtype={dtype} n={n} k={k} m={m}")
    blocks = make_weight(oracle, dtype, n, k, 60 + m)
    x = oracle.randn(61 + m, (m, k))
    dt = qa.GgmlDType(dtype)
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, blocks, (n, k)))
    rows = ((m + 15) // 16) * 16
    y = torch.full((rows + 1, n), 7.0, dtype=torch.float32, device="cuda")
    mm.forward_fused(torch.from_numpy(x).cuda(), out=y[:m])
    torch.cuda.synchronize()
    assert rel_err(y[:m].cpu().numpy(), oracle.qmatmul(dtype, x, blocks, n)) < DECODE_TOL
    assert bool((y[m:] == 7.0).all())


def test_config3_lm_head_full_size(qa, oracle):
    n, k = 151936, 4096
    blocks = make_weight(oracle, Q4_K, n, k, 50)
    x = oracle.randn(51, (1, k))
    y = run_forward(qa, Q4_K, blocks, n, k, x)
    assert rel_err(y, oracle.qmatmul(Q4_K, x, blocks, n)) < DECODE_TOL


def sample_rows(blocks, dtype, n, k, count, seed):
    """Block bytes of `count` weight rows spread over the matrix (first and last included), and
    their indices: rows are independent, so the oracle's product over the subset is the
    corresponding columns of the full product."""
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, n - 1], rng.choice(n, size=count - 2, replace=False)]))
    row_bytes = k // {Q8_0: 32, Q4_K: 256}[dtype] * {Q8_0: 34, Q4_K: 144}[dtype]
    return rows, np.ascontiguousarray(blocks.reshape(n, row_bytes)[rows]).reshape(-1)


@pytest.mark.parametrize("m", [8, 16])
def test_config3_lm_head_full_size_batched(qa, oracle, m):
    # the full 151936 x 4096 matrix on the device; the oracle on ~2k of its rows
    n, k = 151936, 4096
    blocks = make_weight(oracle, Q4_K, n, k, 50)
    x = oracle.randn(52 + m, (m, k))
    _say(f"config3 lm_head m={m}")
    y = run_forward(qa, Q4_K, blocks, n, k, x)
    rows, sub = sample_rows(blocks, Q4_K, n, k, 2048, 53)
    want = oracle.qmatmul(Q4_K, x, sub, rows.size)
    assert rel_err(y[:, rows], want) < DECODE_TOL
    # the rest of the output against the single-row call of every activation row (another kernel)
    y1 = run_forward(qa, Q4_K, blocks, n, k, x[3:4])
    assert rel_err(y[3:4], y1.astype(np.float64)) < DECODE_TOL


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("n,k,m", [(1, 256, 1), (15, 256, 2), (17, 512, 3), (100, 768, 5), (250, 1280, 7),
                                   (33, 2048, 64), (7, 16384, 2), (4100, 256, 1),
                                   # batched (matrix-core) forms: more panels per row-tile than waves
                                   # (streaming form, two activation windows, y accumulated per window),
                                   # several row tiles with one LDS window buffer, ragged row tiles
                                   (20, 16384, 5), (33, 12288, 40), (50, 3072, 17),
                                   (40000, 1024, 9),  # very tall: streaming form with a resident window
                                   # k longer than one window, one row tile of activations: the
                                   # register-direct form (Q4_K), also with 3 units per panel
                                   (100, 12288, 7), (4096, 12288, 16), (33, 9216, 3), (48, 8448, 5)])
def test_ragged_shapes(qa, oracle, dtype, n, k, m):
    _say(f"ragged dtype={dtype} n={n} k={k} m={m}")
    blocks = make_weight(oracle, dtype, n, k, 60 + n)
    x = oracle.randn(61 + k, (m, k))
    y = run_forward(qa, dtype, blocks, n, k, x)
    assert rel_err(y, oracle.qmatmul(dtype, x, blocks, n)) < DECODE_TOL


def test_q8_0_k_not_multiple_of_256(qa, oracle):
    for k in (32, 96, 352):
        blocks = make_weight(oracle, Q8_0, 24, k, 70 + k)
        x = oracle.randn(71, (3, k))
        y = run_forward(qa, Q8_0, blocks, 24, k, x)
        assert rel_err(y, oracle.qmatmul(Q8_0, x, blocks, 24)) < DECODE_TOL


def test_empty_and_zero_inputs(qa, oracle):
    blocks = make_weight(oracle, Q4_K, 32, 512, 80)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks, (32, 512)))
    y0 = q.forward(torch.empty((0, 512), device="cuda"))
    assert tuple(y0.shape) == (0, 32)
    yz = q.forward(torch.zeros((2, 512), device="cuda")).cpu().numpy()
    assert not yz.any()
    # leading dims are flattened: [b, s, k] -> [b, s, n]
    x = oracle.randn(81, (2, 3, 512))
    y = q.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    assert y.shape == (2, 3, 32)
    assert rel_err(y.reshape(6, 32), oracle.qmatmul(Q4_K, x.reshape(6, 512), blocks, 32)) < DECODE_TOL


def test_host_memory_space_matches_device(qa, oracle):
    blocks = make_weight(oracle, Q8_0, 64, 512, 90)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q8_0, blocks, (64, 512)))
    x = torch.from_numpy(oracle.randn(91, (2, 512)))
    assert torch.equal(q.forward(x), q.forward(x.cuda()).cpu())


def test_shape_and_dtype_errors(qa, oracle):
    blocks = make_weight(oracle, Q4_K, 32, 512, 92)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks, (32, 512)))
    with pytest.raises(qa.QmmError):
        q.forward(torch.zeros((2, 256), device="cuda"))
    with pytest.raises(qa.QmmError):
        q.forward(torch.zeros((512, 4), device="cuda").t())
    with pytest.raises(qa.QmmError):
        q.forward(torch.zeros((2, 512), device="cuda", dtype=torch.float16))
    with pytest.raises(qa.QmmError):
        qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks[:-1], (32, 512))


# ------------------------------------------------------- packed projections --
def test_packed_qmatmul_matches_separate_q8_0(qa, oracle):
    # the reference's own test, qwen3/core.rs:3099-3142, plus its known answers
    w1 = ((np.arange(64, dtype=np.float32) - 31.0) / 8.0).reshape(2, 32)
    w2 = ((15.0 - np.arange(32, dtype=np.float32)) / 7.0).reshape(1, 32)
    x = ((np.arange(32, dtype=np.float32) + 1.0) / 16.0).reshape(1, 32)
    q1, q2 = oracle.quantize(Q8_0, w1), oracle.quantize(Q8_0, w2)
    dt = qa.GgmlDType.Q8_0
    packed = qa.packed_qmatmul_from_qtensors([(dt, q1, (2, 32)), (dt, q2, (1, 32))])
    xg = torch.from_numpy(x).cuda()
    got = packed.forward(xg).cpu().numpy()
    sep = np.concatenate([run_forward(qa, Q8_0, q1, 2, 32, x), run_forward(qa, Q8_0, q2, 1, 32, x)], axis=1)
    assert np.abs(got - sep).max() < 1e-5
    assert np.allclose(got[0], [-42.692207, 89.229607, -26.613434], rtol=0, atol=1e-5)
    assert np.array_equal(packed.qtensor.data(), np.concatenate([q1, q2]))
    with pytest.raises(qa.QmmError, match="input mismatch"):
        qa.packed_qmatmul_from_qtensors([(dt, q1, (2, 32)), (dt, oracle.quantize(Q8_0, np.zeros((1, 64), np.float32)), (1, 64))])
    with pytest.raises(qa.QmmError, match="empty"):
        qa.packed_qmatmul_from_qtensors([])


def test_packed_qkv_q4_k_split_offsets(qa, oracle):
    # fused QKV (qwen3/core.rs:1028-1035): one matmul, then narrow at 0, q, q+k
    k, nq, nkv = 1024, 512, 128
    parts = [make_weight(oracle, Q4_K, n, k, 95 + i) for i, n in enumerate((nq, nkv, nkv))]
    dt = qa.GgmlDType.Q4K
    proj = qa.Qwen3Projection.packed_quantized([(dt, p, (n, k)) for p, n in zip(parts, (nq, nkv, nkv))])
    x = oracle.randn(99, (2, k))
    y = proj.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    off = 0
    for p, n in zip(parts, (nq, nkv, nkv)):
        assert rel_err(y[:, off:off + n], oracle.qmatmul(Q4_K, x, p, n)) < DECODE_TOL
        off += n


def test_projection_dtype_policy(qa, oracle):
    blocks = make_weight(oracle, Q4_K, 64, 512, 120)
    proj = qa.Qwen3Projection.quantized(qa.GgmlDType.Q4K, blocks, (64, 512))
    x = oracle.randn(121, (1, 512))
    xb = torch.from_numpy(x).cuda().to(torch.bfloat16)
    y = proj.forward(xb)
    assert y.dtype == torch.bfloat16  # cast back to the activation dtype, qwen3/core.rs:817-828
    want = oracle.qmatmul(Q4_K, xb.float().cpu().numpy(), blocks, 64)
    assert rel_err(y.float().cpu().numpy(), want) < 1e-2


# ----------------------------------------------------------------- prefill --
@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m,n,k", [(512, 1024, 4096), (300, 200, 768), (64, 256, 256), (1, 16, 512)])
def test_prefill_bf16_against_oracle(qa, oracle, dtype, m, n, k):
    _say(f"prefill oracle dtype={dtype} m={m} n={n} k={k}")
    blocks = make_weight(oracle, dtype, n, k, 130 + n)
    xb = torch.from_numpy(oracle.randn(131 + m, (m, k))).cuda().to(torch.bfloat16)
    q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))
    y = q.forward_bf16_to_f32(xb).cpu().numpy()
    yb = q.forward(xb).float().cpu().numpy()
    xf = xb.float().cpu().numpy()
    # (a) the kernel's own arithmetic: exact bf16 activations x bf16-rounded dequantized weights
    dense = xf.astype(np.float64) @ oracle.dequantize(dtype, blocks, n, k).astype(np.float64).T
    assert rel_err(y, dense) < 4e-3
    # (b) the reference's CPU result, which also carries its int8 activation rounding
    # (about 0.5 % of the output scale): the stated 1e-2 bar, normalised by max|y_ref|.
    # With only a handful of outputs max|y_ref| is no larger than that noise's tail, so
    # the bar is applied where the output row is long enough for the normalisation to hold.
    if n >= 128:
        want = oracle.qmatmul(dtype, xf, blocks, n)
        assert rel_err(y, want) < PREFILL_TOL
        assert rel_err(yb, want) < PREFILL_TOL
    else:
        assert rel_err(yb, dense) < 1e-2


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [512, 2048])
def test_config4_prefill_full_shapes(qa, oracle, dtype, m):
    # full 8B shapes: checked against a plain fp32 matmul of the (bit-exact) dequantized weight
    for i, (name, n, k) in enumerate(SHAPES_8B):
        _say(f"config4 dtype={dtype} {name} m={m}")
        blocks = make_weight(oracle, dtype, n, k, 140 + i)
        qt = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
        xb = torch.from_numpy(oracle.randn(150 + i, (m, k))).cuda().to(torch.bfloat16)
        y = qa.QMatMul.from_qtensor(qt).forward_bf16_to_f32(xb)
        ref = xb.float() @ qt.dequantize().t()
        err = float((y - ref).abs().max() / ref.abs().max())
        assert err < 5e-3, (name, err)
        # and against the reference's CPU arithmetic on a spread of 256 weight rows
        rows, sub = sample_rows(blocks, dtype, n, k, 256, 170 + i)
        want = oracle.qmatmul(dtype, xb.float().cpu().numpy(), sub, rows.size)
        assert rel_err(y[:, torch.from_numpy(rows).cuda()].cpu().numpy(), want) < PREFILL_TOL, name
        del qt, y, ref


def test_forward_f32_large_m_uses_prefill_kernel(qa, oracle):
    blocks = make_weight(oracle, Q4_K, 256, 1024, 160)
    x = oracle.randn(161, (200, 1024))
    y = run_forward(qa, Q4_K, blocks, 256, 1024, x)
    assert rel_err(y, oracle.qmatmul(Q4_K, x, blocks, 256)) < PREFILL_TOL


def forward_rows(qa, q, ids, x):
    """izwi_qmm_forward_rows_f32 through the C ABI on device or host tensors."""
    from izwi_amd import capi
    idt = torch.from_numpy(np.asarray(ids, dtype=np.uint32).view(np.int32)).to(x.device)
    y = torch.empty((x.shape[0], len(ids)), dtype=torch.float32, device=x.device)
    capi.check(capi.lib().izwi_qmm_forward_rows_f32(
        q._h, idt.data_ptr(), len(ids), x.data_ptr(), x.shape[0], y.data_ptr(),
        capi.DEVICE if x.is_cuda else capi.HOST, torch.cuda.current_stream().cuda_stream if x.is_cuda else None))
    return y


@pytest.mark.parametrize("dtype,n,k", [(Q4_K, 151936, 4096), (Q4_K, 4096, 4096), (Q4_K, 4096, 12288), (Q8_0, 3072, 1024),
                                       (Q4_K, 1000, 768), (Q8_0, 50, 352)])
def test_selected_rows_equal_full_forward_then_gather(qa, oracle, dtype, n, k):
    """`logits_for_tokens` (qwen3/core.rs:745-758, 2155-2171): the reference runs the full LM head
    and index_selects; the row-subset call must give those bits while reading only the selected tiles."""
    _say(f"rows dtype={dtype} n={n} k={k}")
    blocks = make_weight(oracle, dtype, n, k, 180)
    q = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
    mm = qa.QMatMul.from_qtensor(q)
    rng = np.random.default_rng(181)
    ids = [0, n - 1, n - 1, 17, 16, 15] + [int(v) for v in rng.integers(0, n, size=70)]   # repeats, unsorted, both ends
    for m in (1, 2):
        x = torch.from_numpy(oracle.randn(182 + m, (m, k))).cuda()
        full = mm.forward(x)
        got = forward_rows(qa, q, ids, x)
        torch.cuda.synchronize()
        assert torch.equal(got, full[:, torch.tensor(ids, device="cuda")]), m
    # one id; host pointers (staged), where an id beyond the matrix is refused as index_select refuses it
    assert torch.equal(forward_rows(qa, q, [n // 2], x), full[:, n // 2:n // 2 + 1])
    assert torch.equal(forward_rows(qa, q, ids, x.cpu()), got.cpu())
    from izwi_amd import capi
    with pytest.raises(capi.QmmError, match="out of range"):
        forward_rows(qa, q, [n], x.cpu())
    assert torch.isnan(forward_rows(qa, q, [3, n, 5], x)[:, 1]).all()       # device ids: no host round trip
    with pytest.raises(capi.QmmError, match="selected-token"):
        forward_rows(qa, q, ids, torch.zeros((3, k), device="cuda"))
    # the mirror of Qwen3Projection::logits_for_tokens: pairs (id, value) for one hidden state
    proj = qa.Qwen3Projection(mm, is_lm_head=True)
    pairs = proj.logits_for_tokens(x[:1].view(1, 1, k), ids[:9])
    assert [p[0] for p in pairs] == ids[:9]
    assert pairs == list(zip(ids[:9], mm.forward(x[:1])[0, torch.tensor(ids[:9], device="cuda")].tolist()))
    assert proj.logits_for_tokens(x[:1], []) == []
    with pytest.raises(capi.QmmError, match="selected-token"):
        proj.logits_for_tokens(x, ids)


def test_large_m_arithmetic_switch(qa, oracle):
    """Beyond 64 rows `forward_f32` changes arithmetic (bf16 matrix cores on dequantized weights)
    unless the caller selects the integer dots: the error against the reference's CPU result at
    m = 64 and m = 65 on one shape, in both modes."""
    from izwi_amd import capi
    L = capi.lib()
    n, k = 1024, 4096
    blocks = make_weight(oracle, Q4_K, n, k, 165)
    x = oracle.randn(166, (200, k))
    want = oracle.qmatmul(Q4_K, x, blocks, n)
    assert L.izwi_qmm_get_large_m_arithmetic() == 0
    y64 = run_forward(qa, Q4_K, blocks, n, k, x[:64])
    y65 = run_forward(qa, Q4_K, blocks, n, k, x[:65])
    assert rel_err(y64, want[:64]) < DECODE_TOL
    e65 = rel_err(y65, want[:65])
    _say(f"m=64 err {rel_err(y64, want[:64]):.2e}, m=65 (bf16 matrix cores) err {e65:.2e}")
    assert DECODE_TOL < e65 < PREFILL_TOL
    capi.check(L.izwi_qmm_set_large_m_arithmetic(1))
    try:
        for m in (65, 130, 200):   # tails of 1, 2 and 8 rows behind the 64-row chunks
            y = run_forward(qa, Q4_K, blocks, n, k, x[:m])
            assert rel_err(y, want[:m]) < DECODE_TOL, m
            assert np.array_equal(y[:64], y64), m
        # the fused call (bf16 in, residual, bf16 out) follows the same switch
        q = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(Q4_K), blocks, (n, k)))
        xb = torch.from_numpy(x[:130]).cuda().to(torch.bfloat16)
        res = torch.from_numpy(oracle.randn(167, (130, n))).cuda().to(torch.bfloat16)
        got = q.forward_fused(xb, residual=res)
        plain = q.forward(xb.float())
        assert rel_err(plain.cpu().numpy(), oracle.qmatmul(Q4_K, xb.float().cpu().numpy(), blocks, n)) < DECODE_TOL
        assert torch.equal(got, (plain + res.float()).to(torch.bfloat16))
        # Qwen3Projection.forward on bf16 activations: cast to f32, QMatMul, cast back
        proj = qa.Qwen3Projection(q)
        assert torch.equal(proj.forward(xb), plain.to(torch.bfloat16))
    finally:
        capi.check(L.izwi_qmm_set_large_m_arithmetic(0))
    assert L.izwi_qmm_set_large_m_arithmetic(7) == -1 and L.izwi_qmm_get_large_m_arithmetic() == 0


# --------------------------------------------------------------------- MoE --
@pytest.mark.parametrize("t", [1, 16, 512])
def test_moe_route_and_sort_bit_exact(qa, oracle, t):
    logits = oracle.randn(170 + t, (t, 128))
    if t >= 16:
        logits[3, 10] = logits[3, 90] = logits[3].max() + 1.0
        logits[5, :] = 0.25
    ids, wts = qa.moe_route(torch.from_numpy(logits).cuda(), 8)
    want_ids, want_wts = oracle.moe_route(logits, 8)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.allclose(wts.cpu().numpy(), want_wts, rtol=1e-5, atol=1e-7)
    perm, offsets = qa.moe_sort(ids, 128)
    want_perm, want_off = oracle.moe_sort(want_ids, 128)
    assert np.array_equal(perm.cpu().numpy(), want_perm)
    assert np.array_equal(offsets.cpu().numpy(), want_off)


@pytest.mark.parametrize("rows,experts", [
    (5000, 128),   # 40000 pairs: the three-launch sort
    (1024, 128),   # 8192 pairs: one workgroup, 83 KB of LDS
    (2048, 128),   # 16384 pairs: the most one workgroup takes (149 KB)
    (2049, 128),   # one row more: three launches
    (1500, 200),   # 12000 pairs of 200 experts: 152 KB would not do, three launches
    (700, 512),    # many experts, few runs
])
def test_moe_sort_many_pairs(qa, oracle, rows, experts):
    rng = np.random.default_rng(3 + rows)
    ids = rng.integers(0, experts, size=(rows, 8)).astype(np.int32)
    ids[:, 3] = 5  # an expert with a pair of every row
    perm, offsets = qa.moe_sort(torch.from_numpy(ids).cuda(), experts)
    want_perm, want_off = oracle.moe_sort(ids, experts)
    assert np.array_equal(perm.cpu().numpy(), want_perm) and np.array_equal(offsets.cpu().numpy(), want_off)


@pytest.fixture(scope="module")
def moe_weights(oracle):
    # benchmark configuration 5 at full size: 128 experts, hidden 2048, intermediate 768, Q4_K
    E, hidden, inter = 128, 2048, 768
    gate = oracle.quantize(Q4_K, oracle.randn(180, (E * inter, hidden), std=0.02))
    up = oracle.quantize(Q4_K, oracle.randn(181, (E * inter, hidden), std=0.02))
    down = oracle.quantize(Q4_K, oracle.randn(182, (E * hidden, inter), std=0.02))
    return E, hidden, inter, gate, up, down


@pytest.mark.parametrize("t", [1, 16, 512])
def test_config5_moe_forward(qa, oracle, moe_weights, t):
    E, hidden, inter, gate, up, down = moe_weights
    dt = qa.GgmlDType.Q4K
    experts = qa.MoeExperts(qa.QTensor.from_blocks(dt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, down, (E, hidden, inter)))
    x = oracle.randn(190 + t, (t, hidden))
    logits = oracle.randn(191 + t, (t, E))
    xg = torch.from_numpy(x).cuda()
    ids, wts = qa.moe_route(torch.from_numpy(logits).cuda(), 8)
    perm, offsets = qa.moe_sort(ids, E)
    out = experts.forward(xg, ids, wts, perm, offsets).cpu().numpy()
    # the oracle is scalar: check every token for small t, a spread of 12 tokens at t = 512
    rows = np.arange(t) if t <= 16 else np.linspace(0, t - 1, 12).astype(np.int64)
    want_ids, want_wts = oracle.moe_route(logits, 8)
    want = oracle.moe_forward(Q4_K, x[rows], want_ids[rows], want_wts[rows], gate, up, down, E, inter)
    assert rel_err(out[rows], want) < 1e-3
    assert np.isfinite(out).all()


@pytest.mark.parametrize("t", [1, 2, 3, 16, 17, 24, 40, 63, 100, 128, 129, 512])
def test_config5_moe_layer_one_call_equals_the_three_calls(qa, oracle, moe_weights, t):
    """izwi_moe_layer_f32 = route + sort + forward, bit for bit (ids, weights, outputs): up to
    1024 pairs routing, sort and segment tables come from one launch, beyond from the
    separate kernels."""
    _say(f"moe layer t={t}")
    E, hidden, inter, gate, up, down = moe_weights
    dt = qa.GgmlDType.Q4K
    experts = qa.MoeExperts(qa.QTensor.from_blocks(dt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, down, (E, hidden, inter)))
    x = torch.from_numpy(oracle.randn(290 + t, (t, hidden))).cuda()
    logits_h = oracle.randn(291 + t, (t, E))
    if t >= 3:  # ties, an infinity and a NaN in the logits of some tokens
        logits_h[1, 5] = logits_h[1, 77] = logits_h[1].max() + 1.0
        logits_h[2, 9] = np.inf
        logits_h[2, 100] = np.nan
        logits_h[0, :] = 0.25
    logits = torch.from_numpy(logits_h).cuda()
    ids, wts = qa.moe_route(logits, 8)
    perm, offsets = qa.moe_sort(ids, E)
    want = experts.forward(x, ids, wts, perm, offsets)
    out, ids2, wts2 = experts.layer(logits, x, 8, return_routing=True)
    assert torch.equal(ids2, ids)
    assert torch.equal(wts2.view(torch.int32), wts.view(torch.int32))
    assert torch.equal(out.view(torch.int32), want.view(torch.int32))
    assert torch.equal(experts.layer(logits, x, 8).view(torch.int32), want.view(torch.int32))
    want_ids, _ = oracle.moe_route(logits_h, 8)
    assert np.array_equal(ids2.cpu().numpy(), want_ids)
    if t <= 16:  # host pointers
        out_h = experts.layer(logits.cpu(), x.cpu(), 8)
        assert torch.equal(out_h.view(torch.int32), want.cpu().view(torch.int32))


@pytest.mark.parametrize("dtype,E,hidden,inter,t,top_k", [
    (Q8_0, 64, 512, 256, 20, 4),    # 17..: the routing kernel quantizes the token rows, gate / up copies the blocks
    (Q4_K, 64, 1280, 768, 33, 2),   # the same with five units per row (two rounds of a wave's four groups)
    (Q4_K, 32, 2560, 256, 17, 2),   # ten units per row: units beyond the eight that are loaded ahead of the routing
    (Q8_0, 48, 1056, 256, 40, 3),   # a row that ends inside a unit
])
def test_moe_layer_with_token_rows_quantized_by_the_routing_kernel(qa, oracle, dtype, E, hidden, inter, t, top_k):
    """More than 16 tokens and fewer than four pairs per expert: izwi_moe_layer_f32 quantizes every
    token row once, in the routing kernel; route + sort + forward (rows quantized in the grouped
    kernel's workgroups) must give the same bits."""
    _say(f"moe x blocks dtype={dtype} E={E} hidden={hidden} inter={inter} t={t} top_k={top_k}")
    assert t > 16 and t * top_k < 4 * E
    gate = oracle.quantize(dtype, oracle.randn(311, (E * inter, hidden), std=0.05))
    up = oracle.quantize(dtype, oracle.randn(312, (E * inter, hidden), std=0.05))
    down = oracle.quantize(dtype, oracle.randn(313, (E * hidden, inter), std=0.05))
    dt = qa.GgmlDType(dtype)
    experts = qa.MoeExperts(qa.QTensor.from_blocks(dt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, down, (E, hidden, inter)))
    x_h = oracle.randn(314, (t, hidden))
    x_h[3, :] = 0.0  # a zero row: scale 0
    logits_h = oracle.randn(315, (t, E))
    x, logits = torch.from_numpy(x_h).cuda(), torch.from_numpy(logits_h).cuda()
    ids, wts = qa.moe_route(logits, top_k)
    perm, offsets = qa.moe_sort(ids, E)
    want = experts.forward(x, ids, wts, perm, offsets)
    out = experts.layer(logits, x, top_k)
    assert torch.equal(out.view(torch.int32), want.view(torch.int32))
    want_ids, want_wts = oracle.moe_route(logits_h, top_k)
    ref = oracle.moe_forward(dtype, x_h, want_ids, want_wts, gate, up, down, E, inter)
    assert rel_err(out.cpu().numpy(), ref) < 1e-3


@pytest.mark.parametrize("dtype,E,hidden,inter,t,top_k", [
    (Q8_0, 8, 512, 256, 64, 4),     # 32 pairs per expert: matrix-core tiles, Q8_0, one unit per panel
    (Q4_K, 4, 1280, 768, 40, 2),    # ragged k (5 units), three-unit panels on the way down
    (Q4_K, 16, 512, 512, 6, 8),     # 3 pairs per expert: 4-row segments
    (Q8_0, 8, 512, 256, 2, 4),      # 8 pairs: the two-launch form (routing in gate / up, combine in down)
    (Q4_K, 8, 1280, 1024, 3, 2),    # the same with four units per panel on the way down, ragged k on the way up
])
def test_moe_forward_small_shapes(qa, oracle, dtype, E, hidden, inter, t, top_k):
    gate = oracle.quantize(dtype, oracle.randn(301, (E * inter, hidden), std=0.05))
    up = oracle.quantize(dtype, oracle.randn(302, (E * inter, hidden), std=0.05))
    down = oracle.quantize(dtype, oracle.randn(303, (E * hidden, inter), std=0.05))
    dt = qa.GgmlDType(dtype)
    experts = qa.MoeExperts(qa.QTensor.from_blocks(dt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, down, (E, hidden, inter)))
    x = oracle.randn(304, (t, hidden))
    logits = oracle.randn(305, (t, E))
    ids, wts = qa.moe_route(torch.from_numpy(logits).cuda(), top_k)
    perm, offsets = qa.moe_sort(ids, E)
    out = experts.forward(torch.from_numpy(x).cuda(), ids, wts, perm, offsets).cpu().numpy()
    want_ids, want_wts = oracle.moe_route(logits, top_k)
    want = oracle.moe_forward(dtype, x, want_ids, want_wts, gate, up, down, E, inter)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert rel_err(out, want) < 1e-3


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 16, 40, 80])
def test_projection_group_equals_separate_calls(qa, oracle, dtype, m):
    """Qwen3QkvProjection / Qwen3GateUpProjection `Separate` arms as one call: bit-identical to
    separate forwards (one launch of the decode kernel for m <= 2 and, at this k, for m <= 4; shared
    activation quantization up to 64)."""
    k = 1024
    dt = qa.GgmlDType(dtype)
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, dtype, n, k, 400 + n), (n, k)))
             for n in (2048, 1024, 1000)]
    x = torch.from_numpy(oracle.randn(401 + m, (m, k))).cuda()
    q, kk, v = qa.Qwen3QkvProjection.new_separate(*parts).forward(x)
    for got, p in zip((q, kk, v), parts):
        assert torch.equal(got, p.forward(x))
    # and against the oracle for one of them
    want = oracle.qmatmul(dtype, x.cpu().numpy(), make_weight(oracle, dtype, 1000, k, 1400), 1000)
    tol = DECODE_TOL if m <= 64 else PREFILL_TOL
    assert rel_err(v.cpu().numpy(), want) < tol


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [1, 2, 3, 16, 40])
@pytest.mark.parametrize("k,ns", [(1024, (4000, 1000, 600)), (4096, (4096, 1000, 1048)), (2048, (3000, 3000, 3000, 200)),
                                  (1024, (16, 8200))])
def test_projection_group_workgroups_straddle_weights(qa, oracle, dtype, m, k, ns):
    """More row-tiles than CUs: a workgroup takes several row-tiles, the launch's row-tiles are
    counted over all weights and a workgroup may hold the last row-tile of one weight beside the
    first of the next (m <= 2); every output equals the separate forward bit for bit."""
    _say(f"group straddle dtype={dtype} m={m} k={k} ns={ns}")
    dt = qa.GgmlDType(dtype)
    blocks = [make_weight(oracle, dtype, n, k, 900 + n + i) for i, n in enumerate(ns)]
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b, (n, k))) for b, n in zip(blocks, ns)]
    x = torch.from_numpy(oracle.randn(901 + m, (m, k))).cuda()
    outs = qa.forward_group(parts, x)
    for got, p in zip(outs, parts):
        assert torch.equal(got, p.forward(x))
    want = oracle.qmatmul(dtype, x.cpu().numpy(), blocks[1], ns[1])
    assert rel_err(outs[1].cpu().numpy(), want) < DECODE_TOL


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [17, 32, 33, 64])
@pytest.mark.parametrize("k,ns", [(4096, (4096, 1024, 1024)), (2048, (1536, 1536)), (768, (2000, 48, 16, 512))])
def test_projection_group_on_several_row_tiles(qa, oracle, dtype, m, k, ns):
    """17 <= m <= 64 (two to four 16-row tiles of activations): the group is one launch of the
    batched decode kernel, workgroups of their own for every tile of rows, and equals the separate
    forwards bit for bit."""
    _say(f"group tiles dtype={dtype} m={m} k={k} ns={ns}")
    dt = qa.GgmlDType(dtype)
    blocks = [make_weight(oracle, dtype, n, k, 700 + n + i) for i, n in enumerate(ns)]
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b, (n, k))) for b, n in zip(blocks, ns)]
    x = torch.from_numpy(oracle.randn(701 + m, (m, k))).cuda()
    outs = qa.forward_group(parts, x)
    for got, p in zip(outs, parts):
        assert torch.equal(got, p.forward(x))
    want = oracle.qmatmul(dtype, x.cpu().numpy(), blocks[-1], ns[-1])
    assert rel_err(outs[-1].cpu().numpy(), want) < DECODE_TOL


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m,k,ns", [(512, 4096, (4096, 1024, 1024)), (2048, 4096, (4096, 1024, 1024)),
                                    (300, 768, (300, 200)), (200, 1024, (2048, 1000, 16, 512)), (129, 256, (256, 256))])
def test_projection_group_at_prefill_sizes(qa, oracle, dtype, m, k, ns):
    """Beyond 128 rows a projection group is ONE launch of the bf16 matrix-core kernel (the members'
    column tiles side by side): every member equals its separate call up to the f32 summation order
    (the plan may split k differently), for f32 activations (converted once) and bf16 activations."""
    _say(f"group prefill dtype={dtype} m={m} k={k} ns={ns}")
    dt = qa.GgmlDType(dtype)
    blocks = [make_weight(oracle, dtype, n, k, 420 + n + i) for i, n in enumerate(ns)]
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b, (n, k))) for b, n in zip(blocks, ns)]
    x = torch.from_numpy(oracle.randn(421 + m, (m, k))).cuda()
    xb = x.to(torch.bfloat16)
    got_f32 = qa.forward_group(parts, x)
    got_bf16 = qa.forward_group(parts, xb)
    for i, p in enumerate(parts):
        sep = p.forward(x)
        scale = float(sep.abs().max())
        assert float((got_f32[i] - sep).abs().max()) <= 2e-5 * scale, i
        sep_b = p.forward_bf16_to_f32(xb)
        assert got_bf16[i].dtype == torch.bfloat16 and got_bf16[i].shape == (m, ns[i])
        assert float((got_bf16[i].float() - sep_b).abs().max()) <= 2.0 ** -7 * float(sep_b.abs().max()), i
    # the reference's CPU arithmetic on the narrowest member with at least 128 outputs, on the same
    # (bf16-representable) activations
    i = min((j for j, n in enumerate(ns) if n >= 128), key=lambda j: ns[j])
    want = oracle.qmatmul(dtype, xb.float().cpu().numpy(), blocks[i], ns[i])
    assert rel_err(got_bf16[i].float().cpu().numpy(), want) < PREFILL_TOL
    # gate / up with its activation runs on the same group launch
    if len(ns) >= 2 and ns[0] == ns[1] or len(ns) >= 3 and ns[1] == ns[2]:
        a, b = (parts[1], parts[2]) if len(ns) >= 3 and ns[1] == ns[2] else (parts[0], parts[1])
        h = qa.Qwen3GateUpProjection.new_separate(a, b).forward_silu_mul(x)
        ga, ub = a.forward(x), b.forward(x)
        ref = torch.nn.functional.silu(ga) * ub
        assert float((h - ref).abs().max()) <= 1e-4 * float(ref.abs().max())


@pytest.mark.parametrize("dtype", [Q4_K, Q8_0])
@pytest.mark.parametrize("m", [1, 2, 16, 64, 100])
def test_projection_group_on_bf16_activations_equals_the_members_forwards(qa, oracle, dtype, m):
    """forward_group on bf16 activations gives, bit for bit, what Qwen3Projection.forward gives for
    every member (the reference's Separate arms just call each projection, qwen3/core.rs:1119-1127):
    up to 64 rows that is the integer block-dot arithmetic, not the bf16 matrix-core kernel; with
    the integer arithmetic selected for larger batches too, also beyond."""
    _say(f"group bf16 policy dtype={dtype} m={m}")
    dt = qa.GgmlDType(dtype)
    k, ns = 1024, (512, 256, 48)
    blocks = [make_weight(oracle, dtype, n, k, 470 + n) for n in ns]
    parts = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b, (n, k))) for b, n in zip(blocks, ns)]
    xb = torch.from_numpy(oracle.randn(471 + m, (m, k))).cuda().to(torch.bfloat16)
    lib = qa.lib()
    try:
        if m > 64:
            assert lib.izwi_qmm_set_large_m_arithmetic(1) == 0
        got = qa.forward_group(parts, xb)
        for i, p in enumerate(parts):
            sep = qa.Qwen3Projection(p).forward(xb)
            assert got[i].dtype == torch.bfloat16 and torch.equal(got[i], sep), i
        # and it is the integer arithmetic: the reference's CPU result on the same activations
        want = oracle.qmatmul(dtype, xb.float().cpu().numpy(), blocks[0], ns[0])
        assert rel_err(got[0].float().cpu().numpy(), want) < 5e-3  # bf16 rounding of the output
    finally:
        lib.izwi_qmm_set_large_m_arithmetic(0)


def test_projection_group_8b_gate_up_and_errors(qa, oracle):
    dt = qa.GgmlDType.Q4K
    gate = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, Q4_K, 12288, 4096, 410), (12288, 4096)))
    up = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, Q4_K, 12288, 4096, 411), (12288, 4096)))
    x = torch.from_numpy(oracle.randn(412, (1, 4096))).cuda()
    g, u = qa.Qwen3GateUpProjection.new_separate(gate, up).forward(x)
    assert torch.equal(g, gate.forward(x)) and torch.equal(u, up.forward(x))
    other_k = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, Q4_K, 64, 1024, 413), (64, 1024)))
    with pytest.raises(qa.QmmError, match="input mismatch"):
        qa.forward_group([gate, other_k], x)
    # mixed block types still work (one call per projection inside)
    q8 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q8_0, make_weight(oracle, Q8_0, 96, 4096, 414), (96, 4096)))
    a, b = qa.forward_group([up, q8], x)
    assert torch.equal(a, up.forward(x)) and torch.equal(b, q8.forward(x))


# ------------------------------------------------- gate / up with its activation --
@pytest.mark.parametrize("dtype,n,k", [(Q4_K, 12288, 4096), (Q8_0, 3072, 1024), (Q4_K, 80, 768), (Q8_0, 40, 96)])
@pytest.mark.parametrize("m", [1, 2, 5, 16, 80])
def test_gate_up_silu_matches_separate_projections(qa, oracle, dtype, n, k, m):
    """Qwen3Mlp::forward's gate_up_proj + silu * up (qwen3/core.rs:1786-1796) in one call: the two
    sums are the separate projections' bit for bit, so the result equals silu(g) * u computed
    from them up to the rounding of silu itself; against the oracle within the decode tolerance."""
    _say(f"gate_up_silu dtype={dtype} n={n} k={k} m={m}")
    dt = qa.GgmlDType(dtype)
    wg, wu = make_weight(oracle, dtype, n, k, 500), make_weight(oracle, dtype, n, k, 501)
    gate = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, wg, (n, k)))
    up = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, wu, (n, k)))
    x = torch.from_numpy(oracle.randn(502 + m, (m, k))).cuda()
    proj = qa.Qwen3GateUpProjection.new_separate(gate, up)
    h = proj.forward_silu_mul(x)
    g, u = gate.forward(x), up.forward(x)
    want = (g.double() / (1.0 + torch.exp(-g.double())) * u.double()).float()
    assert h.shape == (m, n)
    assert (h - want).abs().max().item() <= 2e-6 * max(want.abs().max().item(), 1e-30)
    if m <= 16 and n <= 3072:
        xo = x.cpu().numpy()
        go, uo = oracle.qmatmul(dtype, xo, wg, n), oracle.qmatmul(dtype, xo, wu, n)
        ref = go / (1.0 + np.exp(-go.astype(np.float64))) * uo
        assert rel_err(h.cpu().numpy(), ref.astype(np.float32)) < (1e-4 if m <= 64 else 1e-2)


def test_gate_up_silu_mlp_mirror_host_pointers_and_errors(qa, oracle):
    dt = qa.GgmlDType.Q4K
    n, k = 64, 512
    wg, wu, wd = make_weight(oracle, Q4_K, n, k, 510), make_weight(oracle, Q4_K, n, k, 511), make_weight(oracle, Q4_K, k, 256, 512)
    gate = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, wg, (n, k)))
    up = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, wu, (n, k)))
    proj = qa.Qwen3GateUpProjection.new_separate(gate, up)
    x = torch.from_numpy(oracle.randn(513, (3, k)))
    assert torch.equal(proj.forward_silu_mul(x), proj.forward_silu_mul(x.cuda()).cpu())       # host pointers
    # Qwen3Mlp: down(silu(gate x) * up x); inner width 256 here needs its own gate / up
    g2 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, Q4_K, 256, k, 514), (256, k)))
    u2 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, make_weight(oracle, Q4_K, 256, k, 515), (256, k)))
    down = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, wd, (k, 256)))
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(g2, u2), down)
    xc = x.cuda()
    y = mlp.forward(xc)
    assert torch.equal(y, down.forward(qa.Qwen3GateUpProjection.new_separate(g2, u2).forward_silu_mul(xc)))
    assert y.shape == (3, k)
    # shape and type mismatches are errors
    with pytest.raises(qa.QmmError, match="gate is"):
        qa.Qwen3GateUpProjection.new_separate(gate, g2).forward_silu_mul(xc)
    q8 = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q8_0, make_weight(oracle, Q8_0, n, k, 516), (n, k)))
    with pytest.raises(qa.QmmError, match="different ggml dtypes"):
        qa.Qwen3GateUpProjection.new_separate(gate, q8).forward_silu_mul(xc)
    with pytest.raises(qa.QmmError, match="shape mismatch"):
        proj.forward_silu_mul(torch.zeros((1, 256), device="cuda"))


@pytest.mark.parametrize("dtype,n,k", [(Q4_K, 1000, 1024), (Q8_0, 300, 96), (Q4_K, 151936, 256)])
def test_embedding_rows_equal_rows_of_the_dequantized_table(qa, oracle, dtype, n, k):
    """`Embedding::forward(input_ids)` on the dequantized table (qwen3/core.rs:2000-2007, 2083-2085):
    the selected rows bit for bit, f32 and cast to bf16; ids from host and from device memory."""
    w = oracle.randn(4100 + n, (min(n, 4096), k), std=0.05)
    if n > 4096:
        w = np.tile(w, ((n + 4095) // 4096, 1))[:n]
    blocks = oracle.quantize(dtype, w)
    q = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
    table = q.dequantize()
    assert np.array_equal(table.cpu().numpy().view(np.uint32), oracle.dequantize(dtype, blocks, n, k).view(np.uint32))
    ids = np.array([0, n - 1, 17, 17, n // 2, 3, n - 2, 1], dtype=np.int64)
    for where in ("cpu", "cuda"):
        idt = torch.from_numpy(ids).to(where)
        got = q.dequantize_rows(idt)
        assert torch.equal(got.view(torch.int32), table[torch.from_numpy(ids).cuda()].view(torch.int32)), where
        got16 = q.dequantize_rows(idt, torch.bfloat16)
        assert torch.equal(got16.view(torch.int16), table[torch.from_numpy(ids).cuda()].to(torch.bfloat16).view(torch.int16))
    emb = qa.QuantizedEmbedding(q, torch.bfloat16)
    batch = torch.from_numpy(ids.reshape(2, 4)).cuda()
    out = emb.forward(batch)
    assert out.shape == (2, 4, k) and out.dtype == torch.bfloat16
    assert torch.equal(out.view(-1, k).view(torch.int16), got16.view(torch.int16))
    assert q.dequantize_rows(torch.zeros(0, dtype=torch.int64)).shape == (0, k)
    from izwi_amd import capi
    with pytest.raises(capi.QmmError, match="out of range"):
        q.dequantize_rows(torch.tensor([0, n]))
    with pytest.raises(capi.QmmError, match="out of range"):
        q.dequantize_rows(torch.tensor([-1]))
    # ids in device memory are not read by the host: a row of zeros
    z = q.dequantize_rows(torch.tensor([n, 1], device="cuda"))
    assert torch.count_nonzero(z[0]) == 0 and torch.equal(z[1].view(torch.int32), table[1].view(torch.int32))


def test_embedding_rows_q6k(qa, oracle):
    n, k = 200, 512
    blocks = np_ref.random_q6_k_blocks(77, n, k)
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q6K, blocks, (n, k))
    table = q.dequantize()
    ids = torch.tensor([199, 0, 5, 5, 100], device="cuda")
    assert torch.equal(q.dequantize_rows(ids).view(torch.int32), table[ids].view(torch.int32))
    assert torch.equal(q.dequantize_rows(ids, torch.bfloat16).view(torch.int16), table[ids].to(torch.bfloat16).view(torch.int16))
