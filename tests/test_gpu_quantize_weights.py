"""GPU parity of `QTensor::quantize` (pytest -m gpu): the Q8_0 / Q4_K block bytes of f32 matrices are,
byte for byte, those of the oracle's restatement of candle-core's CPU quantizers
(`BlockQ8_0::from_float`, `BlockQ4K::from_float` + `make_qkx1_quants`), on the closed-form blocks of
tests/golden/q4k_quantizer_cases.json and on seeded matrices."""
import ctypes as C
import json
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14
ERR_INVALID, ERR_UNSUPPORTED = -1, -2
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "q4k_quantizer_cases.json")


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


def device_blocks(qa, dtype, w, on_device=True):
    from izwi_amd import capi
    n, k = w.shape
    nbytes = qa.quantized_storage_bytes(n, k, qa.GgmlDType(dtype))
    if on_device:
        wt = torch.from_numpy(np.ascontiguousarray(w, dtype=np.float32)).cuda()
        out = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        capi.check(capi.lib().izwi_qmm_quantize_weights_f32(dtype, wt.data_ptr(), n, k, out.data_ptr(), capi.DEVICE,
                                                            torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        return out.cpu().numpy()
    wh = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty(nbytes, dtype=np.uint8)
    capi.check(capi.lib().izwi_qmm_quantize_weights_f32(dtype, wh.ctypes.data, n, k, out.ctypes.data, capi.HOST, None))
    return out


def test_q4_k_closed_form_blocks(qa):
    cases = json.load(open(GOLDEN))["blocks"]
    for case in cases:
        print(f"q4k quantize golden {case['name']}", flush=True)
        x = np.asarray(case["x"], dtype=np.float32).reshape(1, 256)
        got = device_blocks(qa, Q4_K, x)
        assert bytes(got).hex() == case["block_hex"], case["name"]


@pytest.mark.parametrize("dtype", [Q8_0, Q4_K])
@pytest.mark.parametrize("n,k,std,seed", [(1, 256, 0.02, 1), (7, 512, 0.02, 2), (33, 768, 1.0, 3), (64, 4096, 0.02, 4),
                                          (300, 1280, 5.0, 5), (1024, 4096, 0.02, 6), (17, 12288, 0.02, 7)])
def test_blocks_equal_the_oracle_quantizer(qa, oracle, dtype, n, k, std, seed):
    print(f"quantize dtype={dtype} n={n} k={k} std={std}", flush=True)
    w = oracle.randn(seed, (n, k), std=std)
    want = oracle.quantize(dtype, w)
    got = device_blocks(qa, dtype, w)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [Q8_0, Q4_K])
def test_special_values_and_host_buffers(qa, oracle, dtype):
    k = 1024
    rng = np.random.default_rng(11)
    rows = [np.zeros(k, np.float32), np.full(k, 0.125, np.float32), np.full(k, -3.0, np.float32),
            np.abs(rng.standard_normal(k)).astype(np.float32), -np.abs(rng.standard_normal(k)).astype(np.float32),
            (rng.standard_normal(k) * 1e-30).astype(np.float32), (rng.standard_normal(k) * 1e4).astype(np.float32),
            np.round(rng.standard_normal(k) * 4).astype(np.float32) / 8,  # many ties
            np.where(rng.random(k) < 0.9, 0.0, rng.standard_normal(k)).astype(np.float32)]
    w = np.stack(rows)
    want = oracle.quantize(dtype, w)
    assert np.array_equal(device_blocks(qa, dtype, w), want)
    assert np.array_equal(device_blocks(qa, dtype, w, on_device=False), want)


def test_qtensor_quantize_mirror_and_errors(qa, oracle):
    from izwi_amd import capi
    w = oracle.randn(21, (48, 1024), std=0.02)
    for dtype in (Q8_0, Q4_K):
        q = qa.QTensor.quantize(torch.from_numpy(w).cuda(), qa.GgmlDType(dtype))
        assert q.shape() == (48, 1024) and int(q.dtype()) == dtype
        blocks = oracle.quantize(dtype, w)
        assert np.array_equal(q.data(), blocks)
        want = oracle.dequantize(dtype, blocks, 48, 1024)
        assert np.array_equal(q.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    L = capi.lib()
    buf = torch.zeros(4096, dtype=torch.float32, device="cuda")
    out = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    assert L.izwi_qmm_quantize_weights_f32(Q6_K, buf.data_ptr(), 1, 256, out.data_ptr(), capi.DEVICE, None) == ERR_UNSUPPORTED
    assert L.izwi_qmm_quantize_weights_f32(Q4_K, buf.data_ptr(), 1, 100, out.data_ptr(), capi.DEVICE, None) == ERR_INVALID
    assert L.izwi_qmm_quantize_weights_f32(Q4_K, None, 1, 256, out.data_ptr(), capi.DEVICE, None) == ERR_INVALID
    assert L.izwi_qmm_quantize_weights_f32(Q8_0, buf.data_ptr(), 0, 256, out.data_ptr(), capi.DEVICE, None) == 0
    with pytest.raises(capi.QmmError):
        qa.QTensor.quantize(torch.zeros(2, 3, 256), qa.GgmlDType.Q4K)
