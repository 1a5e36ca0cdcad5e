"""The entry point that allocates nothing (izwi_qmm_forward_f32_noalloc, pytest -m gpu): called
through the C ABI and compared bit for bit with izwi_qmm_forward_f32 on the same inputs, twice in a
row with the second input smaller (the static scratch keeps the first call's contents), plus its
limits.  Collected last on purpose: it passes alone in a fresh process and after the other tests."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


def both(qa, q, x):
    """(noalloc result, forward_f32 result) on device tensors, through the C ABI."""
    from izwi_amd import capi
    L = capi.lib()
    n, k = q.dims2()
    m = x.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    y0 = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    y1 = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    capi.check(L.izwi_qmm_forward_f32_noalloc(q._h, x.data_ptr(), m, y0.data_ptr(), stream))
    capi.check(L.izwi_qmm_forward_f32(q._h, x.data_ptr(), m, y1.data_ptr(), capi.DEVICE, stream))
    torch.cuda.synchronize()
    return y0, y1


@pytest.mark.parametrize("dtype,n,k", [(Q4_K, 4096, 4096), (Q8_0, 1024, 4096), (Q4_K, 4096, 12288), (Q4_K, 100, 768)])
def test_noalloc_matches_forward_f32_twice_in_a_row(qa, oracle, dtype, n, k):
    blocks = oracle.quantize(dtype, oracle.randn(2000 + n, (n, k), std=0.02))
    q = qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))
    xa = torch.from_numpy(oracle.randn(2001 + k, (64, k))).cuda()
    xb = torch.from_numpy(oracle.randn(2002 + k, (5, k))).cuda()
    print(f"noalloc dtype={dtype} n={n} k={k}: m=64 then m=5", flush=True)
    y0, y1 = both(qa, q, xa)            # fills the whole static scratch the shape needs
    assert torch.equal(y0, y1)
    y0, y1 = both(qa, q, xb)            # smaller input on top of the first call's leftovers
    assert torch.equal(y0, y1)
    want = oracle.qmatmul(dtype, xb.cpu().numpy(), blocks, n)
    assert float(np.abs(y0.cpu().numpy() - want).max() / np.abs(want).max()) < 1e-4
    for m in (1, 2, 3, 16, 17):
        y0, y1 = both(qa, q, xa[:m].contiguous())
        assert torch.equal(y0, y1), m


def test_noalloc_allocates_nothing_and_rejects_what_does_not_fit(qa, oracle):
    from izwi_amd import capi
    L = capi.lib()
    n, k = 256, 16384
    blocks = oracle.quantize(Q8_0, oracle.randn(2100, (n, k), std=0.02))
    q = qa.QTensor.from_blocks(qa.GgmlDType(Q8_0), blocks, (n, k))
    x = torch.from_numpy(oracle.randn(2101, (64, k))).cuda()
    y = torch.empty((64, n), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    # 4 tiles x 64 units x 4608 bytes = 1,179,648 > 1 MiB: refused with a message, nothing launched
    rc = L.izwi_qmm_forward_f32_noalloc(q._h, x.data_ptr(), 64, y.data_ptr(), stream)
    assert rc == -2 and b"static scratch" in L.izwi_qmm_last_error()
    assert L.izwi_qmm_forward_f32_noalloc(q._h, x.data_ptr(), 65, y.data_ptr(), stream) == -2
    # 3 tiles fit
    y0, y1 = both(qa, q, x[:48].contiguous())
    assert torch.equal(y0, y1)
    # device memory in use does not move across calls (no hipMalloc / hipFree inside)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for m in (3, 48, 7, 33):
        capi.check(L.izwi_qmm_forward_f32_noalloc(q._h, x.data_ptr(), m, y.data_ptr(), stream))
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free0 == free1
    # and it is legal inside a stream capture on a stream that never ran a library call
    _, want16 = both(qa, q, x[:16].contiguous())
    s = torch.cuda.Stream()
    yg = torch.empty((16, n), dtype=torch.float32, device="cuda")
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            capi.check(L.izwi_qmm_forward_f32_noalloc(q._h, x.data_ptr(), 16, yg.data_ptr(), s.cuda_stream))
        for _ in range(3):
            yg.zero_()
            g.replay()
            s.synchronize()
            assert torch.equal(yg, want16)
