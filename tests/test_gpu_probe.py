"""GPU test of the read-only streaming probe (pytest -m gpu): it runs, leaves its buffer alone, and rejects
bad arguments; its rate is a report of bench.py, not a test."""
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from izwi_amd import capi
    return capi


@pytest.mark.parametrize("nbytes", [16, 4096 + 48, 9 << 20, (40 << 20) + 16, 64 << 20])
def test_probe_reads_and_stores_nothing(lib, nbytes):
    print(f"probe nbytes={nbytes}", flush=True)
    buf = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
    before = buf.clone()
    sp = torch.cuda.current_stream().cuda_stream
    assert lib.lib().izwi_qmm_probe_stream_read(buf.data_ptr(), nbytes, sp) == 0
    torch.cuda.synchronize()
    assert torch.equal(buf, before)


def test_probe_rejects_bad_arguments(lib):
    buf = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    L = lib.lib()
    assert L.izwi_qmm_probe_stream_read(None, 1024, None) != 0
    assert L.izwi_qmm_probe_stream_read(buf.data_ptr() + 4, 512, None) != 0
    assert b"aligned" in L.izwi_qmm_last_error()
    assert L.izwi_qmm_probe_stream_read(buf.data_ptr(), 0, None) == 0
