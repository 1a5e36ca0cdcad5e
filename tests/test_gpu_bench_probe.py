"""The benchmark's own measurement kernels (bench_probe/libbench_probe.so, not part of the library):
they load, reject bad arguments without launching, and the copy kernel copies (pytest -m gpu)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_bench_probe_read_and_copy():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible")
    import bench
    P = bench.probe()
    torch.cuda.set_device(0)
    sp = torch.cuda.current_stream().cuda_stream
    for nbytes in (4096, 1 << 20, 50 << 20, (50 << 20) + 48):
        src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
        dst = torch.zeros_like(src)
        assert P.bench_probe_stream_read(src.data_ptr(), nbytes, sp) == 0
        for wgs in (1, 4, 100):
            dst.zero_()
            assert P.bench_probe_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, wgs, sp) == 0
            torch.cuda.synchronize()
            assert torch.equal(dst[:nbytes // 16 * 16], src[:nbytes // 16 * 16])
    buf = torch.zeros(64, dtype=torch.uint8, device="cuda")
    assert P.bench_probe_stream_read(None, 1024, None) != 0
    assert P.bench_probe_stream_read(buf.data_ptr() + 4, 32, None) != 0
    assert P.bench_probe_stream_copy(buf.data_ptr(), None, 32, 1, None) != 0
    assert P.bench_probe_stream_read(buf.data_ptr(), 0, None) == 0
