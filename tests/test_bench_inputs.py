"""bench.py's own input generator: the synthetic quantizer must write well-formed Q8_0 / Q4_K blocks
whose dequantization (by the oracle) is the input up to the format's step, so that the benchmark
measures the kernels on realistic bytes without any measured leg touching the oracle."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
import bench  # noqa: E402

Q8_0, Q4_K = 8, 12


def test_synthetic_quantizer_writes_valid_blocks(oracle):
    w = bench.synth_normal(3, (48, 1024), std=0.02)
    assert w.dtype == np.float32 and abs(float(w.std()) - 0.02) < 2e-3
    for dtype, step in ((Q8_0, 1 / 127.0), (Q4_K, 1 / 15.0)):
        blocks = bench.quantize_synthetic(dtype, w)
        assert blocks.dtype == np.uint8 and blocks.size == oracle.storage_bytes(dtype, 48, 1024)
        back = oracle.dequantize(dtype, blocks, 48, 1024)
        # error of a value: at most about one step of its block's range
        span = np.abs(w).reshape(48, -1, 32).max(axis=2, keepdims=True) * 2
        err = np.abs(back - w).reshape(48, -1, 32)
        assert float((err / span).max()) <= 0.75 * step + 0.02
        assert float(np.abs(back - w).mean()) <= 0.3 * step * float(np.abs(w).max())
    # all-zero input: zero scales, zero output, no NaN
    z = bench.quantize_synthetic(Q4_K, np.zeros((2, 256), np.float32))
    assert not np.any(oracle.dequantize(Q4_K, z, 2, 256))
    assert bench.make_blocks(Q4_K, 40, 256, 1, pool_rows=16).size == oracle.storage_bytes(Q4_K, 40, 256)
