"""Independent numpy restatements used to pin the C oracle (tests only).

These are written from the public GGUF block formats, vectorised and with
numpy.float16 doing the f16 work, so a slip in the C oracle's loops, indices
or f16 conversion does not repeat here.
"""
import numpy as np


def q8_0_fields(blocks: np.ndarray):
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, 34)
    d = b[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    q = b[:, 2:].copy().view(np.int8)
    return d, q


def dequant_q8_0(blocks: np.ndarray, rows: int, cols: int) -> np.ndarray:
    d, q = q8_0_fields(blocks)
    return (q.astype(np.float32) * d[:, None]).reshape(rows, cols)


def q4_k_fields(blocks: np.ndarray):
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32).reshape(-1)
    s = b[:, 4:16].astype(np.uint8)
    sc = np.empty((b.shape[0], 8), dtype=np.uint8)
    mn = np.empty((b.shape[0], 8), dtype=np.uint8)
    sc[:, :4] = s[:, 0:4] & 63
    mn[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    qs = b[:, 16:]
    # element order: per 64-group g, 32 low nibbles of qs[32g:32g+32] then their high nibbles
    qg = qs.reshape(-1, 4, 32)
    q = np.stack([qg & 0x0F, qg >> 4], axis=2).reshape(-1, 8, 32)  # [blk, sub-block, 32]
    return d, dmin, sc, mn, q


def dequant_q4_k(blocks: np.ndarray, rows: int, cols: int) -> np.ndarray:
    d, dmin, sc, mn, q = q4_k_fields(blocks)
    d1 = d[:, None] * sc.astype(np.float32)          # one rounding
    m1 = dmin[:, None] * mn.astype(np.float32)       # one rounding
    y = d1[:, :, None] * q.astype(np.float32)        # one rounding
    y = y - m1[:, :, None]                           # one rounding
    return y.astype(np.float32).reshape(rows, cols)


def q6_k_fields(blocks: np.ndarray):
    """Q6_K blocks (ql[128], qh[64], int8 scales[16], f16 d = 210 B) -> (d f32 [blk], scales int8
    [blk, 16], q int32 [blk, 256] in element order, already minus 32), from the public block format:
    element 128 h + 32 g + l of a block (g < 4, l < 32) takes nibble g // 2 of ql[64 h + 32 (g % 2) + l]
    and bits 2 g, 2 g + 1 of qh[32 h + l]; scale j belongs to the elements 16 j .. 16 j + 15."""
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, 210)
    ql = b[:, :128].reshape(-1, 2, 2, 32)           # [blk, half, which 32 bytes, l]
    qh = b[:, 128:192].reshape(-1, 2, 32)           # [blk, half, l]
    sc = b[:, 192:208].view(np.int8)
    d = b[:, 208:210].copy().view(np.float16).astype(np.float32).reshape(-1)
    lo = np.stack([ql[:, :, 0] & 0xF, ql[:, :, 1] & 0xF, ql[:, :, 0] >> 4, ql[:, :, 1] >> 4], axis=2)
    hi = np.stack([(qh >> (2 * g)) & 3 for g in range(4)], axis=2)
    q = (lo | (hi << 4)).astype(np.int32) - 32       # [blk, half, g, l]
    return d, sc, q.reshape(-1, 256)


def dequant_q6_k(blocks: np.ndarray, rows: int, cols: int) -> np.ndarray:
    d, sc, q = q6_k_fields(blocks)
    scale = np.repeat(sc.astype(np.float32), 16, axis=1)                 # [blk, 256]
    ds = (d[:, None] * scale).astype(np.float32)                         # one rounding
    y = (ds * q.astype(np.float32)).astype(np.float32)                   # one rounding
    return y.reshape(rows, cols)


def random_q6_k_blocks(seed: int, rows: int, cols: int, d_scale: float = 1e-3) -> np.ndarray:
    """Random but well-formed Q6_K bytes for a [rows, cols] tensor: every quant and scale value
    occurs, d is a finite positive f16 around d_scale (weights of order 0.02 .. 0.1)."""
    rng = np.random.default_rng(seed)
    nb = rows * cols // 256
    b = rng.integers(0, 256, size=(nb, 210), dtype=np.uint8)
    d = (d_scale * rng.uniform(0.5, 2.0, size=nb)).astype(np.float16)
    b[:, 208:210] = d.view(np.uint8).reshape(nb, 2)
    return b.reshape(-1)


def quant_act_q8_0(x: np.ndarray):
    """Q8_0 activation quantization -> (d as f32 of the f16-rounded scale, int8 q)."""
    xb = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    v = (xb * inv[:, None]).astype(np.float32)
    q = np.clip(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)), -128, 127).astype(np.int8)
    return d.astype(np.float16).astype(np.float32), q


def quant_act_q8_k(x: np.ndarray):
    xb = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, 256)
    idx = np.abs(xb).argmax(axis=1)  # first occurrence of the largest |x|
    mx = xb[np.arange(xb.shape[0]), idx]
    d = np.zeros(xb.shape[0], dtype=np.float32)
    q = np.zeros(xb.shape, dtype=np.int8)
    nz = mx != 0
    iscale = (np.float32(-128.0) / mx[nz]).astype(np.float32)
    v = (xb[nz] * iscale[:, None]).astype(np.float32)
    r = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
    q[nz] = np.minimum(r, 127).astype(np.int8)
    d[nz] = (np.float32(1.0) / iscale).astype(np.float32)
    return d, q


def qmatmul_int(dtype: int, x: np.ndarray, blocks: np.ndarray, n: int) -> np.ndarray:
    """Integer-exact block dots, f64 scaling: what the quantized matmul equals
    before f32 accumulation rounding."""
    m, k = x.shape
    y = np.zeros((m, n), dtype=np.float64)
    if dtype == 8:
        dw, qw = q8_0_fields(blocks)
        dw = dw.reshape(n, k // 32).astype(np.float64)
        qw = qw.reshape(n, k // 32, 32).astype(np.int64)
        for r in range(m):
            dx, qx = quant_act_q8_0(x[r])
            qx = qx.reshape(k // 32, 32).astype(np.int64)
            sumi = np.einsum("nbj,bj->nb", qw, qx)
            y[r] = (sumi * dw * dx.astype(np.float64)[None, :]).sum(axis=1)
        return y
    if dtype == 14:
        nb = k // 256
        d, sc, q = q6_k_fields(blocks)
        d = d.reshape(n, nb).astype(np.float64)
        sc = sc.reshape(n, nb, 16).astype(np.int64)
        q = q.reshape(n, nb, 16, 16).astype(np.int64)
        for r in range(m):
            dx, qx = quant_act_q8_k(x[r])
            qx = qx.reshape(nb, 16, 16).astype(np.int64)
            dots = np.einsum("nbsj,bsj->nbs", q, qx)
            y[r] = ((dots * sc).sum(axis=2) * d * dx.astype(np.float64)[None, :]).sum(axis=1)
        return y
    d, dmin, sc, mn, q = q4_k_fields(blocks)
    nb = k // 256
    d = d.reshape(n, nb).astype(np.float64)
    dmin = dmin.reshape(n, nb).astype(np.float64)
    sc = sc.reshape(n, nb, 8).astype(np.int64)
    mn = mn.reshape(n, nb, 8).astype(np.int64)
    q = q.reshape(n, nb, 8, 32).astype(np.int64)
    for r in range(m):
        dx, qx = quant_act_q8_k(x[r])
        qx = qx.reshape(nb, 8, 32).astype(np.int64)
        dots = np.einsum("nbsj,bsj->nbs", q, qx)
        bsum = qx.sum(axis=2)
        pos = (dots * sc).sum(axis=2) * d * dx.astype(np.float64)[None, :]
        neg = (mn * bsum[None]).sum(axis=2) * dmin * dx.astype(np.float64)[None, :]
        y[r] = (pos - neg).sum(axis=1)
    return y
