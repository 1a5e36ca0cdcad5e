"""ctypes binding of the C oracle (oracle/qmm_oracle.c).

TEST INFRASTRUCTURE ONLY: the product package never imports this module.  Each
function forwards to the C restatement of candle-core 0.10.2's scalar CPU path;
see the header of qmm_oracle.c for what pins each of them.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_qmm.so")

GGML_Q8_0 = 8
GGML_Q4_K = 12
GGML_Q6_K = 14  # dequantize and matmul; no quantizer (tests build Q6_K blocks directly)
BLOCK_SIZE = {GGML_Q8_0: 32, GGML_Q4_K: 256, GGML_Q6_K: 256}
TYPE_SIZE = {GGML_Q8_0: 34, GGML_Q4_K: 144, GGML_Q6_K: 210}
# activation-side ("vec dot") block of each weight type
ACT_BLOCK_SIZE = {GGML_Q8_0: 32, GGML_Q4_K: 256, GGML_Q6_K: 256}
ACT_TYPE_SIZE = {GGML_Q8_0: 34, GGML_Q4_K: 292, GGML_Q6_K: 292}


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it (gcc, -ffp-contract=off)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle_qmm.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        i64, f32p, vp = C.c_int64, C.POINTER(C.c_float), C.c_void_p
        L.oracle_f16_to_f32.restype = C.c_float
        L.oracle_f16_to_f32.argtypes = [C.c_uint16]
        L.oracle_f32_to_f16.restype = C.c_uint16
        L.oracle_f32_to_f16.argtypes = [C.c_float]
        L.oracle_storage_bytes.restype = i64
        L.oracle_storage_bytes.argtypes = [C.c_int, i64, i64]
        L.oracle_qmatmul.restype = C.c_int
        L.oracle_qmatmul.argtypes = [C.c_int, i64, i64, i64, vp, vp, vp]
        L.oracle_quantize.restype = C.c_int
        L.oracle_quantize.argtypes = [C.c_int, i64, i64, vp, vp]
        L.oracle_dequantize.restype = C.c_int
        L.oracle_dequantize.argtypes = [C.c_int, i64, i64, vp, vp]
        L.oracle_quantize_activations.restype = C.c_int
        L.oracle_quantize_activations.argtypes = [C.c_int, i64, i64, vp, vp]
        L.oracle_moe_route.restype = None
        L.oracle_moe_route.argtypes = [vp, i64, C.c_int, C.c_int, vp, vp]
        L.oracle_moe_sort.restype = None
        L.oracle_moe_sort.argtypes = [vp, i64, C.c_int, C.c_int, vp, vp]
        L.oracle_moe_forward.restype = C.c_int
        L.oracle_moe_forward.argtypes = [C.c_int, i64, C.c_int, C.c_int, i64, i64,
                                         vp, vp, vp, vp, vp, vp, vp]
        L.oracle_moe_forward_mixed.restype = C.c_int
        L.oracle_moe_forward_mixed.argtypes = [C.c_int, C.c_int, i64, C.c_int, C.c_int, i64, i64,
                                               vp, vp, vp, vp, vp, vp, vp]
        L.oracle_fill_normal.restype = None
        L.oracle_fill_normal.argtypes = [C.c_uint64, i64, i64, C.c_float, C.c_float, vp]
        f32 = C.c_float
        L.oracle_rms_norm.restype = None
        L.oracle_rms_norm.argtypes = [vp, vp, i64, i64, f32, vp]
        L.oracle_qk_rms_norm.restype = None
        L.oracle_qk_rms_norm.argtypes = [vp, vp, vp, i64, i64, i64, f32, vp, vp]
        L.oracle_rope_pair_bshd.restype = None
        L.oracle_rope_pair_bshd.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, vp, vp]
        L.oracle_argmax.restype = None
        L.oracle_argmax.argtypes = [vp, i64, i64, vp]
        L.oracle_decode_gqa_attention.restype = C.c_int
        L.oracle_decode_gqa_attention.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, f32, vp]
        L.oracle_make_qkx1_quants.restype = None
        L.oracle_make_qkx1_quants.argtypes = [C.c_int, C.c_int, vp, C.c_int, vp, vp]
        L.oracle_get_scale_min_k4.restype = None
        L.oracle_get_scale_min_k4.argtypes = [C.c_int, vp, vp, vp]
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def storage_bytes(dtype: int, rows: int, cols: int) -> int:
    """`quantized_storage_bytes` (qwen3/core.rs:891-909); -1 when not divisible."""
    return int(lib().oracle_storage_bytes(dtype, rows, cols))


def f16_to_f32(bits: int) -> float:
    return float(lib().oracle_f16_to_f32(bits))


def f32_to_f16(v: float) -> int:
    return int(lib().oracle_f32_to_f16(v))


def randn(seed: int, shape, mean: float = 0.0, std: float = 1.0, offset: int = 0) -> np.ndarray:
    """Seeded N(mean, std) f32 array from the oracle's counter-based generator."""
    out = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_normal(seed, offset, out.size, mean, std, _ptr(out))
    return out


def quantize(dtype: int, w: np.ndarray) -> np.ndarray:
    """`QTensor::quantize(w, dtype)` -> raw GGUF block bytes, uint8 [rows * bytes_per_row]."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, cols = w.shape
    nbytes = storage_bytes(dtype, rows, cols)
    if nbytes < 0 or cols % BLOCK_SIZE[dtype]:
        raise ValueError("last dim is not a multiple of the block size")
    out = np.empty(nbytes, dtype=np.uint8)
    rc = lib().oracle_quantize(dtype, rows, cols, _ptr(w), _ptr(out))
    if rc:
        raise ValueError("oracle_quantize rejected the shape")
    return out


def make_qkx1_quants(x: np.ndarray, nmax: int = 15, ntry: int = 5):
    """The Q4_K sub-block scale search -> (scale, -min) as f32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(2, dtype=np.float32)
    lib().oracle_make_qkx1_quants(nmax, ntry, _ptr(x), x.size, out.ctypes.data, out.ctypes.data + 4)
    return out[0], out[1]


def dequantize(dtype: int, blocks: np.ndarray, rows: int, cols: int) -> np.ndarray:
    """`QTensor::dequantize` -> f32 [rows, cols]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    assert blocks.size == storage_bytes(dtype, rows, cols)
    out = np.empty((rows, cols), dtype=np.float32)
    rc = lib().oracle_dequantize(dtype, rows, cols, _ptr(blocks), _ptr(out))
    if rc:
        raise ValueError("oracle_dequantize rejected the shape")
    return out


def quantize_activations(weight_dtype: int, x: np.ndarray) -> np.ndarray:
    """Rows of x quantized to the weight type's dot type (Q8_0 -> Q8_0, Q4_K -> Q8_K)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    nb = k // ACT_BLOCK_SIZE[weight_dtype]
    out = np.zeros(m * nb * ACT_TYPE_SIZE[weight_dtype], dtype=np.uint8)
    rc = lib().oracle_quantize_activations(weight_dtype, m, k, _ptr(x), _ptr(out))
    if rc:
        raise ValueError("oracle_quantize_activations rejected the shape")
    return out


def qmatmul(dtype: int, x: np.ndarray, blocks: np.ndarray, n: int) -> np.ndarray:
    """`QMatMul::forward` on CPU: x [m, k] f32, weight [n, k] blocks -> y [m, n] f32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    assert blocks.size == storage_bytes(dtype, n, k), "weight byte count does not match [n, k]"
    y = np.empty((m, n), dtype=np.float32)
    rc = lib().oracle_qmatmul(dtype, m, k, n, _ptr(x), _ptr(blocks), _ptr(y))
    if rc:
        raise ValueError("oracle_qmatmul rejected the shape")
    return y


def moe_route(logits: np.ndarray, top_k: int):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = logits.shape
    ids = np.empty((T, top_k), dtype=np.int32)
    wts = np.empty((T, top_k), dtype=np.float32)
    lib().oracle_moe_route(_ptr(logits), T, E, top_k, _ptr(ids), _ptr(wts))
    return ids, wts


def moe_sort(ids: np.ndarray, n_experts: int):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    T, top_k = ids.shape
    perm = np.empty(T * top_k, dtype=np.int32)
    offsets = np.empty(n_experts + 1, dtype=np.int32)
    lib().oracle_moe_sort(_ptr(ids), T, top_k, n_experts, _ptr(perm), _ptr(offsets))
    return perm, offsets


def moe_forward(dtype: int, x: np.ndarray, ids: np.ndarray, wts: np.ndarray, gate: np.ndarray,
                up: np.ndarray, down: np.ndarray, n_experts: int, inter: int, down_dtype: int | None = None) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    T, hidden = x.shape
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    wts = np.ascontiguousarray(wts, dtype=np.float32)
    top_k = ids.shape[1]
    out = np.empty((T, hidden), dtype=np.float32)
    rc = lib().oracle_moe_forward_mixed(dtype, dtype if down_dtype is None else down_dtype, T, n_experts, top_k,
                                        hidden, inter, _ptr(x), _ptr(ids), _ptr(wts), _ptr(gate), _ptr(up),
                                        _ptr(down), _ptr(out))
    if rc:
        raise ValueError("oracle_moe_forward rejected the shape")
    return out


# ---- decode-step neighbours (decode_ops_oracle.c) ---------------------------------------

def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """`try_fused_rms_norm`: x [..., hidden], weight [hidden]."""
    x, weight = _f32(x), _f32(weight)
    out = np.empty_like(x)
    hidden = x.shape[-1]
    lib().oracle_rms_norm(_ptr(x), _ptr(weight), x.size // hidden, hidden, eps, _ptr(out))
    return out


def qk_rms_norm(q: np.ndarray, k: np.ndarray, qk_weight: np.ndarray, eps: float):
    """`try_fused_qk_rms_norm`: q, k [..., head_dim], qk_weight [2 * head_dim]."""
    q, k, qk_weight = _f32(q), _f32(k), _f32(qk_weight)
    d = q.shape[-1]
    qo, ko = np.empty_like(q), np.empty_like(k)
    lib().oracle_qk_rms_norm(_ptr(q), _ptr(k), _ptr(qk_weight), q.size // d, k.size // d, d, eps, _ptr(qo), _ptr(ko))
    return qo, ko


def rope_pair_bshd(q: np.ndarray, k: np.ndarray, cos_sin: np.ndarray):
    """`try_fused_rope_pair_bshd`: q [b, s, hq, d], k [b, s, hk, d], cos_sin [s, d]."""
    q, k, cos_sin = _f32(q), _f32(k), _f32(cos_sin)
    b, s, hq, d = q.shape
    qo, ko = np.empty_like(q), np.empty_like(k)
    lib().oracle_rope_pair_bshd(_ptr(q), _ptr(k), _ptr(cos_sin), b, s, hq, k.shape[2], d, _ptr(qo), _ptr(ko))
    return qo, ko


def decode_gqa_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, kv_len: int, scale: float) -> np.ndarray:
    """`try_fused_decode_gqa_attention_with_kv_len`: q [1, heads, 1, d], k / v [1, kv_heads, capacity, d]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    _, heads, _, d = q.shape
    _, kv_heads, cap, _ = k.shape
    out = np.empty_like(q)
    rc = lib().oracle_decode_gqa_attention(_ptr(q), _ptr(k), _ptr(v), heads, kv_heads, d, kv_len, cap, scale, _ptr(out))
    if rc:
        raise ValueError("oracle_decode_gqa_attention rejected the shape")
    return out


def argmax(x: np.ndarray) -> np.ndarray:
    """First index of each row's maximum, uint32 [rows]."""
    x = _f32(x)
    n = x.shape[-1]
    out = np.empty(x.size // n, dtype=np.uint32)
    lib().oracle_argmax(_ptr(x), x.size // n, n, _ptr(out))
    return out.reshape(x.shape[:-1])
