"""Host-side mirror of the reference's fused-kernel hooks for the decode step
(crates/izwi-core/src/kernels/mod.rs:109-225): the same names, argument meaning and "return None
when the fused path does not apply" behaviour, over the C ABI of include/izwi_decode_ops.h.

A hook returns None (the caller then runs its own eager operators, as the reference does) when
its preconditions do not hold: f32 or f16 throughout, contiguous, on one GPU, the shapes the reference's wrapper
checks (metal.rs:1921-1945, 1991-2003, 2043-2062, 2141-2172).  When they hold the HIP kernel runs;
a failure inside it raises (there is no silent CPU path)."""
from __future__ import annotations

import torch

from .capi import DEVICE, check, lib
from .qmatmul import _stream_ptr


def _ok(*tensors: torch.Tensor) -> bool:
    """All on one GPU, contiguous, one dtype, f32 or f16 (the hooks' `matches!(dtype, F32 | F16)`)."""
    dev, dt = tensors[0].device, tensors[0].dtype
    return dt in (torch.float32, torch.float16) and all(
        t.is_cuda and t.device == dev and t.dtype == dt and t.is_contiguous() for t in tensors)


def _fn(name: str, t: torch.Tensor):
    return getattr(lib(), f"izwi_{name}_{'f16' if t.dtype == torch.float16 else 'f32'}")


def try_fused_rms_norm(input: torch.Tensor, weight: torch.Tensor, eps: float):  # noqa: A002
    """kernels/mod.rs:141-155: input [..., hidden], weight [hidden] -> x * rsqrt(mean(x^2) + eps) * weight."""
    if input.dim() < 1 or not _ok(input, weight):
        return None
    hidden = input.shape[-1]
    if hidden == 0 or tuple(weight.shape) != (hidden,) or input.numel() == 0:
        return None
    out = torch.empty_like(input)
    check(_fn('rms_norm', input)(input.data_ptr(), weight.data_ptr(), input.numel() // hidden, hidden, eps,
                                  out.data_ptr(), DEVICE, _stream_ptr(input)))
    return out


def try_fused_qk_rms_norm(q: torch.Tensor, k: torch.Tensor, qk_weight: torch.Tensor, eps: float):
    """kernels/mod.rs:109-123: q [b, 1, heads, d], k [b, 1, kv_heads, d], qk_weight [2 d] -> (q_norm, k_norm)."""
    if q.dim() != 4 or k.dim() != 4 or not _ok(q, k, qk_weight):
        return None
    if q.shape[1] != 1 or k.shape[1] != 1 or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
        return None
    d = q.shape[3]
    if d == 0 or tuple(qk_weight.shape) != (2 * d,):
        return None
    q_out, k_out = torch.empty_like(q), torch.empty_like(k)
    check(_fn('qk_rms_norm', q)(q.data_ptr(), k.data_ptr(), qk_weight.data_ptr(), q.numel() // d, k.numel() // d,
                                     d, eps, q_out.data_ptr(), k_out.data_ptr(), DEVICE, _stream_ptr(q)))
    return q_out, k_out


def try_fused_rope_pair_bshd(q: torch.Tensor, k: torch.Tensor, cos_sin: torch.Tensor):
    """kernels/mod.rs:157-171: q [b, s, hq, d], k [b, s, hk, d], cos_sin [s, d] (cos | sin) -> (q_rot, k_rot)."""
    if q.dim() != 4 or k.dim() != 4 or not _ok(q, k, cos_sin):
        return None
    b, s, hq, d = q.shape
    if k.shape[0] != b or k.shape[1] != s or k.shape[3] != d or d == 0 or d % 2 or tuple(cos_sin.shape) != (s, d):
        return None
    q_out, k_out = torch.empty_like(q), torch.empty_like(k)
    check(_fn('rope_pair_bshd', q)(q.data_ptr(), k.data_ptr(), cos_sin.data_ptr(), b, s, hq, k.shape[2], d,
                                        q_out.data_ptr(), k_out.data_ptr(), DEVICE, _stream_ptr(q)))
    return q_out, k_out


def try_fused_decode_gqa_attention_with_kv_len(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_heads: int,
                                               num_kv_heads: int, head_dim: int, kv_len: int, scale: float):
    """kernels/mod.rs:199-225: q [1, heads, 1, d], k / v [1, kv_heads, capacity, d], the first kv_len positions
    count -> [1, heads, 1, d].  No limit on kv_len (the reference's shader stops at 2048)."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or not _ok(q, k, v):
        return None
    if (tuple(q.shape) != (1, num_heads, 1, head_dim) or k.shape[0] != 1 or k.shape[1] != num_kv_heads
            or k.shape[3] != head_dim or tuple(v.shape) != tuple(k.shape) or kv_len == 0 or kv_len > k.shape[2]
            or num_heads == 0 or num_kv_heads == 0 or num_heads % num_kv_heads or head_dim not in (64, 128, 256)):
        return None
    out = torch.empty_like(q)
    check(_fn('decode_gqa_attention', q)(q.data_ptr(), k.data_ptr(), v.data_ptr(), num_heads, num_kv_heads,
                                              head_dim, kv_len, k.shape[2], scale, out.data_ptr(), DEVICE,
                                              _stream_ptr(q)))
    return out


def try_fused_decode_gqa_attention(q, k, v, num_heads: int, num_kv_heads: int, head_dim: int, scale: float):
    """kernels/mod.rs:173-197: all cached positions count."""
    if k.dim() != 4:
        return None
    return try_fused_decode_gqa_attention_with_kv_len(q, k, v, num_heads, num_kv_heads, head_dim, k.shape[2], scale)


def qk_norm_rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qk_weight: torch.Tensor,
                        cos_sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: int, eps: float):
    """apply_qk_norm_pair + apply_rope_pair + cache append of Qwen3Attention::forward for one token
    (qwen3/core.rs:1464-1575) in one launch.  q [heads * d], k / v [kv_heads * d] (any shape with that many
    elements), caches [1, kv_heads, capacity, d].  Returns the normed, rotated q as [1, heads, 1, d]; the caches
    gain position `pos`."""
    from .capi import QmmError
    if (not _ok(q, k, v, qk_weight, cos_sin, k_cache, v_cache) or q.dtype != torch.float32 or k_cache.dim() != 4
            or tuple(v_cache.shape) != tuple(k_cache.shape)):
        raise QmmError(-1, "qk_norm_rope_append: contiguous f32 CUDA tensors on one device expected")
    _, kv_heads, cap, d = k_cache.shape
    heads = q.numel() // d
    if (q.numel() != heads * d or k.numel() != kv_heads * d or v.numel() != kv_heads * d or qk_weight.numel() != 2 * d
            or cos_sin.numel() != d):
        raise QmmError(-1, "qk_norm_rope_append: shapes do not match the caches")
    q_out = torch.empty((1, heads, 1, d), dtype=torch.float32, device=q.device)
    check(lib().izwi_qk_norm_rope_append_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), qk_weight.data_ptr(),
                                             cos_sin.data_ptr(), heads, kv_heads, d, eps, q_out.data_ptr(),
                                             k_cache.data_ptr(), v_cache.data_ptr(), cap, pos, _stream_ptr(q)))
    return q_out


def decode_attention_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qk_weight: torch.Tensor,
                          cos_sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: int, eps: float,
                          scale: float) -> torch.Tensor:
    """`qk_norm_rope_append` and the attention over positions 0 .. pos behind it as one call: the attention
    kernel prepares its query heads and the new key itself and appends the new key / value to the caches.
    Arguments as `qk_norm_rope_append`; returns the attention output [1, heads, 1, d]."""
    from .capi import QmmError
    if (not _ok(q, k, v, qk_weight, cos_sin, k_cache, v_cache) or q.dtype != torch.float32 or k_cache.dim() != 4
            or tuple(v_cache.shape) != tuple(k_cache.shape)):
        raise QmmError(-1, "decode_attention_step: contiguous f32 CUDA tensors on one device expected")
    _, kv_heads, cap, d = k_cache.shape
    heads = q.numel() // d
    if (q.numel() != heads * d or k.numel() != kv_heads * d or v.numel() != kv_heads * d or qk_weight.numel() != 2 * d
            or cos_sin.numel() != d):
        raise QmmError(-1, "decode_attention_step: shapes do not match the caches")
    out = torch.empty((1, heads, 1, d), dtype=torch.float32, device=q.device)
    check(lib().izwi_decode_attention_step_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), qk_weight.data_ptr(),
                                               cos_sin.data_ptr(), heads, kv_heads, d, eps, k_cache.data_ptr(),
                                               v_cache.data_ptr(), cap, pos, scale, out.data_ptr(), _stream_ptr(q)))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """`logits.argmax(D::Minus1)` of the greedy samplers (qwen3/chat.rs:574-597): logits [..., n] f32 on the
    GPU -> int32 indices [...] (first index of the maximum), computed on the device."""
    from .capi import QmmError
    if not _ok(logits) or logits.dtype != torch.float32 or logits.dim() < 1 or logits.shape[-1] == 0:
        raise QmmError(-1, "argmax: a contiguous f32 CUDA tensor with a non-empty last dimension expected")
    n = logits.shape[-1]
    out = torch.empty(logits.shape[:-1], dtype=torch.int32, device=logits.device)
    check(lib().izwi_argmax_f32(logits.data_ptr(), logits.numel() // n, n, out.data_ptr(), DEVICE, _stream_ptr(logits)))
    return out
