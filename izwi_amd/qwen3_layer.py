"""One decoder layer of izwi-core's Qwen3 model at one token, composed from the library's calls.

Mirror of `Qwen3Layer::forward` (qwen3/core.rs:1863-1881) with `Qwen3Attention::forward`'s
single-token path (core.rs:1446-1575: q/k/v projections, per-head q/k norm, rotary embedding, cache
append, grouped-query attention, output projection) and `Qwen3Mlp::forward` (core.rs:1786-1798),
f32 activations.  Every arithmetic step is one library call; torch only appends the new key /
value rows to the caches in the unfused form and owns the tensors.  Per layer: 6 kernel launches
(the two RMSNorms ride in the projection launches behind them; q/k norm, rotary and the cache
append ride in the attention launch), or 12 with the reference's separate hooks and two copies,
where the reference's eager path issues one per operator.
"""
from __future__ import annotations

import torch

from .decode_ops import (decode_attention_step, qk_norm_rope_append, try_fused_decode_gqa_attention_with_kv_len, try_fused_qk_rms_norm,
                         try_fused_rms_norm, try_fused_rope_pair_bshd)
from .qmatmul import QMatMul, Qwen3GateUpProjection, forward_group


class Qwen3DecodeLayer:
    def __init__(self, input_layernorm: torch.Tensor, post_attention_layernorm: torch.Tensor, q_proj: QMatMul,
                 k_proj: QMatMul, v_proj: QMatMul, qk_norm_weight: torch.Tensor, o_proj: QMatMul, gate_proj: QMatMul,
                 up_proj: QMatMul, down_proj: QMatMul, num_heads: int, num_kv_heads: int, head_dim: int,
                 rms_norm_eps: float = 1e-6, fuse_prep: bool = True, fuse_norm: bool = True, fuse_step: bool = True):
        self.w_in, self.w_post, self.qk_w = input_layernorm, post_attention_layernorm, qk_norm_weight
        self.qkv = (q_proj, k_proj, v_proj)
        self.o_proj, self.down_proj = o_proj, down_proj
        self.gate_up = Qwen3GateUpProjection.new_separate(gate_proj, up_proj)
        self.heads, self.kv_heads, self.d, self.eps = num_heads, num_kv_heads, head_dim, rms_norm_eps
        self.fuse_prep = fuse_prep  # q/k norm, rotary and cache append as one launch instead of four
        self.fuse_norm = fuse_norm  # the two RMSNorms inside the projection launches that follow them
        self.fuse_step = fuse_step  # q/k norm, rotary and cache append inside the attention launch

    def forward(self, x: torch.Tensor, cos_sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                pos: int) -> torch.Tensor:
        """x [1, hidden] f32; cos_sin [1, head_dim] for position `pos`; caches [1, kv_heads, capacity,
        head_dim] holding positions < pos.  Returns the layer's output [1, hidden]; the caches gain
        position `pos`."""
        h, kv, d = self.heads, self.kv_heads, self.d
        if self.fuse_norm:  # input_layernorm inside the q|k|v launch
            q, k, v = forward_group(self.qkv, x, norm_weight=self.w_in, eps=self.eps)
        else:
            q, k, v = forward_group(self.qkv, try_fused_rms_norm(x, self.w_in, self.eps))
        if self.fuse_prep and self.fuse_step:
            attn = decode_attention_step(q, k, v, self.qk_w, cos_sin, k_cache, v_cache, pos, self.eps, d ** -0.5)
        else:
            if self.fuse_prep:
                q4 = qk_norm_rope_append(q, k, v, self.qk_w, cos_sin, k_cache, v_cache, pos, self.eps)
            else:  # the same steps as the reference's separate hooks
                q4, k4 = try_fused_qk_rms_norm(q.view(1, 1, h, d), k.view(1, 1, kv, d), self.qk_w, self.eps)
                q4, k4 = try_fused_rope_pair_bshd(q4, k4, cos_sin)
                k_cache[0, :, pos] = k4.view(kv, d)
                v_cache[0, :, pos] = v.view(kv, d)
            attn = try_fused_decode_gqa_attention_with_kv_len(q4.view(1, h, 1, d), k_cache, v_cache, h, kv, d, pos + 1,
                                                              d ** -0.5)
        x = self.o_proj.forward_fused(attn.view(1, h * d), residual=x)       # x + o_proj(attn)
        if self.fuse_norm:  # post_attention_layernorm inside the gate|up launch
            hidden = self.gate_up.forward_silu_mul(x, norm_weight=self.w_post, eps=self.eps)
        else:
            hidden = self.gate_up.forward_silu_mul(try_fused_rms_norm(x, self.w_post, self.eps))  # silu(gate) * up
        return self.down_proj.forward_fused(hidden, residual=x)              # x + down_proj(hidden)
