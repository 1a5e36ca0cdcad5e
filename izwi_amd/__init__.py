"""izwi_amd: MI355X-native quantized linear layer (Candle ``QMatMul`` forward).

The package is a thin host-side mirror of the reference's operator interface
(``QTensor`` / ``QMatMul`` / ``Qwen3Projection``) over the C ABI of
``libizwi_qmm.so`` (include/izwi_qmm.h).  All arithmetic runs in hand-written
HIP kernels for gfx950; there is no CPU or PyTorch fallback: if the library is
missing or no GPU is present, calls raise.
"""
from .capi import QmmError, lib, library_path  # noqa: F401
from .decode_ops import (  # noqa: F401
    argmax,
    decode_attention_step,
    qk_norm_rope_append,
    try_fused_decode_gqa_attention,
    try_fused_decode_gqa_attention_with_kv_len,
    try_fused_qk_rms_norm,
    try_fused_rms_norm,
    try_fused_rope_pair_bshd,
)
from .gguf import GgufLoader, GgufMmapMode, GgufModelInfo, GgufReaderKind, is_gguf_file, resolve_gguf_mmap_mode  # noqa: F401
from .qmatmul import (  # noqa: F401
    ActivationRecords,
    DecodeChain,
    GgmlDType,
    MoeExperts,
    QMatMul,
    QTensor,
    QuantizedEmbedding,
    Qwen3GateUpProjection,
    Qwen3Mlp,
    Qwen3Projection,
    Qwen3QkvProjection,
    asr_profile_diagnostics,
    forward_group,
    get_prefill_form,
    moe_route,
    moe_sort,
    packed_qmatmul_from_qtensors,
    profile_snapshot,
    quantize_activations,
    quantized_storage_bytes,
    set_prefill_form,
)
