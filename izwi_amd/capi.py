"""ctypes binding of include/izwi_qmm.h and include/izwi_gguf.h (one prototype per exported symbol)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

OK = 0
DEVICE, HOST = 0, 1
OUT_F32, OUT_BF16 = 0, 1
LARGE_M_BF16, LARGE_M_INT8 = 0, 1  # izwi_qmm_large_m


class QmmError(RuntimeError):
    """A failing izwi_qmm call; mirrors the reference's Error::InferenceError."""

    def __init__(self, code: int, message: str):
        super().__init__(f"izwi_qmm error {code}: {message}")
        self.code = code
        self.message = message


class WeightInfo(C.Structure):
    _fields_ = [("ggml_dtype", C.c_int32), ("n_stacked", C.c_int32), ("n", C.c_int64),
                ("k", C.c_int64), ("nbytes", C.c_uint64), ("device", C.c_int32),
                ("reserved", C.c_int32)]


class ProfileSnapshot(C.Structure):
    _fields_ = [(name, C.c_uint64) for name in (
        "qmatmul_calls", "qmatmul_ns", "qmatmul_input_casts", "qmatmul_input_cast_ns",
        "qmatmul_output_casts", "qmatmul_output_cast_ns", "lm_head_calls", "lm_head_ns",
        "silu_mul_fused_calls", "silu_mul_fallback_calls")]


class GgufTensorInfo(C.Structure):
    """izwi_gguf_tensor_info (include/izwi_gguf.h)."""
    _fields_ = [("ggml_dtype", C.c_int32), ("n_dims", C.c_int32), ("dims", C.c_int64 * 8),
                ("offset", C.c_uint64), ("nbytes", C.c_uint64), ("data", C.c_void_p)]


_i32, _i64, _u64, _vp = C.c_int32, C.c_int64, C.c_uint64, C.c_void_p
_pp = C.POINTER(C.c_void_p)
_cpp = C.POINTER(C.c_char_p)

class ChainStep(C.Structure):
    """izwi_qmm_chain_step"""
    _fields_ = [("weights", C.c_void_p * 4), ("n_weights", C.c_int32), ("reserved", C.c_int32),
                ("x", C.c_void_p), ("ys", C.c_void_p * 4)]


# name -> (restype, argtypes); must list every symbol include/izwi_qmm.h and include/izwi_gguf.h declare
PROTOTYPES = {
    "izwi_qmm_abi_version": (C.c_int, []),
    "izwi_qmm_init": (C.c_int, [C.c_int]),
    "izwi_qmm_last_error": (C.c_char_p, []),
    "izwi_qmm_storage_bytes": (C.c_int, [C.c_int, _i64, _i64, C.POINTER(_u64)]),
    "izwi_qmm_weight_create": (C.c_int, [C.c_int, _i64, _i64, _vp, _u64, C.c_int, _pp]),
    "izwi_qmm_weight_create_packed": (C.c_int, [C.c_int, _i32, C.POINTER(_i64), _i64, _pp,
                                                C.POINTER(_u64), C.c_int, _pp]),
    "izwi_qmm_weight_create_stacked": (C.c_int, [C.c_int, _i32, _i64, _i64, _vp, _u64, C.c_int, _pp]),
    "izwi_qmm_weight_destroy": (None, [_vp]),
    "izwi_qmm_weight_get_info": (C.c_int, [_vp, C.POINTER(WeightInfo)]),
    "izwi_qmm_weight_data": (C.c_int, [_vp, _vp, _u64, C.c_int, _vp]),
    "izwi_qmm_dequantize_f32": (C.c_int, [_vp, _vp, C.c_int, _vp]),
    "izwi_qmm_dequantize_rows": (C.c_int, [_vp, _vp, _i64, C.c_int, _vp, C.c_int, C.c_int, _vp]),
    "izwi_qmm_forward_f32": (C.c_int, [_vp, _vp, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_records_bytes": (_u64, [C.c_int, _i64, _i64]),
    "izwi_qmm_quantize_records_f32": (C.c_int, [C.c_int, _vp, _i64, _i64, _vp, _vp]),
    "izwi_qmm_silu_mul_quantize_records_f32": (C.c_int, [C.c_int, _vp, _vp, _i64, _i64, _vp, _vp]),
    "izwi_qmm_forward_group_records_f32": (C.c_int, [_vp, _i32, _vp, _i64, _vp, _vp]),
    "izwi_rms_norm_quantize_records_f32": (C.c_int, [C.c_int, _vp, _vp, _i64, _i64, C.c_float, _vp, _vp]),
    "izwi_qmm_chain_create": (C.c_int, [_vp, _i32, _pp]),
    "izwi_qmm_chain_destroy": (None, [_vp]),
    "izwi_qmm_chain_run": (C.c_int, [_vp, _vp]),
    "izwi_qmm_chain_status": (C.c_int, [_vp, _vp]),
    "izwi_qmm_chain_set_spin_limit": (C.c_int, [_vp, C.c_uint32]),
    "izwi_qmm_forward_rows_f32": (C.c_int, [_vp, _vp, _i64, _vp, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_f32_noalloc": (C.c_int, [_vp, _vp, _i64, _vp, _vp]),
    "izwi_qmm_quantize_weights_f32": (C.c_int, [C.c_int, _vp, _i64, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_group_f32": (C.c_int, [_vp, _i32, _vp, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_group_bf16": (C.c_int, [_vp, _i32, _vp, _i64, _vp, C.c_int, C.c_int, _vp]),
    "izwi_qmm_forward_gate_up_silu_f32": (C.c_int, [_vp, _vp, _vp, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_mlp_forward_f32": (C.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_normed_f32": (C.c_int, [_vp, _vp, _i64, _vp, C.c_float, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_group_normed_f32": (C.c_int, [_vp, _i32, _vp, _i64, _vp, C.c_float, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_gate_up_silu_normed_f32": (C.c_int, [_vp, _vp, _vp, _i64, _vp, C.c_float, _vp, C.c_int, _vp]),
    "izwi_qmm_forward_bf16": (C.c_int, [_vp, _vp, _i64, _vp, C.c_int, C.c_int, _vp]),
    "izwi_qmm_forward_fused": (C.c_int, [_vp, _vp, C.c_int, _i64, _vp, _vp, C.c_int, C.c_int, _vp]),
    "izwi_qmm_quantize_activations": (C.c_int, [C.c_int, _vp, _i64, _i64, _vp, C.c_int, _vp]),
    "izwi_rms_norm_f32": (C.c_int, [_vp, _vp, _i64, _i64, C.c_float, _vp, C.c_int, _vp]),
    "izwi_qk_rms_norm_f32": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, C.c_float, _vp, _vp, C.c_int, _vp]),
    "izwi_rope_pair_bshd_f32": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, C.c_int, _vp]),
    "izwi_rms_norm_f16": (C.c_int, [_vp, _vp, _i64, _i64, C.c_float, _vp, C.c_int, _vp]),
    "izwi_qk_rms_norm_f16": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, C.c_float, _vp, _vp, C.c_int, _vp]),
    "izwi_rope_pair_bshd_f16": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, C.c_int, _vp]),
    "izwi_decode_gqa_attention_f16": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float, _vp,
                                                C.c_int, _vp]),
    "izwi_argmax_f32": (C.c_int, [_vp, _i64, _i64, _vp, C.c_int, _vp]),
    "izwi_qk_norm_rope_append_f32": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, C.c_float, _vp, _vp, _vp,
                                               _i64, _i64, _vp]),
    "izwi_decode_attention_step_f32": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, C.c_float, _vp, _vp, _i64,
                                                 _i64, C.c_float, _vp, _vp]),
    "izwi_decode_gqa_attention_f32": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float, _vp,
                                                C.c_int, _vp]),
    "izwi_moe_route": (C.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, C.c_int, _vp]),
    "izwi_moe_sort": (C.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, C.c_int, _vp]),
    "izwi_moe_layer_f32": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _vp, _vp, _vp, C.c_int, _vp]),
    "izwi_moe_forward_f32": (C.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _i32, _vp, _vp, _vp,
                                       C.c_int, _vp]),
    "izwi_qmm_set_large_m_arithmetic": (C.c_int, [C.c_int]),
    "izwi_qmm_get_large_m_arithmetic": (C.c_int, []),
    "izwi_qmm_set_prefill_form": (C.c_int, [C.c_int]),
    "izwi_qmm_get_prefill_form": (C.c_int, []),
    "izwi_qmm_set_moe_expert_form": (C.c_int, [C.c_int]),
    "izwi_qmm_scratch_reserve": (C.c_int, [_u64, _vp]),
    "izwi_qmm_profile_enable": (C.c_int, [C.c_int]),
    "izwi_qmm_profile_enabled": (C.c_int, []),
    "izwi_qmm_profile_snapshot_get": (C.c_int, [C.POINTER(ProfileSnapshot)]),
    "izwi_qmm_profile_reset": (C.c_int, []),
    "izwi_qmm_profile_argmax_get": (C.c_int, [C.POINTER(_u64), C.POINTER(_u64)]),
    "izwi_qmm_weight_set_lm_head": (C.c_int, [_vp, C.c_int]),
    # include/izwi_gguf.h
    "izwi_gguf_is_gguf_file": (C.c_int, [C.c_char_p]),
    "izwi_gguf_open": (C.c_int, [C.c_char_p, _pp]),
    "izwi_gguf_close": (None, [_vp]),
    "izwi_gguf_open_with_mode": (C.c_int, [C.c_char_p, C.c_int, _pp]),
    "izwi_gguf_parse_mmap_mode": (C.c_int, [C.c_char_p]),
    "izwi_gguf_resolve_mmap_mode": (C.c_int, [C.c_int]),
    "izwi_gguf_reader_kind": (C.c_int, [_vp]),
    "izwi_gguf_header": (C.c_int, [_vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(_u64)]),
    "izwi_gguf_tensor_count": (_i64, [_vp]),
    "izwi_gguf_tensor_name": (C.c_int, [_vp, _i64, _cpp]),
    "izwi_gguf_tensor_info_get": (C.c_int, [_vp, C.c_char_p, C.POINTER(GgufTensorInfo)]),
    "izwi_gguf_metadata_count": (_i64, [_vp]),
    "izwi_gguf_metadata_key": (C.c_int, [_vp, _i64, _cpp]),
    "izwi_gguf_metadata_type": (C.c_int, [_vp, C.c_char_p]),
    "izwi_gguf_metadata_string": (C.c_int, [_vp, C.c_char_p, _pp, C.POINTER(_u64)]),
    "izwi_gguf_metadata_u64": (C.c_int, [_vp, C.c_char_p, C.POINTER(_u64)]),
    "izwi_gguf_metadata_f64": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_double)]),
    "izwi_gguf_metadata_array": (C.c_int, [_vp, C.c_char_p, C.POINTER(_i32), C.POINTER(_u64), _pp]),
    "izwi_gguf_metadata_array_string": (C.c_int, [_vp, C.c_char_p, _u64, _pp, C.POINTER(_u64)]),
    "izwi_gguf_load_weight": (C.c_int, [_vp, C.c_char_p, _pp]),
    "izwi_gguf_load_packed": (C.c_int, [_vp, _cpp, _i32, _pp]),
    "izwi_gguf_load_tensor_f32": (C.c_int, [_vp, C.c_char_p, _vp, _u64, C.c_int, _vp]),
}

_lib = None


def library_path() -> str:
    return os.path.join(_HERE, "libizwi_qmm.so")


def lib() -> C.CDLL:
    """Loads the in-tree HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise QmmError(-4, f"{path} is missing: build it with __graft_entry__.build() "
                               "(make -C izwi_amd/csrc); there is no fallback path")
        L = C.CDLL(path)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != OK:
        raise QmmError(rc, lib().izwi_qmm_last_error().decode("utf-8", "replace"))
