"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and argument errors that need no GPU are reported as errors."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    names = set()
    for header in ("izwi_qmm.h", "izwi_gguf.h", "izwi_decode_ops.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(izwi_(?:qmm|moe|gguf|rms|qk|rope|decode|argmax)_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def capi():
    from izwi_amd import capi as c
    if not os.path.exists(c.library_path()):
        import __graft_entry__
        __graft_entry__.build()
    return c


def test_library_exports_every_declared_symbol(capi):
    L = C.CDLL(capi.library_path())
    names = header_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/*.h but not exported"


def test_binding_covers_every_declared_symbol(capi):
    assert sorted(capi.PROTOTYPES) == header_symbols()


def test_abi_version_and_storage_bytes_rule(capi):
    L = capi.lib()
    assert L.izwi_qmm_abi_version() == 1
    out = C.c_uint64()
    # qwen3/core.rs:891-909
    assert L.izwi_qmm_storage_bytes(8, 3072, 1024, C.byref(out)) == 0 and out.value == 3_342_336
    assert L.izwi_qmm_storage_bytes(12, 151936, 4096, C.byref(out)) == 0 and out.value == 350_060_544
    assert L.izwi_qmm_storage_bytes(12, 3, 100, C.byref(out)) == -1
    assert b"not divisible by block size 256" in L.izwi_qmm_last_error()
    assert L.izwi_qmm_storage_bytes(14, 4, 256, C.byref(out)) == 0 and out.value == 4 * 210  # Q6_K
    assert L.izwi_qmm_storage_bytes(13, 4, 256, C.byref(out)) == -2  # Q5_K: no kernel for it
    assert L.izwi_qmm_storage_bytes(8, -1, 32, C.byref(out)) == -1


def test_errors_without_touching_the_gpu(capi):
    L = capi.lib()
    h = C.c_void_p()
    # byte count mismatch is caught before any device work
    assert L.izwi_qmm_weight_create(8, 2, 32, None, 10, capi.HOST, C.byref(h)) == -1
    assert b"expected 68" in L.izwi_qmm_last_error()
    # empty packed group, as packed_qmatmul_from_qtensors rejects it
    assert L.izwi_qmm_weight_create_packed(8, 0, None, 32, None, None, capi.HOST, C.byref(h)) == -1
    assert b"Cannot pack empty" in L.izwi_qmm_last_error()
    assert L.izwi_qmm_forward_f32(None, None, 1, None, capi.DEVICE, None) == -1
    assert L.izwi_moe_route(None, 4, 128, 200, None, None, capi.DEVICE, None) == -1
    L.izwi_qmm_weight_destroy(None)  # NULL is ignored


def test_no_gpu_means_loud_failure_not_fallback(capi):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import numpy as np
    L = capi.lib()
    h = C.c_void_p()
    blocks = np.zeros(68, dtype=np.uint8)
    rc = L.izwi_qmm_weight_create(8, 2, 32, blocks.ctypes.data, 68, capi.HOST, C.byref(h))
    assert rc in (-3, -4) and not h.value
    assert L.izwi_qmm_last_error() != b""


def test_profile_snapshot_fields_match_reference(capi):
    # Qwen3RuntimeProfileSnapshot, qwen3/core.rs:571-582
    names = [n for n, _ in capi.ProfileSnapshot._fields_]
    assert names == ["qmatmul_calls", "qmatmul_ns", "qmatmul_input_casts", "qmatmul_input_cast_ns",
                     "qmatmul_output_casts", "qmatmul_output_cast_ns", "lm_head_calls", "lm_head_ns",
                     "silu_mul_fused_calls", "silu_mul_fallback_calls"]
    L = capi.lib()
    snap = capi.ProfileSnapshot()
    assert L.izwi_qmm_profile_reset() == 0
    assert L.izwi_qmm_profile_snapshot_get(C.byref(snap)) == 0
    assert snap.qmatmul_calls == 0
