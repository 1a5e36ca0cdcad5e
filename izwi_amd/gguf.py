"""Host-side mirror of the reference's GGUF loader over include/izwi_gguf.h.

``GgufLoader`` follows crates/izwi-core/src/models/shared/weights/gguf.rs:36-203 name for
name: ``from_path``, ``get_model_info``, ``has_tensor``, ``tensor_shape``, ``load_qtensor``,
``load_tensor``, ``tensor_names``, ``tensor_count``, ``metadata_value``, ``get_metadata_string``,
``get_metadata_u64``; ``is_gguf_file`` is gguf.rs:366-377.  Parsing is done by the C library
(host only, no GPU needed); ``load_qtensor`` / ``load_tensor`` upload to the current HIP device.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import os
import struct
from typing import Dict, List, Optional

import torch

from . import capi
from .capi import DEVICE, HOST, check, lib
from .qmatmul import QMatMul, QTensor, _stream_ptr

# ggml type id -> the name candle-core's GgmlDType prints with {:?}
GGML_TYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1",
                   10: "Q2K", 11: "Q3K", 12: "Q4K", 13: "Q5K", 14: "Q6K", 15: "Q8K", 30: "BF16"}

_SCALAR_FORMATS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q",
                   12: "<d"}
_STRING, _ARRAY = 8, 9


class GgufMmapMode:
    """backends/model_io.rs:13-45."""
    AUTO, ON, OFF = 0, 1, 2
    _NAMES = {0: "auto", 1: "on", 2: "off"}

    @staticmethod
    def parse(raw: str):
        """GgufMmapMode::parse: the mode, or None for the empty string and unknown words."""
        mode = lib().izwi_gguf_parse_mmap_mode(raw.encode("utf-8"))
        return None if mode < 0 else mode

    @classmethod
    def as_str(cls, mode: int) -> str:
        return cls._NAMES[mode]


class GgufReaderKind:
    """backends/model_io.rs:85-89."""
    BUFFERED, MAPPED = 0, 1


def resolve_gguf_mmap_mode(configured=None) -> int:
    """model_io.rs:63-67: the configured mode, else IZWI_GGUF_MMAP, else auto."""
    return lib().izwi_gguf_resolve_mmap_mode(-1 if configured is None else configured)


def is_gguf_file(path) -> bool:
    """gguf.rs:366-377: true if the file starts with the magic bytes "GGUF"."""
    return bool(lib().izwi_gguf_is_gguf_file(os.fsencode(path)))


@dataclasses.dataclass
class GgufModelInfo:
    """gguf.rs:21-33."""
    path: str
    architecture: Optional[str]
    parameter_count: Optional[int]
    quantization: Optional[str]
    metadata: Dict[str, str]


class GgufLoader:
    """gguf.rs:36-203 over the C ABI: one mapped GGUF file."""

    def __init__(self, handle: int, path: str):
        self._h = C.c_void_p(handle)
        self.path = path

    @classmethod
    def from_path(cls, path, mmap_mode=None) -> "GgufLoader":
        """GgufLoader::from_path (gguf.rs:44-70) over `open_gguf_reader_with_mode`
        (model_io.rs:127-160); parse errors raise (ModelLoadError upstream)."""
        h = C.c_void_p()
        check(lib().izwi_gguf_open_with_mode(os.fsencode(path), -1 if mmap_mode is None else mmap_mode, C.byref(h)))
        return cls(h.value, os.fspath(path))

    def reader_kind(self) -> int:
        """GgufReader::kind (model_io.rs:96-103)."""
        return lib().izwi_gguf_reader_kind(self._h)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                lib().izwi_gguf_close(h)
            except Exception:
                pass

    # -- header ---------------------------------------------------------------------------
    def header(self):
        """(version, alignment, offset of the tensor data section)."""
        v, a, o = C.c_uint32(), C.c_uint32(), C.c_uint64()
        check(lib().izwi_gguf_header(self._h, C.byref(v), C.byref(a), C.byref(o)))
        return v.value, a.value, o.value

    # -- tensors --------------------------------------------------------------------------
    def tensor_count(self) -> int:
        return lib().izwi_gguf_tensor_count(self._h)

    def tensor_names(self) -> List[str]:
        out = []
        for i in range(self.tensor_count()):
            p = C.c_char_p()
            check(lib().izwi_gguf_tensor_name(self._h, i, C.byref(p)))
            out.append(p.value.decode("utf-8"))
        return out

    def _info(self, name: str) -> Optional[capi.GgufTensorInfo]:
        info = capi.GgufTensorInfo()
        rc = lib().izwi_gguf_tensor_info_get(self._h, name.encode("utf-8"), C.byref(info))
        return info if rc == capi.OK else None

    def has_tensor(self, name: str) -> bool:
        return self._info(name) is not None

    def tensor_shape(self, name: str) -> Optional[List[int]]:
        info = self._info(name)
        return None if info is None else [info.dims[i] for i in range(info.n_dims)]

    def tensor_dtype(self, name: str) -> Optional[int]:
        """ggml type id of the tensor (TensorInfo::ggml_dtype)."""
        info = self._info(name)
        return None if info is None else info.ggml_dtype

    def tensor_bytes(self, name: str) -> Optional[bytes]:
        """The tensor's raw bytes in the file."""
        info = self._info(name)
        if info is None or not info.data:
            return None
        return C.string_at(info.data, info.nbytes)

    def load_qtensor(self, name: str) -> QTensor:
        """load_qtensor (gguf.rs:117-124): the tensor's blocks as a QTensor on the GPU."""
        h = C.c_void_p()
        check(lib().izwi_gguf_load_weight(self._h, name.encode("utf-8"), C.byref(h)))
        return QTensor(h.value)

    def load_packed_qmatmul(self, names: List[str]) -> QMatMul:
        """packed_quantized_qmatmul (qwen3/core.rs:834-845): tensors concatenated along rows."""
        arr = (C.c_char_p * len(names))(*[n.encode("utf-8") for n in names])
        h = C.c_void_p()
        check(lib().izwi_gguf_load_packed(self._h, arr, len(names), C.byref(h)))
        return QMatMul.from_qtensor(QTensor(h.value))

    def load_tensor(self, name: str, dtype: torch.dtype = torch.float32,
                    device: str | torch.device = "cuda") -> torch.Tensor:
        """load_tensor (gguf.rs:127-144): dequantized to f32, then cast to `dtype`."""
        shape = self.tensor_shape(name)
        if shape is None:
            raise capi.QmmError(-1, f"Failed to load tensor '{name}' from GGUF: tensor not found")
        out = torch.empty(shape, dtype=torch.float32, device=device)
        space = DEVICE if out.is_cuda else HOST
        check(lib().izwi_gguf_load_tensor_f32(self._h, name.encode("utf-8"), out.data_ptr(), out.numel(), space,
                                              _stream_ptr(out)))
        return out if dtype == torch.float32 else out.to(dtype)

    # -- metadata -------------------------------------------------------------------------
    def metadata_keys(self) -> List[str]:
        out = []
        for i in range(lib().izwi_gguf_metadata_count(self._h)):
            p = C.c_char_p()
            check(lib().izwi_gguf_metadata_key(self._h, i, C.byref(p)))
            out.append(p.value.decode("utf-8"))
        return out

    def metadata_value(self, key: str):
        """metadata_value (gguf.rs:157-159) as a Python value, None if the key is absent."""
        k = key.encode("utf-8")
        t = lib().izwi_gguf_metadata_type(self._h, k)
        if t < 0:
            return None
        if t == _STRING:
            return self.get_metadata_string(key)
        if t == _ARRAY:
            et, n, data = C.c_int32(), C.c_uint64(), C.c_void_p()
            check(lib().izwi_gguf_metadata_array(self._h, k, C.byref(et), C.byref(n), C.byref(data)))
            if et.value == _STRING:
                out = []
                for i in range(n.value):
                    p, ln = C.c_void_p(), C.c_uint64()
                    check(lib().izwi_gguf_metadata_array_string(self._h, k, i, C.byref(p), C.byref(ln)))
                    out.append(C.string_at(p.value, ln.value).decode("utf-8", "replace"))
                return out
            fmt = _SCALAR_FORMATS.get(et.value)
            if fmt is None or not data.value:
                return [None] * n.value
            size = struct.calcsize(fmt)
            raw = C.string_at(data.value, size * n.value)
            return [struct.unpack_from(fmt, raw, i * size)[0] for i in range(n.value)]
        if t in (4, 10, 11):
            v = C.c_uint64()
            check(lib().izwi_gguf_metadata_u64(self._h, k, C.byref(v)))
            return C.c_int64(v.value).value if t == 11 else v.value
        d = C.c_double()
        check(lib().izwi_gguf_metadata_f64(self._h, k, C.byref(d)))
        if t == 7:
            return bool(d.value)
        return d.value if t in (6, 12) else int(d.value)

    def get_metadata_string(self, key: str) -> Optional[str]:
        """gguf.rs:162-170: the value if it is a string, else None."""
        p, n = C.c_void_p(), C.c_uint64()
        rc = lib().izwi_gguf_metadata_string(self._h, key.encode("utf-8"), C.byref(p), C.byref(n))
        return C.string_at(p.value, n.value).decode("utf-8", "replace") if rc == capi.OK else None

    def get_metadata_u64(self, key: str) -> Optional[int]:
        """gguf.rs:172-181: U64, I64 (cast) and U32 values, else None."""
        v = C.c_uint64()
        rc = lib().izwi_gguf_metadata_u64(self._h, key.encode("utf-8"), C.byref(v))
        return v.value if rc == capi.OK else None

    def _detect_quantization_from_tensors(self) -> Optional[str]:
        """gguf.rs:184-203: the single non-F32/F16 tensor type, or "mixed:a,b"."""
        names = {GGML_TYPE_NAMES.get(self.tensor_dtype(n), f"type{self.tensor_dtype(n)}") for n in self.tensor_names()}
        quant = sorted(d for d in names if "F32" not in d and "F16" not in d)
        if len(quant) == 1:
            return quant[0]
        return "mixed:" + ",".join(quant) if quant else None

    def get_model_info(self) -> GgufModelInfo:
        """gguf.rs:73-97."""
        architecture = self.get_metadata_string("general.architecture") or self.get_metadata_string("general.name")
        quantization = (self.get_metadata_string("general.quantization_type")
                        or self._detect_quantization_from_tensors())
        metadata = {}
        for key in self.metadata_keys():
            v = self.metadata_value(key)
            if isinstance(v, list):
                metadata[key] = f"[{len(v)} elements]"
            elif isinstance(v, bool):
                metadata[key] = "true" if v else "false"
            else:
                metadata[key] = str(v)
        return GgufModelInfo(self.path, architecture, self.get_metadata_u64("general.parameter_count"),
                             quantization, metadata)
