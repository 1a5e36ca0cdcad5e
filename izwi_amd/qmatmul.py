"""Host-side mirror of the reference's quantized projection interface.

Names and error behaviour follow the reference (izwi-core, qwen3/core.rs, and
the Candle types it calls): ``QTensor`` carries GGUF block bytes and a 2-D
shape, ``QMatMul.forward`` multiplies activations by the transposed weight,
``Qwen3Projection`` adds the activation-dtype policy and
``packed_qmatmul_from_qtensors`` row-concatenates projections.  torch tensors
only supply device memory and the current HIP stream; every operation is a
call into libizwi_qmm.
"""
from __future__ import annotations

import ctypes as C
import enum
from typing import Sequence

import numpy as np
import torch

from . import capi
from .capi import DEVICE, HOST, check, lib


class GgmlDType(enum.IntEnum):
    """candle_core::quantized::GgmlDType, the block formats of the path (Q6K: single projections
    only, no projection-group launch and no expert stacks)."""
    Q8_0 = 8
    Q4K = 12
    Q6K = 14

    def block_size(self) -> int:
        return 32 if self == GgmlDType.Q8_0 else 256

    def type_size(self) -> int:
        return {GgmlDType.Q8_0: 34, GgmlDType.Q4K: 144, GgmlDType.Q6K: 210}[self]


def quantized_storage_bytes(rows: int, cols: int, dtype: GgmlDType) -> int:
    """qwen3/core.rs:891-909: bytes of a [rows, cols] tensor, or an error."""
    out = C.c_uint64()
    check(lib().izwi_qmm_storage_bytes(int(dtype), rows, cols, C.byref(out)))
    return out.value


def _stream_ptr(t: torch.Tensor | None = None) -> int:
    if t is not None and not t.is_cuda:
        return 0
    return torch.cuda.current_stream().cuda_stream


def _space(t: torch.Tensor) -> int:
    return DEVICE if t.is_cuda else HOST


def _blocks_arg(blocks):
    """(pointer, nbytes, mem_space, keepalive) for numpy / bytes / torch uint8 input."""
    if isinstance(blocks, torch.Tensor):
        if blocks.dtype != torch.uint8 or not blocks.is_contiguous():
            raise ValueError("block bytes must be a contiguous uint8 tensor")
        return blocks.data_ptr(), blocks.numel(), _space(blocks), blocks
    arr = np.ascontiguousarray(np.frombuffer(blocks, dtype=np.uint8) if isinstance(blocks, (bytes, bytearray)) else blocks)
    if arr.dtype != np.uint8:
        raise ValueError("block bytes must be uint8")
    return arr.ctypes.data, arr.size, HOST, arr


class QTensor:
    """candle_core::quantized::QTensor for a [n, k] (or stacked [e, n, k]) weight on the GPU."""

    def __init__(self, handle: int, keep=None):
        self._h = C.c_void_p(handle)
        info = capi.WeightInfo()
        check(lib().izwi_qmm_weight_get_info(self._h, C.byref(info)))
        self._dtype = GgmlDType(info.ggml_dtype)
        self._n, self._k, self._e = info.n, info.k, info.n_stacked
        self._nbytes = info.nbytes

    # -- constructors --------------------------------------------------------
    @classmethod
    def from_blocks(cls, dtype: GgmlDType, blocks, shape: Sequence[int]) -> "QTensor":
        """ggml_file::qtensor_from_ggml(dtype, raw, dims, device): raw GGUF bytes -> tensor."""
        if len(shape) == 2:
            e, (n, k) = 1, shape
        elif len(shape) == 3:
            e, n, k = shape
        else:
            raise capi.QmmError(-1, f"unexpected rank, expected: 2, got: {len(shape)} ({tuple(shape)})")
        ptr, nbytes, space, keep = _blocks_arg(blocks)
        h = C.c_void_p()
        if e == 1 and len(shape) == 2:
            check(lib().izwi_qmm_weight_create(int(dtype), n, k, ptr, nbytes, space, C.byref(h)))
        else:
            check(lib().izwi_qmm_weight_create_stacked(int(dtype), e, n, k, ptr, nbytes, space, C.byref(h)))
        del keep
        return cls(h.value)

    @classmethod
    def quantize(cls, tensor: torch.Tensor, dtype: GgmlDType) -> "QTensor":
        """QTensor::quantize(&tensor, dtype) (candle-core quantized/mod.rs; the reference's use:
        qwen3/core.rs:3112): an f32 [n, k] matrix (host or device) -> Q8_0 / Q4_K tensor on the GPU,
        the blocks value for value those of the reference's CPU quantizer.  The last dimension
        must divide by the block size (the reference's own requirement)."""
        if tensor.dim() != 2:
            raise capi.QmmError(-1, f"unexpected rank, expected: 2, got: {tensor.dim()} ({tuple(tensor.shape)})")
        w = tensor.to(torch.float32).contiguous()
        n, k = w.shape
        nbytes = quantized_storage_bytes(n, k, dtype)
        blocks = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
        check(lib().izwi_qmm_quantize_weights_f32(int(dtype), w.data_ptr(), n, k, blocks.data_ptr(), _space(w),
                                                  _stream_ptr(w)))
        if w.is_cuda:
            torch.cuda.current_stream().synchronize()
        return cls.from_blocks(dtype, blocks, (n, k))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                lib().izwi_qmm_weight_destroy(h)
            except Exception:
                pass

    # -- QTensor accessors ---------------------------------------------------
    def dtype(self) -> GgmlDType:
        return self._dtype

    def shape(self):
        return (self._n, self._k) if self._e == 1 else (self._e, self._n, self._k)

    def dims2(self):
        if self._e != 1:
            raise capi.QmmError(-1, f"unexpected rank, expected: 2, got: 3 ({self.shape()})")
        return self._n, self._k

    def storage_size_in_bytes(self) -> int:
        return self._nbytes

    def data(self) -> np.ndarray:
        """QTensor::data(): the GGUF block bytes this tensor was built from."""
        out = np.empty(self._nbytes, dtype=np.uint8)
        check(lib().izwi_qmm_weight_data(self._h, out.ctypes.data, out.size, HOST, None))
        return out

    def dequantize(self, device: str | torch.device = "cuda") -> torch.Tensor:
        """QTensor::dequantize: f32 tensor, bit-identical to candle-core's to_float."""
        out = torch.empty((self._e * self._n, self._k), dtype=torch.float32, device=device)
        check(lib().izwi_qmm_dequantize_f32(self._h, out.data_ptr(), _space(out), _stream_ptr(out)))
        return out if self._e == 1 else out.view(self._e, self._n, self._k)


    def dequantize_rows(self, row_ids: torch.Tensor, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """Rows ``row_ids`` (int32 / int64 tensor, host or device) of ``dequantize()``, value for value,
        as f32 or bf16, without building the dense matrix."""
        if dtype not in (torch.float32, torch.bfloat16):
            raise capi.QmmError(-1, f"dequantize_rows gives f32 or bf16, not {dtype}")
        self.dims2()
        ids = row_ids.to(torch.int32).contiguous().view(-1)
        device = ids.device if ids.is_cuda else torch.device("cuda")
        out = torch.empty((ids.numel(), self._k), dtype=dtype, device=device)
        check(lib().izwi_qmm_dequantize_rows(self._h, ids.data_ptr(), ids.numel(), _space(ids), out.data_ptr(),
                                             1 if dtype == torch.bfloat16 else 0, _space(out), _stream_ptr(out)))
        return out


class QuantizedEmbedding:
    """The embedding lookup of the reference's decoders: ``Embedding::new(loader.load_tensor(name, dtype,
    device), hidden)`` followed by ``forward(input_ids)`` (qwen3/core.rs:2000-2007, 2083-2085) - the rows
    of the dequantized table, cast to the model dtype - read from the quantized tensor itself."""

    def __init__(self, qtensor: QTensor, dtype: torch.dtype = torch.float32):
        self.qtensor = qtensor
        self.dtype = dtype
        self.vocab_size, self.hidden_size = qtensor.dims2()

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """[..., hidden] for ids of any shape (index_select + reshape, as candle_nn's Embedding)."""
        rows = self.qtensor.dequantize_rows(input_ids.reshape(-1), self.dtype)
        return rows.view(*input_ids.shape, self.hidden_size)

    def embeddings(self) -> torch.Tensor:
        """The dense table (what a tied LM head multiplies by when a checkpoint has no lm_head)."""
        return self.qtensor.dequantize().to(self.dtype)


class QMatMul:
    """candle_core::quantized::QMatMul (the QTensor arm): ``forward(x) = x @ W^T``."""

    def __init__(self, qtensor: QTensor):
        self.qtensor = qtensor

    @classmethod
    def from_qtensor(cls, qtensor: QTensor) -> "QMatMul":
        qtensor.dims2()
        return cls(qtensor)

    from_arc = from_qtensor

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, k = self.qtensor.dims2()
        if x.dim() < 1 or x.shape[-1] != k:
            raise capi.QmmError(-1, f"shape mismatch in qmatmul, lhs: {tuple(x.shape)}, rhs: ({n}, {k})")
        if not x.is_contiguous():
            raise capi.QmmError(-1, "qmatmul requires a contiguous input")
        m = x.numel() // k if k else 0
        out_shape = tuple(x.shape[:-1]) + (n,)
        h = self.qtensor._h
        if x.dtype == torch.float32:
            y = torch.empty(out_shape, dtype=torch.float32, device=x.device)
            check(lib().izwi_qmm_forward_f32(h, x.data_ptr(), m, y.data_ptr(), _space(x), _stream_ptr(x)))
            return y
        if x.dtype == torch.bfloat16:
            y = torch.empty(out_shape, dtype=torch.bfloat16, device=x.device)
            check(lib().izwi_qmm_forward_bf16(h, x.data_ptr(), m, y.data_ptr(), capi.OUT_BF16,
                                              _space(x), _stream_ptr(x)))
            return y
        raise capi.QmmError(-1, f"unsupported dtype {x.dtype} for qmatmul, expected f32 or bf16")

    def forward_normed(self, x: torch.Tensor, norm_weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
        """forward(rms_norm(x, norm_weight, eps)) in one call (the final norm in front of the LM head)."""
        n, k = self.qtensor.dims2()
        if x.dtype != torch.float32 or x.dim() < 1 or x.shape[-1] != k or not x.is_contiguous():
            raise capi.QmmError(-1, f"expected a contiguous f32 input with last dim {k}")
        assert norm_weight.dtype == torch.float32 and norm_weight.is_contiguous() and norm_weight.numel() == k
        y = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=torch.float32, device=x.device)
        check(lib().izwi_qmm_forward_normed_f32(self.qtensor._h, x.data_ptr(), x.numel() // k if k else 0,
                                                norm_weight.data_ptr(), eps, y.data_ptr(), _space(x), _stream_ptr(x)))
        return y

    def forward_fused(self, x: torch.Tensor, residual: torch.Tensor | None = None,
                      out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        """Qwen3Projection::forward (qwen3/core.rs:795-829) plus the layer's residual add
        (core.rs:1875, 1879) in one call: x is f32 or bf16 and is read in its own type, the result is
        ``x @ W^T (+ residual)`` in ``out_dtype`` (default: x's type, as the reference casts back).
        ``out`` may be ``residual`` itself (in-place add)."""
        n, k = self.qtensor.dims2()
        code = {torch.float32: capi.OUT_F32, torch.bfloat16: capi.OUT_BF16}
        if x.dtype not in code or x.dim() < 1 or x.shape[-1] != k or not x.is_contiguous():
            raise capi.QmmError(-1, f"expected a contiguous f32 or bf16 input with last dim {k}, got {x.dtype} {tuple(x.shape)}")
        out_dtype = out_dtype or x.dtype
        if out_dtype not in code:
            raise capi.QmmError(-1, f"unsupported output dtype {out_dtype}")
        out_shape = tuple(x.shape[:-1]) + (n,)
        if residual is not None and (residual.dtype != out_dtype or tuple(residual.shape) != out_shape
                                     or not residual.is_contiguous() or residual.device != x.device):
            raise capi.QmmError(-1, f"residual must be a contiguous {out_dtype} tensor of shape {out_shape} on {x.device}")
        y = out if out is not None else torch.empty(out_shape, dtype=out_dtype, device=x.device)
        if y.dtype != out_dtype or tuple(y.shape) != out_shape or not y.is_contiguous() or y.device != x.device:
            raise capi.QmmError(-1, f"out must be a contiguous {out_dtype} tensor of shape {out_shape} on {x.device}")
        check(lib().izwi_qmm_forward_fused(self.qtensor._h, x.data_ptr(), code[x.dtype], x.numel() // k if k else 0,
                                           residual.data_ptr() if residual is not None else None, y.data_ptr(),
                                           code[out_dtype], _space(x), _stream_ptr(x)))
        return y

    def forward_bf16_to_f32(self, x: torch.Tensor) -> torch.Tensor:
        """bf16 activations, f32 result (the MFMA kernel's accumulators, unrounded)."""
        n, k = self.qtensor.dims2()
        if x.dtype != torch.bfloat16 or x.shape[-1] != k or not x.is_contiguous():
            raise capi.QmmError(-1, "expected a contiguous bf16 input with last dim k")
        y = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=torch.float32, device=x.device)
        check(lib().izwi_qmm_forward_bf16(self.qtensor._h, x.data_ptr(), x.numel() // k, y.data_ptr(),
                                          capi.OUT_F32, _space(x), _stream_ptr(x)))
        return y


def packed_qmatmul_from_qtensors(parts: Sequence[tuple]) -> QMatMul:
    """qwen3/core.rs:846-889 over (dtype, blocks, (rows, cols)) triples: byte-concatenate
    projections of equal input width and dtype into one QMatMul (fused QKV / gate-up)."""
    if len(parts) == 0:
        raise capi.QmmError(-1, "Cannot pack empty Qwen3 quantized projection group")
    dtype, _, (_, common_cols) = parts[0]
    rows, ptrs, sizes, keep, spaces = [], [], [], [], set()
    for dt, blocks, (r, c) in parts:
        if c != common_cols:
            raise capi.QmmError(-1, f"Qwen3 quantized projection group input mismatch: expected {common_cols}, got {c}")
        if dt != dtype:
            raise capi.QmmError(-1, f"Qwen3 quantized projection group dtype mismatch: expected {dtype!r}, got {dt!r}")
        ptr, nbytes, space, ka = _blocks_arg(blocks)
        rows.append(r)
        ptrs.append(ptr)
        sizes.append(nbytes)
        keep.append(ka)
        spaces.add(space)
    if len(spaces) != 1:
        raise ValueError("all parts must live in the same memory space")
    n = len(parts)
    h = C.c_void_p()
    check(lib().izwi_qmm_weight_create_packed(
        int(dtype), n, (C.c_int64 * n)(*rows), common_cols, (C.c_void_p * n)(*ptrs),
        (C.c_uint64 * n)(*sizes), spaces.pop(), C.byref(h)))
    return QMatMul(QTensor(h.value))


class Qwen3Projection:
    """The Quantized arm of izwi-core's Qwen3Projection (qwen3/core.rs:671-832)."""

    def __init__(self, qmatmul: QMatMul, is_lm_head: bool = False):
        self.qmatmul = qmatmul
        if is_lm_head:
            check(lib().izwi_qmm_weight_set_lm_head(qmatmul.qtensor._h, 1))

    @classmethod
    def quantized(cls, dtype: GgmlDType, blocks, shape, is_lm_head: bool = False) -> "Qwen3Projection":
        return cls(QMatMul.from_arc(QTensor.from_blocks(dtype, blocks, shape)), is_lm_head)

    @classmethod
    def packed_quantized(cls, parts) -> "Qwen3Projection":
        return cls(packed_qmatmul_from_qtensors(parts))

    def diagnostics(self) -> dict:
        """Qwen3Projection::diagnostics (qwen3/core.rs:729-742) for the Quantized arm: the counts that
        feed `qmatmul_projection_count` / `dense_projection_count` of the ASR execution diagnostics."""
        return {"dense_projection_count": 0, "dense_bias_projection_count": 0, "quantized_projection_count": 1}

    def logits_for_tokens(self, hidden: torch.Tensor, token_ids) -> list:
        """qwen3/core.rs:745-758: [(token id, logit)] for the given ids of one hidden state
        ([1, k] or [1, 1, k]); only the weight rows of those ids are read."""
        ids = [int(t) for t in token_ids]
        if not ids:
            return []
        k = hidden.shape[-1]
        if hidden.numel() != k:
            raise capi.QmmError(-1, f"Qwen3 selected-token logits expected [1,vocab] or [1,1,vocab], got {list(hidden.shape)[:-1] + ['vocab']}")
        n = self.qmatmul.qtensor.dims2()[0]
        if max(ids) >= n or min(ids) < 0:
            raise capi.QmmError(-1, f"token id out of range for a vocabulary of {n}")
        x = hidden.to(torch.float32).contiguous().view(1, k)
        import numpy as np
        idt = torch.from_numpy(np.asarray(ids, dtype=np.uint32).view(np.int32)).to(x.device)
        y = torch.empty((1, len(ids)), dtype=torch.float32, device=x.device)
        check(lib().izwi_qmm_forward_rows_f32(self.qmatmul.qtensor._h, idt.data_ptr(), len(ids), x.data_ptr(), 1,
                                              y.data_ptr(), _space(x), _stream_ptr(x)))
        return list(zip(ids, y.view(-1).tolist()))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """qwen3/core.rs:791-831.  f32 goes straight to the op.  bf16 inputs go through the
        fused call, which reads them as they are and rounds the f32 sums back to bf16 (the
        reference's cast to f32, QMatMul, cast back, with both casts inside the kernels); beyond 64
        rows that call runs the bf16 matrix-core kernel unless the integer arithmetic was selected
        (izwi_qmm_set_large_m_arithmetic).  Other dtypes are cast to f32 and back as the reference
        does on accelerators."""
        if x.dtype == torch.float32:
            return self.qmatmul.forward(x)
        if x.dtype == torch.bfloat16 and x.is_cuda:
            return self.qmatmul.forward_fused(x)
        return self.qmatmul.forward(x.to(torch.float32)).to(x.dtype)


def forward_group(projections: Sequence["QMatMul"], x: torch.Tensor, norm_weight: torch.Tensor | None = None,
                  eps: float = 1e-6):
    """Several projections on the same activations in one call (the `Separate` arms of
    Qwen3QkvProjection::forward / Qwen3GateUpProjection::forward, qwen3/core.rs:1119-1127,
    1274-1282).  Returns one output per projection, identical to separate forwards.
    With ``norm_weight`` the projections see rms_norm(x, norm_weight, eps) (the layer norm in front of
    them, core.rs:1872), folded into the same launch for one or two rows."""
    assert x.dtype in (torch.float32, torch.bfloat16) and x.is_contiguous()
    k = x.shape[-1]
    m = x.numel() // k if k else 0
    n = len(projections)
    ys = [torch.empty(tuple(x.shape[:-1]) + (p.qtensor.dims2()[0],), dtype=x.dtype, device=x.device)
          for p in projections]
    if x.dtype == torch.bfloat16:
        assert norm_weight is None
        # Up to 64 rows (or with the integer arithmetic selected for larger batches) a projection on bf16
        # activations runs the reference's integer block dots (Qwen3Projection.forward -> forward_fused);
        # the group must give the same bits as its members' separate forwards, so it takes that path
        # member by member.  Beyond: one launch of the bf16 matrix-core kernel for the whole group.
        if m <= 64 or lib().izwi_qmm_get_large_m_arithmetic() == capi.LARGE_M_INT8:
            for p, y in zip(projections, ys):
                p.forward_fused(x, out=y)
            return tuple(ys)
        handles = (C.c_void_p * n)(*[p.qtensor._h for p in projections])
        outs = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
        check(lib().izwi_qmm_forward_group_bf16(handles, n, x.data_ptr(), m, outs, capi.OUT_BF16, _space(x), _stream_ptr(x)))
        return tuple(ys)
    handles = (C.c_void_p * n)(*[p.qtensor._h for p in projections])
    outs = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
    if norm_weight is not None:
        assert norm_weight.dtype == torch.float32 and norm_weight.is_contiguous() and norm_weight.numel() == k
        check(lib().izwi_qmm_forward_group_normed_f32(handles, n, x.data_ptr(), m, norm_weight.data_ptr(), eps, outs,
                                                      _space(x), _stream_ptr(x)))
    else:
        check(lib().izwi_qmm_forward_group_f32(handles, n, x.data_ptr(), m, outs, _space(x), _stream_ptr(x)))
    return tuple(ys)


class ActivationRecords:
    """Quantized activations in the layout the batched decode kernels read (3..64 rows), written by the
    kernel that produces the activations instead of a quantizer launch of their own:
    ``from_rms_norm`` (the layer norm in front of q|k|v and gate|up), ``from_silu_mul`` (silu(gate) * up in
    front of down), ``quantize`` (anything else).  ``forward_group(projections)`` is `forward_group` on
    them, bit-identical to the calls on the f32 activations."""

    def __init__(self, weight_dtype: GgmlDType, m: int, k: int, device):
        self.weight_dtype, self.m, self.k = GgmlDType(weight_dtype), m, k
        nbytes = lib().izwi_qmm_records_bytes(int(weight_dtype), m, k)
        self.data = torch.empty(nbytes, dtype=torch.uint8, device=device)

    @staticmethod
    def _sp():
        return torch.cuda.current_stream().cuda_stream

    @classmethod
    def quantize(cls, weight_dtype, x: torch.Tensor) -> "ActivationRecords":
        assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
        r = cls(weight_dtype, x.shape[0], x.shape[1], x.device)
        check(lib().izwi_qmm_quantize_records_f32(int(weight_dtype), x.data_ptr(), r.m, r.k, r.data.data_ptr(), cls._sp()))
        return r

    @classmethod
    def from_rms_norm(cls, weight_dtype, x: torch.Tensor, norm_weight: torch.Tensor, eps: float = 1e-6) -> "ActivationRecords":
        assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
        assert norm_weight.dtype == torch.float32 and norm_weight.is_contiguous() and norm_weight.numel() == x.shape[1]
        r = cls(weight_dtype, x.shape[0], x.shape[1], x.device)
        check(lib().izwi_rms_norm_quantize_records_f32(int(weight_dtype), x.data_ptr(), norm_weight.data_ptr(), r.m, r.k, eps,
                                                       r.data.data_ptr(), cls._sp()))
        return r

    @classmethod
    def from_silu_mul(cls, weight_dtype, gate: torch.Tensor, up: torch.Tensor) -> "ActivationRecords":
        assert gate.is_cuda and gate.dtype == torch.float32 and gate.is_contiguous() and gate.dim() == 2
        assert up.shape == gate.shape and up.dtype == torch.float32 and up.is_contiguous()
        r = cls(weight_dtype, gate.shape[0], gate.shape[1], gate.device)
        check(lib().izwi_qmm_silu_mul_quantize_records_f32(int(weight_dtype), gate.data_ptr(), up.data_ptr(), r.m, r.k,
                                                           r.data.data_ptr(), cls._sp()))
        return r

    def forward_group(self, projections: Sequence["QMatMul"], outs=None):
        n = len(projections)
        for p in projections:
            # the C entry takes the records as a bare pointer: records made for another k or for the other
            # record type (Q8_0 blocks against Q8_K blocks) would be read out of bounds or as garbage
            if p.qtensor.dims2()[1] != self.k:
                raise capi.QmmError(-1, f"records of k = {self.k} given to a projection of k = {p.qtensor.dims2()[1]}")
            if (p.qtensor.dtype() == GgmlDType.Q8_0) != (self.weight_dtype == GgmlDType.Q8_0):
                raise capi.QmmError(-1, f"records for {self.weight_dtype.name} weights given to a {p.qtensor.dtype().name} projection")
        ys = outs if outs is not None else [torch.empty((self.m, p.qtensor.dims2()[0]), dtype=torch.float32,
                                                        device=self.data.device) for p in projections]
        handles = (C.c_void_p * n)(*[p.qtensor._h for p in projections])
        ptrs = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
        check(lib().izwi_qmm_forward_group_records_f32(handles, n, self.data.data_ptr(), self.m, ptrs, self._sp()))
        return tuple(ys)


class DecodeChain:
    """One token's projections as one launch (izwi_qmm_chain_*): ``steps`` is a list of
    ``(projections, x, ys)`` with 1..4 QMatMul of equal k, x a device f32 tensor of k values and one
    device f32 output tensor per projection.  Step i reads x after step i - 1 has completed, as the
    same calls issued one after the other on a stream would; results are those of `forward_group`
    bit for bit.  The tensors must stay alive and in place while the chain exists."""

    def __init__(self, steps):
        n = len(steps)
        arr = (capi.ChainStep * n)()
        self._keep = []
        for i, (projections, x, ys) in enumerate(steps):
            assert 1 <= len(projections) <= 4 and len(ys) == len(projections)
            assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
            k = projections[0].qtensor.dims2()[1]
            assert x.numel() == k, (x.shape, k)
            arr[i].n_weights = len(projections)
            arr[i].x = x.data_ptr()
            for j, (p, y) in enumerate(zip(projections, ys)):
                assert y.is_cuda and y.dtype == torch.float32 and y.is_contiguous() and y.numel() == p.qtensor.dims2()[0]
                arr[i].weights[j] = p.qtensor._h
                arr[i].ys[j] = y.data_ptr()
            self._keep.append((projections, x, ys))
        h = C.c_void_p()
        check(lib().izwi_qmm_chain_create(arr, n, C.byref(h)))
        self._h = h

    def run(self) -> None:
        check(lib().izwi_qmm_chain_run(self._h, torch.cuda.current_stream().cuda_stream))

    def status(self) -> None:
        """Waits for the current stream; raises if a wait inside a run gave up."""
        check(lib().izwi_qmm_chain_status(self._h, torch.cuda.current_stream().cuda_stream))

    def set_spin_limit(self, polls: int) -> None:
        check(lib().izwi_qmm_chain_set_spin_limit(self._h, polls))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                lib().izwi_qmm_chain_destroy(h)
            except Exception:
                pass


class Qwen3QkvProjection:
    """izwi-core's Qwen3QkvProjection with quantized weights: `new_separate` keeps q, k, v as
    three weights (the reference's default off Metal), `new_quantized_grouped` packs them."""

    def __init__(self, parts=None, fused=None, splits=None):
        self._parts, self._fused, self._splits = parts, fused, splits

    @classmethod
    def new_separate(cls, q_proj: "QMatMul", k_proj: "QMatMul", v_proj: "QMatMul"):
        return cls(parts=(q_proj, k_proj, v_proj))

    @classmethod
    def new_quantized_grouped(cls, parts: Sequence[tuple]):
        fused = packed_qmatmul_from_qtensors(parts)
        return cls(fused=fused, splits=[shape[0] for _, _, shape in parts])

    def forward(self, x: torch.Tensor):
        if self._fused is None:
            return forward_group(self._parts, x)
        y = self._fused.forward(x)  # one matmul, then `narrow` on the last dim
        outs, off = [], 0
        for rows in self._splits:
            outs.append(y.narrow(-1, off, rows))
            off += rows
        return tuple(outs)


class Qwen3GateUpProjection(Qwen3QkvProjection):
    """izwi-core's Qwen3GateUpProjection (gate, up) with quantized weights."""

    @classmethod
    def new_separate(cls, gate_proj: "QMatMul", up_proj: "QMatMul"):  # noqa: D102
        return cls(parts=(gate_proj, up_proj))

    def forward_silu_mul(self, x: torch.Tensor, norm_weight: torch.Tensor | None = None, eps: float = 1e-6) -> torch.Tensor:
        """`forward(x)` followed by `try_fused_silu_mul(gate, up)` (qwen3/core.rs:1786-1796,
        kernels/mod.rs:94-108) in one call: silu(gate x) * (up x).  With ``norm_weight`` x is replaced by
        rms_norm(x, norm_weight, eps) (post_attention_layernorm, core.rs:1877) in the same call."""
        if self._fused is not None:
            assert norm_weight is None
            gate, up = self.forward(x)
            return torch.nn.functional.silu(gate) * up
        gate_proj, up_proj = self._parts
        assert x.dtype == torch.float32 and x.is_contiguous()
        n, k = gate_proj.qtensor.dims2()
        if x.dim() < 1 or x.shape[-1] != k:
            raise capi.QmmError(-1, f"shape mismatch in qmatmul, lhs: {tuple(x.shape)}, rhs: ({n}, {k})")
        m = x.numel() // k if k else 0
        h = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=torch.float32, device=x.device)
        if norm_weight is not None:
            assert norm_weight.dtype == torch.float32 and norm_weight.is_contiguous() and norm_weight.numel() == k
            check(lib().izwi_qmm_forward_gate_up_silu_normed_f32(gate_proj.qtensor._h, up_proj.qtensor._h, x.data_ptr(), m,
                                                                 norm_weight.data_ptr(), eps, h.data_ptr(), _space(x),
                                                                 _stream_ptr(x)))
        else:
            check(lib().izwi_qmm_forward_gate_up_silu_f32(gate_proj.qtensor._h, up_proj.qtensor._h, x.data_ptr(), m,
                                                          h.data_ptr(), _space(x), _stream_ptr(x)))
        return h


class Qwen3Mlp:
    """izwi-core's Qwen3Mlp (qwen3/core.rs:1740-1798) with quantized weights:
    down(silu(gate x) * (up x))."""

    def __init__(self, gate_up_proj: Qwen3GateUpProjection, down_proj: "QMatMul"):
        self.gate_up_proj, self.down_proj = gate_up_proj, down_proj

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        parts = self.gate_up_proj._parts
        if parts is None or x.dtype != torch.float32:
            return self.down_proj.forward(self.gate_up_proj.forward_silu_mul(x))
        # separate gate / up weights, f32 activations: the three projections as one library call
        gate_proj, up_proj = parts
        n, k = gate_proj.qtensor.dims2()
        if x.dim() < 1 or x.shape[-1] != k:
            raise capi.QmmError(-1, f"shape mismatch in qmatmul, lhs: {tuple(x.shape)}, rhs: ({n}, {k})")
        if not x.is_contiguous():
            raise capi.QmmError(-1, "qmatmul requires a contiguous input")
        m = x.numel() // k if k else 0
        y = torch.empty(tuple(x.shape[:-1]) + (self.down_proj.qtensor.dims2()[0],), dtype=torch.float32, device=x.device)
        check(lib().izwi_qmm_mlp_forward_f32(gate_proj.qtensor._h, up_proj.qtensor._h, self.down_proj.qtensor._h,
                                             x.data_ptr(), m, y.data_ptr(), _space(x), _stream_ptr(x)))
        return y


def quantize_activations(weight_dtype: GgmlDType, x: torch.Tensor) -> torch.Tensor:
    """The activation blocks the decode kernel builds (reference block layout, uint8)."""
    assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
    m, k = x.shape
    per = 34 if weight_dtype == GgmlDType.Q8_0 else 292
    out = torch.empty(m * (k // weight_dtype.block_size()) * per, dtype=torch.uint8, device=x.device)
    check(lib().izwi_qmm_quantize_activations(int(weight_dtype), x.data_ptr(), m, k, out.data_ptr(),
                                              _space(x), _stream_ptr(x)))
    return out


def moe_route(logits: torch.Tensor, top_k: int):
    assert logits.dtype == torch.float32 and logits.is_contiguous() and logits.dim() == 2
    t, e = logits.shape
    ids = torch.empty((t, top_k), dtype=torch.int32, device=logits.device)
    wts = torch.empty((t, top_k), dtype=torch.float32, device=logits.device)
    check(lib().izwi_moe_route(logits.data_ptr(), t, e, top_k, ids.data_ptr(), wts.data_ptr(),
                               _space(logits), _stream_ptr(logits)))
    return ids, wts


def moe_sort(ids: torch.Tensor, n_experts: int):
    assert ids.dtype == torch.int32 and ids.is_contiguous() and ids.dim() == 2
    t, top_k = ids.shape
    perm = torch.empty(t * top_k, dtype=torch.int32, device=ids.device)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=ids.device)
    check(lib().izwi_moe_sort(ids.data_ptr(), t, top_k, n_experts, perm.data_ptr(), offsets.data_ptr(),
                              _space(ids), _stream_ptr(ids)))
    return perm, offsets


class MoeExperts:
    """Expert stacks of one MoE layer: gate/up [e, inter, hidden], down [e, hidden, inter]."""

    def __init__(self, gate: QTensor, up: QTensor, down: QTensor):
        self.gate, self.up, self.down = gate, up, down

    def forward(self, x, ids, wts, perm, offsets) -> torch.Tensor:
        assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
        t = x.shape[0]
        out = torch.empty_like(x)
        check(lib().izwi_moe_forward_f32(self.gate._h, self.up._h, self.down._h, x.data_ptr(), t,
                                         ids.data_ptr(), wts.data_ptr(), ids.shape[1], perm.data_ptr(),
                                         offsets.data_ptr(), out.data_ptr(), _space(x), _stream_ptr(x)))
        return out

    def layer(self, logits: torch.Tensor, x: torch.Tensor, top_k: int, return_routing: bool = False):
        """Route, sort, expert MLP and combine in one call (izwi_moe_layer_f32): the same results
        as moe_route + moe_sort + forward."""
        assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
        assert logits.dtype == torch.float32 and logits.is_contiguous() and logits.shape[0] == x.shape[0]
        t = x.shape[0]
        out = torch.empty_like(x)
        ids = wts = None
        if return_routing:
            ids = torch.empty((t, top_k), dtype=torch.int32, device=x.device)
            wts = torch.empty((t, top_k), dtype=torch.float32, device=x.device)
        check(lib().izwi_moe_layer_f32(self.gate._h, self.up._h, self.down._h, logits.data_ptr(), x.data_ptr(), t,
                                       top_k, out.data_ptr(), ids.data_ptr() if return_routing else None,
                                       wts.data_ptr() if return_routing else None, _space(x), _stream_ptr(x)))
        return (out, ids, wts) if return_routing else out


def profile_snapshot() -> dict:
    snap = capi.ProfileSnapshot()
    check(lib().izwi_qmm_profile_snapshot_get(C.byref(snap)))
    return {name: getattr(snap, name) for name, _ in snap._fields_}


def asr_profile_diagnostics() -> dict:
    """The fields of Qwen3AsrProfileDiagnostics (qwen3/asr/mod.rs:116-147) that `izwi bench` reads
    (crates/izwi-cli/src/commands/bench.rs:281-295), filled from the library's counters the way
    `update_from_runtime_delta` fills them: ns -> ms, plus the device argmax."""
    snap = profile_snapshot()
    calls, ns = C.c_uint64(), C.c_uint64()
    check(lib().izwi_qmm_profile_argmax_get(C.byref(calls), C.byref(ns)))
    ms = lambda v: v / 1e6  # noqa: E731
    return {
        "qwen3_profile_enabled": capi_profile_enabled(),
        "qmatmul_calls": snap["qmatmul_calls"], "qmatmul_ms": ms(snap["qmatmul_ns"]),
        "qmatmul_input_casts": snap["qmatmul_input_casts"], "qmatmul_input_cast_ms": ms(snap["qmatmul_input_cast_ns"]),
        "qmatmul_output_casts": snap["qmatmul_output_casts"], "qmatmul_output_cast_ms": ms(snap["qmatmul_output_cast_ns"]),
        "lm_head_calls": snap["lm_head_calls"], "lm_head_ms": ms(snap["lm_head_ns"]),
        "silu_mul_fused_calls": snap["silu_mul_fused_calls"], "silu_mul_fallback_calls": snap["silu_mul_fallback_calls"],
        "argmax_calls": calls.value, "argmax_ms": ms(ns.value),
    }


PREFILL_AUTO, PREFILL_LDS, PREFILL_PLANE = -1, 0, 1


def set_prefill_form(form: int) -> None:
    """Form of the bf16 prefill product, process-wide (izwi_qmm_set_prefill_form): PREFILL_LDS
    dequantizes the weights inside the matmul kernel on their way into LDS, PREFILL_PLANE once per
    call into a bf16 plane in scratch memory that a plain bf16 matrix-core loop then reads."""
    capi.check(capi.lib().izwi_qmm_set_prefill_form(int(form)))


def get_prefill_form() -> int:
    return int(capi.lib().izwi_qmm_get_prefill_form())


def capi_profile_enabled() -> bool:
    return bool(lib().izwi_qmm_profile_enabled())
