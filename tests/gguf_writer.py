"""Test-side GGUF writer: a restatement of the public GGUF container format (versions 1-3),
independent of the reader under test.  It is the checker of the GGUF ingress tests: the
reference holds no GGUF fixture (only `is_gguf_file` cases, gguf.rs:390-420) and its reader,
candle-core's gguf_file, is not in its tree.

Layout (little-endian): "GGUF", u32 version, tensor count, metadata count (u64; u32 in version 1);
metadata entries {string key, u32 value type, value}; tensor infos {string name, u32 n_dims,
dims innermost first (u64; u32 in version 1), u32 ggml type, u64 offset}; zero padding to the
next multiple of general.alignment (default 32); tensor data at their offsets.
"""
import struct

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?", U64: "<Q",
        I64: "<q", F64: "<d"}


def _length(n, version):
    return struct.pack("<I" if version == 1 else "<Q", n)


def _string(s, version):
    b = s if isinstance(s, bytes) else s.encode("utf-8")
    return _length(len(b), version) + b


def _value(vtype, value, version):
    if vtype in _FMT:
        return struct.pack(_FMT[vtype], value)
    if vtype == STRING:
        return _string(value, version)
    if vtype == ARRAY:
        elem_type, elems = value
        out = struct.pack("<I", elem_type) + _length(len(elems), version)
        for e in elems:
            out += _value(elem_type, e, version)
        return out
    raise ValueError(vtype)


def write_gguf(path, metadata, tensors, version=3, alignment=None, magic=b"GGUF", pad_data=0):
    """metadata: list of (key, value_type, value); ARRAY values are (elem_type, [elems]).
    tensors: list of (name, row_major_dims, ggml_type, raw_bytes).  Returns {name: offset}."""
    metadata = list(metadata)
    if alignment is not None:
        metadata.append(("general.alignment", U32, alignment))
    align = alignment or 32
    head = magic + struct.pack("<I", version) + _length(len(tensors), version) + _length(len(metadata), version)
    for key, vtype, value in metadata:
        head += _string(key, version) + struct.pack("<I", vtype) + _value(vtype, value, version)
    offsets, infos, data = {}, b"", b""
    for name, dims, ggml_type, raw in tensors:
        data += b"\0" * (-len(data) % align)
        offsets[name] = len(data)
        infos += _string(name, version) + struct.pack("<I", len(dims))
        for d in reversed(dims):  # the file lists the innermost dimension first
            infos += _length(d, version)
        infos += struct.pack("<I", ggml_type) + struct.pack("<Q", len(data))
        data += bytes(raw)
    body = head + infos
    body += b"\0" * (-len(body) % align)
    with open(path, "wb") as f:
        f.write(body + data + b"\0" * pad_data)
    return offsets, len(body)
