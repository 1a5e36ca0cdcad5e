"""GGUF ingress (include/izwi_gguf.h, izwi_amd/gguf.py) against files written by the
test-side writer (tests/gguf_writer.py, a restatement of the public container format) and
against the committed fixture tests/golden/tiny.gguf.  Parsing needs no GPU; the load tests
do.  The reference's own tests for this row are the two `is_gguf_file` cases
(crates/izwi-core/src/models/shared/weights/gguf.rs:390-420), repeated here."""
import json
import os
import struct

import numpy as np

import np_ref
import pytest

import gguf_writer as gw

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def qa():
    import izwi_amd
    from izwi_amd import capi
    if not os.path.exists(capi.library_path()):
        import __graft_entry__
        __graft_entry__.build()
    return izwi_amd


def _sample(tmp_path, version=3, alignment=None, name="sample.gguf"):
    rng = np.random.default_rng(5)
    f32 = rng.standard_normal((2, 3)).astype(np.float32)
    q8 = rng.integers(0, 256, 4 * 2 * 34, dtype=np.uint8)       # [4, 64] Q8_0: 2 blocks per row
    q4 = rng.integers(0, 256, 2 * 144, dtype=np.uint8)           # [2, 256] Q4_K
    f16 = rng.standard_normal(5).astype(np.float16)
    metadata = [
        ("general.architecture", gw.STRING, "qwen3"),
        ("general.name", gw.STRING, "tiny"),
        ("general.parameter_count", gw.U64, 123456789012),
        ("a.u8", gw.U8, 200), ("a.i8", gw.I8, -100), ("a.u16", gw.U16, 60000), ("a.i16", gw.I16, -30000),
        ("a.u32", gw.U32, 4000000000), ("a.i32", gw.I32, -2000000000), ("a.f32", gw.F32, 1.5),
        ("a.bool", gw.BOOL, True), ("a.i64", gw.I64, -5), ("a.f64", gw.F64, 2.25),
        ("tokens", gw.ARRAY, (gw.STRING, ["a", "bc", "", "déf"])),
        ("ids", gw.ARRAY, (gw.U32, [7, 8, 9])),
        ("scores", gw.ARRAY, (gw.F32, [0.5, -1.0])),
        ("nested", gw.ARRAY, (gw.ARRAY, [(gw.U8, [1, 2]), (gw.U8, [3])])),
    ]
    tensors = [
        ("dense.weight", (2, 3), 0, f32.tobytes()),
        ("blk.0.attn_q.weight", (4, 64), 8, q8.tobytes()),
        ("blk.0.ffn_gate.weight", (2, 256), 12, q4.tobytes()),
        ("norm.weight", (5,), 1, f16.tobytes()),
        ("exotic", (256,), 16, b""),                                # a type this library has no size for
    ]
    path = str(tmp_path / name)
    offsets, data_offset = gw.write_gguf(path, metadata, tensors, version=version, alignment=alignment)
    return path, metadata, tensors, offsets, data_offset


# ---------------------------------------------------------------- no GPU needed --
def test_is_gguf_file_reference_cases(qa, tmp_path):
    # gguf.rs:394-419
    a = tmp_path / "test.gguf"
    a.write_bytes(b"GGUF\x00\x00\x00\x00")
    b = tmp_path / "test.txt"
    b.write_bytes(b"This is not a GGUF file")
    c = tmp_path / "short"
    c.write_bytes(b"GG")
    assert qa.is_gguf_file(a) and not qa.is_gguf_file(b) and not qa.is_gguf_file(c)
    assert not qa.is_gguf_file(tmp_path / "missing")


@pytest.mark.parametrize("version", [1, 2, 3])
@pytest.mark.parametrize("alignment", [None, 64, 4096])
def test_parse_container(qa, tmp_path, version, alignment):
    path, metadata, tensors, offsets, data_offset = _sample(tmp_path, version, alignment)
    g = qa.GgufLoader.from_path(path)
    assert g.header() == (version, alignment or 32, data_offset)
    assert g.tensor_count() == len(tensors)
    assert g.tensor_names() == [t[0] for t in tensors]
    for name, dims, ggml_type, raw in tensors:
        assert g.has_tensor(name)
        assert g.tensor_shape(name) == list(dims)
        assert g.tensor_dtype(name) == ggml_type
        info = g._info(name)
        assert info.offset == offsets[name] and info.offset % (alignment or 32) == 0
        if ggml_type == 16:
            assert info.nbytes == 0 and g.tensor_bytes(name) is None
        else:
            assert info.nbytes == len(raw) and g.tensor_bytes(name) == raw
    assert not g.has_tensor("nope") and g.tensor_shape("nope") is None
    # metadata
    keys = [m[0] for m in metadata] + (["general.alignment"] if alignment else [])
    assert g.metadata_keys() == keys
    assert g.get_metadata_string("general.architecture") == "qwen3"
    assert g.get_metadata_string("a.u32") is None and g.get_metadata_string("absent") is None
    assert g.get_metadata_u64("general.parameter_count") == 123456789012
    assert g.get_metadata_u64("a.u32") == 4000000000
    assert g.get_metadata_u64("a.i64") == 2 ** 64 - 5          # `*n as u64`, gguf.rs:176
    assert g.get_metadata_u64("a.u8") is None and g.get_metadata_u64("a.i32") is None
    want = {"a.u8": 200, "a.i8": -100, "a.u16": 60000, "a.i16": -30000, "a.u32": 4000000000,
            "a.i32": -2000000000, "a.f32": 1.5, "a.bool": True, "a.i64": -5, "a.f64": 2.25,
            "tokens": ["a", "bc", "", "déf"], "ids": [7, 8, 9], "scores": [0.5, -1.0]}
    for k, v in want.items():
        assert g.metadata_value(k) == v, k
    assert g.metadata_value("nested") == [None, None] and g.metadata_value("absent") is None


def test_model_info(qa, tmp_path):
    path, *_ = _sample(tmp_path)
    info = qa.GgufLoader.from_path(path).get_model_info()
    assert info.architecture == "qwen3" and info.parameter_count == 123456789012
    assert info.quantization == "mixed:Q4K,Q8_0,type16"
    assert info.metadata["tokens"] == "[4 elements]" and info.metadata["a.bool"] == "true"
    assert info.metadata["a.i32"] == "-2000000000"
    # architecture falls back to general.name; one quantized type is named as such (gguf.rs:73-97, 184-203)
    p2 = str(tmp_path / "b.gguf")
    gw.write_gguf(p2, [("general.name", gw.STRING, "fallback"), ("general.parameter_count", gw.U32, 7)],
                  [("w", (1, 256), 12, bytes(144)), ("n", (4,), 0, bytes(16))])
    info = qa.GgufLoader.from_path(p2).get_model_info()
    assert (info.architecture, info.parameter_count, info.quantization) == ("fallback", 7, "Q4K")
    p3 = str(tmp_path / "c.gguf")
    gw.write_gguf(p3, [("general.quantization_type", gw.STRING, "Q4_K_M")], [("n", (4,), 0, bytes(16))])
    info = qa.GgufLoader.from_path(p3).get_model_info()
    assert (info.architecture, info.parameter_count, info.quantization) == (None, None, "Q4_K_M")


def test_malformed_files_are_errors(qa, tmp_path):
    from izwi_amd.capi import QmmError
    path, *_ = _sample(tmp_path)
    blob = open(path, "rb").read()

    def opens(data):
        p = tmp_path / "m.gguf"
        p.write_bytes(data)
        try:
            qa.GgufLoader.from_path(p)
            return True
        except QmmError as e:
            assert e.code == -1 and "GGUF" in e.message
            return False

    assert opens(blob)
    assert not opens(b"GGML" + blob[4:])                                    # magic
    assert not opens(blob[:4] + struct.pack("<I", 4) + blob[8:])            # version
    assert not opens(blob[:4] + struct.pack("<I", 0) + blob[8:])
    assert not opens(b"")
    with pytest.raises(QmmError):
        qa.GgufLoader.from_path(tmp_path / "does-not-exist.gguf")
    # every truncation inside the header, the metadata, the tensor infos or a tensor's data is an error
    g = qa.GgufLoader.from_path(path)
    _, _, data_offset = g.header()
    info = g._info("norm.weight")                                   # the last tensor that has data
    data_end = data_offset + info.offset + info.nbytes
    for cut in list(range(0, data_offset, 7)) + [data_end - 1]:
        assert not opens(blob[:cut]), cut
    assert opens(blob[:data_end])
    # counts that cannot fit the file
    assert not opens(blob[:8] + struct.pack("<Q", 1 << 60) + blob[16:])
    assert not opens(blob[:16] + struct.pack("<Q", 1 << 60) + blob[24:])
    # element count that is not a multiple of the block size; too many dimensions; bad alignment
    p = str(tmp_path / "x.gguf")
    gw.write_gguf(p, [], [("w", (3, 100), 12, bytes(144))])
    with pytest.raises(QmmError, match="multiple of its block size"):
        qa.GgufLoader.from_path(p)
    gw.write_gguf(p, [], [("w", (1,) * 9, 0, bytes(4))])
    with pytest.raises(QmmError, match="too many dimensions"):
        qa.GgufLoader.from_path(p)
    gw.write_gguf(p, [("general.alignment", gw.U32, 0)], [("w", (1,), 0, bytes(4))])
    with pytest.raises(QmmError, match="alignment"):
        qa.GgufLoader.from_path(p)
    gw.write_gguf(p, [("general.alignment", gw.STRING, "32")], [("w", (1,), 0, bytes(4))])
    with pytest.raises(QmmError, match="alignment"):
        qa.GgufLoader.from_path(p)


def test_reader_policy_follows_the_reference(qa, tmp_path, monkeypatch):
    """backends/model_io.rs:13-160 and its tests (`parse_mode_supports_aliases`,
    `parse_mode_rejects_unknown_values`, `resolve_mode_prefers_explicit_value_then_env_then_auto_default`,
    `open_reader_uses_buffered_mode_when_explicitly_disabled`), plus the fallback to buffered I/O
    when the mapping fails (model_io.rs:146-160)."""
    from izwi_amd.gguf import GgufMmapMode as M, GgufReaderKind as K, resolve_gguf_mmap_mode
    assert M.parse("auto") == M.AUTO
    for word in ("on", "true", "1", "yes", " ON ", "Yes"):
        assert M.parse(word) == M.ON, word
    for word in ("off", "false", "0", "no", "OFF\n"):
        assert M.parse(word) == M.OFF, word
    assert M.parse("") is None and M.parse("invalid") is None
    assert [M.as_str(m) for m in (M.AUTO, M.ON, M.OFF)] == ["auto", "on", "off"]
    monkeypatch.delenv("IZWI_GGUF_MMAP", raising=False)
    assert resolve_gguf_mmap_mode(None) == M.AUTO
    monkeypatch.setenv("IZWI_GGUF_MMAP", "off")
    assert resolve_gguf_mmap_mode(None) == M.OFF
    assert resolve_gguf_mmap_mode(M.ON) == M.ON
    monkeypatch.setenv("IZWI_GGUF_MMAP", "nonsense")
    assert resolve_gguf_mmap_mode(None) == M.AUTO

    path, metadata, tensors, *_ = _sample(tmp_path)

    def contents(g):
        return (g.header(), g.tensor_names(), [g.tensor_bytes(n) for n in g.tensor_names()],
                {k: g.metadata_value(k) for k in g.metadata_keys()} if hasattr(g, "metadata_keys") else None)

    monkeypatch.delenv("IZWI_GGUF_MMAP", raising=False)
    mapped = qa.GgufLoader.from_path(path)
    assert mapped.reader_kind() == K.MAPPED                       # auto maps on every backend
    assert qa.GgufLoader.from_path(path, M.ON).reader_kind() == K.MAPPED
    buffered = qa.GgufLoader.from_path(path, M.OFF)
    assert buffered.reader_kind() == K.BUFFERED
    assert contents(buffered) == contents(mapped)
    monkeypatch.setenv("IZWI_GGUF_MMAP", "0")                     # the environment when nothing is configured
    assert qa.GgufLoader.from_path(path).reader_kind() == K.BUFFERED
    assert qa.GgufLoader.from_path(path, M.ON).reader_kind() == K.MAPPED
    monkeypatch.delenv("IZWI_GGUF_MMAP")
    # a mapping that fails falls back to buffered I/O, with the same contents
    monkeypatch.setenv("_IZWI_GGUF_PRIVATE_TEST_FAIL_MMAP", "1")
    fell_back = qa.GgufLoader.from_path(path, M.ON)
    assert fell_back.reader_kind() == K.BUFFERED and contents(fell_back) == contents(mapped)
    monkeypatch.delenv("_IZWI_GGUF_PRIVATE_TEST_FAIL_MMAP")
    # malformed input is an error in buffered mode too
    from izwi_amd.capi import QmmError
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(open(path, "rb").read()[:40])
    with pytest.raises(QmmError):
        qa.GgufLoader.from_path(bad, M.OFF)


def test_crafted_counts_do_not_exhaust_memory(qa, tmp_path):
    """An array-of-strings count far beyond what the file can hold is refused before anything is
    reserved for it (8 bytes per entry at least, 4 in version 1)."""
    from izwi_amd.capi import QmmError
    for version, ln in ((3, "<Q"), (1, "<I")):
        key = b"general.name"
        head = b"GGUF" + struct.pack("<I", version) + struct.pack(ln, 0) + struct.pack(ln, 1)
        kv = struct.pack(ln, len(key)) + key + struct.pack("<I", 9) + struct.pack("<I", 8)
        body = bytes(64 * 1024)
        # the count that would just pass a bytes-remaining bound but not the bytes / entry-size one
        count = len(body) // (2 if version == 3 else 1)
        p = tmp_path / f"crafted{version}.gguf"
        p.write_bytes(head + kv + struct.pack(ln, count) + body)
        with pytest.raises(QmmError, match="GGUF"):
            qa.GgufLoader.from_path(p)


def test_committed_fixture(qa):
    """tests/golden/tiny.gguf is data: the bytes of a small GGUF file and, beside it, what a
    reader must find in it (written once by tests/golden/make_fixtures.py)."""
    want = json.load(open(os.path.join(HERE, "golden", "tiny_gguf.json")))
    g = qa.GgufLoader.from_path(os.path.join(HERE, "golden", "tiny.gguf"))
    assert list(g.header()) == want["header"]
    assert g.tensor_names() == [t["name"] for t in want["tensors"]]
    for t in want["tensors"]:
        assert g.tensor_shape(t["name"]) == t["shape"] and g.tensor_dtype(t["name"]) == t["ggml_dtype"]
        assert g._info(t["name"]).offset == t["offset"]
        assert g.tensor_bytes(t["name"]).hex() == t["bytes_hex"]
    for k, v in want["metadata"].items():
        assert g.metadata_value(k) == v, k


def test_load_without_gpu_fails_loudly(qa, tmp_path):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from izwi_amd.capi import QmmError
    path, *_ = _sample(tmp_path)
    g = qa.GgufLoader.from_path(path)
    with pytest.raises(QmmError) as e:
        g.load_qtensor("blk.0.attn_q.weight")
    assert e.value.code in (-3, -4)
    # argument errors come before any device work
    with pytest.raises(QmmError, match="not supported"):
        g.load_qtensor("dense.weight")
    with pytest.raises(QmmError, match="tensor not found"):
        g.load_qtensor("absent")


# ------------------------------------------------------------------------- GPU --
def _model_file(tmp_path, oracle):
    shapes = {"blk.0.attn_q.weight": (8, 96, 64), "blk.0.attn_k.weight": (8, 32, 64), "blk.0.attn_v.weight": (8, 32, 64),
              "blk.0.ffn_gate.weight": (12, 48, 512), "blk.0.ffn_up.weight": (12, 48, 512),
              "blk.0.ffn_down.weight": (12, 40, 768)}
    tensors, blocks = [], {}
    for i, (name, (dtype, n, k)) in enumerate(shapes.items()):
        b = oracle.quantize(dtype, oracle.randn(100 + i, (n, k), std=0.05))
        blocks[name] = (dtype, n, k, np.ascontiguousarray(b).view(np.uint8).reshape(-1))
        tensors.append((name, (n, k), dtype, blocks[name][3].tobytes()))
    dense = oracle.randn(7, (3, 10))
    tensors.append(("output_norm.weight", (3, 10), 0, dense.astype(np.float32).tobytes()))
    tensors.append(("half.weight", (3, 10), 1, dense.astype(np.float16).tobytes()))
    bf = (dense.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    tensors.append(("bf.weight", (3, 10), 30, bf.tobytes()))
    tensors.append(("vec.q8", (64,), 8, blocks["blk.0.attn_q.weight"][3][:68].tobytes()))
    path = str(tmp_path / "model.gguf")
    gw.write_gguf(path, [("general.architecture", gw.STRING, "qwen3")], tensors)
    return path, blocks, dense, bf


@pytest.mark.gpu
def test_load_qtensor_and_forward(qa, oracle, tmp_path):
    import torch
    path, blocks, _, _ = _model_file(tmp_path, oracle)
    g = qa.GgufLoader.from_path(path)
    for name, (dtype, n, k, raw) in blocks.items():
        print("gguf load", name, flush=True)
        qt = g.load_qtensor(name)
        assert qt.dtype() == qa.GgmlDType(dtype) and qt.shape() == (n, k)
        assert np.array_equal(qt.data(), raw)                      # QTensor::data(): the file's bytes
        direct = qa.QTensor.from_blocks(qa.GgmlDType(dtype), raw, (n, k))
        for m in (1, 5):
            x = torch.from_numpy(oracle.randn(9 + m, (m, k))).cuda()
            y = qa.QMatMul.from_qtensor(qt).forward(x)
            assert torch.equal(y, qa.QMatMul.from_qtensor(direct).forward(x))
            want = oracle.qmatmul(dtype, x.cpu().numpy(), raw, n)
            assert np.abs(y.cpu().numpy() - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.gpu
def test_load_tensor_dequantizes_bit_exactly(qa, oracle, tmp_path):
    import torch
    path, blocks, dense, bf = _model_file(tmp_path, oracle)
    g = qa.GgufLoader.from_path(path)
    for name, (dtype, n, k, raw) in blocks.items():
        print("gguf dequant", name, flush=True)
        want = oracle.dequantize(dtype, raw, n, k)
        for device in ("cuda", "cpu"):
            got = g.load_tensor(name, device=device).cpu().numpy()
            assert got.shape == (n, k) and np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(g.load_tensor("output_norm.weight").cpu().numpy(), dense.astype(np.float32))
    assert np.array_equal(g.load_tensor("output_norm.weight", device="cpu").numpy(), dense.astype(np.float32))
    for device in ("cuda", "cpu"):
        assert np.array_equal(g.load_tensor("half.weight", device=device).cpu().numpy(),
                              dense.astype(np.float16).astype(np.float32))
        assert np.array_equal(g.load_tensor("bf.weight", device=device).cpu().numpy().view(np.uint32),
                              bf.astype(np.uint32) << 16)
    # a one-dimensional quantized tensor dequantizes (load_tensor) but is no projection (load_qtensor)
    v = g.load_tensor("vec.q8").cpu().numpy()
    dtype, n, k, raw = blocks["blk.0.attn_q.weight"]
    assert np.array_equal(v, oracle.dequantize(8, raw[:68], 1, 64).reshape(-1))
    assert g.load_tensor("half.weight", dtype=torch.bfloat16).dtype == torch.bfloat16
    from izwi_amd.capi import QmmError
    with pytest.raises(QmmError, match="2"):
        g.load_qtensor("vec.q8")
    with pytest.raises(QmmError) as e:
        g.load_qtensor("half.weight")
    assert e.value.code == -2


@pytest.mark.gpu
def test_committed_fixture_dequantizes_to_its_closed_form(qa):
    want = json.load(open(os.path.join(HERE, "golden", "tiny_gguf.json")))
    g = qa.GgufLoader.from_path(os.path.join(HERE, "golden", "tiny.gguf"))
    for name, values in want["dequantized"].items():
        got = g.load_tensor(name).cpu().numpy().reshape(-1)
        assert np.array_equal(got, np.array(values, dtype=np.float32)), name


@pytest.mark.gpu
def test_q6_k_tensors_load_dense_and_as_projections(qa, oracle, tmp_path):
    """Q4_K_M files keep some tensors in Q6_K: they are listed with shape, type and size, load as
    dense f32 bit-exactly (device kernel against the oracle's BlockQ6K::to_float) and as projections;
    a type the library has no kernel for (Q5_K) is refused."""
    import torch
    from izwi_amd.capi import QmmError
    n, k = 24, 1024
    nb = n * k // 256
    b = np_ref.random_q6_k_blocks(16, n, k).reshape(nb, 210)
    hand = bytes.fromhex(json.load(open(os.path.join(HERE, "golden", "q6k_hand_block.json")))["block_hex"])
    path = str(tmp_path / "q6.gguf")
    gw.write_gguf(path, [], [("blk.0.ffn_down.weight", (n, k), 14, b.tobytes()), ("hand", (1, 256), 14, hand),
                             ("q5", (2, 256), 13, bytes(2 * 176))])
    g = qa.GgufLoader.from_path(path)
    assert g.tensor_dtype("blk.0.ffn_down.weight") == 14 and g._info("blk.0.ffn_down.weight").nbytes == nb * 210
    assert g.get_model_info().quantization == "mixed:Q5K,Q6K"
    want = oracle.dequantize(14, b.reshape(-1), n, k)
    for device in ("cuda", "cpu"):
        got = g.load_tensor("blk.0.ffn_down.weight", device=device).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    fx = json.load(open(os.path.join(HERE, "golden", "q6k_hand_block.json")))
    assert np.array_equal(g.load_tensor("hand").cpu().numpy().reshape(-1), np.array(fx["expected_f32"], dtype=np.float32))
    q = g.load_qtensor("blk.0.ffn_down.weight")
    assert q.dtype() == qa.GgmlDType.Q6K and q.shape() == (n, k) and np.array_equal(q.data(), b.reshape(-1))
    assert np.array_equal(q.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    x = oracle.randn(17, (2, k))
    y = qa.QMatMul.from_qtensor(q).forward(torch.from_numpy(x).cuda()).cpu().numpy()
    ref = oracle.qmatmul(14, x, b.reshape(-1), n)
    assert np.abs(y - ref).max() <= 1e-4 * np.abs(ref).max()
    with pytest.raises(QmmError) as e:
        g.load_qtensor("q5")
    assert e.value.code == -2


@pytest.mark.gpu
def test_load_packed_matches_packing_separately_loaded_tensors(qa, oracle, tmp_path):
    import torch
    path, blocks, _, _ = _model_file(tmp_path, oracle)
    g = qa.GgufLoader.from_path(path)
    names = ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.attn_v.weight"]
    packed = g.load_packed_qmatmul(names)
    want = qa.packed_qmatmul_from_qtensors([(qa.GgmlDType(blocks[n][0]), blocks[n][3], blocks[n][1:3]) for n in names])
    x = torch.from_numpy(oracle.randn(3, (2, 64))).cuda()
    assert torch.equal(packed.forward(x), want.forward(x))
    assert packed.forward(x).shape == (2, 160)
    from izwi_amd.capi import QmmError
    with pytest.raises(QmmError, match="mismatch"):
        g.load_packed_qmatmul(["blk.0.attn_q.weight", "blk.0.ffn_gate.weight"])
    with pytest.raises(QmmError, match="mismatch"):
        g.load_packed_qmatmul(["blk.0.ffn_gate.weight", "blk.0.ffn_down.weight"])
