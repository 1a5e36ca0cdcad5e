"""Writes the golden fixtures of this directory.

Neither fixture comes from running the reference (it cannot be built here, and the crate
that holds the arithmetic is not in its tree).  They restate, as data:

* q4k_hand_block.json - one Q4_K block built from the public GGUF block format with the
  answers of its closed form y = d * sc * q - dmin * m worked out independently of any
  code under test (all 256 values; the scale bytes exercise both branches of the 6-bit
  unpacking).
* packed_q8_0_case.json - the inputs of the reference's own unit test
  `packed_qmatmul_matches_separate_q8_0_on_cpu`
  (crates/izwi-core/src/models/architectures/qwen3/core.rs:3099-3142), their Q8_0 block
  bytes and the outputs of candle-core's algorithm on them, computed here with plain
  numpy arithmetic (no code of the oracle or of the library is used).

* q6k_hand_block.json - one Q6_K block (a load-time codec: GGUF ingress to dense f32) built
  the same way, all 256 values of y = d * scale * (q - 32) from per-element index arithmetic.
* tiny.gguf + tiny_gguf.json - a small GGUF version 3 file assembled byte by byte from the
  public container format (no writer or reader of this repository is used), and what a
  reader must report for it; its Q4_K tensor is the hand block above.

Run:  python tests/golden/make_fixtures.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def q4k_hand_block():
    d, dmin = np.float16(1.0), np.float16(0.5)
    scales = bytes([0x41, 0x82, 0xC3, 0xC4, 0x40, 0x85, 0xCA, 0xCF, 0x41, 0x82, 0xC3, 0xFF])
    qs = bytes(range(128))
    block = d.tobytes() + dmin.tobytes() + scales + qs
    assert len(block) == 144
    sc = [1, 2, 3, 4, 17, 34, 51, 63]   # what the twelve scale bytes encode
    mn = [0, 5, 10, 15, 20, 40, 60, 63]
    y = np.zeros(256, dtype=np.float64)
    for g in range(4):                   # 64 elements: 32 low nibbles, then 32 high nibbles
        for l in range(32):
            b = qs[32 * g + l]
            y[64 * g + l] = 1.0 * sc[2 * g] * (b & 15) - 0.5 * mn[2 * g]
            y[64 * g + 32 + l] = 1.0 * sc[2 * g + 1] * (b >> 4) - 0.5 * mn[2 * g + 1]
    assert y.sum() == 32224.0 and y[224] == 346.5 and y[255] == 409.5 and y[32] == -2.5
    return {"ggml_dtype": 12, "rows": 1, "cols": 256, "block_hex": block.hex(),
            "scales": sc, "mins": mn, "expected_f32": [float(v) for v in y], "expected_sum": 32224.0}


def q8_0_quantize_rows(w):
    """BlockQ8_0::from_float: d = amax / 127 (stored as f16), q = round(x / d) with d in f32."""
    rows, cols = w.shape
    out = bytearray()
    scale_bits = []
    for r in range(rows):
        for b in range(cols // 32):
            v = w[r, 32 * b:32 * b + 32].astype(np.float32)
            amax = np.float32(np.abs(v).max())
            d = np.float32(amax / np.float32(127.0))
            inv = np.float32(1.0) / d if d != 0 else np.float32(0.0)
            q = np.clip(np.sign(v * inv) * np.floor(np.abs(v * inv) + np.float32(0.5)), -128, 127).astype(np.int8)
            h = np.float16(d)
            scale_bits.append(int(h.view(np.uint16)))
            out += h.tobytes() + q.tobytes()
    return bytes(out), scale_bits


def q8_0_vec_dot(wblocks, xblocks, k):
    """sum over blocks of (sum q_w * q_x) * d_w * d_x, accumulated in f32 in block order."""
    acc = np.float32(0.0)
    for b in range(k // 32):
        wb, xb = wblocks[34 * b:34 * b + 34], xblocks[34 * b:34 * b + 34]
        dw = np.float32(np.frombuffer(wb[:2], np.float16)[0])
        dx = np.float32(np.frombuffer(xb[:2], np.float16)[0])
        s = int(np.dot(np.frombuffer(wb[2:], np.int8).astype(np.int32), np.frombuffer(xb[2:], np.int8).astype(np.int32)))
        acc = np.float32(acc + np.float32(s) * np.float32(dw * dx))
    return acc


def packed_case():
    idx = np.arange(64, dtype=np.float32)
    w1 = ((idx - 31.0) / 8.0).reshape(2, 32)
    w2 = ((15.0 - idx[:32]) / 7.0).reshape(1, 32)
    x = ((idx[:32] + 1.0) / 16.0).reshape(1, 32)
    b1, s1 = q8_0_quantize_rows(w1)
    b2, s2 = q8_0_quantize_rows(w2)
    bx, sx = q8_0_quantize_rows(x)      # the activation row is quantized the same way
    packed = b1 + b2                     # packed_qmatmul_from_qtensors: byte concatenation
    y = [float(q8_0_vec_dot(packed[34 * r:34 * r + 34], bx, 32)) for r in range(3)]
    assert s1 + s2 == [10192, 10248, 9372] and sx == [9224]
    assert np.allclose(y, [-42.692207, 89.229607, -26.613434], rtol=0, atol=2e-6)
    return {"ggml_dtype": 8, "k": 32,
            "w1_f32": [float(v) for v in w1.reshape(-1)], "w1_rows": 2,
            "w2_f32": [float(v) for v in w2.reshape(-1)], "w2_rows": 1,
            "x_f32": [float(v) for v in x.reshape(-1)],
            "w1_blocks_hex": b1.hex(), "w2_blocks_hex": b2.hex(), "x_blocks_hex": bx.hex(),
            "weight_scale_f16_bits": s1 + s2, "activation_scale_f16_bits": sx,
            "expected_y": y, "exact_math_y": [-42.625, 89.375, -26.714286],
            "reference_tolerance_packed_vs_separate": 1e-5}


def q6k_hand_block():
    """One Q6_K block from the public block format (ql[128], qh[64], int8 scales[16], f16 d) with
    every value of y = d * scale * (q - 32) worked out element by element."""
    ql = bytes((7 * i + 3) % 256 for i in range(128))
    qh = bytes((13 * i + 5) % 256 for i in range(64))
    scales = [1, -2, 3, -4, 5, -6, 7, -8, 9, 10, -11, 12, 127, -128, 64, -1]
    d = np.float16(0.25)
    block = ql + qh + bytes(v & 0xFF for v in scales) + d.tobytes()
    assert len(block) == 210
    y = np.zeros(256, dtype=np.float64)
    for e in range(256):
        half, r = divmod(e, 128)      # which 128-element half
        g, l = divmod(r, 32)          # group 0..3 inside the half, position 0..31
        byte = ql[64 * half + 32 * (g % 2) + l]
        low = (byte & 0xF) if g < 2 else (byte >> 4)
        high = (qh[32 * half + l] >> (2 * g)) & 3
        q = (low | (high << 4)) - 32
        y[e] = 0.25 * scales[8 * half + 2 * g + l // 16] * q   # exact in f32: small integers times 2^-2
    return {"ggml_dtype": 14, "rows": 1, "cols": 256, "block_hex": block.hex(), "scales": scales,
            "expected_f32": [float(v) for v in y], "expected_sum": float(y.sum())}


def tiny_gguf():
    """A GGUF version 3 file laid out by hand from the public container format: header, three
    metadata entries (alignment 64), three tensor infos, padding, data.  Returns the file's
    bytes and what a reader must report."""
    import struct

    def s(text):
        b = text.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    f32 = np.array([[1.0, 2.0], [3.0, 4.0]], dtype=np.float32).tobytes()
    q8 = np.float16(1.0).tobytes() + bytes(np.arange(-16, 16, dtype=np.int8).view(np.uint8))
    q4 = bytes.fromhex(q4k_hand_block()["block_hex"])
    head = b"GGUF" + struct.pack("<IQQ", 3, 3, 3)
    head += s("general.architecture") + struct.pack("<I", 8) + s("qwen3")
    head += s("general.alignment") + struct.pack("<I", 4) + struct.pack("<I", 64)
    head += s("test.ids") + struct.pack("<I", 9) + struct.pack("<IQ", 2, 3) + struct.pack("<HHH", 1, 2, 3)
    # dims are written innermost first; offsets are multiples of the alignment
    head += s("a") + struct.pack("<I", 2) + struct.pack("<QQ", 2, 2) + struct.pack("<IQ", 0, 0)
    head += s("blk.q") + struct.pack("<I", 2) + struct.pack("<QQ", 32, 1) + struct.pack("<IQ", 8, 64)
    head += s("hand.q4k") + struct.pack("<I", 2) + struct.pack("<QQ", 256, 1) + struct.pack("<IQ", 12, 128)
    data_offset = (len(head) + 63) // 64 * 64
    blob = head + bytes(data_offset - len(head))
    blob += f32 + bytes(64 - len(f32)) + q8 + bytes(64 - len(q8)) + q4
    want = {"header": [3, 64, data_offset],
            "metadata": {"general.architecture": "qwen3", "general.alignment": 64, "test.ids": [1, 2, 3]},
            "tensors": [
                {"name": "a", "shape": [2, 2], "ggml_dtype": 0, "offset": 0, "bytes_hex": f32.hex()},
                {"name": "blk.q", "shape": [1, 32], "ggml_dtype": 8, "offset": 64, "bytes_hex": q8.hex()},
                {"name": "hand.q4k", "shape": [1, 256], "ggml_dtype": 12, "offset": 128, "bytes_hex": q4.hex()}],
            "dequantized": {"a": [1.0, 2.0, 3.0, 4.0], "blk.q": [float(v) for v in range(-16, 16)],
                            "hand.q4k": q4k_hand_block()["expected_f32"]}}
    return blob, want


if __name__ == "__main__":
    blob, want = tiny_gguf()
    with open(os.path.join(HERE, "tiny.gguf"), "wb") as f:
        f.write(blob)
    with open(os.path.join(HERE, "tiny_gguf.json"), "w") as f:
        json.dump(want, f, indent=1)
    print("wrote tiny.gguf, tiny_gguf.json")
    for name, rec in (("q4k_hand_block.json", q4k_hand_block()), ("packed_q8_0_case.json", packed_case()),
                      ("q6k_hand_block.json", q6k_hand_block())):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(rec, f, indent=1)
        print("wrote", name)
