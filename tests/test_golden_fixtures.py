"""The committed golden fixtures (tests/golden/*.json, written by tests/golden/make_fixtures.py)
against the CPU oracle and, on a GPU, against the library through its C ABI."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
Q8_0, Q4_K = 8, 12


def load(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def blocks(hex_string):
    return np.frombuffer(bytes.fromhex(hex_string), dtype=np.uint8).copy()


# ---- CPU: the oracle ----------------------------------------------------------
def test_oracle_q4k_hand_block_fixture(oracle):
    fx = load("q4k_hand_block.json")
    y = oracle.dequantize(Q4_K, blocks(fx["block_hex"]), fx["rows"], fx["cols"])[0]
    assert np.array_equal(y, np.array(fx["expected_f32"], dtype=np.float32))
    assert float(y.astype(np.float64).sum()) == fx["expected_sum"]


def test_oracle_q6k_hand_block_fixture(oracle):
    """Q6_K is a load-time codec (GGUF ingress to dense f32); the oracle's restatement of
    BlockQ6K::to_float against the hand-built block and against an independent numpy version."""
    import np_ref
    fx = load("q6k_hand_block.json")
    want = np.array(fx["expected_f32"], dtype=np.float32)
    y = oracle.dequantize(14, blocks(fx["block_hex"]), 1, 256)[0]
    assert np.array_equal(y, want) and float(y.astype(np.float64).sum()) == fx["expected_sum"]
    assert np.array_equal(np_ref.dequant_q6_k(blocks(fx["block_hex"]), 1, 256)[0], want)
    # random block bytes with finite scales: the two restatements agree bit for bit
    rng = np.random.default_rng(6)
    nb = 64
    b = rng.integers(0, 256, nb * 210, dtype=np.uint8).reshape(nb, 210)
    b[:, 208:210] = (rng.standard_normal(nb) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
    a = oracle.dequantize(14, b.reshape(-1), 8, 2048)
    c = np_ref.dequant_q6_k(b.reshape(-1), 8, 2048)
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    assert oracle.storage_bytes(14, 8, 2048) == nb * 210


def test_oracle_packed_q8_0_fixture(oracle):
    fx = load("packed_q8_0_case.json")
    k = fx["k"]
    w1 = np.array(fx["w1_f32"], dtype=np.float32).reshape(fx["w1_rows"], k)
    w2 = np.array(fx["w2_f32"], dtype=np.float32).reshape(fx["w2_rows"], k)
    x = np.array(fx["x_f32"], dtype=np.float32).reshape(1, k)
    # the oracle's quantizers reproduce the fixture's block bytes
    assert np.array_equal(oracle.quantize(Q8_0, w1), blocks(fx["w1_blocks_hex"]))
    assert np.array_equal(oracle.quantize(Q8_0, w2), blocks(fx["w2_blocks_hex"]))
    assert np.array_equal(oracle.quantize_activations(Q8_0, x), blocks(fx["x_blocks_hex"]))
    packed = np.concatenate([blocks(fx["w1_blocks_hex"]), blocks(fx["w2_blocks_hex"])])
    y = oracle.qmatmul(Q8_0, x, packed, 3)[0]
    assert np.allclose(y, np.array(fx["expected_y"], dtype=np.float32), rtol=0, atol=2e-6)


def test_oracle_q4k_scale_search_closed_forms(oracle):
    """`make_qkx1_quants` against sub-blocks whose answer the algorithm's mathematics fixes
    (tests/golden/make_q4k_quantizer_vectors.py: exact grids, the clamp of min, a constant, a
    three-pass and a cut-off five-pass refinement, a round-half-away tie)."""
    fx = load("q4k_quantizer_cases.json")
    assert (fx["nmax"], fx["ntry"]) == (15, 5)
    for case in fx["sub_blocks"]:
        x = np.array(case["x"], dtype=np.float32)
        assert np.array_equal(x.astype(np.float64), np.array(case["x"])), "inputs are exact in f32"
        scale, neg_min = oracle.make_qkx1_quants(x)
        if case["exact_in_f32"]:
            num, den = (np.float32(v) for v in case["scale_num_den"])
            want = np.float32(0.0) if den == 0 or num == 0 else num / den
            assert scale == want and np.float32(case["neg_min"]) == neg_min, case["name"]
        else:
            # f32 sums of 32 terms of size <= 15 round on the way: a few 1e-6; a wrong variant of
            # the search is off by more than 4e-3
            assert abs(scale - case["scale"]) <= 1e-5 * case["scale"], case["name"]
            assert abs(neg_min - case["neg_min"]) <= 2e-5, case["name"]
    # what the cases rule out: no refinement, a shorter or longer search, ties to even
    by = {c["name"]: c for c in fx["sub_blocks"]}
    three = np.array(by["three_passes"]["x"], dtype=np.float32)
    assert [float(oracle.make_qkx1_quants(three, ntry=t)[0]) for t in (1, 2, 3)] == [
        float(np.float32(266.25) / np.float32(255)), float(np.float32(251.25) / np.float32(226)),
        float(np.float32(236.25) / np.float32(199))]
    cut = np.array(by["five_pass_cutoff"]["x"], dtype=np.float32)
    assert abs(oracle.make_qkx1_quants(cut, ntry=6)[0] - by["five_pass_cutoff"]["scale"]) > 4e-3


def test_oracle_q4k_quantizer_block_vectors(oracle):
    """`BlockQ4K::from_float` byte for byte on blocks whose bytes follow in closed form."""
    import np_ref
    fx = load("q4k_quantizer_cases.json")
    for case in fx["blocks"]:
        x = np.array(case["x"], dtype=np.float32).reshape(1, 256)
        assert np.array_equal(x.astype(np.float64).reshape(-1), np.array(case["x"]))
        got = oracle.quantize(Q4_K, x)
        want = blocks(case["block_hex"])
        d, dmin, sc, mn, q = np_ref.q4_k_fields(got)
        assert list(sc[0]) == case["scale_codes"] and list(mn[0]) == case["min_codes"], case["name"]
        assert list(q.reshape(-1)) == case["quants"], case["name"]
        assert np.array_equal(got, want), case["name"]
    # grid blocks dequantize back to their inputs exactly when d and dmin are exact
    case = fx["blocks"][0]
    back = oracle.dequantize(Q4_K, blocks(case["block_hex"]), 1, 256)[0]
    assert np.array_equal(back, np.array(case["x"], dtype=np.float32))


# ---- GPU: the library ---------------------------------------------------------
@pytest.fixture(scope="module")
def qa():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import izwi_amd
    izwi_amd.lib()
    return izwi_amd


@pytest.mark.gpu
def test_device_q4k_hand_block_fixture(qa):
    fx = load("q4k_hand_block.json")
    q = qa.QTensor.from_blocks(qa.GgmlDType.Q4K, blocks(fx["block_hex"]), (fx["rows"], fx["cols"]))
    y = q.dequantize().cpu().numpy()[0]
    assert np.array_equal(y, np.array(fx["expected_f32"], dtype=np.float32))
    assert np.array_equal(q.data(), blocks(fx["block_hex"]))


@pytest.mark.gpu
def test_device_packed_q8_0_fixture(qa):
    import torch
    fx = load("packed_q8_0_case.json")
    k = fx["k"]
    dt = qa.GgmlDType.Q8_0
    x = torch.tensor(fx["x_f32"], dtype=torch.float32).reshape(1, k).cuda()
    b1, b2 = blocks(fx["w1_blocks_hex"]), blocks(fx["w2_blocks_hex"])
    packed = qa.packed_qmatmul_from_qtensors([(dt, b1, (fx["w1_rows"], k)), (dt, b2, (fx["w2_rows"], k))])
    y = packed.forward(x).cpu().numpy()[0]
    sep = np.concatenate([qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b1, (fx["w1_rows"], k))).forward(x).cpu().numpy()[0],
                          qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(dt, b2, (fx["w2_rows"], k))).forward(x).cpu().numpy()[0]])
    # the reference's own assertion, then the absolute values
    assert np.abs(y - sep).max() <= fx["reference_tolerance_packed_vs_separate"]
    assert np.allclose(y, np.array(fx["expected_y"], dtype=np.float32), rtol=0, atol=1e-5)
    # the on-chip activation quantizer writes the fixture's activation block
    xq = qa.quantize_activations(dt, x)
    assert np.array_equal(np.asarray(xq.cpu()).reshape(-1), blocks(fx["x_blocks_hex"]))
