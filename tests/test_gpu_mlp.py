"""GPU tests of the whole-MLP call (pytest -m gpu): `Qwen3Mlp::forward`
(crates/izwi-core/src/models/architectures/qwen3/core.rs:1786-1798) through izwi_qmm_mlp_forward_f32
against the two calls it stands for (gate/up with the activation, then down), bit for bit, over the
row counts that take its different routes, and against the oracle's composition of the same steps."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import izwi_amd
    return izwi_amd


def _mm(qa, dtype, n, k, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    return qa.QMatMul.from_qtensor(qa.QTensor.quantize(w.cuda(), qa.GgmlDType(dtype)))


# (gate / up type, down type, hidden, intermediate)
STACKS = [(12, 12, 1024, 3072), (8, 8, 512, 1024), (12, 8, 768, 2048), (8, 12, 256, 512)]
ROWS = [1, 2, 3, 7, 16, 33, 64, 65, 130]


@pytest.mark.parametrize("gu_type,d_type,hidden,inter", STACKS)
def test_mlp_call_equals_the_two_calls(qa, gu_type, d_type, hidden, inter):
    gate, up = _mm(qa, gu_type, inter, hidden, 1), _mm(qa, gu_type, inter, hidden, 2)
    down = _mm(qa, d_type, hidden, inter, 3)
    gate_up = qa.Qwen3GateUpProjection.new_separate(gate, up)
    mlp = qa.Qwen3Mlp(gate_up, down)
    for m in ROWS:
        print(f"mlp types={gu_type}/{d_type} hidden={hidden} inter={inter} m={m}", flush=True)
        x = torch.randn(m, hidden, generator=torch.Generator(device="cpu").manual_seed(10 + m)).cuda()
        want = down.forward(gate_up.forward_silu_mul(x))
        got = mlp.forward(x)
        assert torch.equal(got, want)
        assert torch.equal(mlp.forward(x), got)  # and again on the same scratch


def test_mlp_call_with_gate_and_up_of_two_block_types_is_refused_like_the_pair_call(qa):
    from izwi_amd import capi
    gate, up, down = _mm(qa, 12, 1024, 512, 4), _mm(qa, 8, 1024, 512, 5), _mm(qa, 12, 512, 1024, 6)
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up), down)
    for m in (1, 5, 100):
        with pytest.raises(capi.QmmError, match="different ggml dtypes"):
            mlp.forward(torch.randn(m, 512).cuda())


def test_mlp_call_on_host_pointers_and_after_other_sizes(qa):
    gate, up, down = _mm(qa, 12, 2048, 1024, 7), _mm(qa, 12, 2048, 1024, 8), _mm(qa, 12, 1024, 2048, 9)
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up), down)
    for m in (130, 5, 1, 64, 3):
        x = torch.randn(m, 1024, generator=torch.Generator(device="cpu").manual_seed(20 + m))
        assert torch.equal(mlp.forward(x), mlp.forward(x.cuda()).cpu())


def test_mlp_call_against_the_oracle(qa):
    from oracle import oracle
    hidden, inter = 512, 768
    gate, up, down = _mm(qa, 12, inter, hidden, 11), _mm(qa, 12, inter, hidden, 12), _mm(qa, 12, hidden, inter, 13)
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up), down)
    for m in (1, 6):
        x = torch.randn(m, hidden, generator=torch.Generator(device="cpu").manual_seed(30 + m))
        g = oracle.qmatmul(12, x.numpy(), gate.qtensor.data(), inter)
        u = oracle.qmatmul(12, x.numpy(), up.qtensor.data(), inter)
        h = (g / (1.0 + np.exp(-g.astype(np.float32)))).astype(np.float32) * u
        want = oracle.qmatmul(12, h, down.qtensor.data(), hidden)
        got = mlp.forward(x.cuda()).cpu().numpy()
        # the intermediate is quantized again for down: one int8 step of h where silu's last bit differs
        assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max()


def test_mlp_call_rejects_shapes_that_do_not_chain(qa):
    from izwi_amd import capi
    gate, up = _mm(qa, 8, 512, 256, 1), _mm(qa, 8, 512, 256, 2)
    down_bad = _mm(qa, 8, 256, 1024, 3)
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up), down_bad)
    with pytest.raises(capi.QmmError, match="shape mismatch in qmatmul"):
        mlp.forward(torch.randn(2, 256).cuda())
    up_bad = _mm(qa, 8, 768, 256, 4)
    mlp = qa.Qwen3Mlp(qa.Qwen3GateUpProjection.new_separate(gate, up_bad), _mm(qa, 8, 256, 512, 5))
    with pytest.raises(capi.QmmError, match="gate is"):
        mlp.forward(torch.randn(2, 256).cuda())
