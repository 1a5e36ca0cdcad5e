"""The two forms of the grouped matrix-core kernel (izwi_qmm_set_moe_expert_form /
IZWI_QMM_MOE_EXPERT_FORM): by default the library picks one per call from the number of pairs per
expert; here the MoE parity tests run once more, in this process, with each form forced, so that every
case reports on its own."""
import pytest

# the tests themselves (collected here a second time, with their parameters) and the fixtures they use
from test_gpu_parity import (  # noqa: F401
    moe_weights,
    qa,
    test_config5_moe_forward,
    test_config5_moe_layer_one_call_equals_the_three_calls,
    test_moe_forward_small_shapes,
)
from test_gpu_q6k import test_moe_with_q6_k_expert_stacks  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=[1, 0], ids=["expert_form", "one_shot_form"])
def forced_form(request):
    from izwi_amd import capi
    capi.check(capi.lib().izwi_qmm_set_moe_expert_form(request.param))
    yield
    capi.check(capi.lib().izwi_qmm_set_moe_expert_form(-1))  # back to the choice by size


@pytest.mark.parametrize("t", [128, 512])
def test_tile_path_is_repeatable(qa, oracle, moe_weights, t):
    """The same call four times: identical bits.  (A counted wait on the weight panel's loads that was
    one short - the compiler drops the load of a header nobody uses - let a workgroup start before the
    last piece of its activation tiles had landed: results changed from run to run at 8 pairs per
    expert, where the tiles are one short copy.)"""
    import torch
    E, hidden, inter, gate, up, down = moe_weights
    dt = qa.GgmlDType.Q4K
    experts = qa.MoeExperts(qa.QTensor.from_blocks(dt, gate, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, up, (E, inter, hidden)),
                            qa.QTensor.from_blocks(dt, down, (E, hidden, inter)))
    x = torch.from_numpy(oracle.randn(690 + t, (t, hidden))).cuda()
    logits = torch.from_numpy(oracle.randn(691 + t, (t, E))).cuda()
    outs = [experts.layer(logits, x, 8) for _ in range(4)]
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o.view(torch.int32), outs[0].view(torch.int32))
