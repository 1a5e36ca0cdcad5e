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
