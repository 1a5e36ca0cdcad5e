"""The optional expert form of the grouped matrix-core kernel (IZWI_QMM_MOE_EXPERT_FORM=1, read once per
process): the MoE parity tests once more in a child process with the switch on."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_moe_parity_with_the_expert_form():
    here = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, IZWI_QMM_MOE_EXPERT_FORM="1")
    cmd = [sys.executable, "-u", "-m", "pytest", "-x", "-q", "-m", "gpu", "--timeout", "120", "--timeout-method", "thread",
           "-k", "moe_forward_small_shapes or moe_with_q6_k_expert_stacks or config5_moe_forward",
           os.path.join(here, "test_gpu_parity.py"), os.path.join(here, "test_gpu_q6k.py")]
    out = subprocess.run(cmd, env=env, cwd=os.path.dirname(here), capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-2000:]
    assert " passed" in out.stdout and "failed" not in out.stdout
