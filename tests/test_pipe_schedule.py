"""The compiled form of the hand-scheduled matmul kernels: no spill traffic and no compiler-made wait for vector
memory between a kernel's first and last MFMA (either one silently drains the operand loads that the schedule keeps
in flight; results stay right, the kernel gets slower).  Compiles each instantiation to assembly with hipcc; nothing
runs on a GPU."""
import importlib.util
import os
import shutil

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SCRIPT = os.path.join(HERE, "check_pipe_schedule.py")
spec = importlib.util.spec_from_file_location("check_pipe_schedule", SCRIPT)
chk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(chk)

pytestmark = pytest.mark.skipif(not (os.path.exists(chk.HIPCC) or shutil.which("hipcc")), reason="needs hipcc")


@pytest.mark.parametrize("kernel,own_waits", chk.KERNELS, ids=[k for k, _ in chk.KERNELS])
def test_scheduled_stream_is_free_of_spills_and_foreign_waits(kernel, own_waits, tmp_path):
    problems = chk.check(kernel, own_waits, str(tmp_path))
    assert not problems, "\n".join(problems[:10])
