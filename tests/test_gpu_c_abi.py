"""Runs the plain-C ABI program (tests/c/abi_layer_ops.c) on the GPU: the
library linked and called from C, with the system HIP runtime and no Python or
torch in the process, the way the reference's C engine would use it."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "c", "abi_layer_ops")


@pytest.mark.gpu
def test_c_program_links_and_passes():
    assert os.path.exists(EXE), "tests/c/abi_layer_ops is not built: run __graft_entry__.build()"
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-4000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-2000:]
    assert "all C ABI checks passed" in res.stdout and "FAIL" not in res.stdout


def test_c_program_is_built_against_the_public_header():
    src = open(os.path.join(HERE, "c", "abi_layer_ops.c")).read()
    assert '#include "vibevoice_hip.h"' in src and "hip_runtime" not in src
