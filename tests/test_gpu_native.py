"""The C ABI used without Python or torch: a stand-alone C++ program
(tests/native/cabi_smoke.cc, built by `python -m shmtensor_amd.build native`)
links libshmt.so and checks every operator family against host loops."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "cabi_smoke.bin")


def test_c_abi_standalone_program():
    assert os.path.exists(BIN), "tests/native/cabi_smoke.bin is not built (python -m shmtensor_amd.build native)"
    res = subprocess.run([BIN], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout
    assert "all checks passed" in res.stdout
