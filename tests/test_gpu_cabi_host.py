"""The C ABI from a host that is not Python: tests/cabi_host (plain C++, HIP runtime memory, no PyTorch)
runs forward, values-only forward, backward with the hand-over and the selection count, and compares
them with the C oracle itself.  The program is built beforehand by tests/Makefile."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
PROGRAM = os.path.join(HERE, "cabi_host")


@pytest.mark.parametrize("shape", [(64, 784, 256), (70, 123, 45), (256, 4096, 512)])
def test_plain_cpp_host(shape):
    if not os.path.exists(PROGRAM):
        pytest.fail("tests/cabi_host is not built: run `make -C tests` (or __graft_entry__.build())")
    r = subprocess.run([PROGRAM] + [str(v) for v in shape] + ["7"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.rstrip().endswith("PASS"), r.stdout
