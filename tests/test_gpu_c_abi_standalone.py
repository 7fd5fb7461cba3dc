"""The C ABI from a caller that is neither Python nor torch: tests/c_abi/standalone.cpp (built beforehand by
__graft_entry__.build()) appends, evicts and attends with hipMalloc'd buffers and checks the results against its own loops."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "standalone")


def test_standalone_cpp_caller():
    assert os.path.exists(BINARY), "tests/c_abi/standalone is not built: run __graft_entry__.build()"
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0 and "C-ABI standalone: OK" in proc.stdout, proc.stdout
