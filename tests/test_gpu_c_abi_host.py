"""Runs tests/c_abi_host.cpp: a compiled C++ caller of the C ABI (hipMalloc'd buffers, a HIP stream, no Python and no
torch in the process) that checks quantise / dequantise bit for bit against the scalar C oracle and the fused forward
and backward against double-precision loops.  The executable is built by ``__graft_entry__.build()``."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "_build", "c_abi_host")


def test_cpp_host_of_the_c_abi_passes_its_parity_checks():
    if not os.path.exists(EXE):
        pytest.fail("tests/_build/c_abi_host is missing: run `python -c 'import __graft_entry__ as g; g.build()'` first")
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all checks passed" in proc.stdout
    assert proc.stdout.count(" ok") >= 10 and "FAILED" not in proc.stdout
