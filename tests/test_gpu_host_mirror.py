"""GPU: runs the C++ host-mirror test binary (tests/cpp/test_host_mirror, built by
__graft_entry__.build()): prefill through NTsAttn::TAttentionComputer against the oracle, then a
token-by-token replay through NTsAttn::TAttentionVecHistory + ComputeValLookup."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_host_mirror")


def test_cpp_host_mirror():
    assert os.path.exists(BIN), "build it with `make -C tests/cpp` (done by __graft_entry__.build())"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ALL OK" in r.stdout
