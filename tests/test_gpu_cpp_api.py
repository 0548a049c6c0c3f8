"""The C++ host API (include/mi355_fused_moe.hpp: fused_moe_traits / fused_moe_args / fused_moe())
driven from a compiled C++ program, as CK's example main drives its own API."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "host_api_check")


def test_cpp_host_api_matches_oracle():
    assert os.path.exists(EXE), "tests/cpp/host_api_check is not built (run __graft_entry__.build())"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
