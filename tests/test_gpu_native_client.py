"""Runs the C++ client of the C ABI (tests/native/abi_client.cpp): a compiled caller that sees only include/yka_abi.h,
as the reference engine would.  It checks device-pointer calls against the host-pointer hooks and a captured pass
replayed at a new position; here its exit status and last line are checked."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CLIENT = os.path.join(HERE, "native", "abi_client")


def test_cpp_client_of_the_c_abi():
    assert os.path.exists(CLIENT), "tests/native/abi_client is not built: run `python -c 'import __graft_entry__ as g; g.build()'`"
    p = subprocess.run([CLIENT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert p.returncode == 0, p.stdout[-2000:]
    assert p.stdout.strip().splitlines()[-1] == "abi_client ok", p.stdout[-2000:]
