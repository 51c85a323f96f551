"""Runs the C++ host-mirror test program (tests/host_mirror_test.cpp, built in-tree by
__graft_entry__.build()) on the GPU: the reference's test recipes written against
burn_dragon_amd/host/bdh_host.hpp, values checked against the C oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host_mirror_test.bin")


@pytest.mark.gpu
def test_cpp_host_mirror():
    assert os.path.exists(BIN), "tests/host_mirror_test.bin is not built (python -c 'import __graft_entry__ as g; g.build()')"
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.pathsep.join([os.path.join(ROOT, "burn_dragon_amd"), os.path.join(ROOT, "oracle"),
                                              "/opt/rocm/lib", env.get("LD_LIBRARY_PATH", "")])
    proc = subprocess.run([BIN, os.path.join(ROOT, "tests", "golden", "tiny_shakespeare")], capture_output=True, text=True, timeout=120, env=env)
    print(proc.stdout, proc.stderr)
    assert proc.returncode == 0, f"exit status {proc.returncode}\n{proc.stdout}{proc.stderr}"
    assert proc.stdout.strip().endswith("OK")
