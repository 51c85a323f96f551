"""Builds (g++, AddressSanitizer + UBSan, host only) and runs tests/host_io_test.cpp: the C++ record reader,
tokenizers and generation helpers of burn_dragon_amd/host/bdh_host_io.hpp on the CPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_host_io_helpers(tmp_path):
    exe = str(tmp_path / "host_io_test")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", os.path.join(ROOT, "tests", "host_io_test.cpp"), "-o", exe]
    subprocess.check_call(cmd)
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "verify_asan_link_order=0:detect_leaks=0"  # other preloaded libraries may come first
    proc = subprocess.run([exe, os.path.join(ROOT, "tests", "golden", "tiny_shakespeare")], capture_output=True,
                          text=True, timeout=120, env=env)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip().endswith("OK")
