"""Builds tests/host_mirror_test.bin (test infrastructure: links the product library and, as the
checker, the C oracle).  Called by __graft_entry__.build()."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def build_host_test(verbose: bool = False) -> str:
    """Builds tests/host_mirror_test.bin: the C++ host mirror (host/bdh_host.hpp) exercised with the
    reference's test recipes; links the library and, as the checker, the C oracle."""
    root = ROOT
    PKG = os.path.join(ROOT, 'burn_dragon_amd')
    out = os.path.join(root, "tests", "host_mirror_test.bin")
    cmd = [HIPCC, "-O2", "-std=c++17", "-x", "c++", os.path.join(root, "tests", "host_mirror_test.cpp"), "-o", out,
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-L" + PKG, "-lbdh_mi355x", "-L" + os.path.join(root, "oracle"), "-lbdh_oracle", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../burn_dragon_amd", "-Wl,-rpath,$ORIGIN/../oracle", "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    print(build_host_test(verbose=True))
