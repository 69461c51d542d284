"""The C++ host side (tessera_amd/host: Backend, ProjectBatch, GemmVecSplit) through the C ABI.

tests/host/host_parity.cpp drives the reference's regime table over the C++ Backend mirror and
checks every case against the oracle; this file builds it where a compiler is present, checks
the split rule's documented values on the CPU, and runs the program on the GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "tests", "host")
BIN = os.path.join(HOST, "host_parity")


def ensure_built():
    if not os.path.exists(BIN) and shutil.which("g++"):
        subprocess.run(["make", "-C", HOST], check=True, capture_output=True)
    return os.path.exists(BIN)


def test_host_program_builds_and_lists_cases():
    assert ensure_built(), "tests/host/host_parity is not built and no g++ is available"
    out = subprocess.run([BIN, "--list"], check=True, capture_output=True, text=True).stdout
    assert "gemm_q4k_wmma" in out and "gemm_mxfp4_wmma" in out and len(out.splitlines()) >= 9


def test_split_rule_values():
    """GemmVecSplit (src/core/decode_internal.hpp:864-885) on the shapes the reference documents:
    N=17408 -> 2176 blocks >= 2048 -> 1; N=5120, K=17408 -> 640 blocks, want 4, 68 % 4 == 0 -> 4;
    N=K=5120 -> 20 super-blocks, want 4 -> 4.  Evaluated from the C++ header via a tiny program."""
    src = os.path.join(HOST, "_split_check.cpp")
    exe = os.path.join(HOST, "_split_check")
    with open(src, "w") as f:
        f.write('#include "../../tessera_amd/host/project.hpp"\n#include <cstdio>\n'
                'int main(){using namespace tessera_amd; std::printf("%zu %zu %zu %zu\\n", GemmVecSplit(17408,5120),'
                ' GemmVecSplit(5120,17408), GemmVecSplit(5120,5120), GemmVecSplit(64,256));}\n')
    try:
        subprocess.run(["g++", "-std=c++20", "-fsyntax-only", src], check=True, capture_output=True)
        subprocess.run(["g++", "-std=c++20", "-o", exe, src, "-L" + os.path.join(ROOT, "tessera_amd"), "-ltessera_qmm",
                        "-Wl,-rpath," + os.path.join(ROOT, "tessera_amd"), "-Wl,-rpath,/opt/rocm/lib"],
                       check=True, capture_output=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
        assert out == ["1", "4", "4", "1"]
    finally:
        for p in (src, exe):
            if os.path.exists(p):
                os.remove(p)


@pytest.mark.gpu
def test_host_parity_on_gpu():
    assert os.path.exists(BIN), "build tests/host/host_parity before the GPU run"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
