"""Register budgets of the kernels that count their own outstanding loads or were sized against a
register limit: none of them may spill to scratch memory.  A spill would cost a scratch segment at
every dispatch, and in `q4k_rows16_kernel` it could copy a register that a hand-issued load has not
filled yet.  Compiles the device code only (no GPU needed) with the library's own flags and reads the
compiler's resource remarks."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tessera_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# file -> kernels (substring of the mangled name) that must not use scratch memory
NO_SCRATCH = {
    "gemv_q4k_rows16.hip": ["q4k_rows16_kernel"],
    "gemv_kquant_rows.hip": ["kquant_rows_kernel"],
    "gemv_q4k_i8.hip": ["q4k_i8_gemv_kernel"],
}


def resource_remarks(src):
    makefile = open(os.path.join(CSRC, "Makefile")).read()
    assert "-packed-fp32-ops" in makefile      # the flags below restate the library's
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++20", "-fno-gpu-rdc", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "--cuda-device-only", "-c", "-o", os.devnull, "-Rpass-analysis=kernel-resource-usage",
           os.path.join(CSRC, src)]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    kernels, name = {}, None
    for line in out.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
        m = re.search(r"(ScratchSize \[bytes/lane\]|VGPRs|VGPR Spill): (\d+)", line)
        if m and name is not None:
            kernels[name][m.group(1)] = int(m.group(2))
    return kernels


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not found")
@pytest.mark.parametrize("src", sorted(NO_SCRATCH))
def test_no_scratch_memory(src):
    kernels = resource_remarks(src)
    for want in NO_SCRATCH[src]:
        hits = {k: v for k, v in kernels.items() if want in k}
        assert hits, f"no kernel named *{want}* in {src}"
        for name, res in hits.items():
            assert res.get("ScratchSize [bytes/lane]", 0) == 0, (name, res)
            assert res.get("VGPR Spill", 0) == 0, (name, res)
