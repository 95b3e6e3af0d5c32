"""No MFMA kernel may spill registers to scratch memory: the device code is compiled with
-Rpass-analysis=kernel-resource-usage (no GPU needed) and every la_* / la32_* kernel has to report
ScratchSize 0 and at least two waves per SIMD.  A spilling instantiation still computes the right
thing, only slower, so nothing else would notice."""
import os
import re
import subprocess

import pytest

from lasp_amd import build

SOURCES = ["lasp_mfma.hip", "lasp_mfma_f32.hip"]


def _resource_report(src):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [hipcc, *flags, "--cuda-device-only", "-c", os.path.join(build.CSRC, src), "-o", os.devnull,
           "-Rpass-analysis=kernel-resource-usage"]
    err = subprocess.run(cmd, check=True, capture_output=True, text=True).stderr
    kernels, name = {}, None
    for line in err.splitlines():
        m = re.search(r"remark: .*Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+(VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]): (\d+)", line)
        if m and name:
            kernels[name][m.group(1).split(" ")[0]] = int(m.group(2))
    return kernels


@pytest.mark.parametrize("src", SOURCES)
def test_mfma_kernels_use_no_scratch(src):
    kernels = {k: v for k, v in _resource_report(src).items() if re.search(r"\d+la(32)?_[a-z0-9_]+I", k)}
    assert len(kernels) >= 8, f"expected the la_* kernels of {src} in the compiler's report, got {sorted(kernels)}"
    spilling = {k: v for k, v in kernels.items() if v.get("ScratchSize", -1) != 0}
    assert not spilling, f"kernels with scratch: {spilling}"
    low = {k: v for k, v in kernels.items() if v.get("Occupancy", 0) < 2}
    assert not low, f"kernels below two waves per SIMD: {low}"
