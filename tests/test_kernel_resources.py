"""Register budget of the hot kernels, from the compiler's own resource report (no GPU needed).

A spill to scratch memory inside a streaming loop puts a memory round trip in front of every
tile: measured at +40 % on a layer-sized launch.  Some builds sit exactly at a register limit
(the five-wave form of the lean kernel at 96 VGPRs), so a small edit can tip them over without any
test of results noticing.  This test recompiles both GEMV libraries with
-Rpass-analysis=kernel-resource-usage and checks the kernels the dispatcher picks by default."""
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from bitmtp_amd import build

CSRC = build.CSRC


def _resource_report(source: str) -> dict:
    cmd = [os.environ.get("HIPCC", "hipcc")] + build.HIPCC_FLAGS + [
        "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, source), "-o", os.devnull]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    demangle = subprocess.run(["c++filt"], input=proc.stdout, stdout=subprocess.PIPE, text=True).stdout
    report, cur = {}, None
    for line in demangle.splitlines():
        m = re.search(r"Function Name: (.*?) \[-Rpass", line)
        if m:
            cur = re.sub(r"^void ", "", m.group(1))
            cur = re.sub(r"\(.*$", "", cur)          # drop the argument list
            report[cur] = {}
            continue
        for key, tag in (("VGPRs", "vgprs"), (r"ScratchSize \[bytes/lane\]", "scratch"),
                         (r"Occupancy \[waves/SIMD\]", "occupancy")):
            m = re.search(key + r": (\d+)", line)
            if m and cur is not None:
                report[cur][tag] = int(m.group(1))
    return report


@pytest.fixture(scope="module")
def reports():
    with ThreadPoolExecutor(max_workers=2) as pool:
        t2, q1 = pool.map(_resource_report, ("t2g128_kernels.hip", "q1g128_kernels.hip"))
    assert any("gemv_mxl_kernel" in k for k in t2) and any("gemv_mxl_kernel" in k for k in q1)
    return {2: t2, 1: q1}


def _select(report, pattern):
    return {k: v for k, v in report.items() if re.search(pattern, k)}


@pytest.mark.parametrize("bits", [2, 1])
def test_default_kernels_do_not_spill(reports, bits):
    rep = reports[bits]
    hot = {}
    hot.update(_select(rep, r"gemv_mxl_kernel<"))                      # lean matrix-core kernel, every build
    hot.update(_select(rep, r"gemv_mxs_kernel<"))                      # streaming kernel
    hot.update(_select(rep, r"gemv_rowreg_kernel<"))                   # single-token head kernel (T2 only)
    hot.update(_select(rep, rf"gemv_dot4_grouped_kernel<{bits}, 1, "))  # grouped dot4, one token
    hot.update(_select(rep, rf"gemv_dot4_grouped_kernel<{bits}, 2, [12],"))
    hot.update(_select(rep, rf"gemv_dot4_kernel<{bits}, 1, \d, false"))  # single GEMV, one token
    hot.update(_select(rep, rf"gemv_dot4_kernel<{bits}, 2, [12], false"))
    assert len(hot) >= 20
    spilled = {k: v["scratch"] for k, v in hot.items() if v["scratch"] != 0}
    assert not spilled, f"kernels with scratch memory: {spilled}"


@pytest.mark.parametrize("bits", [2, 1])
def test_lean_kernel_residency(reports, bits):
    """Blocks of at most eight tokens (NB = 1, four waves per workgroup) leave room for five waves
    per SIMD, which is what makes the 1280 workgroups of a layer-sized launch resident at once."""
    # (the last template argument is the output kind: false = scaled result, true = group sums)
    rep = _select(reports[bits], rf"gemv_mxl_kernel<{bits}, 4, (true|false), 4, 1, 5, false>")
    assert len(rep) == 2
    for name, v in rep.items():
        assert v["occupancy"] >= 5 and v["vgprs"] <= 96, (name, v)
    five_wave_two_batch = _select(reports[bits], rf"gemv_mxl_kernel<{bits}, 4, (true|false), 4, 2, 5, (true|false)>")
    assert len(five_wave_two_batch) == 3
    for name, v in five_wave_two_batch.items():
        assert v["occupancy"] >= 5 and v["scratch"] == 0, (name, v)
