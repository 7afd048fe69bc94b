"""Register, scratch and LDS budget of the join kernels, read from the compiler's resource remarks.

The join kernels keep the next tile's global->LDS transfers in flight across their epilogue; a register
spill there would be reloaded from scratch memory, and a scratch reload waits for every outstanding
vector-memory operation of the wave.  So "no scratch" is a property the design depends on, and one that a
compiler or source change can lose silently.  hipcc cross-compiles for gfx950 without a GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LDS_PER_CU = 160 * 1024


def kernel_resources():
    """{demangled-ish kernel name: {field: int}} from `make resources`."""
    proc = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "fasted_amd", "csrc"), "resources"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out, current = {}, None
    for line in proc.stderr.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            current = out.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z /\[\]]+?)(?: \[[^\]]*\])?: (\d+) \[-Rpass", line)
        if m and current is not None:
            current[m.group(1).strip()] = int(m.group(2))
    return out


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not installed")
def test_join_kernels_use_no_scratch_and_fit_one_cu():
    res = kernel_resources()
    joins = {k: v for k, v in res.items() if "join_kernel" in k}
    # both instantiations (with and without the fused epilogue) of every tile variant
    assert len(joins) >= 2, sorted(res)
    for name, r in joins.items():
        assert r["ScratchSize"] == 0, (name, r)
        assert r["VGPRs Spill"] == 0, (name, r)
        # scalar registers that do not fit are parked in lanes of a vector register, not in memory: harmless in
        # small numbers (each costs a vector instruction where it is used)
        assert r["SGPRs Spill"] <= 12, (name, r)
        assert r["VGPRs"] + r["AGPRs"] <= 256, (name, r)  # two waves per SIMD
        assert r["Occupancy"] >= 2, (name, r)
        assert 0 < r["LDS Size"] <= LDS_PER_CU, (name, r)
    # the other kernels are small: nothing spills anywhere in the file
    for name, r in res.items():
        assert r["ScratchSize"] == 0, (name, r)
