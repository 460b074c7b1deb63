"""Compile-time guard for the hand-scheduled kernels (no GPU needed: hipcc cross-compiles).

The table-major kernels issue global -> LDS copies as inline assembly and wait for them with
hand-counted `s_waitcnt vmcnt(n)`.  Two things keep that sound and neither is visible in the source:

  * the four-lanes-per-token gather (lookup_gather_quad.hip) and the score-gradient kernel
    (lookup_inner_quad.hip) must not spill: a spilling variant of the former once moved registers
    to scratch while loads into them were in flight and ended in a GPU memory fault, and the
    latter's wait leaves an exact number of compiler-visible loads in flight across a barrier;
  * the older LDS kernels (lookup_gather.hip, lookup_gather_pair.hip, lookup_inner.hip) write no
    register from inline assembly and wait with vmcnt(0) / vmcnt(1) only, where an extra scratch
    access makes a wait stricter, never weaker; their largest tiles are known to spill a few
    registers, which costs time, not correctness.  Any other instantiation that starts to spill
    is reported here.

The compiler's own remark (-Rpass-analysis=kernel-resource-usage) is the evidence.
"""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from lookupffn_amd import _build

STRICT = ["lookup_gather_quad.hip", "lookup_inner_quad.hip"]
LDS_FORMS = ["lookup_gather.hip", "lookup_gather_pair.hip", "lookup_inner.hip"]
# instantiations of the older kernels that are known to spill (fp32 rows, 13 and 16 passes)
MAY_SPILL = re.compile(r"lookup_gather_lds_kernelILb0ELi1[36]E|lookup_gather_pair_kernelILb0ELi16E")


def _resource_usage(src):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    cmd = [hipcc, *_build.HIPCC_FLAGS, "--cuda-device-only", "-c", os.path.join(_build.CSRC, src), "-o", os.devnull,
           "-Rpass-analysis=kernel-resource-usage"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    kernels, name = {}, None
    for line in res.stderr.splitlines():
        m = re.search(r"remark:\s+Function Name:\s+(\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?:\s+(\S+) \[-Rpass", line)
        if m and name is not None:
            kernels[name][m.group(1).strip()] = m.group(2)
    return src, kernels


@pytest.fixture(scope="module")
def usage():
    with ThreadPoolExecutor(max_workers=4) as ex:
        return dict(ex.map(_resource_usage, STRICT + LDS_FORMS))


def _uses_scratch(k):
    return int(k["ScratchSize"]) != 0 or int(k["VGPRs Spill"]) != 0 or k["Dynamic Stack"] != "False"


def test_remarks_are_parsed(usage):
    for src, kernels in usage.items():
        assert kernels, src
        for name, k in kernels.items():
            assert {"ScratchSize", "VGPRs Spill", "SGPRs Spill", "VGPRs", "Dynamic Stack"} <= set(k), (src, name, k)
    assert sum("lookup_gather_quad_kernel" in n for n in usage["lookup_gather_quad.hip"]) >= 4
    assert sum("lookup_inner_quad_kernel" in n for n in usage["lookup_inner_quad.hip"]) >= 2


@pytest.mark.parametrize("src", STRICT)
def test_hand_scheduled_kernels_do_not_spill(usage, src):
    bad = {n: k for n, k in usage[src].items() if _uses_scratch(k) or int(k["SGPRs Spill"]) != 0}
    assert not bad, f"{src}: these kernels spill: {bad}"


@pytest.mark.parametrize("src", LDS_FORMS)
def test_lds_kernels_spill_only_where_known(usage, src):
    # (scalar registers spilled into vector-register lanes touch no memory and are not counted)
    bad = {n: k for n, k in usage[src].items() if _uses_scratch(k) and not MAY_SPILL.search(n)}
    assert not bad, f"{src}: new spills: {bad}"
