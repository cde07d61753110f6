"""No compiled kernel may spill registers to scratch memory.  The build passes
-Rpass-analysis=kernel-resource-usage to hipcc and keeps the compiler's report of every kernel instantiation in
flashrnn_amd/csrc/build/*.o.log; this test reads those reports.  A tiling that would spill at some batch-tile
height is not compiled that tall (the MTR column of csrc/frnn_plan.h), so a new instantiation that spills fails
here instead of shipping."""
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LOGS = os.path.join(ROOT, "flashrnn_amd", "csrc", "build", "*.o.log")


def _reports():
    out = {}
    for path in sorted(glob.glob(LOGS)):
        name = None
        for line in open(path, errors="replace"):
            m = re.search(r"remark: Function Name: (\S+)", line)
            if m:
                name = m.group(1)
                out[name] = {"file": os.path.basename(path)}
                continue
            m = re.search(r"remark:\s+(ScratchSize \[bytes/lane\]|VGPRs Spill|SGPRs Spill|VGPRs|AGPRs|Dynamic Stack): (\S+)", line)
            if m and name:
                out[name][m.group(1)] = m.group(2)
    return out


def test_no_kernel_uses_scratch_memory():
    rep = _reports()
    if not rep:
        pytest.fail(f"no compiler reports under {LOGS}: build the library first (make -C flashrnn_amd/csrc)")
    fused = [k for k in rep if "fused_fwd_kernel" in k or "fused_bwd_kernel" in k]
    assert len(fused) > 500, len(fused)          # every (cell, type, tiling, tile height) is there
    assert any("grad_gemm16_kernel" in k for k in rep) and any("alt_step_fwd_kernel" in k for k in rep)
    # (the report's "VGPRs Spill" also counts values parked in accumulation registers, which cost a move, not a
    # memory access: the large-head kernels do that by design; scratch memory is what must not happen)
    bad = {k: v for k, v in rep.items()
           if int(v.get("ScratchSize [bytes/lane]", "0")) > 0 or v.get("Dynamic Stack", "False") != "False"}
    assert not bad, "kernels that spill:\n" + "\n".join(f"  {k} ({v['file']}): {v}" for k, v in sorted(bad.items()))
