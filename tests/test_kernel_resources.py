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


# ---- generated code: no wide store whose data registers are overwritten in the next slot -------------------------
# A buffer or global store of 12 or 16 bytes reads its data registers a cycle after it issues.  The compiler lets a
# vector instruction overwrite the first data register in the very next slot when the store takes its offset from a
# scalar register; on gfx950 the stored dword was then the overwriting instruction's result (found in a wave that
# stored 16-byte pieces in a loop: the first dword of every piece was the LDS address of the next one).  The kernels
# put an s_nop that names the data registers behind such stores (buf_store_then_nop in csrc/frnn_common.h); this test
# disassembles the device code of every object of the build and looks for the pattern, so that a kernel that acquires
# it with some later change fails here and not as a rare wrong value.
LLVM = "/opt/rocm/lib/llvm/bin"
OBJS = os.path.join(ROOT, "flashrnn_amd", "csrc", "build", "*.o")


def _vregs(op):
    m = re.match(r"v\[(\d+):(\d+)\]", op)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", op)
    return {int(m.group(1))} if m else set()


def _store_hazards(disassembly):
    hits, kernel, prev = [], "?", None
    for line in disassembly.splitlines():
        m = re.match(r"[0-9a-f]+ <(\S+)>:", line)
        if m:
            kernel, prev = m.group(1), None
            continue
        t = line.split("//")[0].strip()
        if not t or t.endswith(":"):
            continue
        parts = t.split(None, 1)
        op = parts[0]
        args = [a.strip() for a in parts[1].split(",")] if len(parts) > 1 else []
        if prev is not None and args and op.startswith(("v_", "ds_read", "buffer_load", "global_load")) \
                and not op.startswith(("v_cmp", "v_nop")):
            if _vregs(args[0]) & prev[1]:
                hits.append(f"{kernel}: {prev[0]}  ->  {t}")
        prev = None
        if re.match(r"(buffer|global)_store_dwordx[34]\b", op):
            prev = (t, _vregs(args[0] if op.startswith("buffer") else args[1]))
    return hits


def _disassemble(obj, tmp):
    import subprocess

    base = os.path.join(tmp, os.path.basename(obj))
    r = subprocess.run([f"{LLVM}/llvm-objcopy", "--dump-section", f".hip_fatbin={base}.fatbin", obj, f"{base}.copy"],
                       capture_output=True, text=True)
    if r.returncode != 0 or not os.path.exists(f"{base}.fatbin"):
        return None  # (an object without device code)
    subprocess.run([f"{LLVM}/clang-offload-bundler", "--unbundle", "--type=o", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
                    f"--input={base}.fatbin", f"--output={base}.co"], check=True, capture_output=True)
    return subprocess.run([f"{LLVM}/llvm-objdump", "-d", f"{base}.co"], check=True, capture_output=True, text=True).stdout


def test_the_scanner_finds_the_pattern_it_is_looking_for():
    bad = """0000000000001000 <k>:
\tbuffer_store_dwordx4 v[2:5], v36, s[4:7], s0 offen        // 0000: E07C1000
\tv_lshl_add_u32 v2, v32, 1, s3                             // 0008: D1FD0002
\tbuffer_store_dwordx4 v[6:9], v36, s[4:7], s0 offen        // 0010: E07C1000
\ts_nop 0                                                   // 0018: BF800000
\tv_lshl_add_u32 v6, v32, 1, s3                             // 001c: D1FD0002
\tglobal_store_dwordx3 v1, v[10:12], s[0:1]                 // 0024: DC000000
\tds_read_b128 v[12:15], v0                                 // 002c: D9FE0000
\tbuffer_store_dwordx2 v[2:3], v36, s[4:7], s0 offen        // 0034: E0741000
\tv_mov_b32_e32 v2, 0                                       // 003c: 7E040280
"""
    hits = _store_hazards(bad)
    assert len(hits) == 2 and "v_lshl_add_u32 v2" in hits[0] and "ds_read_b128" in hits[1], hits


def test_no_wide_store_has_its_data_registers_overwritten_in_the_next_slot(tmp_path):
    from concurrent.futures import ThreadPoolExecutor

    objs = sorted(glob.glob(OBJS))
    if not objs:
        pytest.fail(f"no objects under {OBJS}: build the library first (make -C flashrnn_amd/csrc)")
    if not os.path.exists(f"{LLVM}/llvm-objdump"):
        pytest.skip("no llvm-objdump in this image")
    with ThreadPoolExecutor(max_workers=8) as pool:
        texts = list(pool.map(lambda o: _disassemble(o, str(tmp_path)), objs))
    scanned = [t for t in texts if t]
    assert len(scanned) >= 40, len(scanned)
    assert sum(t.count("buffer_store_dwordx4") for t in scanned) > 1000     # (the scan saw real code)
    hits = [h for t in scanned for h in _store_hazards(t)]
    assert not hits, f"{len(hits)} stores whose data registers are overwritten in the next slot:\n" + "\n".join(hits[:40])
