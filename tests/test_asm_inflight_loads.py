"""The attention kernels issue some loads as asm that the compiler does not count (the Q
operands; the token ids): their destination registers are valid only behind a hand-placed
vmcnt wait.  To the compiler those registers hold their values from the moment the asm
statement ends, so nothing stops it from copying or spilling them while the load is still in
flight.  This test compiles the three attention translation units to assembly (no GPU needed)
and checks that between every such load and the first wait that covers it no other instruction
names its destination registers.

The HBM -> LDS copies set m0 inside their asm statement without telling the compiler (naming a
reserved register as clobbered only draws a warning).  That is sound as long as the compiler
itself never uses m0 in these kernels: the second check asserts that no instruction outside an
asm statement names m0 in any translation unit that issues such copies."""
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

import pytest

from fgattn_tk_cuda_amd import build

CSRC = Path(build.__file__).resolve().parent / "csrc"
UNITS = ["attn_inst_blocks.hip", "attn_inst_tokens.hip", "attn_inst_dense.hip"]
M0_UNITS = UNITS + ["mask_kernels.hip"]


def _regs(text):
    out = set()
    for m in re.finditer(r"\b([va])\[(\d+):(\d+)\]", text):
        out.update(m.group(1) + str(i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
    for m in re.finditer(r"\b([va])(\d+)\b", text):
        out.add(m.group(1) + m.group(2))
    return out


def _is_vmem(op):
    return op.startswith(("global_load", "global_store", "scratch_load", "scratch_store", "buffer_", "flat_"))


def inflight_accesses(listing):
    """[(line of the access, line of the load)] for a straight-line scan of an assembly listing."""
    lines = listing.split("\n")
    found = []
    for n, raw in enumerate(lines):
        t = raw.strip().split(";")[0].strip()
        if not t.startswith("global_load_dword") or t.startswith("global_load_lds"):
            continue
        dst = _regs(t.split(None, 1)[1].split(",")[0])
        younger = 0
        for j in range(n + 1, min(n + 6000, len(lines))):
            t2 = lines[j].strip().split(";")[0].strip()
            if not t2 or t2.startswith("."):
                continue
            if re.match(r"^_Z\w+:", lines[j]):
                break
            op = t2.split()[0]
            if op == "s_endpgm":
                break
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", t2)
                if m and int(m.group(1)) <= younger:
                    break          # every load up to ours has landed
                continue
            if " " in t2 and _regs(t2.split(None, 1)[1]) & dst:
                found.append((j + 1, n + 1, t2, t))
                break
            if _is_vmem(op):
                younger += 1
    return found


def m0_uses_outside_asm(listing):
    """Lines outside ASMSTART/ASMEND blocks whose instruction names m0."""
    found, inside = [], False
    for n, raw in enumerate(listing.split("\n")):
        if "#ASMSTART" in raw:
            inside = True
            continue
        if "#ASMEND" in raw:
            inside = False
            continue
        t = raw.split(";")[0].strip()
        if not inside and t and not t.startswith(".") and re.search(r"\bm0\b", t):
            found.append((n + 1, t))
    return found


def test_m0_checker_sees_a_compiler_use():
    ok = "\t;;#ASMSTART\n\ts_mov_b32 m0, s3\n\tglobal_load_lds_dwordx4 v1, s[0:1]\n\t;;#ASMEND\n\tv_mov_b32_e32 v2, v3\n"
    bad = ok + "\ts_mov_b32 m0, -1\n"
    assert m0_uses_outside_asm(ok) == []
    assert len(m0_uses_outside_asm(bad)) == 1


def test_checker_sees_an_access_to_a_register_in_flight():
    bad = "\tglobal_load_dwordx4 v[4:7], v[2:3], off\n\tglobal_load_lds_dwordx4 v9, s[0:1]\n\tv_mov_b32_e32 v20, v5\n\ts_waitcnt vmcnt(0)\n"
    good = "\tglobal_load_dwordx4 v[4:7], v[2:3], off\n\tglobal_load_lds_dwordx4 v9, s[0:1]\n\ts_waitcnt vmcnt(1)\n\tv_mov_b32_e32 v20, v5\n"
    assert len(inflight_accesses(bad)) == 1
    assert inflight_accesses(good) == []


@pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(), reason="hipcc not found")
def test_no_instruction_touches_a_register_with_a_load_in_flight(tmp_path):
    hipcc = build._hipcc()

    def listing(unit):
        out = tmp_path / (unit + ".s")
        subprocess.run([hipcc, *build.HIPCC_FLAGS, "-S", "--cuda-device-only", "-o", str(out), str(CSRC / unit)],
                       check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        return out.read_text()

    with ThreadPoolExecutor(max_workers=4) as ex:
        texts = list(ex.map(listing, M0_UNITS))
    for unit, text in zip(M0_UNITS, texts):
        assert "global_load_lds_dwordx4" in text, unit
        uses = m0_uses_outside_asm(text)
        assert not uses, "%s: the compiler uses m0 next to hand-written copies: %s" % (unit, uses[:3])
        if unit not in UNITS:
            continue
        assert "global_load_dword" in text, unit
        found = inflight_accesses(text)
        assert not found, "%s: %s" % (unit, found[:3])
