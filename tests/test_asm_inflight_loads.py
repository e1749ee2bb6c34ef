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
asm statement names m0 in any translation unit that issues such copies.

The tile loop of the attention kernels waits for its copies with hand-counted vmcnt values: that
holds only while the compiler puts no vector-memory instruction of its own into the loop.  The
third check finds the tile loop of every instantiation (one inner loop, closed by a branch back to
its header) and asserts that it holds no scratch access (a spill) and no s_waitcnt vmcnt outside
the asm statements (the compiler waiting for a load of its own)."""
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


def tile_loop_findings(listing):
    """{kernel: (scratch accesses, compiler vmcnt waits)} inside the tile loop of every attn_fwd_kernel
    instantiation of a listing; a kernel whose loop is not found maps to None."""
    out, name, cur = {}, None, []
    for line in listing.split("\n"):
        m = re.match(r"^(_ZN6spattn15attn_fwd_kernel\w+):", line)
        if m:
            name, cur = m.group(1), []
        if name is None:
            continue
        cur.append(line)
        if not line.startswith(".Lfunc_end"):
            continue
        hdr = next(((i, l.split(":")[0]) for i, l in enumerate(cur) if l.startswith(".LBB") and "Loop Header" in l), None)
        last = None
        if hdr is not None:
            back = re.compile(r"s_c?branch\w*\s+" + re.escape(hdr[1]) + r"\b")
            last = max((i for i in range(hdr[0], len(cur)) if back.match(cur[i].strip())), default=None)
        if hdr is None or last is None:
            out[name] = None
        else:
            scratch = waits = 0
            inside = False
            for l in cur[hdr[0]:last + 1]:
                if "#ASMSTART" in l:
                    inside = True
                elif "#ASMEND" in l:
                    inside = False
                t = l.split(";")[0].strip()
                scratch += t.startswith("scratch_")
                waits += (not inside) and t.startswith("s_waitcnt") and "vmcnt" in t
            out[name] = (scratch, waits)
        name = None
    return out


def test_tile_loop_checker():
    body = ("_ZN6spattn15attn_fwd_kernelILi64EEEvNS_10AttnParamsE:\n\ts_nop 0\n.LBB0_3:   ; =>This Inner Loop Header: Depth=1\n"
            "\t;;#ASMSTART\n\ts_waitcnt vmcnt(4)\n\t;;#ASMEND\n%s\ts_cbranch_scc1 .LBB0_3\n\ts_endpgm\n.Lfunc_end0:\n")
    assert tile_loop_findings(body % "") == {"_ZN6spattn15attn_fwd_kernelILi64EEEvNS_10AttnParamsE": (0, 0)}
    assert list(tile_loop_findings(body % "\tscratch_load_dword v1, off, off\n\ts_waitcnt vmcnt(0)\n").values()) == [(1, 1)]
    assert list(tile_loop_findings(body.replace("s_cbranch_scc1 .LBB0_3", "s_nop 1") % "").values()) == [None]


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
        loops = tile_loop_findings(text)
        assert len(loops) >= 4, "%s: %d attention kernels found" % (unit, len(loops))
        for kernel, f in loops.items():
            assert f == (0, 0), "%s %s: tile loop not found, or scratch accesses / compiler vmcnt waits inside it: %s" % (unit, kernel, f)
