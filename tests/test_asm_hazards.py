"""The prefill attention kernel issues LDS reads and MFMAs as hand-written instructions whose results the compiler
believes to be present as soon as the instruction has been issued.  Two classes of mistakes follow from that, both
silent at compile time and sporadic at run time:

  * an instruction the compiler places (a register copy on a branch edge, a spill, an address computation in a register
    it considers free) touches a register while the read that fills it is still in flight;
  * an instruction the compiler places reads an MFMA's result without the wait states the hardware needs between the
    two, because the compiler keeps that distance only for MFMAs it can see.

This test compiles the kernels' translation unit to gfx950 assembly (no GPU needed) and scans every instance of the
kernel for both.  The scanners are themselves checked against short listings that contain each mistake.
"""
import os
import re
import subprocess

import pytest

from seq2seqsharp_amd import build as B

KERNEL = re.compile(r"^(_ZN5tship24attn_mfma_prefill_kernel\w+):")


def _regs(tok):
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", tok)
    return {int(m.group(1))} if m else set()


def _kernels(text):
    """-> {name: [(line number, instruction text, written by hand)]}"""
    out, name, inasm = {}, None, False
    for ln, line in enumerate(text.split("\n"), 1):
        m = KERNEL.match(line)
        if m:
            name = m.group(1)
            out[name] = []
            continue
        if name is None:
            continue
        if line.startswith(".Lfunc_end"):
            name = None
            continue
        s = line.strip()
        if s.startswith(";;#ASMSTART"):
            inasm = True
        elif s.startswith(";;#ASMEND"):
            inasm = False
        elif s and not s.startswith(";") and (not s.startswith(".") or s.startswith(".LBB")):
            out[name].append((ln, s, inasm))
    return out


def reads_in_flight(instrs):
    """Findings: instructions that touch the destination of a hand-written ds_read_b128 before an lgkmcnt wait covers
    it, and branches or labels reached with such reads pending (the compiler may copy registers on an edge)."""
    pend, bad = [], []
    for ln, s, inasm in instrs:
        op = s.split()[0]
        toks = [t.strip(",") for t in s.split()[1:]]
        if s.startswith(".LBB"):
            if pend:
                bad.append((ln, "label with %d reads pending" % len(pend)))
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", s)
            if m:
                n = int(m.group(1))
                pend = pend[len(pend) - n:] if n else []
            continue
        if op == "ds_read_b128" and inasm:
            pend.append(_regs(toks[0]))
            continue
        if op.startswith("s_cbranch") or op == "s_branch":
            if pend:
                bad.append((ln, "branch with %d reads pending" % len(pend)))
            continue
        used = set().union(*[_regs(t) for t in toks]) if toks else set()
        hot = set().union(*pend) if pend else set()
        if used & hot:
            bad.append((ln, "'%s' touches registers of a read in flight" % s))
    return bad


def mfma_results_read_early(instrs, distance=20):
    """Findings: instructions other than MFMAs that use the destination of a hand-written MFMA fewer than `distance`
    issue slots behind it (s_nop n counts n + 1; the hardware's largest requirement for this MFMA shape is below 20)."""
    bad, n = [], len(instrs)
    for i, (l0, s0, a0) in enumerate(instrs):
        if not (a0 and s0.startswith("v_mfma")):
            continue
        dst = _regs(s0.split()[1].strip(","))
        dist = 0
        for j in range(i + 1, min(n, i + 60)):
            l1, s1, _ = instrs[j]
            op = s1.split()[0]
            if op == "s_nop":
                dist += int(s1.split()[1]) + 1
            elif op == "s_branch":
                break
            elif op.startswith("s_") or s1.startswith(".LBB") or op.startswith("ds_") or op.startswith("global_"):
                dist += 1
            else:
                used = set().union(*[_regs(t.strip(",")) for t in s1.split()[1:]])
                if used & dst and not op.startswith("v_mfma"):
                    bad.append((l1, "'%s' %d slots behind the MFMA at line %d" % (s1, dist, l0)))
                dist += 4 if op.startswith("v_mfma") else 1
            if dist >= distance:
                break
    return bad


def _listing(body):
    return "_ZN5tship24attn_mfma_prefill_kernelILi64ELi4ELb0ELi1EEEvNS_8AttnArgsE:\n" + body + "\n.Lfunc_end0:\n"


def test_scanners_find_each_mistake():
    asm = lambda s: ";;#ASMSTART\n\t%s\n;;#ASMEND" % s
    ok = _listing("\n".join([asm("ds_read_b128 v[2:5], v9 offset:0"), "\tv_add_f32_e32 v8, v7, v6",
                             asm("s_waitcnt lgkmcnt(0)"), "\tv_mov_b32_e32 v4, v10"]))
    assert reads_in_flight(_kernels(ok).popitem()[1]) == []
    # a register of the read used as an address before the wait
    late = _listing("\n".join([asm("ds_read_b128 v[2:5], v9 offset:0"), "\tv_lshl_add_u64 v[4:5], s[4:5], 0, v[68:69]",
                               asm("s_waitcnt lgkmcnt(0)")]))
    assert reads_in_flight(_kernels(late).popitem()[1])
    # a wait count that leaves the read outstanding
    count = _listing("\n".join([asm("ds_read_b128 v[2:5], v9 offset:0"), asm("ds_read_b128 v[12:15], v9 offset:1024"),
                                asm("s_waitcnt lgkmcnt(1)"), "\tv_mov_b32_e32 v20, v13"]))
    assert reads_in_flight(_kernels(count).popitem()[1])
    # a copy on a branch edge before the wait
    edge = _listing("\n".join([asm("ds_read_b128 v[2:5], v9 offset:0"), "\ts_cbranch_scc1 .LBB0_2", ".LBB0_2:",
                               "\tv_mov_b64_e32 v[20:21], v[2:3]", asm("s_waitcnt lgkmcnt(0)")]))
    assert reads_in_flight(_kernels(edge).popitem()[1])
    # an MFMA's result copied two instructions behind it; fine behind enough idle instructions
    mf = asm("v_mfma_f32_16x16x32_f16 v[26:29], v[50:53], v[60:63], v[26:29]")
    early = _listing("\n".join([mf, "\tv_max_f32_e32 v1, v2, v3", "\tv_mov_b32_e32 v40, v27"]))
    assert mfma_results_read_early(_kernels(early).popitem()[1])
    padded = _listing("\n".join([mf, asm("s_nop 15\n\ts_nop 15"), "\tv_mov_b32_e32 v40, v27"]))
    assert mfma_results_read_early(_kernels(padded).popitem()[1]) == []


@pytest.mark.timeout(900)
def test_prefill_attention_assembly_has_neither_mistake(tmp_path):
    if not os.path.exists(B.HIPCC):
        pytest.skip("hipcc is not installed")
    out = tmp_path / "tship_gpt.s"
    cmd = [B.HIPCC] + B.FLAGS + ["--cuda-device-only", "-S", os.path.join(B.CSRC, "tship_gpt.hip"), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    kernels = _kernels(out.read_text())
    assert len(kernels) >= 32                      # head sizes 64 / 128, 1 / 2 / 4 / 8 query heads per KV head, plain / padded, one / two column groups
    for name, instrs in kernels.items():
        assert any(a and s.startswith("ds_read_b128") for _, s, a in instrs), name
        assert any(a and s.startswith("v_mfma") for _, s, a in instrs), name
        assert reads_in_flight(instrs) == [], name
        assert mfma_results_read_early(instrs) == [], name
