"""The bf16 / e4m3 GEMM issues some of its global loads from inline assembly (operand half-stages on their way to LDS
through registers, the E8M0 scale dwords of block-scaled activations), so that the only waits on them are the
explicit `s_waitcnt vmcnt(N)` of the loop.  The compiler keeps no book on such a load: it takes the destination
registers for written when the instruction issues.  Two things can then go wrong without any diagnostic, and did
once: a register whose load is still in flight is handed to another value (at the loop's exit, where the loads
asked for past the last stage have no reader), or a value is read, copied or spilled before it has landed.

This test compiles the kernel file for gfx950 and walks every kernel's instruction stream: from an untracked load
until the point that is known to be behind its wait (the LDS write or the scale shift that consumes it, or a full
`vmcnt(0)`), no other instruction may name the load's destination registers.  CPU only: hipcc cross-compiles."""
import os
import re
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "..", "glades-ml_amd", "csrc", "gemm_lp.hip")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def vregs(tok):
    out = set()
    for a, b in re.findall(r"v\[(\d+):(\d+)\]", tok):
        out.update(range(int(a), int(b) + 1))
    for a in re.findall(r"\bv(\d+)\b", tok):
        out.add(int(a))
    return out


def kernels(lines):
    """(name, first line, last line) of every kernel of the file"""
    starts = [(i, l.split(":")[0]) for i, l in enumerate(lines) if re.match(r"^_Z\w*gemm_lp\w*:", l)]
    for i, name in starts:
        end = next(k for k in range(i, len(lines)) if "s_endpgm" in lines[k])
        yield name, i, end


def violations(lines):
    found, loads = [], 0
    for name, lo, hi in kernels(lines):
        fp8 = "ILb1E" in name
        inflight = {}
        for i in range(lo, hi):
            ins = lines[i].split(";")[0].strip()
            m = re.match(r"(\S+)\s+(.*)", ins)
            if not m or ins.endswith(":") or ins.startswith("."):
                continue
            op, parts = m.group(1), [a.strip() for a in m.group(2).split(",")]
            # the untracked loads: scalar base + per-lane offset, into registers
            if op in ("global_load_dwordx4", "global_load_dword") and len(parts) >= 3 and parts[2].startswith("s["):
                for r in vregs(parts[0]):
                    inflight[r] = i
                loads += 1
                continue
            if op == "s_waitcnt" and "vmcnt(0)" in m.group(2):
                inflight.clear()
                continue
            if op == "ds_write_b128":          # the half-stage's way on into LDS, behind its counted wait
                for r in vregs(parts[1]):
                    inflight.pop(r, None)
                continue
            if fp8 and op == "v_lshrrev_b32_e32":   # a stage's scale dword, two stages after it was asked for
                for r in vregs(parts[2]):
                    inflight.pop(r, None)
                continue
            touched = set()
            for p in parts:
                touched |= vregs(p)
            hit = sorted(r for r in touched if r in inflight)
            if hit:
                found.append((name, i - lo, ins, hit, inflight[hit[0]] - lo))
                for r in hit:
                    inflight.pop(r, None)
    return found, loads


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_no_instruction_touches_a_register_whose_untracked_load_is_in_flight(tmp_path):
    asm = tmp_path / "gemm_lp.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-gpu-rdc", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-inline-asm", "--cuda-device-only", "-I", os.path.join(HERE, "..", "include"),
           "-S", SRC, "-o", str(asm)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    lines = asm.read_text().split("\n")
    found, loads = violations(lines)
    assert loads >= 50, loads          # the walk did see the loads it is about (register half-stages and scale dwords)
    assert not found, found[:5]


def test_the_walk_finds_a_planted_case():
    """the checker on a hand-made stream: a value computed into a register whose load has not been waited for"""
    stream = """_ZN1x7gemm_lp_kE:
        global_load_dwordx4 v[34:37], v5, s[2:3]
        v_mfma_f32_32x32x16_bf16 v[0:15], v[40:43], v[44:47], v[0:15]
        v_or_b32_e32 v34, s33, v65
        s_waitcnt vmcnt(0) lgkmcnt(0)
        v_mov_b32_e32 v35, 0
        s_endpgm""".split("\n")
    found, loads = violations(stream)
    assert loads == 1 and len(found) == 1 and found[0][3] == [34]
    ok = [l for l in stream if "v_or_b32" not in l]
    assert violations(ok)[0] == []
