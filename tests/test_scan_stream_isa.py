"""The table lookups of scan_stream.hip, scan_slab_len*.hip and scan_nibble_pack.hip are issued and waited for in
inline assembly, so that the adds of one group overlap the reads of the next.  From the compiler's
point of view a read's destination register holds its value as soon as the read is issued; nothing
stops it from copying or reusing that register before the data has arrived.  Both files therefore
keep a whole tile (or step) of lookups in one assembly block.  This test compiles them for gfx950
and checks the generated code for what that is meant to guarantee: between an inline `ds_read_u16` / `ds_read_u8`
and the inline `s_waitcnt` that covers it, no compiler-generated instruction, label or branch
touches the destination register, and no other inline instruction reads it.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# file: inline reads at least expected
SOURCES = {"scan_stream.hip": 48 * 32, "scan_nibble_pack.hip": 128 * 24, "scan_slab_len2.hip": 64 * 32 * 4}
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _registers(text):
    """VGPR numbers an operand string mentions: v12, v[4:7]."""
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", text))
    return regs


def check_lookup_windows(asm_text):
    """Returns (number of inline reads seen, list of violations)."""
    pending = []  # destination registers of inline reads in issue order
    in_asm = False
    n_reads = 0
    problems = []
    for no, raw in enumerate(asm_text.splitlines(), 1):
        line = raw.split(";")[0].strip() if not raw.strip().startswith(";;#") else raw.strip()
        if line.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if line.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not line:
            continue
        if in_asm:
            m = re.match(r"ds_read_u(?:16|8)\s+v(\d+),", line)
            if m:
                pending.append(int(m.group(1)))
                n_reads += 1
                continue
            m = re.match(r"s_waitcnt\s+.*lgkmcnt\((\d+)\)", line)
            if m:
                keep = int(m.group(1))
                pending = pending[len(pending) - keep:] if keep < len(pending) else pending
                if keep == 0:
                    pending = []
                continue
            if pending and (_registers(line.split(None, 1)[1] if " " in line else "") & set(pending)):
                # another inline instruction: only address computations, which use other registers
                problems.append((no, raw))
            continue
        if not pending:
            continue
        if line.endswith(":") or re.match(r"s_(c?branch|setpc|endpgm)", line):
            problems.append((no, raw))
        elif _registers(line) & set(pending):
            problems.append((no, raw))
    return n_reads, problems


@pytest.mark.skipif(shutil.which(HIPCC) is None and not os.path.exists(HIPCC), reason="needs hipcc")
@pytest.mark.parametrize("name", sorted(SOURCES))
def test_no_instruction_touches_a_lookup_in_flight(tmp_path, name):
    out = tmp_path / (name + ".s")
    subprocess.check_call([HIPCC, "-O3", "-std=c++17", "--offload-arch=gfx950", "--cuda-device-only", "-S",
                           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "cuvs_amd", "csrc"),
                           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fvisibility=hidden",
                           os.path.join(ROOT, "cuvs_amd", "csrc", name), "-o", str(out)], stderr=subprocess.DEVNULL)
    n_reads, problems = check_lookup_windows(out.read_text())
    assert n_reads >= SOURCES[name], "the kernels' inline lookups were not found in the generated code"
    assert not problems, "instructions inside a lookup window:\n" + "\n".join(f"{n}: {t}" for n, t in problems[:20])


def test_the_checker_sees_a_copy_of_a_register_in_flight():
    bad = """
\t;;#ASMSTART
\tds_read_u16 v5, v9 offset:512
\t;;#ASMEND
\tv_mov_b32_e32 v7, v5
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(0)
\t;;#ASMEND
"""
    assert check_lookup_windows(bad)[1]
    good = bad.replace("v_mov_b32_e32 v7, v5", "v_mov_b32_e32 v7, v6")
    assert not check_lookup_windows(good)[1]
    branch = bad.replace("v_mov_b32_e32 v7, v5", "s_cbranch_vccz .LBB0_3")
    assert check_lookup_windows(branch)[1]
