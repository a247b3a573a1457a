"""Static check of the generated gfx950 code: the attention kernels keep tile loads in flight across loop iterations
as hand-written instructions with their own counter waits, which the compiler does not know about.  Nothing may read
or overwrite a register such a load will write until a `s_waitcnt vmcnt(N)` has retired the load - a register copy
the compiler places between a load and its wait would copy the register's previous contents.  The check compiles each
source that contains such loads to assembly (device code only, the flags of the library's Makefile) and walks every
kernel in layout order.  It runs on the CPU (hipcc cross-compiles); it does not prove the absence of the problem on every
path through the control flow, it catches the forms that were seen (copies in front of a wait, copies at a loop's end).
"""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "yasakani_amd", "csrc")
SOURCES = ("attend_narrow.hip", "attend_mid.hip", "attend_wide.hip", "attend256_wide.hip", "attend_tb_wide.hip")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-S", "--cuda-device-only"]

VMEM = re.compile(r"^(global|buffer|scratch|flat)_(load|store|atomic)")
REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _regs(text):
    out = set()
    for a, b, c in REG.findall(text):
        if c:
            out.add(int(c))
        else:
            out.update(range(int(a), int(b) + 1))
    return out


def check_kernel(lines):
    """lines: the instructions of one kernel.  Returns a list of (line number, text, registers) violations."""
    inflight = []            # VMEM operations not yet retired, oldest first: (is_asm_load, dst registers, line)
    bad = []
    in_asm = False
    for n, raw in enumerate(lines):
        t = raw.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t[0] in ";./" or t.endswith(":"):
            continue
        t = t.split(";")[0].strip()
        op = t.split()[0]
        pending = set().union(*[d for a, d, _ in inflight if a]) if inflight else set()
        if VMEM.match(op):
            dst = set()
            if "_load" in op:
                m = re.match(r"\S+\s+(v\[\d+:\d+\]|v\d+)", t)
                dst = _regs(m.group(1)) if m else set()
            # address / data operands of the new operation must not be in flight either
            used = _regs(t) - dst
            hit = used & pending
            if hit:
                bad.append((n + 1, t, sorted(hit)))
            if dst & pending:
                bad.append((n + 1, t, sorted(dst & pending)))
            inflight.append((in_asm and "_load" in op, dst, n + 1))
            continue
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", t)
            if m:
                keep = int(m.group(1))
                inflight = inflight[len(inflight) - keep:] if keep else []
            continue
        if op.startswith("s_") and not _regs(t):
            continue
        hit = _regs(t) & pending
        if hit:
            bad.append((n + 1, t, sorted(hit)))
    return bad


def kernels_of(asm_text):
    """Splits an assembly file into (name, lines) per kernel."""
    out, name, cur = [], None, []
    for line in asm_text.split("\n"):
        m = re.match(r"^(_Z\w+):\s*(;.*)?$", line)
        if m and name is None:
            name, cur = m.group(1), []
            continue
        if name is not None:
            if line.strip().startswith(".end_amdhsa_kernel") or line.strip().startswith("s_endpgm") and False:
                pass
            if re.match(r"^\s*\.section\s+\.rodata", line) or line.strip().startswith(".amdhsa_kernel"):
                out.append((name, cur))
                name, cur = None, []
                continue
            cur.append(line)
    return out


def test_checker_sees_a_copy_in_front_of_a_wait():
    good = """
	;;#ASMSTART
	global_load_dwordx4 v[10:13], v2, s[4:5] offset:0 nt
	;;#ASMEND
	v_add_u32_e32 v3, v4, v5
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v20, v10
"""
    bad = good.replace("v_add_u32_e32 v3, v4, v5", "v_mov_b64_e32 v[60:61], v[10:11]")
    assert check_kernel(good.split("\n")) == []
    assert len(check_kernel(bad.split("\n"))) == 1
    # a wait that leaves the youngest load in flight retires only the older one
    two = """
	;;#ASMSTART
	global_load_dword v10, v2, s[4:5]
	;;#ASMEND
	;;#ASMSTART
	global_load_dword v11, v2, s[4:5] offset:64
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mov_b32_e32 v20, v10
	v_mov_b32_e32 v21, v11
"""
    v = check_kernel(two.split("\n"))
    assert len(v) == 1 and v[0][2] == [11]


@pytest.mark.skipif(shutil.which(HIPCC) is None and not os.path.exists(HIPCC), reason="hipcc not found")
def test_no_instruction_touches_a_register_with_a_load_in_flight(tmp_path):
    def compile_one(src):
        out = tmp_path / (src + ".s")
        p = subprocess.run([HIPCC, *FLAGS, src, "-o", str(out)], cwd=CSRC, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        assert p.returncode == 0, p.stderr[-2000:]
        return src, out.read_text()

    with ThreadPoolExecutor(max_workers=5) as ex:
        results = list(ex.map(compile_one, SOURCES))
    seen_asm_loads = 0
    problems = []
    for src, text in results:
        ks = kernels_of(text)
        assert ks, f"no kernel found in the assembly of {src}"
        for name, lines in ks:
            seen_asm_loads += sum(1 for i, l in enumerate(lines) if "global_load" in l and i and "ASMSTART" in lines[i - 1])
            for n, t, regs in check_kernel(lines):
                problems.append(f"{src} {name[:60]} line {n}: `{t[:80]}` touches v{regs} while their loads are in flight")
    assert seen_asm_loads > 100, "the hand-written loads were not found: the check looked at nothing"
    assert not problems, "\n".join(problems[:40])
