"""Static check of the generated gfx950 code (a build step; the tests and `__graft_entry__.build()` run it).

The attention kernels keep tile loads in flight across loop iterations as hand-written instructions with their own
counter waits, which the compiler does not know about.  Nothing may read or overwrite a register such a load will write
until a `s_waitcnt vmcnt(N)` has retired the load: a register copy (or a spill) the compiler places between a load and its
wait copies the register's previous contents, and the data that arrives later lands in a register that has been given
to something else - an address, for instance.  The same kernels write out their PV matrix instructions by hand (so that the
accumulators stay in the accumulator registers); the compiler does not know these are matrix instructions and keeps none
of the wait states a vector instruction needs before it may read their results, so a register copy it places right behind
one (where control flow joins, for instance) copies values the last passes have not written yet: `check_mfma_results`
walks the instructions behind every hand-written matrix instruction for as many wait states as its passes need.  `check_sources()` compiles each source it covers to assembly (device code
only, the flags of the library's Makefile) and walks every kernel along every path of its control flow.  It needs hipcc
and no GPU.  Loads are assumed to return in the order issued.
"""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
# Walked: the kernel whose waits are unconditional (one register set, `s_waitcnt vmcnt(0)` at one site).  The other
# attention kernels leave a number of loads in flight that depends on wave-uniform conditions correlated across branches
# (a younger tile was requested or not; a wave group has tiles or not), which a walk over all branch outcomes cannot
# follow: it reports paths that no wave takes.
SOURCES = ("attend_mid.hip",)
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-S", "--cuda-device-only"]
EXTRA = {"attend_mid.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}      # as in the library's Makefile

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


def _parse(lines):
    """Instructions of one kernel as (line number, text, from hand-written block) plus the index each label points at."""
    ins, labels, in_asm = [], {}, False
    for n, raw in enumerate(lines):
        t = raw.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = re.match(r"^(\.L\w+):", t)
        if m:
            labels[m.group(1)] = len(ins)
            continue
        if not t or t[0] in ";./" or t.endswith(":"):
            continue
        ins.append((n + 1, t.split(";")[0].strip(), in_asm))
    return ins, labels


def check_kernel(lines):
    """Walks every path through the kernel's control flow (a state = the ordered list of memory operations not yet
    retired; states are merged per instruction by identity, loops end when no new state appears).  Returns a list of
    (line number, text, registers) violations."""
    ins, labels = _parse(lines)
    seen = [set() for _ in ins]
    bad = {}
    work = [(0, ())]
    while work:
        pc, st = work.pop()
        while pc < len(ins):
            if st in seen[pc]:
                break
            seen[pc].add(st)
            if len(seen[pc]) > 64:
                raise AssertionError("too many distinct in-flight states at one instruction: the walk does not converge")
            n, t, in_asm = ins[pc]
            op = t.split()[0]
            pending = set()
            for a, d in st:
                if a:
                    pending |= d
            if VMEM.match(op):
                dst = frozenset()
                if "_load" in op:
                    m = re.match(r"\S+\s+(v\[\d+:\d+\]|v\d+)", t)
                    dst = frozenset(_regs(m.group(1))) if m else frozenset()
                hit = (_regs(t) - dst) & pending | (dst & pending)
                if hit:
                    bad[n] = (n, t, sorted(hit))
                is_asm = in_asm and "_load" in op
                st = st + ((is_asm, dst if is_asm else frozenset()),)      # the compiler's own loads only count
                while st and not st[0][0]:            # operations older than the oldest hand-written load decide nothing
                    st = st[1:]
            elif op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", t)
                if m:
                    keep = int(m.group(1))
                    st = st[len(st) - keep:] if keep else ()
                    while st and not st[0][0]:
                        st = st[1:]
            elif op == "s_endpgm":
                break
            elif op == "s_branch":
                pc = labels[t.split()[1]]
                continue
            elif op.startswith("s_cbranch"):
                work.append((labels[t.split()[1]], st))
            elif not (op.startswith("s_") and not _regs(t)):
                hit = _regs(t) & pending
                if hit:
                    bad[n] = (n, t, sorted(hit))
            pc += 1
    return [bad[k] for k in sorted(bad)]


AREG = re.compile(r"\ba\[(\d+):(\d+)\]|\ba(\d+)\b")
# wait states between a matrix instruction and a vector instruction that touches its result registers: 4-pass / 8-pass
# instructions (one more than the hazard tables say)
MFMA_WAIT = {"v_mfma_f32_16x16x32_f16": 8, "v_mfma_f32_32x32x16_f16": 12}


def _aregs(text):
    out = set()
    for a, b, c in AREG.findall(text):
        if c:
            out.add(int(c))
        else:
            out.update(range(int(a), int(b) + 1))
    return out


def check_mfma_results(lines):
    """For every hand-written matrix instruction: no other kind of instruction touches its result registers within the wait
    states its passes need, along any path.  Returns (hand-written matrix instructions seen, violations)."""
    ins, labels = _parse(lines)
    bad, count = {}, 0
    for p, (n, t, in_asm) in enumerate(ins):
        op = t.split()[0]
        if not (in_asm and op in MFMA_WAIT):
            continue
        count += 1
        first = t.split(",")[0]
        dst_a, dst_v = _aregs(first), _regs(first)         # the result lies in accumulator registers or in ordinary ones
        work, seen = [(p + 1, MFMA_WAIT[op])], set()
        while work:
            pc, left = work.pop()
            while pc < len(ins) and left > 0 and (pc, left) not in seen:
                seen.add((pc, left))
                n2, t2, _ = ins[pc]
                op2 = t2.split()[0]
                if op2 == "s_endpgm":
                    break
                if op2 == "s_nop":
                    left -= int(t2.split()[1]) + 1
                    pc += 1
                    continue
                if op2 == "s_branch":
                    pc = labels[t2.split()[1]]
                    left -= 1
                    continue
                if op2.startswith("s_cbranch"):
                    work.append((labels[t2.split()[1]], left - 1))
                elif not op2.startswith("v_mfma") and (_aregs(t2) & dst_a or _regs(t2) & dst_v):
                    bad[(n, n2)] = (n2, t2, n, sorted(_aregs(t2) & dst_a) + sorted(_regs(t2) & dst_v))
                left -= 1
                pc += 1
    return count, [bad[k] for k in sorted(bad)]


def check_mfma_operands(lines):
    """For every hand-written matrix instruction: none of the two instructions in front of it (wait states of `s_nop`
    counted) is a vector instruction that writes one of its operands - a vector result is not forwarded to a matrix
    instruction issued right behind it (the compiler keeps two wait states for its own).  Looks back in straight-line code
    only: a label or a branch in between ends the search.  Returns the violations."""
    bad = []
    stream = []                                   # (kind, text, line) with labels kept, so that a join ends the look-back
    in_asm = False
    for n, raw in enumerate(lines):
        t = raw.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if re.match(r"^\.L\w+:", t):
            stream.append(("label", t, n + 1, False))
            continue
        if not t or t[0] in ";./" or t.endswith(":"):
            continue
        stream.append(("ins", t.split(";")[0].strip(), n + 1, in_asm))
    for p, (kind, t, n, in_asm) in enumerate(stream):
        if kind != "ins" or not in_asm or t.split()[0] not in MFMA_WAIT:
            continue
        ops = t.split(None, 1)[1].split(",")
        srcs = set()
        for o in ops[1:]:
            srcs |= _regs(o)
        left, q = 2, p - 1
        while q >= 0 and left > 0:
            k2, t2, n2, _ = stream[q]
            if k2 == "label":
                break
            op2 = t2.split()[0]
            if op2.startswith("s_cbranch") or op2 == "s_branch":
                break
            if op2 == "s_nop":
                left -= int(t2.split()[1]) + 1
            else:
                if op2.startswith("v_") and not op2.startswith("v_mfma") and not op2.startswith("v_cmp"):
                    w = _regs(t2.split(None, 1)[1].split(",")[0]) if " " in t2 else set()
                    if w & srcs:
                        bad.append((n, t, n2, t2, sorted(w & srcs)))
                left -= 1
            q -= 1
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
            if re.match(r"^\s*\.section\s+\.rodata", line) or line.strip().startswith(".amdhsa_kernel"):
                out.append((name, cur))
                name, cur = None, []
                continue
            cur.append(line)
    return out


def check_sources(workdir, sources=SOURCES):
    """Compiles `sources` to assembly under `workdir` and checks every kernel.  Returns (hand-written loads seen, list of
    problem descriptions)."""
    def compile_one(src):
        out = os.path.join(workdir, src + ".s")
        p = subprocess.run([HIPCC, *FLAGS, *EXTRA.get(src, []), src, "-o", out], cwd=CSRC, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc -S {src} failed:\n" + p.stderr[-2000:])
        with open(out) as f:
            return src, f.read()

    with ThreadPoolExecutor(max_workers=2) as ex:
        results = list(ex.map(compile_one, sources))
    seen, problems = 0, []
    for src, text in results:
        ks = kernels_of(text)
        if not ks:
            problems.append(f"no kernel found in the assembly of {src}")
        for name, lines in ks:
            seen += sum(1 for i, l in enumerate(lines) if "global_load" in l and i and "ASMSTART" in lines[i - 1])
            for n, t, regs in check_kernel(lines):
                problems.append(f"{src} {name[:60]} line {n}: `{t[:80]}` touches v{regs} while their loads are in flight")
            _, late = check_mfma_results(lines)
            for n2, t2, n, regs in late:
                problems.append(f"{src} {name[:60]} line {n2}: `{t2[:80]}` touches a{regs} before the matrix instruction of line {n} has written them")
            for n, t, n2, t2, regs in check_mfma_operands(lines):
                problems.append(f"{src} {name[:60]} line {n}: `{t[:70]}` reads v{regs} which `{t2[:60]}` (line {n2}) has only just written")
    return seen, problems


def main():
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        seen, problems = check_sources(d)
    if seen < 5 * 2 * 14:
        problems.append(f"only {seen} hand-written loads found: the check looked at nothing")
    if problems:
        raise SystemExit("ISA check failed:\n" + "\n".join(problems[:40]))
    print(f"ISA check: {seen} hand-written loads, no register touched while its load is in flight; "
          "no result of a hand-written matrix instruction touched before its passes are through")


if __name__ == "__main__":
    main()
