"""Checks on the compiled ring GEMV kernels (``csrc/nf4_gemv.hip``), run after every build.

Those kernels keep their weight requests in vector registers that are named literally in
asm statements and lie above the compiler's register budget, and they wait for the requests
by count.  That is only sound while the compiler keeps to its side of the contract, which it
does not promise; so the generated assembly of every ``gemv_ring_*`` kernel is read back and
the build fails unless

1. no instruction outside an asm statement names a vector register at or above the kernel's
   budget (the requests in flight write those registers behind the compiler's back);
2. no instruction touches a compiler-allocated register that an asm request is still
   writing (x travels that way), between the request and the asm wait that names it: a
   may-be-in-flight dataflow over the control-flow graph;
3. no scalar register restored with ``v_readlane`` / ``v_readfirstlane`` is used as an
   address by a vector memory instruction inside an asm statement within five wait states
   (the compiler pads its own instructions for that hazard, not the inside of an asm);
4. the kernel has no scratch traffic: a spill's loads and stores would join the in-order
   queue that the waits count.
"""

from __future__ import annotations

import os
import re
import subprocess
import tempfile

KERNEL = re.compile(r"^(_ZN3chr12_GLOBAL__N_1\d+gemv_ring_(rows)\w+):", re.M)
#: first fixed register of each kernel family (``csrc/nf4_gemv_ring_regs.h``)
BUDGET = {"rows": 104}
HAZARD_WAIT_STATES = 5


def vregs(text: str) -> set[int]:
    out: set[int] = set()
    for a, b in re.findall(r"v\[(\d+):(\d+)\]", text):
        out |= set(range(int(a), int(b) + 1))
    for a in re.findall(r"\bv(\d+)\b", text):
        out.add(int(a))
    return out


def _instructions(body: str):
    """[(inside asm?, text)] and {label: index of the instruction that follows it}."""
    ins: list[tuple[bool, str]] = []
    labels: dict[str, int] = {}
    in_asm = False
    for line in body.splitlines():
        s = line.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not s or s.startswith(";"):
            continue
        m = re.match(r"^(\.LBB\w+):", s)
        if m:
            labels[m.group(1)] = len(ins)
            continue
        if s.startswith("."):
            continue
        ins.append((in_asm, s))
    return ins, labels


def _in_flight_violations(ins, labels, budget: int) -> list[str]:
    n = len(ins)
    leaders = {0} | set(labels.values())
    for i, (_, s) in enumerate(ins):
        if s.startswith(("s_cbranch", "s_branch", "s_endpgm")):
            leaders.add(i + 1)
    starts = sorted(x for x in leaders if x < n)
    blocks = [(st, starts[k + 1] if k + 1 < len(starts) else n) for k, st in enumerate(starts)]
    block_of = {}
    for bi, (st, en) in enumerate(blocks):
        for x in range(st, en):
            block_of[x] = bi
    succ: list[list[int]] = [[] for _ in blocks]
    for bi, (st, en) in enumerate(blocks):
        last = ins[en - 1][1]
        if last.startswith("s_endpgm"):
            continue
        if last.startswith(("s_branch", "s_cbranch")):
            succ[bi].append(block_of[labels[last.split()[1]]])
            if last.startswith("s_branch"):
                continue
        if en < n:
            succ[bi].append(block_of[en])

    def walk(state: set[int], bi: int, found: list[str] | None) -> set[int]:
        st, en = blocks[bi]
        state = set(state)
        for i in range(st, en):
            in_asm, s = ins[i]
            if in_asm and s.startswith("global_load"):
                dest = vregs(s.split(None, 1)[1].split(",")[0])
                state |= {r for r in dest if r < budget}
                continue
            if in_asm and s.startswith("s_waitcnt"):
                # the wait's comment names the registers it covers
                state -= vregs(s.split(";", 1)[1]) if ";" in s else set()
                continue
            touched = vregs(s.split(";")[0]) & state
            if touched and found is not None:
                found.append(f'"{s}" touches registers still being written: {sorted(touched)}')
        return state

    entry = [set() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        bi = work.pop()
        out = walk(entry[bi], bi, None)
        for sb in succ[bi]:
            if not out <= entry[sb]:
                entry[sb] |= out
                work.append(sb)
    found: list[str] = []
    for bi in range(len(blocks)):
        walk(entry[bi], bi, found)
    return found


def _hazards(ins) -> list[str]:
    found = []
    for n, (_, s) in enumerate(ins):
        m = re.match(r"v_read(?:first)?lane_b32 s(\d+)", s)
        if not m:
            continue
        sreg = int(m.group(1))
        waited = 0
        k = n + 1
        while k < len(ins) and waited < HAZARD_WAIT_STATES:
            in_asm, t = ins[k]
            k += 1
            nop = re.match(r"s_nop (\d+)", t)
            if nop:
                waited += int(nop.group(1)) + 1
                continue
            if in_asm and t.startswith(("global_", "buffer_", "flat_", "scratch_")):
                for a, b in re.findall(r"s\[(\d+):(\d+)\]", t):
                    if int(a) <= sreg <= int(b):
                        found.append(f'"{t}" reads s{sreg} {waited} wait states after "{s}"')
            waited += 1
    return found


def check_assembly(text: str) -> list[str]:
    """Problems found in the ring kernels of a device assembly listing (empty = sound)."""
    problems: list[str] = []
    kernels = 0
    for m in KERNEL.finditer(text):
        kernels += 1
        name, family = m.group(1), m.group(2)
        budget = BUDGET[family]
        body = text[m.end(): text.index(".Lfunc_end", m.end())]
        ins, labels = _instructions(body)
        for in_asm, s in ins:
            if not in_asm:
                high = sorted(r for r in vregs(s.split(";")[0]) if r >= budget)
                if high:
                    problems.append(f"{name}: compiler code names reserved registers {high}: {s}")
        problems += [f"{name}: {p}" for p in _in_flight_violations(ins, labels, budget)]
        problems += [f"{name}: {p}" for p in _hazards(ins)]
        scratch = sum(1 for _, s in ins if s.startswith("scratch_"))
        if scratch:
            problems.append(f"{name}: {scratch} scratch instructions (register spills)")
    if kernels == 0:
        problems.append("no gemv_ring_* kernel found in the listing")
    return problems


def check_source(hipcc: str, flags: tuple[str, ...], source: str) -> None:
    """Compile ``source`` to device assembly with the build's flags and check it; raises
    RuntimeError with the findings."""
    keep = [f for f in flags if f not in ("-shared", "-fPIC")]
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "ring.s")
        cmd = [hipcc, *keep, "-S", "--cuda-device-only", "-o", out, source]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on {source}:\n{proc.stderr[-2000:]}")
        with open(out) as fh:
            problems = check_assembly(fh.read())
    if problems:
        shown = "\n  ".join(problems[:20])
        raise RuntimeError(f"ring GEMV kernels: {len(problems)} problems in the generated code:\n  {shown}")
