"""Checks the compiled code of the kernels whose MFMAs are written as inline asm WITHOUT wait states
(csrc/qmatmul_wide.hip, csrc/qmatmul_reg.hip): an MFMA must not read a vector register within two wait
states of the vector instruction that wrote it, and inline asm is outside the compiler's own hazard handling.
The kernels arrange their source so that another MFMA always stands between such a write and the read; this
script compiles the files to assembly and verifies it on every MFMA of every instantiation.

    python jax-gptq_amd/check_mfma_hazards.py        # exit status 0: no hazard

An instruction in between counts one wait state, `s_nop n` n + 1, an MFMA two (its issue takes a pass of four
cycles).  Every way into an MFMA is followed: the fall-through path and, through labels, the instructions in front
of the branches to them (a loop's back edge).
"""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as _build  # noqa: E402

FILES = ["qmatmul_wide.hip", "qmatmul_reg.hip"]


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def scan(asm_text):
    """Returns (number of MFMAs, list of (writer, mfma) pairs that are too close).

    The two wait states in front of an MFMA are looked for along every path into it: the fall-through path
    and, where a label lies within them, the instructions in front of every branch to that label (a loop's
    back edge puts the end of the body in front of its head)."""
    raw = [l.strip() for l in asm_text.splitlines()]
    lines, labels = [], {}
    for l in raw:
        if not l or l.startswith(";") or l.startswith("//"):
            continue
        l = l.split(";")[0].strip()
        if l.endswith(":"):
            labels.setdefault(l[:-1], len(lines))          # the label stands in front of instruction len(lines)
            continue
        if l.startswith("."):
            continue
        lines.append(l)
    jumps = {}                                             # instruction index of a label -> branches to it
    for i, l in enumerate(lines):
        if l.startswith("s_cbranch") or l.startswith("s_branch"):
            t = l.split()[-1]
            if t in labels:
                jumps.setdefault(labels[t], []).append(i)
    found, n = [], 0

    def walk(j, states, src, mfma, seen):
        # instruction j and those in front of it, until two wait states are counted
        while j >= 0 and states < 2:
            if j + 1 in jumps:                             # a label in front of instruction j + 1: its other ways in
                for b in jumps[j + 1]:
                    if (b, states) not in seen:
                        seen.add((b, states))
                        walk(b, states, src, mfma, seen)
            p = lines[j]
            if p.startswith("s_branch"):                   # nothing falls through an unconditional branch
                return
            if p.startswith("s_nop"):
                states += int(p.split()[1]) + 1
            else:
                if p.startswith("v_") and not p.startswith("v_mfma"):
                    if _regs(p.split(None, 1)[1].split(",")[0].strip()) & src:
                        found.append((p, mfma))
                states += 2 if p.startswith("v_mfma") else 1
            j -= 1

    for i, l in enumerate(lines):
        if not l.startswith("v_mfma"):
            continue
        n += 1
        ops = [t.strip() for t in l.split(None, 1)[1].split(",")]
        src = _regs(ops[1]) | _regs(ops[2])
        seen = set()
        if i in jumps:                                     # the MFMA is itself a branch target
            for b in jumps[i]:
                seen.add((b, 0))
                walk(b, 0, src, l, seen)
        walk(i - 1, 0, src, l, seen)
    return n, found


def check(files=FILES, verbose=True):
    bad = 0
    with tempfile.TemporaryDirectory() as tmp:
        procs = []
        for f in files:
            out = os.path.join(tmp, f + ".s")
            cmd = [_build._hipcc(), *_build.FLAGS, "-S", "--cuda-device-only", os.path.join(_build.CSRC, f), "-o", out]
            procs.append((f, out, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        for f, out, p in procs:
            log = p.communicate()[0].decode()
            if p.returncode != 0:
                raise RuntimeError(f"hipcc -S failed on {f}:\n{log}")
            n, found = scan(open(out).read())
            if verbose:
                print(f"{f}: {n} MFMAs, {len(found)} operand writes within two wait states")
                for w, m in found[:10]:
                    print("   ", w, "->", m)
            if n == 0:
                raise RuntimeError(f"no MFMA found in {f}: the listing was not understood")
            bad += len(found)
    return bad


if __name__ == "__main__":
    sys.exit(1 if check() else 0)
