"""The streaming kernel polls activations with loads it issues from inline asm.  The compiler believes
an asm statement's outputs valid as soon as the statement ends, so a load and the wait for it must be
one statement; this test compiles k_flow.hip to assembly and checks that no register that such a load
targets is read or written while the load can still be under way (loads complete in order: an asm-issued
`s_waitcnt vmcnt(N)` leaves at most the N youngest; a variant with two polls under way, whose younger
registers the compiler did read in a loop, was caught by this check)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "llama2.jl_amd", "csrc")


def _regs(text):
    out = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def _violations(path):
    """Linear scan: registers written by the asm-issued coherent 16-byte loads (`... sc1`) stay untouched
    until an asm-issued s_waitcnt vmcnt has retired the load."""
    bad, fn, pending, in_asm, n_loads = [], None, [], False, 0   # pending: [(line, regs)], oldest first
    for ln, line in enumerate(open(path), 1):
        t = line.strip()
        m = re.match(r"^(_Z\w+):", t)
        if m:
            fn, pending = m.group(1), []
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t[0] in ";.":
            continue
        m = re.search(r"s_waitcnt vmcnt\((\d+)\)", t)
        if in_asm and m:
            n = int(m.group(1))
            pending = pending[len(pending) - n:] if n else []
            continue
        live = set().union(*[r for _, r in pending]) if pending else set()
        if in_asm and t.startswith("global_load_dwordx4") and t.endswith("sc1"):
            n_loads += 1
            ops = t.split(None, 1)[1].split(",")
            hit = _regs(",".join(ops[1:])) & live   # (asking again into a register whose load is under way is fine)
            if hit:
                bad.append((fn, ln, t, sorted(hit)))
            pending.append((ln, _regs(ops[0])))
            continue
        hit = _regs(t) & live
        if hit:
            bad.append((fn, ln, t, sorted(hit)))
    return bad, n_loads


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_no_register_of_a_pending_poll_is_touched(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path / "k_flow.s"
    cmd = [hipcc, "-S", "--cuda-device-only", os.path.join(CSRC, "k_flow.hip"), "-o", str(out), "--offload-arch=gfx950", "-O3",
           "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    bad, n_loads = _violations(str(out))
    assert n_loads > 0, "no asm-issued polls found: has the kernel changed?"
    assert not bad, bad[:5]
