"""The prompt-pass kernels read LDS with loads issued from inline asm, some of them one step ahead of the
wait that retires them.  The compiler believes an asm statement's outputs valid as soon as the statement
ends, so until that wait nothing may touch the registers such a read targets.  This test compiles
k_prefill.hip to assembly and walks the generated code: LDS reads complete in order, `s_waitcnt
lgkmcnt(N)` leaves at most the N newest under way, and no instruction in between may name a register
that a read still under way writes."""
import os
import re
import shutil
import subprocess

import pytest

from test_flow_asm import CSRC, ROOT, _regs


def _scan(path):
    bad, fn, pending, n_ahead = [], None, [], 0   # pending: [(line, regs)] oldest first
    for ln, line in enumerate(open(path), 1):
        t = line.strip()
        m = re.match(r"^(_Z\w+):", t)
        if m:
            fn, pending = m.group(1), []
        if not t or t[0] in ";.":
            continue
        if t.startswith("s_waitcnt"):
            m = re.search(r"lgkmcnt\((\d+)\)", t)
            if m:
                n = int(m.group(1))
                pending = pending[len(pending) - n:] if n else []
            continue
        live = set().union(*[r for _, r in pending]) if pending else set()
        if t.startswith("ds_read_b128"):
            ops = t.split(None, 1)[1].split(",")
            dst, rest = _regs(ops[0]), _regs(",".join(ops[1:]))
            hit = (dst | rest) & live
            if hit:
                bad.append((fn, ln, t, sorted(hit)))
            if pending:
                n_ahead += 1
            pending.append((ln, dst))
            continue
        hit = _regs(t) & live
        if hit:
            bad.append((fn, ln, t, sorted(hit)))
    return bad, n_ahead


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_no_register_of_a_pending_lds_read_is_touched(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path / "k_prefill.s"
    cmd = [hipcc, "-S", "--cuda-device-only", os.path.join(CSRC, "k_prefill.hip"), "-o", str(out), "--offload-arch=gfx950",
           "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    bad, n_ahead = _scan(str(out))
    assert n_ahead > 0, "no LDS reads issued ahead of a wait found: has the kernel changed?"
    assert not bad, bad[:5]
