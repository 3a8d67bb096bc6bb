"""Builds libl2hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage:  python llama2.jl_amd/build.py [--force]
The objects are compiled in parallel (one hipcc per source file) and linked into
llama2.jl_amd/libl2hip.so.  hipcc cross-compiles: no GPU is needed to build.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libl2hip.so")

SOURCES = ["api.cpp", "synth.cpp", "k_misc.hip", "k_matvec.hip", "k_attn.hip", "k_mega.hip", "k_prefill.hip", "k_flow.hip"]

COMMON = [
    "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]
# device code: gfx950 only; packed-fp32 instructions are switched off for the whole library
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src):
    obj = os.path.join(OBJ, src + ".o")
    cmd = [_hipcc(), "-c", os.path.join(CSRC, src), "-o", obj] + COMMON
    if src.endswith(".hip"):
        cmd += DEVICE
    else:
        cmd += ["-D__HIP_PLATFORM_AMD__"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, r.returncode, r.stdout + r.stderr, obj


def build(force=True, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(ROOT, "include", "l2h.h")]
    if not force and os.path.exists(LIB) and all(os.path.getmtime(LIB) >= os.path.getmtime(d) for d in deps):
        return LIB
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        for src, rc, out, obj in ex.map(_compile, SOURCES):
            text = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, text))
            if verbose and text.strip():
                print("[%s]\n%s" % (src, text))
            objs.append(obj)
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force=True)
    sys.exit(0)
