"""Builds libl2hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage:  python llama2.jl_amd/build.py [--timeline]
The objects are compiled in parallel (one hipcc per source file) and linked into
llama2.jl_amd/libl2hip.so.  hipcc cross-compiles: no GPU is needed to build.

--timeline builds llama2.jl_amd/libl2hip_tl.so instead: the same library with -DL2H_TIMELINE, in which the
streaming decode kernel stamps the wall clock at every phase boundary (llama2.jl_amd/timeline.py prints
the table).  The product library is not touched.
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
LIB_TIMELINE = os.path.join(HERE, "libl2hip_tl.so")

SOURCES = ["api.cpp", "synth.cpp", "pf_lt.cpp", "k_misc.hip", "k_matvec.hip", "k_attn.hip", "k_mega.hip", "k_prefill.hip", "k_flow.hip"]

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


def _compile(src, extra=(), objdir=OBJ):
    obj = os.path.join(objdir, src + ".o")
    cmd = [_hipcc(), "-c", os.path.join(CSRC, src), "-o", obj] + COMMON + list(extra)
    if src.endswith(".hip"):
        cmd += DEVICE
    else:
        cmd += ["-D__HIP_PLATFORM_AMD__"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, r.returncode, r.stdout + r.stderr, obj


def build(force=True, verbose=True, timeline=False):
    objdir = OBJ + "_tl" if timeline else OBJ
    lib = LIB_TIMELINE if timeline else LIB
    extra = ["-DL2H_TIMELINE"] if timeline else []
    os.makedirs(objdir, exist_ok=True)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(ROOT, "include", "l2h.h")]
    if not force and os.path.exists(lib) and all(os.path.getmtime(lib) >= os.path.getmtime(d) for d in deps):
        return lib
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        for src, rc, out, obj in ex.map(lambda s: _compile(s, extra, objdir), SOURCES):
            text = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, text))
            if verbose and text.strip():
                print("[%s]\n%s" % (src, text))
            objs.append(obj)
    # (hipBLASLt is opened at run time by pf_lt.cpp: -ldl, no link-time dependency on it)
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs + ["-ldl"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", lib)
    return lib


if __name__ == "__main__":
    build(force=True, timeline="--timeline" in sys.argv[1:])
    sys.exit(0)
