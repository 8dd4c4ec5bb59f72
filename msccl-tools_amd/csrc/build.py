"""Builds libmscclx.so (gfx950) in-tree with hipcc.  Run: python build.py [--force]"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libmscclx.so")
SOURCES = ["plan.cpp", "exec.hip"]
HEADERS = ["plan.h", os.path.join(ROOT, "include", "mscclx.h")]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def is_stale():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(HERE, s) for s in SOURCES] + [h if os.path.isabs(h) else os.path.join(HERE, h) for h in HEADERS]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=True, verbose=True):
    if not force and not is_stale():
        return LIB
    common = ["-O3", "-std=c++17", "-fPIC", "-I", os.path.join(ROOT, "include"), "-I", HERE, "-Wall", "-Wno-unused-function"]
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(HERE, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmd = [hipcc()] + common
        if src.endswith(".hip"):
            # gfx950 only; packed FP32 instructions are disabled on purpose; no FMA contraction so
            # that reductions are exactly the IEEE operation the oracle performs.
            cmd += ["--offload-arch=gfx950", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
        else:
            cmd += ["-x", "c++"]
        cmd += ["-c", os.path.join(HERE, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)  # host pass does not know the feature
        if out.strip() and verbose:
            print(out)
        if p.returncode:
            raise RuntimeError(f"compiling {src} failed:\n{out}")
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv or is_stale())
    print(LIB)
