"""Builds libmscclx.so (gfx950) in-tree with hipcc.  Run: python build.py [--force] [--flags "-DX ..."] [--out PATH]

The kernels (exec_device.h) are compiled as five translation units of two element types each
(exec_kernels.hip with -DMSCCLX_KERNEL_GROUP=0..4), in parallel with the host sources."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libmscclx.so")
KERNEL_GROUPS = 5
SOURCES = ["plan.cpp", "exec.hip", "exec_kernels.hip"]
HEADERS = ["plan.h", "exec_device.h", os.path.join(ROOT, "include", "mscclx.h")]


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


def build(force=True, verbose=True, extra_flags=(), out=None):
    lib = out or LIB
    if not force and not is_stale() and out is None:
        return lib
    common = ["-O3", "-std=c++17", "-fPIC", "-I", os.path.join(ROOT, "include"), "-I", HERE, "-Wall", "-Wno-unused-function"] + list(extra_flags)
    # gfx950 only; packed FP32 instructions are disabled on purpose; no FMA contraction so that
    # reductions are exactly the IEEE operation the oracle performs.
    device = ["--offload-arch=gfx950", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    tag = "" if out is None else "." + os.path.splitext(os.path.basename(out))[0]
    jobs = [("plan.cpp", ["-x", "c++"], "plan" + tag + ".o"), ("exec.hip", device, "exec" + tag + ".o")]
    jobs += [("exec_kernels.hip", device + [f"-DMSCCLX_KERNEL_GROUP={g}"], f"exec_kernels_{g}{tag}.o") for g in range(KERNEL_GROUPS)]
    objs = []
    procs = []
    for src, flags, obj in jobs:
        obj = os.path.join(HERE, obj)
        objs.append(obj)
        cmd = [hipcc()] + common + flags + ["-c", os.path.join(HERE, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out_text, _ = p.communicate()
        out_text = "\n".join(l for l in out_text.splitlines() if "packed-fp32-ops" not in l)  # host pass does not know the feature
        if out_text.strip() and verbose:
            print(out_text)
        if p.returncode:
            raise RuntimeError(f"compiling {src} failed:\n{out_text}")
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return lib


if __name__ == "__main__":
    argv = sys.argv[1:]
    flags = argv[argv.index("--flags") + 1].split() if "--flags" in argv else []
    out = argv[argv.index("--out") + 1] if "--out" in argv else None
    print(build(force="--force" in argv or is_stale(), extra_flags=flags, out=out))
