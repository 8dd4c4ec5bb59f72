"""Development-container check (needs the read-only msccl-tools checkout at /root/reference): run the
example programs of msccl-tools, unchanged, once against msccl-tools' own `msccl.language` and once
against this repository's `msccl.language`, and compare the MSCCL-IR they print.

This shows two things no committed fixture can: that user programs written for msccl-tools run
unmodified on this package (same names, same arguments), and that both compilers agree on them.
Documents are compared on the canonical form of tests/test_compiler_golden.py (waits in front of a
step form a set), because msccl-tools' own output is not reproducible for multi-wait steps.

usage: python tests/golden/compare_examples.py            # prints one line per example
"""
import contextlib
import io
import json
import os
import runpy
import subprocess
import sys
import types

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))

EXAMPLES = [
    ("allgather_a100_pcie.py", [8, 1]), ("allgather_allpairs.py", [8, 2]), ("allgather_recursive_doubling.py", [8, 1]),
    ("allgather_ring.py", [8, 2, 2]), ("allreduce_1step.py", [4, 1]), ("allreduce_a100_allpairs.py", [8, 2]),
    ("allreduce_a100_allpairs_v2.py", [8, 1]), ("allreduce_a100_multinode_allpairs.py", [16, 1]),
    ("allreduce_a100_ncv4.py", [8, 1]), ("allreduce_a100_ncv4_v2.py", [8, 1]), ("allreduce_a100_pcie_hierarchical.py", [8, 1]),
    ("allreduce_a100_recursive_doubling_halving.py", [2, 1]), ("allreduce_a100_ring.py", [8, 4, 2]),
    ("allreduce_binomial_tree.py", [8, 1, 1]), ("allreduce_recursive_doubling_halving.py", [8, 1]),
    ("alltoall_a100_three_step.py", [3, 4, 1]), ("alltoall_a100_two_step.py", [2, 4]), ("alltoall_allpairs.py", [4, 2]),
    ("alltonext_backward.py", [2, 1]), ("alltonext_forward.py", [2, 1]), ("hierarchical_allreduce.py", [4, 2, 1]),
    ("hierarchical_allreduce.py", [4, 2, 2, "--schedule", "manual"]), ("pipeline_a100_allpairs.py", [8, 1]),
    ("pipeline_a100_ring.py", [8, 2, 1]), ("reducegather.py", [8, 2]), ("simple/allgather_ring.py", []), ("simple/allreduce_ring.py", [8, 2]),
    ("simple/custom_collective.py", []), ("allreduce_dgx1.py", [1, 1]), ("allreduce_ndv2.py", [1]),
]


def child(which, script, argv):
    """Runs in a subprocess: execute one example with the chosen `msccl` and print its XML as JSON."""
    sys.dont_write_bytecode = True
    if which == "reference":
        import xml.etree.ElementTree as ET
        pkg = types.ModuleType("msccl")
        pkg.__path__ = [os.path.join(REF, "msccl")]
        sys.modules["msccl"] = pkg
        lxml = types.ModuleType("lxml")
        lxml.etree = ET
        sys.modules["lxml"] = lxml
        sys.modules["lxml.etree"] = ET
        sys.path.insert(0, REF)
    else:
        sys.path.insert(0, os.path.join(ROOT, "msccl-tools_amd"))
    sys.argv = [script] + [str(a) for a in argv]
    buf = io.StringIO()
    try:
        with contextlib.redirect_stdout(buf):
            runpy.run_path(os.path.join(REF, "examples", "mscclang", script), run_name="__main__")
    except BaseException as e:  # noqa: BLE001 -- report, whatever it was
        print(json.dumps({"error": f"{type(e).__name__}: {e}"[:200]}))
        return
    text = buf.getvalue()
    if "<algo" not in text:
        print(json.dumps({"error": "no XML printed"}))
        return
    print(json.dumps({"xml": text[text.index("<algo"):text.index("</algo>") + 7].replace(" />", "/>")}))


def main():
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    sys.path.insert(0, os.path.join(ROOT, "msccl-tools_amd"))
    from test_compiler_golden import canonical
    same = diff = skipped = 0
    for script, argv in EXAMPLES:
        out = {}
        for which in ("reference", "package"):
            r = subprocess.run([sys.executable, __file__, "--child", which, script, json.dumps(argv)], capture_output=True, text=True,
                               env=dict(os.environ, PYTHONDONTWRITEBYTECODE="1"))
            last = [l for l in r.stdout.splitlines() if l.startswith("{")]
            out[which] = json.loads(last[-1]) if last else {"error": (r.stderr or "no output")[-200:]}
        a, b = out["reference"], out["package"]
        tag = f"{script} {' '.join(map(str, argv))}"
        if "error" in a:
            skipped += 1
            print(f"SKIP  {tag}: fails on msccl-tools itself ({a['error']}); this package: {b.get('error', 'compiles')}")
        elif "error" in b:
            diff += 1
            print(f"FAIL  {tag}: this package: {b['error']}")
        elif canonical(a["xml"]) == canonical(b["xml"]):
            same += 1
            print(f"SAME  {tag}" + ("  (byte-identical)" if a["xml"].split(">", 1)[1] == b["xml"].split(">", 1)[1] else ""))
        else:
            diff += 1
            print(f"DIFF  {tag}")
    print(f"{same} same, {diff} different, {skipped} not runnable upstream")
    return 1 if diff else 0


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "--child":
        child(sys.argv[2], sys.argv[3], json.loads(sys.argv[4]))
    else:
        sys.exit(main())
