"""Writes tests/golden/reference_xml/*.xml.gz: MSCCL-IR emitted by msccl-tools' own MSCCLang compiler.

Runs ONLY in the development container, where the msccl-tools checkout is mounted read-only at
/root/reference; the GPU box has no such checkout and only ever sees the committed XML files.
The fixtures are data (compiler output), used for two things no test of msccl-tools pins:
  * the executor is fed IR the real compiler produced (not only IR from this package's compiler);
  * this package's scheduler is compared, structurally, with the real one on auto-scheduled programs.

msccl-tools imports lxml, z3 and humanfriendly at package import time; none is installed here.
Only msccl.language and msccl.topologies are needed, so the top-level package is entered through an
empty stand-in module object (its __init__ is not executed) and `lxml.etree` is served by the
standard library's ElementTree, of which the emitter uses Element/SubElement/set/indent/tostring.

tests/golden/reference_random_xml/*.xml.gz: the same compiler on random programs of tests/random_programs.py
(instruction fusion on), among them programs it leaves malformed (sends without receives) or with a race:
what this package's compiler is compared with, byte for byte, on shapes no example has.

usage: python tests/golden/make_reference_xml.py [/root/reference] [--only SUBSTRING]
"""
import contextlib
import gzip
import io
import os
import runpy
import sys
import types
import xml.etree.ElementTree as ET

ONLY = sys.argv[sys.argv.index("--only") + 1] if "--only" in sys.argv else None
if ONLY is not None:
    del sys.argv[sys.argv.index("--only"):sys.argv.index("--only") + 2]
REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
RANDOM_OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_random_xml")
# fused random programs: well-formed ones, three that come out with unmatched sends and receives (7, 11, 19), two with a
# race (12, 32), two with an `rrs` (216, 270)
RANDOM_SEEDS = [0, 1, 2, 3, 4, 5, 6, 7, 11, 12, 19, 32, 216, 270]
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_xml")
sys.dont_write_bytecode = True


def install_entry_points():
    pkg = types.ModuleType("msccl")
    pkg.__path__ = [os.path.join(REF, "msccl")]
    sys.modules["msccl"] = pkg
    lxml = types.ModuleType("lxml")
    lxml.etree = ET
    sys.modules["lxml"] = lxml
    sys.modules["lxml.etree"] = ET
    sys.path.insert(0, REF)


def normalise(xml):
    return xml.replace(" />", "/>").strip() + "\n"


def from_example(script, argv, which=0):
    """Run an examples/mscclang script as __main__ and capture the XML it prints (the `which`-th
    document, for scripts that print several)."""
    old = sys.argv
    sys.argv = [script] + [str(a) for a in argv]
    buf = io.StringIO()
    try:
        with contextlib.redirect_stdout(buf):
            runpy.run_path(os.path.join(REF, "examples", "mscclang", script), run_name="__main__")
    finally:
        sys.argv = old
    text = buf.getvalue()
    docs = [d[:d.index("</algo>") + len("</algo>")] for d in text.split("<algo")[1:]]
    return normalise("<algo" + docs[which])


def from_program(build):
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        build()
    text = buf.getvalue()
    return normalise(text[text.index("<algo"):text.index("</algo>") + len("</algo>")])


def main():
    install_entry_points()
    from msccl.language import MSCCLProgram, XML, Check, ThreadblockPolicy
    from msccl.language.collectives import AllReduce, AllToAll
    from msccl.topologies import fully_connected

    def ring(n, channels, instances):
        from msccl.programs.allreduce_a100_ring import allreduce_ring
        with MSCCLProgram("allreduce_ring", fully_connected(n), AllReduce(n, n, True), instances,
                          threadblock_policy=ThreadblockPolicy.manual):
            allreduce_ring(n, channels)
            assert Check()
            XML()

    def chain(n):
        # this repository's msccl/programs/allreduce_chain.py, through msccl-tools' compiler
        from msccl.language import chunk, Buffer
        with MSCCLProgram("allreduce_chain", fully_connected(n), AllReduce(n, 1, True), 1, threadblock_policy=ThreadblockPolicy.manual):
            for hop in range(n - 1):
                chunk(hop + 1, Buffer.input, 0).reduce(chunk(hop, Buffer.input, 0), ch=0, recvtb=0, sendtb=0)
            for hop in range(-1, n - 2):
                chunk(hop % n, Buffer.input, 0).copy(hop + 1, Buffer.input, 0, ch=0, recvtb=0, sendtb=0)
            assert Check()
            XML()

    def allpairs(n, instances):
        from msccl.programs.allreduce_allpairs import allreduce_allpairs
        with MSCCLProgram("allreduce_allpairs", fully_connected(n), AllReduce(n, n * n, True), instances, protocol="LL",
                          threadblock_policy=ThreadblockPolicy.manual, interleaved_replication=False, dependence_nop=True):
            allreduce_allpairs(n)
            assert Check()
            XML()

    def three_step(nodes, gpus):
        from msccl.programs.alltoall_a100_8kp1 import alltoall_three_step
        n = nodes * gpus
        with MSCCLProgram("alltoall_three_step", fully_connected(n), AllToAll(n, 1, False), 1):
            alltoall_three_step(nodes, gpus)
            assert Check()
            XML()

    def registered_hierarchical(nodes):
        from msccl.programs.alltoall_a100_yifan import alltoall_hierarchical
        n = nodes * 8
        with MSCCLProgram("hierarchical_all_to_all", fully_connected(n), AllToAll(n, 1, False), 1):
            alltoall_hierarchical(nodes, 8)
            assert Check()
            XML()

    def reduce_scatter_ring(n, channels, instances):
        # this repository's msccl/programs/reducescatter_ring.py, through msccl-tools' compiler
        from msccl.language import chunk, Buffer
        from msccl.language.collectives import ReduceScatter
        with MSCCLProgram("reducescatter_ring", fully_connected(n), ReduceScatter(n, 1, True), instances, threadblock_policy=ThreadblockPolicy.manual):
            for hop in range(n - 1):
                for k in range(n):
                    lane = k % channels
                    here, there = (k + 1 + hop) % n, (k + 2 + hop) % n
                    chunk(there, Buffer.input, k).reduce(chunk(here, Buffer.input, k), ch=lane, recvtb=lane, sendtb=lane)
            assert Check()
            XML()

    def reduce_scatter_allpairs(n):
        # this repository's msccl/programs/reducescatter_allpairs.py, through msccl-tools' compiler
        from msccl.language import chunk, Buffer
        from msccl.language.collectives import ReduceScatter
        with MSCCLProgram("reducescatter_allpairs", fully_connected(n), ReduceScatter(n, n, True), 1, threadblock_policy=ThreadblockPolicy.manual,
                          dependence_nop=True):
            for src in range(n):
                for dst in range(n):
                    if src != dst:
                        chunk(src, Buffer.input, dst * n, size=n).copy(dst, "scratch", sendtb=dst, recvtb=src)
            for r in range(n):
                for k in range(n * (n - 1)):
                    chunk(r, Buffer.input, r * n + k % n).reduce(chunk(r, "scratch", k), sendtb=k % n)
            assert Check()
            XML()

    jobs = {
        "reducescatter_ring_8r_1ch_4inst": lambda: from_program(lambda: reduce_scatter_ring(8, 1, 4)),
        "reducescatter_allpairs_8r": lambda: from_program(lambda: reduce_scatter_allpairs(8)),
        "c1_allreduce_ring_8r_1ch_1inst": lambda: from_program(lambda: ring(8, 1, 1)),
        "c2_allgather_ring_8r_1ch_4inst": lambda: from_example("allgather_ring.py", [8, 1, 4, "--protocol", "Simple"]),
        "c3_alltoall_two_step_2x8": lambda: from_example("alltoall_a100_two_step.py", [2, 8]),
        "c3_alltoall_registered_2x8": lambda: from_program(lambda: registered_hierarchical(2)),
        "c4_hierarchical_allreduce_8x4_2inst_auto": lambda: from_example("hierarchical_allreduce.py", [8, 4, 2]),
        "c4_hierarchical_allreduce_4x2_1inst_manual": lambda: from_example("hierarchical_allreduce.py", [4, 2, 1, "--schedule", "manual"]),
        "c5_allreduce_ring_64r_1ch_1inst": lambda: from_program(lambda: ring(64, 1, 1)),
        "c5_allreduce_chain_64r": lambda: from_program(lambda: chain(64)),
        "simple_allgather_ring_4r_auto": lambda: from_example("simple/allgather_ring.py", []),
        "simple_allreduce_ring_8r_2inst_auto": lambda: from_example("simple/allreduce_ring.py", [8, 2]),
        "simple_custom_collective_3r_fanout": lambda: from_example("simple/custom_collective.py", [], which=0),
        "simple_custom_collective_3r_relay": lambda: from_example("simple/custom_collective.py", [], which=1),
        "allreduce_a100_allpairs_v2_8r": lambda: from_example("allreduce_a100_allpairs_v2.py", [8, 1]),
        "alltoall_a100_three_step_3x4_example": lambda: from_example("alltoall_a100_three_step.py", [3, 4, 1]),
        "allreduce_ring_8r_4ch_8inst": lambda: from_program(lambda: ring(8, 4, 8)),
        "allreduce_allpairs_8r_2inst": lambda: from_program(lambda: allpairs(8, 2)),
        "alltoall_three_step_3x4": lambda: from_program(lambda: three_step(3, 4)),
        "allgather_recursive_doubling_8r": lambda: from_example("allgather_recursive_doubling.py", [8, 1]),
        "allreduce_recursive_doubling_halving_8r": lambda: from_example("allreduce_recursive_doubling_halving.py", [8, 1]),
        "allgather_allpairs_8r": lambda: from_example("allgather_allpairs.py", [8, 1]),
        "allreduce_a100_allpairs_8r": lambda: from_example("allreduce_a100_allpairs.py", [8, 1]),
        "alltoall_allpairs_4r": lambda: from_example("alltoall_allpairs.py", [4, 1]),
        "allreduce_1step_4r": lambda: from_example("allreduce_1step.py", [4, 1]),
        "allreduce_a100_multinode_allpairs_16r": lambda: from_example("allreduce_a100_multinode_allpairs.py", [16, 1]),
        "allreduce_a100_ncv4_8r": lambda: from_example("allreduce_a100_ncv4.py", [8, 1]),
        "allreduce_a100_pcie_hierarchical_8r": lambda: from_example("allreduce_a100_pcie_hierarchical.py", [8, 1]),
        "alltonext_forward_2x8": lambda: from_example("alltonext_forward.py", [2, 1]),
        "alltonext_backward_2x8": lambda: from_example("alltonext_backward.py", [2, 1]),
        "pipeline_a100_allpairs_8r": lambda: from_example("pipeline_a100_allpairs.py", [8, 1]),
        "pipeline_a100_ring_8r_2ch": lambda: from_example("pipeline_a100_ring.py", [8, 2, 1]),
    }
    os.makedirs(OUT, exist_ok=True)
    for name, job in jobs.items():
        if ONLY is not None and ONLY not in name:
            continue
        try:
            xml = job()
        except (SystemExit, Exception) as e:  # some examples are written against an older DSL and fail upstream too
            print(f"{name}: skipped ({type(e).__name__}: {e})")
            continue
        with open(os.path.join(OUT, name + ".xml.gz"), "wb") as f:
            f.write(gzip.compress(xml.encode(), 9, mtime=0))
        print(f"{name}: {len(xml)} bytes")


def random_programs():
    """tests/random_programs.py's generator, traced and compiled by msccl-tools' msccl.language.  Every seed is
    compiled in six processes: msccl-tools walks sets of objects hashed by address (rank_dag.py:156-174,
    tb_assignment.py:100-128), so where an order is not otherwise fixed its output changes from process to process;
    every distinct document is kept (random_<seed>_fused, random_<seed>_fused_alt1, ...)."""
    import subprocess
    os.makedirs(RANDOM_OUT, exist_ok=True)
    for seed in RANDOM_SEEDS:
        name = f"random_{seed}_fused"
        if ONLY is not None and ONLY not in name:
            continue
        variants = []
        for _ in range(6):
            out = subprocess.run([sys.executable, os.path.abspath(__file__), REF, "--random-child", str(seed)], capture_output=True, text=True, check=True).stdout
            if out not in variants:
                variants.append(out)
        for old in os.listdir(RANDOM_OUT):
            if old.startswith(name + "_alt") or old == name + ".xml.gz":
                os.remove(os.path.join(RANDOM_OUT, old))
        for k, xml in enumerate(sorted(variants)):
            with open(os.path.join(RANDOM_OUT, name + (f"_alt{k}" if k else "") + ".xml.gz"), "wb") as f:
                f.write(gzip.compress(xml.encode(), 9, mtime=0))
        print(f"{name}: {len(variants)} distinct document(s), {len(variants[0])} bytes")


def random_child(seed):
    install_entry_points()
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import random_programs as rp
    sys.stdout.write(normalise(rp.random_program(seed, fusion=True)[0]))


if __name__ == "__main__":
    if "--random-child" in sys.argv:
        random_child(int(sys.argv[sys.argv.index("--random-child") + 1]))
    else:
        main()
        random_programs()
