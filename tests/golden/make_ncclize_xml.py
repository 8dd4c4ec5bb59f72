"""Writes tests/golden/ncclize_xml/*.xml.gz: MSCCL-IR emitted by msccl-tools' SECOND emitter, ncclize
(msccl/ncclize.py:286-722), for hand-built Algorithm objects (msccl/algorithm.py:29-59).

Runs ONLY in the development container, where the msccl-tools checkout is mounted read-only at
/root/reference; the GPU box only ever sees the committed XML files.  The fixtures are data
(emitter output).  Nothing is synthesized: every algorithm below is a list of (address, source,
destination) sends per step, written by hand, and handed to Algorithm.make_implementation, which
checks it against the collective's pre/postcondition, and then to ncclize().

ncclize.py does `from lxml import etree` and `from z3 import *` at import time; neither package is
installed here.  lxml.etree is served by the standard library's ElementTree (the emitter uses
Element / SubElement / set / indent / tostring); z3 by an EMPTY module object -- its names are only
touched by the scratch-remapping pass (ncclize.py:96-205), which stays off (remap_scratch=False;
asking for it would fail with a NameError, not with a wrong answer).  The top-level package is entered
through an empty stand-in so that msccl/__init__.py (autosynth, which wants more absent packages)
does not run.

usage: python tests/golden/make_ncclize_xml.py [/root/reference]
"""
import gzip
import os
import sys
import types
import xml.etree.ElementTree as ET

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ncclize_xml")
sys.dont_write_bytecode = True


def install_entry_points():
    pkg = types.ModuleType("msccl")
    pkg.__path__ = [os.path.join(REF, "msccl")]
    sys.modules["msccl"] = pkg
    lxml = types.ModuleType("lxml")
    lxml.etree = ET
    sys.modules["lxml"] = lxml
    sys.modules["lxml.etree"] = ET
    sys.modules["z3"] = types.ModuleType("z3")
    sys.path.insert(0, REF)


def main():
    install_entry_points()
    from msccl.algorithm import Algorithm, Step
    from msccl.collectives import allgather, allreduce, alltoall, reduce, reduce_scatter, scatter
    from msccl.instance import Instance
    from msccl.ncclize import ChannelPolicy, ncclize
    from msccl.topologies import fully_connected, line, ring

    def allgather_ring(n):
        steps = [Step(1, [((r - k) % n, r, (r + 1) % n) for r in range(n)]) for k in range(n - 1)]
        return Algorithm.make_implementation(allgather(n), ring(n), Instance(n - 1), steps)

    def allgather_allpairs(n):
        steps = [Step(1, [(r, r, p) for r in range(n) for p in range(n) if p != r])]
        return Algorithm.make_implementation(allgather(n), fully_connected(n), Instance(1), steps)

    def reduce_scatter_allpairs(n, chunks):
        # address a*chunks + j belongs to rank a; every other rank sends its contribution straight to a
        steps = [Step(chunks, [(a * chunks + j, r, a) for a in range(n) for j in range(chunks) for r in range(n) if r != a])]
        return Algorithm.make_implementation(reduce_scatter(n), fully_connected(n), Instance(1, extra_rounds=chunks - 1, chunks=chunks), steps)

    def reduce_tree(n):
        # binary tree towards rank 0 on the single address 0: 1->0 and 3->2, then 2->0
        steps = [Step(1, [(0, 1, 0), (0, 3, 2)]), Step(1, [(0, 2, 0)])]
        return Algorithm.make_implementation(reduce(n, 0), fully_connected(n), Instance(2), steps)

    def allreduce_two_step(n):
        # what msccl/composers.py:compose_allreduce builds: the sends of an all-pairs reduce-scatter
        # followed by the sends of an all-pairs all-gather, over allreduce(n) cut into n addresses
        steps = [Step(1, [(a, r, a) for a in range(n) for r in range(n) if r != a]),
                 Step(1, [(a, a, r) for a in range(n) for r in range(n) if r != a])]
        return Algorithm.make_implementation(allreduce(n), fully_connected(n), Instance(2, chunks=n), steps)

    def alltoall_allpairs(n):
        steps = [Step(1, [(c, c % n, c // n) for c in range(n * n) if c % n != c // n])]
        return Algorithm.make_implementation(alltoall(n), fully_connected(n), Instance(1), steps)

    def scatter_line(n):
        # root 0 at the end of a line: chunk k travels 0 -> 1 -> ... -> k, through scratch on the way
        steps = []
        for t in range(n - 1):
            steps.append(Step(1, [(k, t - (n - 1 - k), t - (n - 1 - k) + 1) for k in range(1, n) if 0 <= t - (n - 1 - k) < k]))
        return Algorithm.make_implementation(scatter(n, 0), line(n), Instance(n - 1), steps)

    jobs = {
        "ncclize_allgather_ring_4r": lambda: ncclize(allgather_ring(4)),
        "ncclize_allgather_ring_5r_3inst": lambda: ncclize(allgather_ring(5), instances=3),
        "ncclize_allgather_allpairs_4r_2inst": lambda: ncclize(allgather_allpairs(4), instances=2),
        "ncclize_reduce_scatter_allpairs_4r_2chunks": lambda: ncclize(reduce_scatter_allpairs(4, 2)),
        "ncclize_reduce_scatter_allpairs_3r_unmerged": lambda: ncclize(reduce_scatter_allpairs(3, 2), merge_contiguous=False, channel_policy=ChannelPolicy.One),
        "ncclize_reduce_tree_4r": lambda: ncclize(reduce_tree(4)),
        "ncclize_allreduce_two_step_4r": lambda: ncclize(allreduce_two_step(4)),
        "ncclize_allreduce_two_step_3r_2inst": lambda: ncclize(allreduce_two_step(3), instances=2),
        "ncclize_alltoall_allpairs_3r": lambda: ncclize(alltoall_allpairs(3)),
        "ncclize_scatter_line_4r": lambda: ncclize(scatter_line(4)),
        "ncclize_scatter_line_4r_noscratch": lambda: ncclize(scatter_line(4), use_scratch=False),
    }
    os.makedirs(OUT, exist_ok=True)
    for name, job in jobs.items():
        xml = job().replace(" />", "/>").strip() + "\n"
        with open(os.path.join(OUT, name + ".xml.gz"), "wb") as f:
            f.write(gzip.compress(xml.encode(), 9, mtime=0))
        print(f"{name}: {len(xml)} bytes")


if __name__ == "__main__":
    main()
