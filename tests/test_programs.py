"""Registered programs: the symbolic checks msccl-tools runs on them (tests/test_programs.py:10-59
there) and what the lowered IR looks like."""
import numpy as np

from msccl.executor import Plan, parse_algo_xml
from msccl.language import *
from msccl.language.collectives import *
from msccl.topologies import fully_connected


def test_registered_alltoall_yifan():
    from msccl.programs.alltoall_a100_yifan import alltoall_hierarchical
    num_ranks = 4 * 8
    with MSCCLProgram("hierarchical_all_to_all", fully_connected(num_ranks), AllToAll(num_ranks, 1, inplace=False), 1):
        alltoall_hierarchical(4, 8)
        assert Check()


def test_registered_alltoall_8kp1(capsys):
    from msccl.programs.alltoall_a100_8kp1 import alltoall_three_step
    num_ranks = 9 * 8
    with MSCCLProgram("hierarchical_all_to_all", fully_connected(num_ranks), AllToAll(num_ranks, 1, inplace=False), 1):
        alltoall_three_step(9, 8)
        assert Check()
        XML()
    xml = capsys.readouterr().out
    t = parse_algo_xml(xml)
    assert t.ngpus == 72 and t.coll == "alltoall"
    p = Plan(t)  # 72 ranks: validates, matches every connection
    assert p.min_fifo_depth() >= 1
    assert p.algorithmic_units() > 0


def test_registered_allreduce_ring(capsys):
    from msccl.programs.allreduce_a100_ring import allreduce_ring
    with MSCCLProgram("allreduce_ring", fully_connected(8), AllReduce(8, 8, inplace=True), 4, protocol="LL128",
                      threadblock_policy=ThreadblockPolicy.manual):
        allreduce_ring(8, 8)
        assert Check()
        XML()
    t = parse_algo_xml(capsys.readouterr().out)
    assert (t.proto, t.nchannels, t.nchunksperloop) == ("LL128", 32, 32)
    assert t.ntbs == 8 * 8 * 4


def test_registered_allreduce_allpairs(capsys):
    from msccl.programs.allreduce_allpairs import allreduce_allpairs
    with MSCCLProgram("allreduce_allpairs", fully_connected(8), AllReduce(8, 64, inplace=True), 2, protocol="LL",
                      threadblock_policy=ThreadblockPolicy.manual):
        allreduce_allpairs(8)
        assert Check()
        XML()
    t = parse_algo_xml(capsys.readouterr().out)
    types = np.bincount(t.ops[:, 0], minlength=9)
    assert types[8] == 8 * 56 * 2          # one local reduce per (rank, scratch chunk, instance)
    assert types[1] == types[2] == 8 * 7 * 2 * 2


def test_catalog_builds_the_workloads():
    from msccl.executor.workloads import WORKLOADS
    expect = {"c1": (8, 8, 120), "c2": (8, 32, 256), "c3": (16, 256, 624), "c4": (32, 1920, 4480), "c5": (64, 64, 8128), "c5_chain": (64, 64, 127)}
    for key, w in WORKLOADS.items():
        t = parse_algo_xml(w.build())
        assert (t.ngpus, t.ntbs, t.nops) == expect[key], key
        assert t.algorithmic_units() * w.chunk_bytes == {"c1": 5 * 7 * (1 << 20), "c2": 2 * 7 * 8 * (32 << 20),
                                                         "c3": 3 * 16 * (64 << 20), "c4": 5 * 31 * (128 << 20),
                                                         "c5": 5 * 63 * (256 << 10), "c5_chain": 5 * 63 * (256 << 10)}[key]
