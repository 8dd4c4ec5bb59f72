"""Complete programs: name -> XML, for the benchmark configurations and the tests.

Each builder opens an MSCCLProgram with the collective, replication and threadblock policy the
corresponding msccl-tools program is meant to run with, traces the algorithm, checks the
collective's post-condition symbolically and returns the MSCCL-IR XML.
"""
from __future__ import annotations

from msccl.language import MSCCLProgram, ThreadblockPolicy
from msccl.language.collectives import AllGather, AllReduce, AllToAll, ReduceScatter
from msccl.topologies import fully_connected


def _finish(prog):
    if not prog.check():
        raise RuntimeError(f"program {prog.name} does not implement its collective")
    return prog.generate_xml()


def ring_allreduce(num_ranks, channels=1, instances=1, protocol="Simple"):
    """msccl/programs/allreduce_a100_ring.py as registered in autosynth/ndv4_plans.py:24-32:
    AllReduce(n, n, inplace), manual threadblocks."""
    from msccl.programs.allreduce_a100_ring import allreduce_ring
    prog = MSCCLProgram(f"allreduce_ring_{channels}channelsperring", fully_connected(num_ranks), AllReduce(num_ranks, num_ranks, True),
                        instances, protocol=protocol, threadblock_policy=ThreadblockPolicy.manual)
    with prog:
        allreduce_ring(num_ranks, channels)
    return _finish(prog)


def chain_allreduce(num_ranks, instances=1, protocol="Simple"):
    """AllReduce(n, 1, inplace): the whole buffer is ONE chunk, reduced along a chain of n-1 hops and
    handed on along n-1 more (msccl/programs/allreduce_chain.py) -- what "chunk factor 1" means when
    msccl-tools' registry passes it as the collective's chunk count (autosynth/registry.py:65-66,75-76)."""
    from msccl.programs.allreduce_chain import allreduce_chain
    prog = MSCCLProgram("allreduce_chain", fully_connected(num_ranks), AllReduce(num_ranks, 1, True), instances, protocol=protocol,
                        threadblock_policy=ThreadblockPolicy.manual)
    with prog:
        allreduce_chain(num_ranks)
    return _finish(prog)


def ring_allgather(num_ranks, channels=1, instances=1, protocol="Simple"):
    """examples/mscclang/allgather_ring.py:13-26: AllGather(n, 1, inplace), manual threadblocks."""
    from msccl.programs.allgather_ring import allgather_ring
    prog = MSCCLProgram(f"allgather_ring_{channels}channelsperring", fully_connected(num_ranks), AllGather(num_ranks, 1, True),
                        instances, protocol=protocol, threadblock_policy=ThreadblockPolicy.manual)
    with prog:
        allgather_ring(num_ranks, channels)
    return _finish(prog)


def allpairs_allgather(num_ranks, instances=1, protocol="Simple"):
    """All-pairs all-gather (msccl.programs.allgather_allpairs): AllGather(n, 1, inplace), manual threadblocks."""
    from msccl.programs.allgather_allpairs import allgather_allpairs
    prog = MSCCLProgram("allgather_allpairs", fully_connected(num_ranks), AllGather(num_ranks, 1, True),
                        instances, protocol=protocol, threadblock_policy=ThreadblockPolicy.manual)
    with prog:
        allgather_allpairs(num_ranks)
    return _finish(prog)


def allpairs_alltoall(num_ranks, instances=1, protocol="Simple"):
    """examples/mscclang/alltoall_allpairs.py:10-19: AllToAll(n, 1, out of place), automatic threadblocks."""
    from msccl.programs.alltoall_allpairs import alltoall_allpairs
    prog = MSCCLProgram("alltoall_allpairs", fully_connected(num_ranks), AllToAll(num_ranks, 1, inplace=False), instances, protocol=protocol)
    with prog:
        alltoall_allpairs(num_ranks)
    return _finish(prog)


def hierarchical_alltoall(num_nodes, gpus_per_node, instances=1, protocol="Simple"):
    """examples/mscclang/alltoall_a100_two_step.py:8-48: AllToAll(n, 1, out of place), automatic
    threadblocks."""
    from msccl.programs.alltoall_a100_yifan import alltoall_hierarchical
    n = num_nodes * gpus_per_node
    prog = MSCCLProgram("hierarchical_all_to_all", fully_connected(n), AllToAll(n, 1, False), instances, protocol=protocol)
    with prog:
        alltoall_hierarchical(num_nodes, gpus_per_node)
    return _finish(prog)


def two_level_allreduce(num_local_gpus, num_nodes, instances=1, protocol="Simple", schedule="auto"):
    """examples/mscclang/hierarchical_allreduce.py:26-77: AllReduce(n, n, inplace), batched
    replication, automatic or manual channels."""
    from msccl.programs.hierarchical_allreduce import hierarchical_allreduce
    n = num_local_gpus * num_nodes
    prog = MSCCLProgram("hierarchical_allreduce", fully_connected(n), AllReduce(n, n, True), instances, protocol=protocol,
                        interleaved_replication=False)
    with prog:
        hierarchical_allreduce(num_local_gpus, num_nodes, schedule)
    return _finish(prog)


def allpairs_allreduce(num_ranks, instances=1, protocol="Simple", dependence_nop=True):
    """msccl/programs/allreduce_allpairs.py as registered in autosynth/ndv4_plans.py:14-22."""
    from msccl.programs.allreduce_allpairs import allreduce_allpairs
    prog = MSCCLProgram("allreduce_allpairs", fully_connected(num_ranks), AllReduce(num_ranks, num_ranks * num_ranks, True), instances,
                        protocol=protocol, threadblock_policy=ThreadblockPolicy.manual, interleaved_replication=False,
                        dependence_nop=dependence_nop)
    with prog:
        allreduce_allpairs(num_ranks)
    return _finish(prog)


def three_step_alltoall(num_nodes, gpus_per_node, instances=1, protocol="Simple"):
    """msccl/programs/alltoall_a100_8kp1.py: AllToAll(n, 1, out of place), automatic threadblocks."""
    from msccl.programs.alltoall_a100_8kp1 import alltoall_three_step
    n = num_nodes * gpus_per_node
    prog = MSCCLProgram("alltoall_three_step", fully_connected(n), AllToAll(n, 1, False), 1, protocol=protocol)
    with prog:
        alltoall_three_step(num_nodes, gpus_per_node, instances=instances)
    return _finish(prog)


def ring_reduce_scatter(num_ranks, channels=1, instances=1, protocol="Simple"):
    """Ring reduce-scatter (msccl.programs.reducescatter_ring): ReduceScatter(n, 1, inplace), manual threadblocks."""
    from msccl.programs.reducescatter_ring import reducescatter_ring
    prog = MSCCLProgram(f"reducescatter_ring_{channels}channelsperring", fully_connected(num_ranks), ReduceScatter(num_ranks, 1, True),
                        instances, protocol=protocol, threadblock_policy=ThreadblockPolicy.manual)
    with prog:
        reducescatter_ring(num_ranks, channels)
    return _finish(prog)


def allpairs_reduce_scatter(num_ranks, protocol="Simple"):
    """All-pairs reduce-scatter (msccl.programs.reducescatter_allpairs): ReduceScatter(n, n, inplace), manual
    threadblocks and hoisted reduce dependencies as for the all-pairs all-reduce (msccl-tools'
    msccl/autosynth/ndv4_plans.py:12-22).  One instance only: replication cuts the program's n-chunk copies
    and its one-chunk reduces differently (msccl/language/rank_dag.py:337-340), and rank r's result would
    no longer be the contiguous block the collective defines as its output."""
    from msccl.programs.reducescatter_allpairs import reducescatter_allpairs
    prog = MSCCLProgram("reducescatter_allpairs", fully_connected(num_ranks), ReduceScatter(num_ranks, num_ranks, True), 1,
                        protocol=protocol, threadblock_policy=ThreadblockPolicy.manual, dependence_nop=True)
    with prog:
        reducescatter_allpairs(num_ranks)
    return _finish(prog)


def allpairs_two_level_allreduce(num_groups, group_size, protocol="Simple"):
    """All-pairs inside groups and across them (msccl.programs.allreduce_allpairs_two_level): AllReduce(n, n, inplace),
    manual threadblocks, dependencies of the folds hoisted as for the all-pairs all-reduce."""
    from msccl.programs.allreduce_allpairs_two_level import allreduce_allpairs_two_level
    n = num_groups * group_size
    prog = MSCCLProgram("allreduce_allpairs_two_level", fully_connected(n), AllReduce(n, n, True), 1, protocol=protocol,
                        threadblock_policy=ThreadblockPolicy.manual, dependence_nop=True)
    with prog:
        allreduce_allpairs_two_level(num_groups, group_size)
    return _finish(prog)
