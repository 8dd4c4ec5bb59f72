"""Plan registry: which algorithm serves which (collective, machine type, machine count, size
range).  Same decorators and entry layout as msccl-tools' msccl/autosynth/registry.py:
`register_ef_file` (:42-46), `register_synthesis_plan` (:49-62), `register_msccl_program` (:65-99);
a plan is a callable(machines) -> path of an MSCCL-IR XML file."""
import atexit
import math
import os
import tempfile
from collections import defaultdict

import msccl.language.collectives as lang_collectives
from msccl.autosynth.sizes import parse_size
from msccl.language import MSCCLProgram
from msccl.language.ir import ThreadblockPolicy
from msccl.topologies import distributed_fully_connected

# (collective, machine_type) -> [(description, plan, machines predicate, (low, high), protocol, priority)]
synthesis_plans = defaultdict(list)


def _size_range(sizes):
    if sizes is None:
        return (0, math.inf)
    low, high = sizes
    low = parse_size(low) if isinstance(low, str) else low
    high = math.inf if high is None else parse_size(high) if isinstance(high, str) else high
    return (low, high)


def _register_ef_provider(desc, fun, collective, machine_type, machines, sizes, protocol, priority):
    entry = (desc, fun, machines, _size_range(sizes), protocol, priority)
    for mtype in (machine_type if isinstance(machine_type, list) else [machine_type]):
        synthesis_plans[(collective, mtype)].append(entry)


def _write_temp_xml(xml):
    fd, path = tempfile.mkstemp(suffix=".xml")
    with os.fdopen(fd, "w") as f:
        f.write(xml)
    atexit.register(lambda: os.path.exists(path) and os.remove(path))
    return path


def register_ef_file(path, collective, machine_type, num_machines, sizes=None, protocol="Simple", priority=0):
    _register_ef_provider(f"load {path}", lambda machines: path, collective, machine_type,
                          lambda x: x == num_machines, sizes, protocol, priority)


def register_synthesis_plan(collective, machine_type, machines=lambda x: True, sizes=None, protocol="Simple", priority=0):
    def decorator(fun):
        _register_ef_provider(f"call {fun.__name__}", lambda m: _write_temp_xml(fun(m)), collective, machine_type, machines,
                              sizes, protocol, priority)
        return fun
    return decorator


_COLLECTIVES = {"allreduce": lang_collectives.AllReduce, "allgather": lang_collectives.AllGather,
                "alltoall": lang_collectives.AllToAll, "reduce_scatter": lang_collectives.ReduceScatter}


def register_msccl_program(local_topology, collective, machine_type, machines=lambda x: True, sizes=None, protocol="Simple",
                           chunk_factor=1, priority=0, collective_obj=None, instances=1, inplace=False,
                           threadblock_policy=ThreadblockPolicy.auto, interleaved_replication=True, dependence_nop=False):
    def decorator(fun):
        name = fun.__name__

        def plan(num_machines):
            topology = distributed_fully_connected(local_topology, num_machines, 1)
            co = collective_obj
            if co is None:
                if collective not in _COLLECTIVES:
                    raise RuntimeError(f'No collective_obj in msccl.language.collectives known for "{collective}"')
                co = _COLLECTIVES[collective](topology.num_nodes(), chunk_factor, inplace)
            prog = MSCCLProgram(name, topology, co, instances, protocol, threadblock_policy=threadblock_policy,
                                interleaved_replication=interleaved_replication, dependence_nop=dependence_nop)
            with prog:
                fun(prog, num_machines)
            prog.check()
            return _write_temp_xml(prog.generate_xml())
        _register_ef_provider(f"run {name}", plan, collective, machine_type, machines, sizes, protocol, priority)
        return fun
    return decorator
