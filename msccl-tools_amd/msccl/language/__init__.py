"""MSCCLang: chunk-oriented programs traced into MSCCL-IR.

    with MSCCLProgram("ring", fully_connected(8), AllReduce(8, 8, True), instances=1):
        c = chunk(0, Buffer.input, 0)
        c = chunk(1, Buffer.input, 0).reduce(c)
        ...
        XML(); Check()

The user-facing names and their meaning are msccl-tools' (msccl/language/__init__.py): MSCCLProgram
and its keyword arguments (:23-50), what a copy (dst = src, :65-71) and a reduce (dst = dst (+) src,
:74-82) do to the symbolic buffers, `lower()` (:107-126), `chunk` / `XML` / `Check` (:144-156) and
`Ref.copy` / `Ref.reduce` / `split` / `group` (:171-254).

How this module is put together is its own: a traced program is three things kept apart --

* `SymbolicMemory`: what every slot of every rank's buffers holds (the collective's pre-condition
  at first), with the collective's aliasing of in-place buffers applied where a location is named;
* a list of `Transfer`s as the user issues them -- one record per `copy` / `reduce`, which
  `MSCCLProgram.record` turns into the symbolic effect and into the instruction DAG's nodes (a local
  instruction, or a send matched with its receive);
* `LOWERING`, the ordered passes that take the instruction DAG to per-threadblock step lists.
"""
from __future__ import annotations

import dataclasses

from msccl.language.ir import (Buffer, ChunkInstruction, ChunkRef, Gpu, Instruction, Op, Program, Threadblock,
                               ThreadblockPolicy, ir_to_xml)
from msccl.language.chunk import Chunk, ReduceChunk
from msccl.language.buffer import BufferSlice
from msccl.language.dag import InstructionDAG
from msccl.language.scheduling import auto_assign_tbs, manual_assign_tbs, topo_sort_instrs, channel_assignment
from msccl.language.checks import ScheduleError, check_dependency_cycles, check_threadblock_ordering

PROTOCOLS = ("Simple", "LL", "LL128")

# ---- the program being traced -------------------------------------------------------------------
_active = []  # at most one entry: programs do not nest


def active_program():
    if not _active:
        raise RuntimeError("No Program in context")
    return _active[0]


# ---- symbolic state -------------------------------------------------------------------------------
class SymbolicMemory:
    """Per rank, per buffer, the symbolic chunk every slot holds.  Locations are always resolved
    through the collective first, so that the two names of an aliased in-place buffer mean one slot."""

    def __init__(self, collective):
        self.collective = collective
        self.buffers = collective.init_buffers()

    def resolve(self, rank, buffer, index):
        return self.collective.get_buffer_index(rank, buffer, index)

    def slots(self, rank, buffer, index):
        buffer, index = self.resolve(rank, buffer, index)
        return self.buffers[rank][buffer], index

    def populated_inputs(self, rank):
        """Resolved (buffer, index) of every slot of the rank's input buffer, in order."""
        return [self.resolve(rank, Buffer.input, k) for k in range(len(self.buffers[rank][Buffer.input]))]

    def holds(self, rank, buffer, index):
        return self.buffers[rank][buffer][index] is not None

    def peek(self, rank, buffer, index, size=1):
        store = self.buffers[rank][buffer]
        return [store[index + k] if store and index + k < len(store) else None for k in range(size)]

    def scratch(self, rank, name):
        """The named scratch buffer of a rank, created on first use; standard buffers pass through."""
        if name is not None and name not in self.buffers[rank]:
            self.buffers[rank][name] = BufferSlice(Buffer.scratch, name)
        return self.buffers[rank].get(name)

    def overwrite(self, src, dst, size):
        (sb, si), (db, di) = self.slots(*src), self.slots(*dst)
        for k in range(size):
            db[di + k] = sb[si + k]

    def accumulate(self, src, dst, size):
        (sb, si), (db, di) = self.slots(*src), self.slots(*dst)
        for k in range(size):
            db[di + k] = db[di + k].reduce(dst[0], sb[si + k])


@dataclasses.dataclass(frozen=True)
class Transfer:
    """One `copy` or `reduce` as the user wrote it."""
    reduces: bool
    src: "Ref"
    dst: "Ref"
    sendtb: int = -1
    recvtb: int = -1
    ch: int = -1

    @property
    def local(self):
        return self.src.rank == self.dst.rank


# ---- lowering -----------------------------------------------------------------------------------
def _fuse(prog, dag):
    if prog.instr_fusion:
        dag.optimize()


def _assign_threadblocks(prog, dag):
    (manual_assign_tbs if prog.threadblock_policy == ThreadblockPolicy.manual else auto_assign_tbs)(dag)


def _verify(prog, dag):
    if prog.check_xml:
        check_dependency_cycles(dag.tbs)
        check_threadblock_ordering(dag)


# (name, pass over (program, instruction DAG)); `replicate` is where the per-rank Gpu objects appear
LOWERING = (
    ("normalise", lambda prog, dag: dag.convert_set_list()),
    ("fuse", _fuse),
    ("measure", lambda prog, dag: dag._complete_metadata()),
    ("assign threadblocks", _assign_threadblocks),
    ("order steps", lambda prog, dag: dag.lower_pt1(prog.instances)),
    ("replicate", lambda prog, dag: dag.lower_pt2(prog.instances, prog.interleaved_replication)),
    ("verify", _verify),
)


class MSCCLProgram:
    def __init__(self, name, topo, collective, instances, protocol="Simple", threadblock_policy=ThreadblockPolicy.auto,
                 interleaved_replication=True, instr_fusion=True, check_xml=True, dependence_nop=False):
        assert protocol in PROTOCOLS, f"Given protocol: {protocol}. Must be either Simple, LL, LL128"
        self.name, self.topo, self.collective, self.instances = name, topo, collective, instances
        self.num_ranks = topo.num_nodes()
        self.protocol = protocol
        self.threadblock_policy = threadblock_policy
        self.interleaved_replication = interleaved_replication
        self.instr_fusion = instr_fusion
        self.check_xml = check_xml
        self.dependence_nop = dependence_nop
        self.memory = SymbolicMemory(collective)
        self.buffers = self.memory.buffers  # (user collectives' check() reads prog.buffers)
        self.transfers = []
        self.instr_dag = InstructionDAG(self.num_ranks, self.buffers)
        # every slot of every input buffer starts life written by a `start` pseudo-op
        for rank in range(self.num_ranks):
            for buffer, index in self.memory.populated_inputs(rank):
                self.instr_dag.add_start(rank, buffer, index, Ref(rank, buffer, index, 1, self))

    def __enter__(self):
        if _active:
            raise RuntimeError("There is already a MSCCL Program in context")
        _active.append(self)
        return self

    def __exit__(self, exc_type, exc_value, exc_traceback):
        if not _active or _active[0] is not self:
            raise RuntimeError("This program is not currently in context")
        _active.clear()

    # ---- tracing ----------------------------------------------------------------------------------
    def get_ref(self, rank, buffer, index, size):
        buffer, index = self.memory.resolve(rank, buffer, index)
        return Ref(rank, buffer, index, size, self)

    def get_chunks(self, rank, buffer, index, size=1):
        return self.memory.peek(rank, buffer, index, size)

    def record(self, t):
        """Take one Transfer: it must follow a link of the topology; the symbolic buffers change;
        the instruction DAG gets a local instruction, or a send and the receive that matches it."""
        assert t.local or self.topo.link(t.src.rank, t.dst.rank), f"No link from {t.src.rank} to {t.dst.rank}"
        src_at, dst_at = (t.src.rank, t.src.buffer, t.src.index), (t.dst.rank, t.dst.buffer, t.dst.index)
        (self.memory.accumulate if t.reduces else self.memory.overwrite)(src_at, dst_at, t.dst.size)
        self.transfers.append(t)
        dag = self.instr_dag
        if t.local:
            (dag.add_reduce if t.reduces else dag.add_copy)(t.src.rank, t.src, t.dst, t.sendtb, t.ch)
            return
        send = dag.add_send(t.src.rank, t.src, t.dst, t.sendtb, t.ch)
        receive = (dag.add_recv_reduce_copy if t.reduces else dag.add_recv)(t.dst.rank, t.src, t.dst, t.recvtb, t.ch, send)
        send.recv_match = receive

    def check(self):
        return self.collective.check(self)

    # ---- lowering ---------------------------------------------------------------------------------
    def lower(self):
        gpus = None
        for _stage, run in LOWERING:
            out = run(self, self.instr_dag)
            gpus = out if out is not None else gpus
        return Program(self.name, self.collective.name, self.collective.inplace, self.protocol, gpus)

    def generate_xml(self):
        return ir_to_xml(self.lower(), dependence_nop=self.dependence_nop)


def chunk(rank, buffer, index, size=1):
    prog = active_program()
    return prog.get_ref(rank, buffer, index, size) if prog.memory.holds(rank, buffer, index) else None


def XML():
    print(active_program().generate_xml())


def Check():
    return active_program().check()


class Ref(ChunkRef):
    """A handle on `size` consecutive chunks of one rank's buffer."""

    def __init__(self, rank, buffer, index, size, prog):
        super().__init__(rank, buffer, index, size)
        self.prog = prog

    def _key(self):
        return (self.rank, self.buffer, self.index, self.size)

    def __eq__(self, other):
        return isinstance(other, ChunkRef) and self._key() == (other.rank, other.buffer, other.index, other.size)

    def __hash__(self):
        return hash(self._key())

    def __repr__(self):
        return f"Ref(Buffer:{self.buffer}, Index:{self.index}, Size:{self.size}, Rank:{self.rank})"

    @property
    def end(self):
        return self.index + self.size

    def split(self, num):
        assert self.size % num == 0, f"Trying to split a chunk of {self.size} elements into {num} parts"
        part = self.size // num
        return [self.prog.get_ref(self.rank, self.buffer, self.index + k * part, part) for k in range(num)]

    def group(self, other):
        assert self.rank == other.rank, f"Trying to concatenate chunks on ranks {self.rank} and {other.rank}"
        assert self.buffer == other.buffer, f"Trying to concatenate chunks in {self.buffer} and {other.buffer}"
        first = min(self.index, other.index)
        return Ref(self.rank, self.buffer, first, max(self.end, other.end) - first, self.prog)

    def _destination(self, dst, buffer, index):
        """Where a copy to rank `dst` lands: the same place when nothing is said, the end of a
        scratch buffer named without an index, else as given -- then through the collective's aliasing
        (as seen from the SENDING rank, which is how msccl-tools resolves it, language/__init__.py:203)."""
        memory = self.prog.memory
        store = memory.scratch(dst, buffer)
        if index == -1 and buffer is None:
            buffer, index = self.buffer, self.index
        elif index == -1 and buffer is not Buffer.input and buffer is not Buffer.output:
            index = store.instance_size()
        buffer, index = memory.resolve(self.rank, buffer, index)
        return self.prog.get_ref(dst, buffer, index, self.size)

    def copy(self, dst, buffer=None, index=-1, sendtb=-1, recvtb=-1, ch=-1):
        """Copy these chunks to rank `dst` at (buffer, index); returns the destination handle
        (None when source and destination are the same place)."""
        target = self._destination(dst, buffer, index)
        if target == self:
            return None
        self.prog.record(Transfer(False, self, target, sendtb, recvtb, ch))
        return target

    def reduce(self, other_chunkref, sendtb=-1, recvtb=-1, ch=-1):
        """self = self (+) other; returns self."""
        self.prog.record(Transfer(True, other_chunkref, self, sendtb, recvtb, ch))
        return self

    # ---- what the symbolic chunk at a position of this handle says about itself --------------------
    def _symbolic(self, index):
        return self.prog.buffers[self.rank][self.buffer][self.index + index]

    def get_origin_index(self, index=0):
        return self._symbolic(index).origin_index

    def get_origin_rank(self, index=0):
        return self._symbolic(index).origin_rank

    def get_dst_index(self, index=0):
        return self._symbolic(index).dst_index

    def get_dst_rank(self, index=0):
        return self._symbolic(index).dst_rank

    def print_chunk_info(self, index=0):
        print(self._symbolic(index))


__all__ = ["Buffer", "ChunkInstruction", "ChunkRef", "Gpu", "Instruction", "Op", "Program", "Threadblock", "ThreadblockPolicy",
           "ir_to_xml", "Chunk", "ReduceChunk", "BufferSlice", "InstructionDAG", "MSCCLProgram", "Ref", "chunk", "XML", "Check",
           "ScheduleError", "auto_assign_tbs", "manual_assign_tbs", "topo_sort_instrs", "channel_assignment",
           "check_dependency_cycles", "check_threadblock_ordering", "SymbolicMemory", "Transfer", "LOWERING", "active_program"]
