"""MSCCLang: chunk-oriented programs traced into MSCCL-IR.

    with MSCCLProgram("ring", fully_connected(8), AllReduce(8, 8, True), instances=1):
        c = chunk(0, Buffer.input, 0)
        c = chunk(1, Buffer.input, 0).reduce(c)
        ...
        XML(); Check()

The user-facing names and their meaning follow msccl-tools' msccl/language/__init__.py:
MSCCLProgram and its keyword arguments (:23-50), the symbolic effect of a copy (dst = src, :65-71)
and of a reduce (dst = dst (+) src, :74-82), `lower()` (:107-126), `chunk`/`XML`/`Check`
(:144-156) and `Ref.copy` / `Ref.reduce` / `split` / `group` (:171-254).
"""
from __future__ import annotations

from msccl.language.ir import (Buffer, ChunkInstruction, ChunkRef, Gpu, Instruction, Op, Program, Threadblock,
                               ThreadblockPolicy, ir_to_xml)
from msccl.language.chunk import Chunk, ReduceChunk
from msccl.language.buffer import BufferSlice
from msccl.language.dag import InstructionDAG
from msccl.language.scheduling import auto_assign_tbs, manual_assign_tbs, topo_sort_instrs, channel_assignment
from msccl.language.checks import ScheduleError, check_dependency_cycles, check_threadblock_ordering

_current_program = None


def _curr():
    if _current_program is None:
        raise RuntimeError("No Program in context")
    return _current_program


class MSCCLProgram:
    def __init__(self, name, topo, collective, instances, protocol="Simple", threadblock_policy=ThreadblockPolicy.auto,
                 interleaved_replication=True, instr_fusion=True, check_xml=True, dependence_nop=False):
        assert protocol in ("Simple", "LL", "LL128"), f"Given protocol: {protocol}. Must be either Simple, LL, LL128"
        self.name = name
        self.topo = topo
        self.collective = collective
        self.num_ranks = topo.num_nodes()
        self.instances = instances
        self.protocol = protocol
        self.threadblock_policy = threadblock_policy
        self.interleaved_replication = interleaved_replication
        self.instr_fusion = instr_fusion
        self.check_xml = check_xml
        self.dependence_nop = dependence_nop
        self.buffers = collective.init_buffers()
        self.instr_dag = InstructionDAG(self.num_ranks, self.buffers)
        # every slot of every input buffer starts life written by a `start` pseudo-op
        for r in range(self.num_ranks):
            for k in range(len(self.buffers[r][Buffer.input])):
                buffer, index = collective.get_buffer_index(r, Buffer.input, k)
                self.instr_dag.add_start(r, buffer, index, self.get_ref(r, buffer, index, 1))

    def __enter__(self):
        global _current_program
        if _current_program is not None:
            raise RuntimeError("There is already a MSCCL Program in context")
        _current_program = self
        return self

    def __exit__(self, exc_type, exc_value, exc_traceback):
        global _current_program
        if _current_program is not self:
            raise RuntimeError("This program is not currently in context")
        _current_program = None

    # ---- symbolic execution ---------------------------------------------------------------------
    def _slots(self, rank, buffer, index):
        buffer, index = self.collective.get_buffer_index(rank, buffer, index)
        return self.buffers[rank][buffer], index

    def apply_send(self, src, src_buffer, src_index, dst, dst_buffer, dst_index, size):
        sb, si = self._slots(src, src_buffer, src_index)
        db, di = self._slots(dst, dst_buffer, dst_index)
        for k in range(size):
            db[di + k] = sb[si + k]

    def apply_reduce(self, src, src_buffer, src_index, dst, dst_buffer, dst_index, size):
        sb, si = self._slots(src, src_buffer, src_index)
        db, di = self._slots(dst, dst_buffer, dst_index)
        for k in range(size):
            db[di + k] = db[di + k].reduce(dst, sb[si + k])

    def get_ref(self, rank, buffer, index, size):
        buffer, index = self.collective.get_buffer_index(rank, buffer, index)
        return Ref(rank, buffer, index, size, self)

    def get_chunks(self, rank, buffer, index, size=1):
        buf = self.buffers[rank][buffer]
        return [buf[index + k] if buf and index + k < len(buf) else None for k in range(size)]

    def check_buffer_exists(self, rank, name):
        if name is not None and name not in self.buffers[rank]:
            self.buffers[rank][name] = BufferSlice(Buffer.scratch, name)

    def check(self):
        return self.collective.check(self)

    # ---- lowering ---------------------------------------------------------------------------------
    def lower(self):
        dag = self.instr_dag
        dag.convert_set_list()
        if self.instr_fusion:
            dag.optimize()
        dag._complete_metadata()
        if self.threadblock_policy == ThreadblockPolicy.manual:
            manual_assign_tbs(dag)
        else:
            auto_assign_tbs(dag)
        dag.lower_pt1(self.instances)
        gpus = dag.lower_pt2(self.instances, self.interleaved_replication)
        if self.check_xml:
            check_dependency_cycles(dag.tbs)
            check_threadblock_ordering(dag)
        return Program(self.name, self.collective.name, self.collective.inplace, self.protocol, gpus)

    def generate_xml(self):
        return ir_to_xml(self.lower(), dependence_nop=self.dependence_nop)


def chunk(rank, buffer, index, size=1):
    if _curr().buffers[rank][buffer][index] is None:
        return None
    return _curr().get_ref(rank, buffer, index, size)


def XML():
    print(_curr().generate_xml())


def Check():
    return _curr().check()


class Ref(ChunkRef):
    """A handle on `size` consecutive chunks of one rank's buffer."""

    def __init__(self, rank, buffer, index, size, prog):
        super().__init__(rank, buffer, index, size)
        self.prog = prog

    def __eq__(self, other):
        return (isinstance(other, ChunkRef) and (self.rank, self.buffer, self.index, self.size) ==
                (other.rank, other.buffer, other.index, other.size))

    def __hash__(self):
        return hash((self.rank, self.buffer, self.index, self.size))

    def __repr__(self):
        return f"Ref(Buffer:{self.buffer}, Index:{self.index}, Size:{self.size}, Rank:{self.rank})"

    def _end(self):
        return self.index + self.size

    def _get_chunk(self, index):
        return self.prog.buffers[self.rank][self.buffer][index]

    def split(self, num):
        assert self.size % num == 0, f"Trying to split a chunk of {self.size} elements into {num} parts"
        part = self.size // num
        return [self.prog.get_ref(self.rank, self.buffer, self.index + k * part, part) for k in range(num)]

    def group(self, other):
        assert self.rank == other.rank, f"Trying to concatenate chunks on ranks {self.rank} and {other.rank}"
        assert self.buffer == other.buffer, f"Trying to concatenate chunks in {self.buffer} and {other.buffer}"
        first = min(self.index, other.index)
        return Ref(self.rank, self.buffer, first, max(self._end(), other._end()) - first, self.prog)

    def copy(self, dst, buffer=None, index=-1, sendtb=-1, recvtb=-1, ch=-1):
        """Copy these chunks to rank `dst` at (buffer, index); returns the destination handle.
        Without buffer and index the chunks keep their place; a scratch buffer named without an
        index is appended to."""
        prog = self.prog
        prog.check_buffer_exists(dst, buffer)
        if index == -1 and buffer is None:
            index, buffer = self.index, self.buffer
        elif index == -1 and buffer is not Buffer.input and buffer is not Buffer.output:
            index = prog.buffers[dst][buffer].instance_size()
        buffer, index = prog.collective.get_buffer_index(self.rank, buffer, index)
        assert prog.topo.link(self.rank, dst) or dst == self.rank, f"No link from {self.rank} to {dst}"
        target = prog.get_ref(dst, buffer, index, self.size)
        if target == self:
            return None
        prog.apply_send(self.rank, self.buffer, self.index, dst, buffer, index, self.size)
        if dst != self.rank:
            send = prog.instr_dag.add_send(self.rank, self, target, sendtb, ch)
            recv = prog.instr_dag.add_recv(dst, self, target, recvtb, ch, send)
            send.recv_match = recv
        else:
            prog.instr_dag.add_copy(self.rank, self, target, sendtb, ch)
        return target

    def reduce(self, other_chunkref, sendtb=-1, recvtb=-1, ch=-1):
        """self = self (+) other; returns self."""
        prog = self.prog
        dst, src = self.rank, other_chunkref.rank
        assert prog.topo.link(src, dst) or src == dst, f"No link from {src} to {dst}"
        prog.apply_reduce(src, other_chunkref.buffer, other_chunkref.index, dst, self.buffer, self.index, self.size)
        if src != dst:
            send = prog.instr_dag.add_send(src, other_chunkref, self, sendtb, ch)
            recv = prog.instr_dag.add_recv_reduce_copy(dst, other_chunkref, self, recvtb, ch, send)
            send.recv_match = recv
        else:
            prog.instr_dag.add_reduce(src, other_chunkref, self, sendtb, ch)
        return self

    def get_origin_index(self, index=0):
        return self._get_chunk(index + self.index).origin_index

    def get_origin_rank(self, index=0):
        return self._get_chunk(index + self.index).origin_rank

    def get_dst_index(self, index=0):
        return self._get_chunk(index + self.index).dst_index

    def get_dst_rank(self, index=0):
        return self._get_chunk(index + self.index).dst_rank

    def print_chunk_info(self, index=0):
        print(self._get_chunk(index + self.index))


__all__ = ["Buffer", "ChunkInstruction", "ChunkRef", "Gpu", "Instruction", "Op", "Program", "Threadblock", "ThreadblockPolicy",
           "ir_to_xml", "Chunk", "ReduceChunk", "BufferSlice", "InstructionDAG", "MSCCLProgram", "Ref", "chunk", "XML", "Check",
           "ScheduleError", "auto_assign_tbs", "manual_assign_tbs", "topo_sort_instrs", "channel_assignment",
           "check_dependency_cycles", "check_threadblock_ordering"]
