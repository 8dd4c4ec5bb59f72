"""MSCCL-IR: the per-rank, per-threadblock step lists and their XML form.

Follows the format contract of msccl-tools' msccl/language/ir.py: instruction and buffer names
(ir.py:69-92), the <algo>/<gpu>/<tb>/<step> attributes (ir.py:320-391), threadblock ids assigned
after sorting by (send, recv, channel) (ir.py:229-233), removal of intra-threadblock and redundant
dependencies (ir.py:235-255), `hasdep` marking (ir.py:257-262), one dependency per step with extra
ones carried by `nop` steps placed before it (ir.py:296-311), and the optional hoisting of local
reduce dependencies (`dependence_nop`, ir.py:264-291).
"""
from __future__ import annotations

import enum
import xml.etree.ElementTree as ET
from dataclasses import dataclass, field


class _StrEnum(enum.Enum):
    def __str__(self):
        return self.value


class Instruction(_StrEnum):
    nop = "nop"
    send = "s"
    recv = "r"
    recv_copy_send = "rcs"
    recv_reduce_send = "rrs"
    recv_reduce_copy = "rrc"
    recv_reduce_copy_send = "rrcs"
    copy = "cpy"
    reduce = "re"
    delete = "d"
    start = "st"


class Buffer(_StrEnum):
    input = "i"
    output = "o"
    scratch = "s"

    def __lt__(self, other):
        return self.value < other.value


class ThreadblockPolicy(_StrEnum):
    auto = "auto"
    manual = "manual"


class ChunkInstruction(_StrEnum):
    start = "start"
    reduce = "reduce"
    send = "send"


_SENDING = frozenset({Instruction.send, Instruction.recv_copy_send, Instruction.recv_reduce_send, Instruction.recv_reduce_copy_send})
_RECEIVING = frozenset({Instruction.recv, Instruction.recv_copy_send, Instruction.recv_reduce_send, Instruction.recv_reduce_copy,
                        Instruction.recv_reduce_copy_send})
_FUSED = frozenset({Instruction.recv_copy_send, Instruction.recv_reduce_send, Instruction.recv_reduce_copy_send})
_LOCAL = frozenset({Instruction.copy, Instruction.reduce})
# which side of a step is an address on the executing rank
LOCAL_SOURCE = frozenset({Instruction.send, Instruction.copy, Instruction.reduce})
LOCAL_DESTINATION = _RECEIVING | _LOCAL


@dataclass
class ChunkRef:
    rank: int
    buffer: object  # Buffer, or the name of a scratch buffer before lowering
    index: int
    size: int

    def __hash__(self):
        return hash((self.rank, self.buffer, self.index, self.size))


class Op:
    """One instruction.  `prev`/`next` are the slot-level DAG edges (insertion ordered, no
    duplicates); `depends` are the cross-threadblock waits that end up as depid/deps."""

    __slots__ = ("inst", "rank", "src", "dst", "depends", "step", "tb", "prev", "next", "num", "chunk_step", "priority",
                 "recv_match", "send_match", "channel")

    def __init__(self, inst, rank, src, dst, depends=None, step=-1, tb=-1, channel=-1):
        self.inst, self.rank, self.src, self.dst = inst, rank, src, dst
        self.depends = depends if depends is not None else []
        self.step, self.tb, self.channel = step, tb, channel
        self.prev, self.next = [], []
        self.num = -1
        self.chunk_step = -1
        self.priority = -1
        self.recv_match = None
        self.send_match = None

    def cnt(self):
        if self.src is not None:
            if self.dst is not None:
                assert self.src.size == self.dst.size
            return self.src.size
        return self.dst.size if self.dst is not None else 0

    def is_send(self):
        return self.inst in _SENDING

    def is_recv(self):
        return self.inst in _RECEIVING

    def is_fused(self):
        return self.inst in _FUSED

    def is_local(self):
        return self.inst in _LOCAL

    def send_peer(self):
        return self.dst.rank if self.inst in _SENDING else -1

    def recv_peer(self):
        return self.src.rank if self.inst in _RECEIVING else -1

    def __lt__(self, other):
        # heap tie-break between steps of equal scheduling key: lower source index first
        if self.chunk_step != other.chunk_step:
            return self.chunk_step < other.chunk_step
        if self.priority != other.priority:
            return self.priority > other.priority
        return self.src.index < other.src.index

    def __repr__(self):
        return f"Op({self.inst}, {self.rank}, {self.src}, {self.dst}, step:{self.step}, tb:{self.tb})"


class Threadblock:
    __slots__ = ("channel", "send", "recv", "ops", "rbid")

    def __init__(self, channel=-1, send=-1, recv=-1, ops=None):
        self.channel, self.send, self.recv = channel, send, recv
        self.ops = ops if ops is not None else []
        self.rbid = -1


@dataclass
class Gpu:
    rank: int
    threadblocks: list = field(default_factory=list)
    input_chunks: int = 0
    output_chunks: int = 0
    scratch_chunks: int = 0


@dataclass
class Program:
    name: str
    collective: str
    inplace: bool
    protocol: str
    gpus: list = field(default_factory=list)


# ----------------------------------------------------------------------------------------------
# XML emission
# ----------------------------------------------------------------------------------------------
def _buffer_extents(program):
    """chunks each rank's buffers must hold = furthest chunk any local address reaches."""
    extent = {}
    for gpu in program.gpus:
        for tb in gpu.threadblocks:
            for op in tb.ops:
                if op.inst in LOCAL_SOURCE:
                    key = (gpu.rank, op.src.buffer)
                    extent[key] = max(extent.get(key, 0), op.src.index + op.src.size)
                if op.inst in LOCAL_DESTINATION:
                    key = (gpu.rank, op.dst.buffer)
                    extent[key] = max(extent.get(key, 0), op.dst.index + op.dst.size)
    return extent


def _prune_dependencies(program, tb_index):
    home = {id(op): tb_index[id(tb)] for gpu in program.gpus for tb in gpu.threadblocks for op in tb.ops}
    for gpu in program.gpus:
        for tb in gpu.threadblocks:
            me = tb_index[id(tb)]
            seen = []
            for op in tb.ops:
                # a threadblock runs its steps in order, and a wait satisfied once stays satisfied
                kept = [d for d in op.depends if home[id(d)] != me and not any(d is s for s in seen)]
                op.depends = kept
                seen.extend(kept)
    return home


def _hoist_reduce_dependencies(program):
    """dependence_nop: all waits of the local reduces of a threadblock move in front of its first
    reduce (one on that reduce, the others as nops before it)."""
    for gpu in program.gpus:
        for tb in gpu.threadblocks:
            before, after = [], []
            first_reduce = first_dep = None
            for op in tb.ops:
                if op.inst is Instruction.reduce:
                    for dep in op.depends:
                        if first_dep is None:
                            first_dep = dep
                        else:
                            before.append(Op(Instruction.nop, -1, None, None, [dep]))
                    op.depends = []
                    if first_reduce is None:
                        first_reduce = op
                (after if first_reduce is not None else before).append(op)
            if first_dep is not None:
                first_reduce.depends = [first_dep]
            tb.ops = before + after


def _expand_nops(program):
    position = {}
    for gpu in program.gpus:
        for tb in gpu.threadblocks:
            steps = []
            for op in tb.ops:
                if len(op.depends) > 1:
                    for dep in op.depends[1:]:
                        steps.append(Op(Instruction.nop, -1, None, None, [dep]))
                    op.depends = op.depends[:1]
                steps.append(op)
            for k, op in enumerate(steps):
                position[id(op)] = k
            tb.ops = steps
    return position


def ir_to_xml(program, old_format=True, use_scratch=True, pretty_print=True, dependence_nop=False):
    """Serialise a lowered Program.  Reorders each rank's threadblocks and rewrites dependencies in
    place, like the emitter it mirrors."""
    if not old_format or not use_scratch:
        raise NotImplementedError("only the <step> format with a separate scratch buffer is emitted")
    extent = _buffer_extents(program)
    tb_index = {}
    for gpu in program.gpus:
        gpu.threadblocks = sorted(gpu.threadblocks, key=lambda tb: (tb.send, tb.recv, tb.channel))
        for k, tb in enumerate(gpu.threadblocks):
            tb_index[id(tb)] = k
    home = _prune_dependencies(program, tb_index)
    awaited = {id(d) for gpu in program.gpus for tb in gpu.threadblocks for op in tb.ops for d in op.depends}
    if dependence_nop:
        _hoist_reduce_dependencies(program)
    position = _expand_nops(program)

    nchannels = 0
    for gpu in program.gpus:
        if gpu.threadblocks:
            nchannels = max(nchannels, max(tb.channel + 1 for tb in gpu.threadblocks))
    root = ET.Element("algo")
    root.set("name", program.name)
    root.set("proto", program.protocol)
    root.set("nchannels", str(nchannels))
    root.set("nchunksperloop", str(max(max(extent.get((g.rank, Buffer.input), 0), extent.get((g.rank, Buffer.output), 0))
                                       for g in program.gpus)))
    root.set("ngpus", str(len(program.gpus)))
    root.set("coll", program.collective)
    root.set("inplace", "1" if program.inplace else "0")
    for gpu in program.gpus:
        g = ET.SubElement(root, "gpu")
        g.set("id", str(gpu.rank))
        g.set("i_chunks", str(max(extent.get((gpu.rank, Buffer.input), 0), gpu.input_chunks)))
        g.set("o_chunks", str(max(extent.get((gpu.rank, Buffer.output), 0), gpu.output_chunks)))
        g.set("s_chunks", str(max(extent.get((gpu.rank, Buffer.scratch), 0), gpu.scratch_chunks)))
        for tb in gpu.threadblocks:
            t = ET.SubElement(g, "tb")
            t.set("id", str(tb_index[id(tb)]))
            t.set("send", str(tb.send))
            t.set("recv", str(tb.recv))
            t.set("chan", str(tb.channel))
            for op in tb.ops:
                s = ET.SubElement(t, "step")
                s.set("s", str(position[id(op)]))
                s.set("type", str(op.inst))
                s.set("srcbuf", str(op.src.buffer) if op.src is not None else "i")
                s.set("srcoff", str(op.src.index) if op.src is not None else "-1")
                s.set("dstbuf", str(op.dst.buffer) if op.dst is not None else "o")
                s.set("dstoff", str(op.dst.index) if op.dst is not None else "-1")
                s.set("cnt", str(op.cnt()))
                assert len(op.depends) <= 1
                if op.depends:
                    s.set("depid", str(home[id(op.depends[0])]))
                    s.set("deps", str(position[id(op.depends[0])]))
                else:
                    s.set("depid", "-1")
                    s.set("deps", "-1")
                s.set("hasdep", "1" if id(op) in awaited else "0")
    if pretty_print:
        ET.indent(root, space="  ")
    # lxml writes empty elements as <step .../> without a space before the slash
    return ET.tostring(root, encoding="unicode").replace(" />", "/>")
