"""Instruction DAG of an MSCCLang program: slot-level hazards, instruction fusion, scheduling
metadata, dependency inference, scratch lowering and instance replication.

Behaviour follows msccl-tools' msccl/language/rank_dag.py: `_write`/`_read` hazard rules
(rank_dag.py:47-89), node constructors (:92-154), fusion into rcs / rrs / rrcs (:209-251),
chunk_step / priority (:181-200), `infer_dependencies` (:262-277), scratch offsets (:280-294) and
`replicate` (:318-378).  Edge lists are insertion ordered, so the emitted IR is reproducible.
"""
from __future__ import annotations

from .ir import Buffer, ChunkRef, Gpu, Instruction, Op, Threadblock


def _link(before, after):
    if not any(x is after for x in before.next):
        before.next.append(after)
    if not any(x is before for x in after.prev):
        after.prev.append(before)


def _splice_out(op):
    """Remove `op` from the DAG, connecting its predecessors to its successors."""
    for p in op.prev:
        p.next = [x for x in p.next if x is not op]
        for n in op.next:
            if not any(x is n for x in p.next):
                p.next.append(n)
    for n in op.next:
        n.prev = [x for x in n.prev if x is not op]
        for p in op.prev:
            if not any(x is p for x in n.prev):
                n.prev.insert(0, p)


def _same_tb(a, b):
    return a.tb == b.tb and a.channel == b.channel


def _fusable(recv_like, send):
    return (_same_tb(recv_like, send) and recv_like.cnt() == send.cnt()
            and recv_like.dst.buffer == send.dst.buffer and recv_like.dst.index == send.dst.index)


def _is_scratch(buffer):
    return buffer is not Buffer.input and buffer is not Buffer.output


class InstructionDAG:
    def __init__(self, num_ranks, buffers):
        self.num_ranks = num_ranks
        self.buffers = buffers
        self.operations = {}    # slot -> first op that touches it (the `start` op for inputs)
        self.last_writer = {}   # slot -> op
        self.last_readers = {}  # slot -> [ops] since the last write
        self.tbs = [dict() for _ in range(num_ranks)]
        self.num_channels = [1] * num_ranks
        self.instanced_tbs = None

    # ---- hazards ----------------------------------------------------------------------------
    def _write(self, rank, buffer, index, size, op, read=False):
        befores = []
        for i in range(index, index + size):
            slot = (rank, buffer, i)
            if read:
                assert slot in self.last_writer, f"Destination slot has never been written before a reduce {op}"
            self.operations.setdefault(slot, op)
            readers = self.last_readers.get(slot)
            if readers:
                befores.extend(readers)          # write after read
            elif slot in self.last_writer:
                befores.append(self.last_writer[slot])  # write after write / read-modify-write
            self.last_writer[slot] = op
            self.last_readers[slot] = []
        for b in befores:
            _link(b, op)

    def _read(self, rank, buffer, index, size, op):
        befores = []
        for i in range(index, index + size):
            slot = (rank, buffer, i)
            assert slot in self.last_writer, f"Slot has never been written before a read-type {op}"
            befores.append(self.last_writer[slot])
            self.last_readers.setdefault(slot, []).append(op)
        for b in befores:
            _link(b, op)

    # ---- node constructors --------------------------------------------------------------------
    def add_start(self, rank, buffer, index, ref):
        op = Op(Instruction.start, rank, ref, ref)
        slot = (rank, buffer, index)
        self.operations[slot] = op
        self.last_writer[slot] = op
        return op

    def add_copy(self, rank, send_ref, recv_ref, tb, ch):
        op = Op(Instruction.copy, rank, send_ref, recv_ref, tb=tb, channel=ch)
        self._read(rank, send_ref.buffer, send_ref.index, recv_ref.size, op)
        self._write(rank, recv_ref.buffer, recv_ref.index, recv_ref.size, op)
        return op

    def add_reduce(self, rank, send_ref, recv_ref, tb, ch):
        op = Op(Instruction.reduce, rank, send_ref, recv_ref, tb=tb, channel=ch)
        self._read(rank, send_ref.buffer, send_ref.index, recv_ref.size, op)
        self._write(rank, recv_ref.buffer, recv_ref.index, recv_ref.size, op, read=True)
        return op

    def add_send(self, rank, send_ref, recv_ref, tb, ch):
        op = Op(Instruction.send, rank, send_ref, recv_ref, tb=tb, channel=ch)
        self._read(rank, send_ref.buffer, send_ref.index, send_ref.size, op)
        return op

    def add_recv(self, rank, send_ref, recv_ref, tb, ch, send_op):
        op = Op(Instruction.recv, rank, send_ref, recv_ref, tb=tb, channel=ch)
        self._write(rank, recv_ref.buffer, recv_ref.index, recv_ref.size, op)
        op.send_match = send_op
        return op

    def add_recv_reduce_copy(self, rank, send_ref, recv_ref, tb, ch, send_op):
        op = Op(Instruction.recv_reduce_copy, rank, send_ref, recv_ref, tb=tb, channel=ch)
        self._write(rank, recv_ref.buffer, recv_ref.index, recv_ref.size, op, read=True)
        op.send_match = send_op
        return op

    def convert_set_list(self):
        """Edge lists are lists from the start; kept for callers written against msccl-tools."""

    # ---- traversal ----------------------------------------------------------------------------
    def _all_ops(self):
        """Every op reachable from the first op of any slot, each once, in discovery order."""
        seen, order = set(), []
        for first in self.operations.values():
            stack = [first]
            while stack:
                op = stack.pop()
                if id(op) in seen:
                    continue
                seen.add(id(op))
                order.append(op)
                stack.extend(reversed(op.next))
        return order

    # ---- fusion -------------------------------------------------------------------------------
    def optimize(self):
        self._fuse_reduce_chains()
        self._fuse_copy_chains()

    @staticmethod
    def _absorb_send(op, send, inst):
        op.inst = inst
        op.dst = send.dst
        send.recv_match.send_match = op
        op.recv_match = send.recv_match
        _splice_out(send)

    def _fuse_reduce_chains(self):
        """rrc whose only successor is a matching send becomes rrs when the next thing that happens
        to the slot is a receive overwriting it (the local result is dead), else rrcs."""
        for op in self._all_ops():
            if op.inst is not Instruction.recv_reduce_copy or len(op.next) != 1:
                continue
            send = op.next[0]
            if send.inst is not Instruction.send or not _fusable(op, send):
                continue
            if len(send.next) == 1 and send.next[0].inst is Instruction.recv:
                self._absorb_send(op, send, Instruction.recv_reduce_send)
            else:
                self._absorb_send(op, send, Instruction.recv_reduce_copy_send)

    def _fuse_copy_chains(self):
        """recv followed by a matching send of the same data becomes rcs (first matching successor)."""
        for op in self._all_ops():
            if op.inst is not Instruction.recv:
                continue
            for send in op.next:
                if send.inst is Instruction.send and _fusable(op, send):
                    self._absorb_send(op, send, Instruction.recv_copy_send)
                    break

    # ---- scheduling metadata --------------------------------------------------------------------
    def _complete_metadata(self):
        """chunk_step = longest distance from a start op, priority = longest distance to a sink,
        both over DAG edges plus the edge from a send to its matching receive."""
        ops = self._all_ops()
        # matching receives are reachable only through their send when they are the first op of no slot
        known = {id(o) for o in ops}
        frontier = list(ops)
        while frontier:
            o = frontier.pop()
            m = o.recv_match if o.is_send() else None
            if m is not None and id(m) not in known:
                known.add(id(m))
                ops.append(m)
                frontier.append(m)
                for n in m.next:
                    if id(n) not in known:
                        known.add(id(n)); ops.append(n); frontier.append(n)

        def succ(o):
            out = list(o.next)
            if o.is_send() and o.recv_match is not None:
                out.append(o.recv_match)
            return out

        indeg = {id(o): 0 for o in ops}
        for o in ops:
            for n in succ(o):
                indeg[id(n)] += 1
        ready = [o for o in ops if indeg[id(o)] == 0]
        topo = []
        while ready:
            o = ready.pop()
            topo.append(o)
            for n in succ(o):
                indeg[id(n)] -= 1
                if indeg[id(n)] == 0:
                    ready.append(n)
        assert len(topo) == len(ops), "the instruction DAG has a cycle"
        reached = set()
        for o in topo:
            if o.inst is Instruction.start:
                o.chunk_step = max(o.chunk_step, -1)
                reached.add(id(o))
            if id(o) not in reached:
                continue
            for n in succ(o):
                n.chunk_step = max(n.chunk_step, o.chunk_step + 1)
                reached.add(id(n))
        for o in reversed(topo):
            if id(o) not in reached:
                continue
            nxt = succ(o)
            if not nxt:
                o.priority = 0
            else:
                o.priority = max(o.priority, max(n.priority + 1 for n in nxt))

    # ---- lowering -----------------------------------------------------------------------------
    def lower_pt1(self, instances):
        self.infer_dependencies()
        self.lower_buffers(instances)

    def lower_pt2(self, instances, interleaved):
        self.replicate(instances, interleaved)
        return self.lower_tbs()

    def infer_dependencies(self):
        """An op waits for its DAG predecessors; per predecessor threadblock only the latest step."""
        for op in self._all_ops():
            latest = {}
            for dep in op.prev:
                if dep.inst is Instruction.start:
                    continue
                if dep.tb not in latest or dep.step > latest[dep.tb].step:
                    latest[dep.tb] = dep
            op.depends = list(latest.values())

    def lower_buffers(self, instances):
        for rank_buffers in self.buffers:
            offset = 0
            for key, buf in rank_buffers.items():
                if _is_scratch(key):
                    buf.set_offset(offset)
                    offset += buf.instance_size() * instances

    def lower_chunk(self, ref):
        if ref is not None and _is_scratch(ref.buffer):
            slice_ = self.buffers[ref.rank][ref.buffer]
            return ChunkRef(ref.rank, slice_.get_buffer(), slice_.get_global_index(ref.index), ref.size)
        return ref

    def lower_tbs(self):
        gpus = []
        for rank, rank_tbs in enumerate(self.instanced_tbs):
            for tb in rank_tbs.values():
                for op in tb.ops:
                    op.src = self.lower_chunk(op.src)
                    op.dst = self.lower_chunk(op.dst)
            gpus.append(Gpu(rank, list(rank_tbs.values())))
        return gpus

    def replicate(self, instances, interleaved):
        """Run `instances` copies of the program side by side, each on its own 1/instances of every
        chunk: threadblock t -> t*instances+i, channel c -> max_channels*i+c.  Input/output indices
        are interleaved (index*instances + i*size) or batched (len(buffer)*i + index); scratch is
        always batched."""
        if instances == 1:
            self.instanced_tbs = self.tbs
            return
        self.instanced_tbs = [dict() for _ in range(self.num_ranks)]
        max_channels = max(self.num_channels)

        def instance_ref(ref, i):
            if _is_scratch(ref.buffer):
                index = self.buffers[ref.rank][ref.buffer].instance_size() * i + ref.index
            elif interleaved:
                index = ref.index * instances + i * ref.size
            else:
                index = len(self.buffers[ref.rank][ref.buffer]) * i + ref.index
            return ChunkRef(ref.rank, ref.buffer, index, ref.size)

        for i in range(instances):
            for rank, rank_tbs in enumerate(self.tbs):
                for tbid, tb in rank_tbs.items():
                    itbid = tbid * instances + i
                    itb = Threadblock(max_channels * i + tb.channel, tb.send, tb.recv)
                    itb.ops = [Op(op.inst, op.rank, instance_ref(op.src, i), instance_ref(op.dst, i), [], op.step, itbid)
                               for op in tb.ops]
                    self.instanced_tbs[rank][itbid] = itb
        for rank, rank_tbs in enumerate(self.tbs):
            for tbid, tb in rank_tbs.items():
                for i in range(instances):
                    itb = self.instanced_tbs[rank][tbid * instances + i]
                    for op, iop in zip(tb.ops, itb.ops):
                        iop.depends = [self.instanced_tbs[rank][dep.tb * instances + i].ops[dep.step] for dep in op.depends]
