"""Ordering of instructions, channel assignment and threadblock assignment.

Behaviour follows msccl-tools' msccl/language/tb_assignment.py: `topo_sort_instrs` (heap keyed by
(chunk_step, -priority, dst.index), seeded with the sends/copies that follow a start,
tb_assignment.py:100-128), `channel_assignment` for fused flows and the send/receive order fix-up
(:130-224), `manual_assign_tbs` (:22-41) and `auto_assign_tbs` (:43-96).
"""
from __future__ import annotations

import heapq
from collections import defaultdict

from .ir import Instruction, Threadblock

MAX_CHANNELS = 32


def _compatible(tb, op):
    s = op.dst.rank if op.is_send() else -1
    r = op.src.rank if op.is_recv() else -1
    return ((tb.send == s or s == -1 or tb.send == -1) and (tb.recv == r or r == -1 or tb.recv == -1)
            and (tb.channel == op.channel or tb.channel == -1 or op.channel == -1))


def topo_sort_instrs(dag):
    """Order in which instructions are handed to threadblocks: a send before its receive,
    predecessors before successors, otherwise earliest chunk_step, then highest priority, then
    lowest destination index."""
    def key(op):
        return (op.chunk_step, -op.priority, op.dst.index)

    visited = set()
    heap, ordered = [], []
    for first in dag.operations.values():
        if first.inst is Instruction.start:
            visited.add(id(first))
            for o in first.next:
                if o.inst is Instruction.send or o.inst is Instruction.copy:
                    heapq.heappush(heap, (key(o), o))
    while heap:
        _, op = heapq.heappop(heap)
        if id(op) in visited:
            continue
        ordered.append(op)
        visited.add(id(op))
        match = op.recv_match
        if match is not None and all(id(p) in visited for p in match.prev):
            heapq.heappush(heap, (key(match), match))
        for o in op.next:
            if all(id(p) in visited for p in o.prev):
                heapq.heappush(heap, (key(o), o))
    return ordered


def channel_assignment(instrs, dag):
    """Fused receivers forward on the channel they receive on, so two chains ("flows") that share
    an edge but differ elsewhere need different channels; afterwards channels are bumped until, on
    every (sender, receiver, channel), receives happen in the order of the sends."""
    free_send = [defaultdict(lambda: set(range(MAX_CHANNELS))) for _ in range(dag.num_ranks)]
    free_recv = [defaultdict(lambda: set(range(MAX_CHANNELS))) for _ in range(dag.num_ranks)]
    flows, flow_channels = [], []

    def reserve(sender, receiver, ch):
        free_send[sender][receiver].discard(ch)
        free_recv[receiver][sender].discard(ch)

    def walk(op, channels, path):
        if op.is_local():
            op.channel = 0
            return
        if not op.is_send():
            return
        match = op.recv_match
        sender, receiver = op.rank, match.rank
        channels = free_send[sender][receiver] & free_recv[receiver][sender] & channels
        path.append(op.rank)
        if not match.is_fused():
            path.append(match.rank)
            flow = {(path[i - 1], path[i]) for i in range(1, len(path))}
            if op.channel != -1:
                ch = op.channel
            elif flow in flows:
                ch = flow_channels[flows.index(flow)]
            else:
                ch = min(channels)
                flows.append(flow)
                flow_channels.append(ch)
            op.channel = ch
            match.channel = ch
        else:
            walk(match, channels, path)
            ch = match.channel
            op.channel = ch
        reserve(sender, receiver, ch)

    for op in instrs:
        if op.inst is Instruction.send and op.recv_match.is_fused():
            walk(op, set(range(MAX_CHANNELS)), [])

    again = True
    while again:
        again = False
        pending = defaultdict(list)  # (sender, receiver, channel) -> receives in send order
        for op in instrs:
            ch = 0 if op.channel == -1 else op.channel
            if op.is_send():
                pending[(op.rank, op.dst.rank, ch)].append(op.recv_match)
            if op.is_recv():
                queue = pending[(op.src.rank, op.rank, ch)]
                at = next((k for k, x in enumerate(queue) if x is op), None)
                if at is None:
                    continue
                if at == 0:
                    del queue[0]
                else:
                    again = True
                    op.channel += 1
                    op.send_match.channel += 1
                    del queue[at]


def manual_assign_tbs(dag):
    """Threadblock and channel are the user's (sendtb / recvtb / ch); conflicts raise."""
    for op in topo_sort_instrs(dag):
        tbs = dag.tbs[op.rank]
        if op.tb not in tbs:
            tbs[op.tb] = Threadblock()
        tb = tbs[op.tb]
        if not _compatible(tb, op):
            raise Exception(
                f"Illegal threadblock assignment. Trying to add {op} to threadblock {op.tb}\n"
                f"Threadblock {op.tb} send:{tb.send} recv:{tb.recv} channel:{tb.channel}\n"
                f"Operation send:{op.dst.rank if op.is_send() else -1} recv:{op.src.rank if op.is_recv() else -1} channel:{op.channel}")
        tb.ops.append(op)
        tb.channel = op.channel if op.channel != -1 else 0
        if op.is_send():
            tb.send = op.dst.rank
        if op.is_recv():
            tb.recv = op.src.rank
        op.step = len(tb.ops) - 1
        dag.num_channels[op.rank] = max(op.channel + 1, dag.num_channels[op.rank])


def _candidates(tbs, send, recv, channel):
    options = []
    for tbid, tb in tbs.items():
        channel_ok = channel == -1 or channel == tb.channel
        # a peer's connection on this channel is already owned by a threadblock: it must be that one
        if channel_ok and ((tb.send == send and send != -1) or (tb.recv == recv and recv != -1)):
            return [tbid]
        if (send == -1 or tb.send == send) and (recv == -1 or tb.recv == recv) and channel_ok:
            options.append(tbid)
    return options


def auto_assign_tbs(dag):
    instrs = topo_sort_instrs(dag)
    channel_assignment(instrs, dag)
    next_id = [0] * dag.num_ranks
    progress = [dict() for _ in range(dag.num_ranks)]  # tb -> chunk_step of its last op
    for op in instrs:
        rank = op.rank
        s, r = op.send_peer(), op.recv_peer()
        channel = 0 if op.channel == -1 else op.channel
        options = _candidates(dag.tbs[rank], s, r, channel)
        if not options:
            tbid = next_id[rank]
            dag.tbs[rank][tbid] = Threadblock(send=s, recv=r, channel=channel)
            next_id[rank] += 1
        else:
            tbid = options[0]
            for cand in options:
                if progress[rank][cand] < progress[rank][tbid] and _compatible(dag.tbs[rank][tbid], op):
                    tbid = cand
        tb = dag.tbs[rank][tbid]
        assert _compatible(tb, op), (f"Failing: Operations uses channel {op.channel}, send:{s} recv:{r} {op}\n"
                                     f"Threadblock uses send:{tb.send} recv:{tb.recv} channel:{tb.channel}")
        dag.num_channels[rank] = max(dag.num_channels[rank], channel + 1)
        tb.ops.append(op)
        if op.is_send():
            tb.send = op.dst.rank
        if op.is_recv():
            tb.recv = op.src.rank
        op.step = len(tb.ops) - 1
        op.tb = tbid
        progress[rank][tbid] = op.chunk_step
