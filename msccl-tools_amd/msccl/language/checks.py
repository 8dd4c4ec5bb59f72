"""Static checks on a scheduled program (msccl-tools' msccl/language/passes.py): the waits between
threadblocks of a rank form no cycle (passes.py:8-27), and two threadblocks that exchange several
messages send and receive them in the same order (passes.py:31-55)."""
from __future__ import annotations


class ScheduleError(Exception):
    pass


def check_dependency_cycles(tbs):
    """`tbs`: per rank, {tb id: Threadblock}.  Raises ScheduleError on a cycle of waits, counting
    the implicit wait of every step for its predecessor in the same threadblock."""
    for rank, rank_tbs in enumerate(tbs):
        WHITE, GREY, BLACK = 0, 1, 2
        colour = {}
        for tbid, tb in rank_tbs.items():
            for root in tb.ops:
                if colour.get(id(root), WHITE) != WHITE:
                    continue
                stack = [(root, iter(_waits(rank_tbs, root)))]
                colour[id(root)] = GREY
                while stack:
                    op, it = stack[-1]
                    nxt = next(it, None)
                    if nxt is None:
                        colour[id(op)] = BLACK
                        stack.pop()
                        continue
                    c = colour.get(id(nxt), WHITE)
                    if c == GREY:
                        raise ScheduleError(f"Cyclic dependency in rank {rank} threadblock {tbid} at {nxt}")
                    if c == WHITE:
                        colour[id(nxt)] = GREY
                        stack.append((nxt, iter(_waits(rank_tbs, nxt))))


def _waits(rank_tbs, op):
    out = list(op.depends)
    tb = rank_tbs.get(op.tb)
    if tb is not None and 0 < op.step < len(tb.ops) and tb.ops[op.step] is op:
        out.append(tb.ops[op.step - 1])
    return out


def check_threadblock_ordering(dag):
    for rank in range(dag.num_ranks):
        for tb in dag.tbs[rank].values():
            last = {}  # (receiver rank, receiver tb) -> step of the last matched receive
            for op in tb.ops:
                if not op.is_send():
                    continue
                match = op.recv_match
                assert op.dst.rank == match.rank, "Bug in MSCCLang: Sends don't match receives"
                key = (match.rank, match.tb)
                if key in last and match.step <= last[key]:
                    raise ScheduleError(f"Rank {op.rank} sends op1 then op2 but {match.rank} receives op2 then op1 "
                                        f"(threadblock {match.tb}, steps {last[key]} and {match.step})")
                last[key] = match.step
