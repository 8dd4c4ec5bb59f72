"""In-place all-pairs all-gather: every rank copies its chunk straight to every other rank -- one hand-off
deep, the same 2(n-1)nS bytes a ring moves.  (The schedule of msccl-tools' examples/mscclang/allgather_allpairs.py:10-25,
one threadblock per peer; the copies here land at the output index the collective asks for.)"""
from msccl.language import Buffer, chunk


def allgather_allpairs(size):
    """Rank k's chunk already sits at output index k (in place); threadblock p of a rank sends to peer p,
    threadblock k of the peer receives from k."""
    for owner in range(size):
        mine = chunk(owner, Buffer.output, owner)
        for peer in range(size):
            if peer != owner:
                mine.copy(peer, Buffer.output, owner, sendtb=peer, recvtb=owner)
