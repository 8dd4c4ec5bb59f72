"""All-pairs all-reduce through scratch (msccl-tools' msccl/programs/allreduce_allpairs.py:6-28)."""
from msccl.language import Buffer, chunk


def allreduce_allpairs(size):
    """size*size chunks.  Rank r owns the block of `size` chunks starting at r*size: every peer
    sends its copy of that block into r's scratch, r folds the copies in, and r sends the reduced
    block back to every peer.  Threadblock p of a rank talks to peer p; the local folds are spread
    over `size` threadblocks by chunk position."""
    for src in range(size):
        for dst in range(size):
            if src != dst:
                chunk(src, Buffer.input, dst * size, size=size).copy(dst, "scratch", sendtb=dst, recvtb=src)
    for r in range(size):
        for k in range(size * (size - 1)):
            lane = k % size
            chunk(r, Buffer.input, r * size + lane).reduce(chunk(r, "scratch", k), sendtb=lane)
    for src in range(size):
        for dst in range(size):
            if src != dst:
                chunk(src, Buffer.input, src * size, size).copy(dst, Buffer.input, src * size, sendtb=dst, recvtb=src)
