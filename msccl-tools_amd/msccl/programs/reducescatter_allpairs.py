"""In-place all-pairs reduce-scatter through scratch: the first two of the three phases of the all-pairs
all-reduce (msccl-tools' msccl/programs/allreduce_allpairs.py:6-21), which leave the sum of rank r's block
on rank r -- the post-condition of msccl/language/collectives.py:172-225."""
from msccl.language import Buffer, chunk


def reducescatter_allpairs(size):
    """ReduceScatter(size, size, inplace): size*size input chunks per rank, rank r owns the block of `size`
    chunks starting at r*size.  Every peer sends its copy of that block into r's scratch (threadblock p of
    a rank talks to peer p) and r folds the copies in, own value first, then the peers in ascending
    order; the folds are spread over `size` threadblocks by chunk position."""
    for src in range(size):
        for dst in range(size):
            if src != dst:
                chunk(src, Buffer.input, dst * size, size=size).copy(dst, "scratch", sendtb=dst, recvtb=src)
    for r in range(size):
        for k in range(size * (size - 1)):
            lane = k % size
            chunk(r, Buffer.input, r * size + lane).reduce(chunk(r, "scratch", k), sendtb=lane)
