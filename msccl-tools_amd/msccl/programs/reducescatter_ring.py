"""In-place ring reduce-scatter: the reducing half of the ring all-reduce
(msccl-tools' msccl/programs/allreduce_a100_ring.py:12-18) with the start of every chunk's walk moved on
by one rank, so that the sum of chunk k ends on rank k -- where the collective wants it
(msccl/language/collectives.py:172-225; in place, rank k's output is its input chunk k, :220-225)."""
from msccl.language import Buffer, chunk


def reducescatter_ring(size, channels):
    """ReduceScatter(size, 1, inplace): `size` input chunks per rank.  Chunk k starts on rank k+1 and is
    summed around the ring k+1 -> k+2 -> ... -> k; chunk k uses channel and threadblock k % channels."""
    for hop in range(size - 1):
        for k in range(size):
            lane = k % channels
            here, there = (k + 1 + hop) % size, (k + 2 + hop) % size
            chunk(there, Buffer.input, k).reduce(chunk(here, Buffer.input, k), ch=lane, recvtb=lane, sendtb=lane)
