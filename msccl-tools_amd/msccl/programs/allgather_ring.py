"""In-place ring all-gather (msccl-tools' examples/mscclang/allgather_ring.py:13-26)."""
from msccl.language import Buffer, chunk


def allgather_ring(size, channels):
    """Rank k's chunk sits at output index k and hops k -> k+1 -> ... size-1 times; chunk k uses
    channel and threadblock k % channels."""
    for hop in range(size - 1):
        for k in range(size):
            lane = k % channels
            here, there = (k + hop) % size, (k + hop + 1) % size
            chunk(here, Buffer.output, k).copy(there, Buffer.output, k, sendtb=lane, recvtb=lane, ch=lane)
