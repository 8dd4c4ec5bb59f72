"""Ring all-reduce (msccl-tools' msccl/programs/allreduce_a100_ring.py:10-26)."""
from msccl.language import Buffer, chunk


def allreduce_ring(size, channels):
    """`size` ranks, `size` chunks.  Chunk k starts on rank k, is summed around the ring
    (k -> k+1 -> ...), then the total travels the ring once more.  Chunk k uses channel and
    threadblock k % channels, so channels=1 puts the whole ring on one threadblock per rank."""
    # reduce phase: after hop h, rank (k+h+1) holds the sum of ranks k..k+h+1 of chunk k
    for hop in range(size - 1):
        for k in range(size):
            lane = k % channels
            here, there = (k + hop) % size, (k + hop + 1) % size
            chunk(there, Buffer.input, k).reduce(chunk(here, Buffer.input, k), ch=lane, recvtb=lane, sendtb=lane)
    # broadcast phase: the total of chunk k sits on rank k-1 and visits the other size-1 ranks
    for hop in range(-1, size - 2):
        for k in range(size):
            lane = k % channels
            here, there = (k + hop) % size, (k + hop + 1) % size
            chunk(here, Buffer.input, k).copy(there, Buffer.input, k, ch=lane, recvtb=lane, sendtb=lane)
