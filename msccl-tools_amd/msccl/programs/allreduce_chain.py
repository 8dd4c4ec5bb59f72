"""All-reduce of one chunk along a chain: the ring all-reduce of msccl-tools
(msccl/programs/allreduce_a100_ring.py:10-26) when the buffer is a single chunk -- that program
indexes one chunk per rank, so with AllReduce(size, 1) only its chunk 0 exists."""
from msccl.language import Buffer, chunk


def allreduce_chain(size):
    """The chunk is summed from rank 0 to rank size-1 (size-1 dependent hops), then the total
    travels on round the ring, size-1 -> 0 -> 1 -> ... -> size-2 (size-1 more hops).  One
    threadblock and one channel per rank."""
    for hop in range(size - 1):
        chunk(hop + 1, Buffer.input, 0).reduce(chunk(hop, Buffer.input, 0), ch=0, recvtb=0, sendtb=0)
    for hop in range(-1, size - 2):
        chunk(hop % size, Buffer.input, 0).copy(hop + 1, Buffer.input, 0, ch=0, recvtb=0, sendtb=0)
