"""Reusable program fragments (msccl-tools' msccl/language/routines.py:8-27): rings among the ranks
[gpu_offset, gpu_offset + gpus), written as walks -- a chunk that starts on a ring member and visits
the members after it."""
from msccl.language import Buffer, chunk


def _walks(gpus, gpu_offset, index_offset):
    """One walk per ring member: (member, the buffer index that belongs to it, a function from a
    range of hops to the ranks that many steps round the ring).  The peer formula is msccl-tools' own,
    offsets and all."""
    for member in range(gpu_offset, gpu_offset + gpus):
        yield member, index_offset + member - gpu_offset, lambda hops, member=member: [(member + hop) % gpus + gpu_offset for hop in hops]


def allgather_ring_inplace(gpus, gpu_offset=0, index_offset=0, ch=0):
    """Ring all-gather: every member's input chunk travels the ring and lands at that member's output
    index on every rank.  (Always on channel 0, whatever `ch` says: msccl-tools does the same, and the
    XML has to come out the same.)"""
    for member, index, ranks_at in _walks(gpus, gpu_offset, index_offset):
        travelling = chunk(member, Buffer.input, 0)
        for peer in ranks_at(range(1, gpus)):
            travelling = travelling.copy(peer, Buffer.output, index, ch=0)


def allreduce_ring_inplace(gpus, gpu_offset=0, index_offset=0, ch=0):
    """Ring all-reduce on `gpus` consecutive chunks: chunk k is summed along the ring starting at
    member k, and the total is passed round once more."""
    for member, index, ranks_at in _walks(gpus, gpu_offset, index_offset):
        total = chunk(member, Buffer.input, index)
        for peer in ranks_at(range(1, gpus)):
            total = chunk(peer, Buffer.input, index).reduce(total, ch=ch)
        for peer in ranks_at(range(gpus - 1)):  # the total sits on the last rank of the sum: round once more from hop 0
            total = total.copy(peer, Buffer.input, index, ch=ch)
