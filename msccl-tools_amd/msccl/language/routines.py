"""Reusable program fragments (msccl-tools' msccl/language/routines.py:8-27)."""
from msccl.language import Buffer, chunk


def allgather_ring_inplace(gpus, gpu_offset=0, index_offset=0, ch=0):
    """Ring all-gather among ranks [gpu_offset, gpu_offset+gpus): rank k's input chunk travels the
    ring and lands at output index index_offset+k everywhere."""
    for rank in range(gpu_offset, gpu_offset + gpus):
        index = index_offset + rank - gpu_offset
        c = chunk(rank, Buffer.input, 0)
        for hop in range(1, gpus):
            c = c.copy((rank + hop) % gpus + gpu_offset, Buffer.output, index, ch=0)


def allreduce_ring_inplace(gpus, gpu_offset=0, index_offset=0, ch=0):
    """Ring all-reduce among ranks [gpu_offset, gpu_offset+gpus) on `gpus` consecutive chunks."""
    for rank in range(gpu_offset, gpu_offset + gpus):
        index = index_offset + rank - gpu_offset
        c = chunk(rank, Buffer.input, index)
        for hop in range(1, gpus):
            c = chunk((rank + hop) % gpus + gpu_offset, Buffer.input, index).reduce(c, ch=ch)
        for hop in range(0, gpus - 1):
            c = c.copy((rank + hop) % gpus + gpu_offset, Buffer.input, index, ch=ch)
