"""Two-level all-reduce: reduce-scatter inside each node, reduce-scatter and all-gather across
nodes, all-gather inside each node (msccl-tools' examples/mscclang/hierarchical_allreduce.py:13-77)."""
from msccl.language import Buffer, chunk


def ring_reduce_scatter(size, rank_offset=0, rank_step=1, local_chunk_size=1, chunk_offset=0, chunk_stride=1, chan=-1):
    """Ring over ranks rank_offset + k*rank_step.  Block b (at index b*chunk_stride*local_chunk_size +
    chunk_offset) starts on ring position b+1 and is summed around the ring to end on position b."""
    for b in range(size):
        index = b * chunk_stride * local_chunk_size + chunk_offset
        for hop in range(size - 1):
            src = ((hop + 1 + b) % size) * rank_step + rank_offset
            dst = ((hop + 2 + b) % size) * rank_step + rank_offset
            chunk(dst, Buffer.input, index, local_chunk_size).reduce(chunk(src, Buffer.input, index, local_chunk_size), ch=chan)


def ring_all_gather(size, rank_offset=0, rank_step=1, local_chunk_size=1, chunk_offset=0, chunk_stride=1, chan=-1):
    """Ring over the same ranks: block b starts on ring position b and visits the others."""
    for b in range(size):
        index = b * chunk_stride * local_chunk_size + chunk_offset
        for hop in range(size - 1):
            src = ((hop + b) % size) * rank_step + rank_offset
            dst = ((hop + 1 + b) % size) * rank_step + rank_offset
            chunk(src, Buffer.input, index, local_chunk_size).copy(dst, Buffer.input, index, ch=chan)


def hierarchical_allreduce(num_local_gpus, num_nodes, schedule="auto"):
    """num_local_gpus*num_nodes ranks and as many chunks.  schedule='manual' pins channels the way
    the reference example does; 'auto' leaves channels and threadblocks to the compiler."""
    manual = schedule != "auto"
    for node in range(num_nodes):
        for off in range(num_nodes):
            ring_reduce_scatter(num_local_gpus, rank_offset=node * num_local_gpus, chunk_offset=off, chunk_stride=num_nodes,
                                chan=off if manual else -1)
    for g in range(num_local_gpus):
        ring_reduce_scatter(num_nodes, rank_offset=g, rank_step=num_local_gpus, chunk_offset=g * num_nodes,
                            chan=g % 2 + num_nodes * 2 if manual else -1)
    for g in range(num_local_gpus):
        ring_all_gather(num_nodes, rank_offset=g, rank_step=num_local_gpus, chunk_offset=g * num_nodes,
                        chan=g % 2 + num_nodes * 2 if manual else -1)
    for node in range(num_nodes):
        for off in range(num_nodes):
            ring_all_gather(num_local_gpus, rank_offset=node * num_local_gpus, chunk_offset=off, chunk_stride=num_nodes,
                            chan=off + num_nodes if manual else -1)
