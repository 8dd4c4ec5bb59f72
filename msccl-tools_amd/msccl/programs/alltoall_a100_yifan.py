"""Two-step hierarchical all-to-all (msccl-tools' msccl/programs/alltoall_a100_yifan.py:6-39 and its
parametric twin examples/mscclang/alltoall_a100_two_step.py:8-48)."""
from msccl.language import Buffer, chunk


def alltoall_hierarchical(num_nodes, gpus_per_node):
    """Step 1 (inside a node): for every other node m, local gpu g collects from its node-mates the
    chunks addressed to gpu g of node m, appending them to scratch buffer copy_<m>.  Step 2 (across
    nodes): g ships that whole buffer in one message to gpu g of node m.  Chunks addressed to the own
    node go straight to their output slot."""
    num_ranks = num_nodes * gpus_per_node
    for node in range(num_nodes):
        others = [(node + d) % num_nodes for d in range(1, num_nodes)]
        for other in others:
            for g_from in range(gpus_per_node):
                for g_via in range(gpus_per_node):
                    src = node * gpus_per_node + g_from
                    via = node * gpus_per_node + g_via
                    chunk(src, Buffer.input, other * gpus_per_node + g_via).copy(via, f"copy_{other}")
        for other in others:
            for g in range(gpus_per_node):
                rank = node * gpus_per_node + g
                peer = other * gpus_per_node + g
                gathered = chunk(rank, f"copy_{other}", 0, gpus_per_node)
                gathered.copy(peer, Buffer.output, gathered.get_dst_index(),
                              ch=((node + other) % gpus_per_node) * 2 + (rank % 2) + 2)
    for rank in range(num_ranks):
        base = (rank // gpus_per_node) * gpus_per_node
        for g in range(gpus_per_node):
            c = chunk(rank, Buffer.input, base + g)
            c.copy(c.get_dst_rank(), Buffer.output, c.get_dst_index())
