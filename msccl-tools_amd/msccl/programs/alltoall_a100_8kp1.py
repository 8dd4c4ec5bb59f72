"""Three-step all-to-all: gather per node pair, one cross-node transfer, local scatter
(msccl-tools' msccl/programs/alltoall_a100_8kp1.py:6-78)."""
from msccl.language import Buffer, chunk


def alltoall_three_step(num_nodes, gpus_per_node, instances=1, ib_connections=1):
    def rank_of(node, gpu):
        return node * gpus_per_node + gpu

    def gateway(n_from, n_to):
        """(rank on n_from that gathers traffic for n_to, rank on n_to that scatters it)."""
        def local(a, b):
            return (b if a > b else b - 1) % gpus_per_node
        return rank_of(n_from, local(n_from, n_to)), rank_of(n_to, local(n_to, n_from))

    staged = {}  # (n_from, n_to) -> handle on everything gathered for that node pair
    for n1 in range(num_nodes):
        for g1 in range(gpus_per_node):
            for inst in range(instances):
                for n2 in range(num_nodes):
                    r1 = rank_of(n1, g1)
                    if n1 != n2:
                        block = chunk(r1, Buffer.input, n2 * gpus_per_node * instances + inst * gpus_per_node, gpus_per_node)
                        gather_rank, _ = gateway(n1, n2)
                        landed = block.copy(gather_rank, buffer=(n1, n2), ch=inst * 2)
                        staged[(n1, n2)] = staged[(n1, n2)].group(landed) if (n1, n2) in staged else landed
                    else:
                        for g2 in range(gpus_per_node):
                            r2 = rank_of(n2, g2)
                            c = chunk(r1, Buffer.input, r2 * instances + inst)
                            c.copy(r2, buffer=Buffer.output, index=c.get_dst_index(), ch=inst * 2)
    for (n1, n2), everything in staged.items():
        _, scatter_rank = gateway(n1, n2)
        for part_no, part in enumerate(everything.split(ib_connections)):
            link = part.rank % 2 if ib_connections == 1 else part_no
            arrived = part.copy(scatter_rank, buffer=(n1, n2), ch=link)
            for piece in arrived.split(gpus_per_node * gpus_per_node):
                piece.copy(piece.get_dst_rank(), buffer=Buffer.output, index=piece.get_dst_index(), ch=part_no * 2 + 1)
