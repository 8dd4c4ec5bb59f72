"""Link matrices the MSCCLang front-end consults (`topo.link(src, dst)`, `topo.num_nodes()`).

On one MI355X every virtual rank reaches every other through HBM, so `fully_connected` is the
natural topology; `line`, `ring` and `distributed_fully_connected` exist because programs and
tests written for msccl-tools name them (msccl/topologies/generic.py, distributed.py).
"""


class Topology:
    """links[dst][src] > 0 means src can send to dst."""

    def __init__(self, name, links):
        self.name = name
        self.links = links

    def link(self, src, dst):
        return self.links[dst][src]

    def num_nodes(self):
        return len(self.links)

    def nodes(self):
        return range(len(self.links))

    def sources(self, dst):
        return (s for s, bw in enumerate(self.links[dst]) if bw > 0)

    def destinations(self, src):
        return (d for d, row in enumerate(self.links) if row[src] > 0)


def _matrix(n, connected):
    return [[1 if connected(src, dst) else 0 for src in range(n)] for dst in range(n)]


def fully_connected(num_nodes):
    return Topology(f"FullyConnected(n={num_nodes})", _matrix(num_nodes, lambda s, d: s != d))


def ring(num_nodes):
    return Topology(f"Ring(n={num_nodes})", _matrix(num_nodes, lambda s, d: s != d and (s - d) % num_nodes in (1, num_nodes - 1)))


def line(num_nodes):
    return Topology(f"Line(n={num_nodes})", _matrix(num_nodes, lambda s, d: abs(s - d) == 1))


def distributed_fully_connected(local_topology, num_copies, remote_bw):
    """num_copies machines with `local_topology` inside each and `remote_bw` between any two ranks
    of different machines."""
    k = local_topology.num_nodes()
    n = k * num_copies
    links = [[remote_bw if src // k != dst // k else local_topology.links[dst % k][src % k] for src in range(n)]
             for dst in range(n)]
    return Topology(f"DistributedFullyConnected(local={local_topology.name},copies={num_copies},bw={remote_bw})", links)


def mi355x_virtual_ranks(num_ranks):
    """All ranks are partitions of one GPU's HBM: any rank reaches any other."""
    t = fully_connected(num_ranks)
    t.name = f"MI355XVirtualRanks(n={num_ranks})"
    return t
