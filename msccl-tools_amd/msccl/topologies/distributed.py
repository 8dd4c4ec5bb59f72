"""`from msccl.topologies.distributed import *`, as programs written for msccl-tools spell it."""
from msccl.topologies import Topology, distributed_fully_connected  # noqa: F401

__all__ = ["distributed_fully_connected"]
