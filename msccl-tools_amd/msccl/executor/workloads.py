"""The five benchmark workloads: which compiled algorithm, how many virtual ranks, element type,
bytes per rank, how inputs are drawn, and how algbw/busbw are derived from a launch time.

algbw = S / t and busbw = algbw * f with the nccl-tests conventions: all-reduce S = bytes per rank,
f = 2(n-1)/n; all-gather S = n * input bytes per rank, f = (n-1)/n; all-to-all S = bytes per rank,
f = (n-1)/n.  hbm_fraction = algorithmic_bytes / t / 8e12.
"""
from __future__ import annotations

import dataclasses

import numpy as np

HBM_PEAK_BYTES_PER_S = 8.0e12  # MI355X HBM3E


@dataclasses.dataclass(frozen=True)
class Workload:
    key: str
    cfg: int             # seeds: default_rng(1000*cfg + rank)
    description: str
    coll: str
    ranks: int
    dtype: str
    bytes_per_rank: int  # send-buffer bytes of one rank
    nchunks: int         # chunks the per-rank reference buffer is cut into (all-gather: output chunks)
    build: object        # () -> XML

    @property
    def chunk_bytes(self):
        total = self.bytes_per_rank * self.ranks if self.coll == "allgather" else self.bytes_per_rank
        return total // self.nchunks

    def scaled(self, bytes_per_rank):
        """Same algorithm on smaller buffers (parity tests, smoke)."""
        return dataclasses.replace(self, bytes_per_rank=bytes_per_rank)

    def bandwidths(self, seconds, algorithmic_bytes):
        n = self.ranks
        if self.coll == "allreduce":
            S, f = self.bytes_per_rank, 2.0 * (n - 1) / n
        elif self.coll == "allgather":
            S, f = self.bytes_per_rank * n, (n - 1) / n
        else:
            S, f = self.bytes_per_rank, (n - 1) / n
        algbw = S / seconds
        return {"algbw_GBps": algbw / 1e9, "busbw_GBps": algbw * f / 1e9,
                "algorithmic_GBps": algorithmic_bytes / seconds / 1e9,
                "hbm_fraction": algorithmic_bytes / seconds / HBM_PEAK_BYTES_PER_S}


def _catalog():
    from msccl.programs import catalog
    return catalog


WORKLOADS = {
    "c1": Workload("c1", 1, "ring AllReduce, 8 ranks, 1 channel, 1 instance, 8 chunks; fp32 1 MiB/rank", "allreduce", 8, "float32",
                   1 << 20, 8, lambda: _catalog().ring_allreduce(8, channels=1, instances=1)),
    "c2": Workload("c2", 2, "ring AllGather, 8 ranks, 4 instances; int32 32 MiB/rank", "allgather", 8, "int32",
                   32 << 20, 32, lambda: _catalog().ring_allgather(8, channels=1, instances=4)),
    "c3": Workload("c3", 3, "hierarchical AllToAll, 2 groups x 8 = 16 ranks; uint8 64 MiB/rank", "alltoall", 16, "uint8",
                   64 << 20, 16, lambda: _catalog().hierarchical_alltoall(2, 8)),
    "c4": Workload("c4", 4, "two-level AllReduce, 4 x 8 = 32 ranks, 2 instances; bf16 128 MiB/rank", "allreduce", 32, "bfloat16",
                   128 << 20, 64, lambda: _catalog().two_level_allreduce(8, 4, instances=2)),
    "c5": Workload("c5", 5, "small-message ring AllReduce, 64 ranks, one chunk per ring slot; fp16 256 KiB/rank", "allreduce", 64,
                   "float16", 256 << 10, 64, lambda: _catalog().ring_allreduce(64, channels=1, instances=1)),
    # the other reading of "chunk factor 1" for the 64-rank configuration: the buffer is ONE chunk
    "c5_chain": Workload("c5_chain", 5, "small-message chain AllReduce, 64 ranks, one 256 KiB chunk on a 63-hop reduce chain and a 63-hop "
                         "broadcast chain; fp16 256 KiB/rank", "allreduce", 64, "float16", 256 << 10, 1,
                         lambda: _catalog().chain_allreduce(64)),
}


def _f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + (((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) >> np.uint32(16)).astype(np.uint16)


def numpy_input(w, rank, nbytes=None):
    """Rank `rank`'s send buffer, drawn as the benchmark definition says.  bf16 comes back as
    uint16 bit patterns."""
    nbytes = w.bytes_per_rank if nbytes is None else nbytes
    rng = np.random.default_rng(1000 * w.cfg + rank)
    if w.dtype == "float32":
        return rng.random(nbytes // 4, dtype=np.float32) * 2 - 1
    if w.dtype == "int32":
        return rng.integers(-2 ** 31, 2 ** 31, nbytes // 4, dtype=np.int64).astype(np.int32)
    if w.dtype == "uint8":
        return rng.integers(0, 256, nbytes, dtype=np.uint8)
    if w.dtype == "bfloat16":
        return _f32_to_bf16_bits(rng.standard_normal(nbytes // 2, dtype=np.float32))
    if w.dtype == "float16":
        return (rng.random(nbytes // 2, dtype=np.float32) * 2 - 1).astype(np.float16)
    raise ValueError(w.dtype)


def torch_input(w, rank, device, nbytes=None):
    """Same distributions drawn on the device (full-size runs; not the numpy stream)."""
    import torch
    nbytes = w.bytes_per_rank if nbytes is None else nbytes
    g = torch.Generator(device=device)
    g.manual_seed(1000 * w.cfg + rank)
    if w.dtype == "float32":
        return torch.rand(nbytes // 4, generator=g, device=device, dtype=torch.float32) * 2 - 1
    if w.dtype == "int32":
        return torch.randint(-2 ** 31, 2 ** 31, (nbytes // 4,), generator=g, device=device, dtype=torch.int64).to(torch.int32)
    if w.dtype == "uint8":
        return torch.randint(0, 256, (nbytes,), generator=g, device=device, dtype=torch.uint8)
    if w.dtype == "bfloat16":
        return torch.randn(nbytes // 2, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    if w.dtype == "float16":
        return (torch.rand(nbytes // 2, generator=g, device=device, dtype=torch.float32) * 2 - 1).to(torch.float16)
    raise ValueError(w.dtype)
