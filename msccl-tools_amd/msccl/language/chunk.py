"""Symbolic chunks: what a buffer slot holds while a program is traced, so that `Check()` can
compare the final placement with the collective's post-condition (msccl/language/chunk.py)."""
from dataclasses import dataclass


@dataclass
class Chunk:
    origin_rank: int
    origin_index: int
    dst_rank: int = -1
    dst_index: int = -1

    def reduce(self, dst, chunk):
        if type(chunk) is ReduceChunk:
            return chunk.reduce(dst, self)
        if type(chunk) is Chunk:
            return ReduceChunk(dst, [self, chunk])
        return None

    def __hash__(self):
        return hash((self.origin_rank, self.origin_index))

    def __eq__(self, other):
        return type(other) is Chunk and (self.origin_rank, self.origin_index) == (other.origin_rank, other.origin_index)

    def __lt__(self, other):
        return (self.origin_rank, self.origin_index) < (other.origin_rank, other.origin_index)


@dataclass
class ReduceChunk:
    """A multiset of input chunks summed together; `creation_rank` records where it was formed."""
    creation_rank: int
    chunks: list

    def reduce(self, dst, chunk):
        if type(chunk) is ReduceChunk:
            merged = self.chunks + chunk.chunks
        elif type(chunk) is Chunk:
            merged = self.chunks + [chunk]
        else:
            merged = self.chunks
        return ReduceChunk(self.creation_rank, merged)

    def sort(self):
        self.chunks.sort()

    def __hash__(self):
        self.sort()
        return hash((self.creation_rank,) + tuple(self.chunks))

    def __eq__(self, other):
        if type(other) is not ReduceChunk:
            return False
        self.sort()
        other.sort()
        return self.chunks == other.chunks
