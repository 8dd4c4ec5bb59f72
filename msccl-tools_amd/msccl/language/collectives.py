"""Collectives as seen by the MSCCLang front-end: initial symbolic buffers, the aliasing rule of
in-place variants and the post-condition `Check()` asserts (msccl-tools'
msccl/language/collectives.py: AllToAll :22-60, AllGather :63-115, AllReduce :119-169,
ReduceScatter :172-225)."""
from msccl.language.ir import Buffer
from msccl.language.chunk import Chunk, ReduceChunk


class Collective:
    def __init__(self, num_ranks, chunk_factor, inplace):
        self.num_ranks = num_ranks
        self.chunk_factor = chunk_factor
        self.inplace = inplace
        self.name = "custom"

    def init_buffers(self):
        pass

    def check(self, prog):
        pass

    def get_buffer_index(self, rank, buffer, index):
        return buffer, index


def _sum_of_all_ranks(num_ranks, index):
    total = ReduceChunk(-1, [])
    for r in range(num_ranks):
        total = total.reduce(-1, Chunk(r, index))
    return total


class AllToAll(Collective):
    """out_r[i*cf + c] = in_i[r*cf + c]."""

    def __init__(self, num_ranks, chunk_factor, inplace):
        super().__init__(num_ranks, chunk_factor, inplace)
        self.name = "alltoall"

    def init_buffers(self):
        n, cf = self.num_ranks, self.chunk_factor
        result = []
        for r in range(n):
            inp = [Chunk(r, k, k // cf, k % cf + r * cf) for k in range(n * cf)]
            out = inp if self.inplace else [None] * (n * cf)
            result.append({Buffer.input: inp, Buffer.output: out})
        return result

    def check(self, prog):
        ok = True
        for r in range(self.num_ranks):
            out = prog.buffers[r][Buffer.output]
            for i in range(self.num_ranks):
                for c in range(self.chunk_factor):
                    k = i * self.chunk_factor + c
                    got, want = out[k], (i, r * self.chunk_factor + c)
                    if got is None or (got.origin_rank, got.origin_index) != want:
                        print(f"Rank {r} chunk {k} is incorrect should be chunk({want[0]},{want[1]}) given {got}")
                        ok = False
        return ok


class AllGather(Collective):
    """out_r[i*cf + c] = in_i[c]; in place, rank r's input IS output chunks [r*cf, (r+1)*cf)."""

    def __init__(self, num_ranks, chunk_factor, inplace):
        super().__init__(num_ranks, chunk_factor, inplace)
        self.name = "allgather"

    def init_buffers(self):
        n, cf = self.num_ranks, self.chunk_factor
        result = []
        for r in range(n):
            out = [None] * (n * cf)
            if self.inplace:
                for c in range(cf):
                    out[r * cf + c] = Chunk(r, c, -1, r * cf + c)
                inp = out[r * cf:(r + 1) * cf]
            else:
                inp = [Chunk(r, c, -1, r * cf + c) for c in range(cf)]
            result.append({Buffer.input: inp, Buffer.output: out})
        return result

    def check(self, prog):
        ok = True
        for r in range(self.num_ranks):
            out = prog.buffers[r][Buffer.output]
            for i in range(self.num_ranks):
                for c in range(self.chunk_factor):
                    k = i * self.chunk_factor + c
                    got = out[k]
                    if got is None:
                        print(f"Rank {r} chunk {k} is incorrect should be ({i}, {c}) given None")
                        ok = False
                    elif (got.origin_rank, got.origin_index) != (i, c):
                        print(f"Rank {r} chunk {k} is incorrect should be ({i}, {c}) given ({got.origin_rank}, {got.origin_index})")
                        ok = False
        return ok

    def get_buffer_index(self, rank, buffer, index):
        if self.inplace and buffer == Buffer.input:
            return Buffer.output, index + rank * self.chunk_factor
        return buffer, index


class AllReduce(Collective):
    """out_r[c] = sum over ranks of in_i[c]; in place, the output is the input buffer."""

    def __init__(self, num_ranks, chunk_factor, inplace):
        super().__init__(num_ranks, chunk_factor, inplace)
        self.name = "allreduce"

    def init_buffers(self):
        result = []
        for r in range(self.num_ranks):
            inp = [Chunk(r, c, -1, c) for c in range(self.chunk_factor)]
            out = inp if self.inplace else [None] * self.chunk_factor
            result.append({Buffer.input: inp, Buffer.output: out})
        return result

    def check(self, prog):
        buf = Buffer.input if self.inplace else Buffer.output
        want = [_sum_of_all_ranks(self.num_ranks, c) for c in range(self.chunk_factor)]
        ok = True
        for r in range(self.num_ranks):
            out = prog.buffers[r][buf]
            for c in range(self.chunk_factor):
                if out[c] is None or out[c] != want[c]:
                    print(f"Rank {r} chunk {c} is incorrect should be ReduceChunk index {c} from all ranks, given {out[c]}")
                    ok = False
        return ok

    def get_buffer_index(self, rank, buffer, index):
        if self.inplace and buffer == Buffer.output:
            return Buffer.input, index
        return buffer, index


class ReduceScatter(Collective):
    """out_r[c] = sum over ranks of in_i[r*cf + c]; in place, the output of rank r is input
    chunks [r*cf, (r+1)*cf)."""

    def __init__(self, num_ranks, chunk_factor, inplace):
        super().__init__(num_ranks, chunk_factor, inplace)
        self.name = "reduce_scatter"

    def init_buffers(self):
        n, cf = self.num_ranks, self.chunk_factor
        result = []
        for r in range(n):
            inp = [Chunk(r, i * cf + c, i, c) for i in range(n) for c in range(cf)]
            bufs = {Buffer.input: inp}
            if not self.inplace:
                bufs[Buffer.output] = [None] * cf
            result.append(bufs)
        return result

    def check(self, prog):
        buf = Buffer.input if self.inplace else Buffer.output
        want = [_sum_of_all_ranks(self.num_ranks, k) for k in range(self.num_ranks * self.chunk_factor)]
        ok = True
        for r in range(self.num_ranks):
            out = prog.buffers[r][buf]
            for c in range(self.chunk_factor):
                k = r * self.chunk_factor + c
                at = k if self.inplace else c
                if out[at] is None or out[at] != want[k]:
                    print(f"Rank {r} chunk {at} is incorrect should be index {k} from all ranks given {out[at]}")
                    ok = False
        return ok

    def get_buffer_index(self, rank, buffer, index):
        if self.inplace and buffer == Buffer.output:
            return Buffer.input, index + rank * self.chunk_factor
        return buffer, index


# programs written for msccl-tools expect `from msccl.language.collectives import *` to bring the
# language itself along
from msccl.language import *  # noqa: E402,F401,F403
