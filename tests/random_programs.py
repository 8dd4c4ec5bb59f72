"""Random MSCCLang programs for end-to-end parity: a seeded sequence of copies and reduces between
the buffers of a few ranks, traced by this package's front-end into MSCCL-IR, together with what the
sequence means when its statements are executed one after the other on NumPy arrays.  The compiler
(fusion into rcs / rrs / rrc / rrcs, dependencies and their nops, scratch allocation, threadblock and
channel assignment, instance replication), the interpreter and the device must all agree with that."""
import numpy as np

from msccl.language import Buffer, MSCCLProgram, chunk
from msccl.language.chunk import Chunk
from msccl.language.collectives import Collective
from msccl.topologies import fully_connected


class Anything(Collective):
    """Every rank starts with `chunk_factor` chunks in its input buffer; nothing is promised about the end."""

    def init_buffers(self):
        cf = self.chunk_factor
        return [{Buffer.input: [Chunk(r, c, -1, c) for c in range(cf)], Buffer.output: [None] * cf} for r in range(self.num_ranks)]

    def check(self, prog):
        return True


def random_program(seed, fusion=None):
    """-> (xml, statements, ranks, chunks per buffer, instances).  statements: ("copy" | "reduce",
    (rank, buffer, index), (rank, buffer, index), size) with buffer "i" | "o" | a scratch name.
    fusion: True / False, or None for the seed's own choice (on three times out of four)."""
    rng = np.random.default_rng(seed)
    ranks, cf = int(rng.integers(2, 6)), int(rng.integers(2, 5))
    instances = int(rng.integers(1, 3))
    steps = int(rng.integers(8, 28))
    names = {"i": Buffer.input, "o": Buffer.output}
    held = {(r, "i", c) for r in range(ranks) for c in range(cf)}  # slots that hold a chunk
    written = set()                                                # ... because a statement put it there
    scratch_len = {}                                               # (rank, name) -> slots so far
    statements = []
    prog = MSCCLProgram(f"random_{seed}", fully_connected(ranks), Anything(ranks, cf, False), instances,
                        instr_fusion=bool(rng.integers(0, 4)) if fusion is None else fusion, dependence_nop=False)
    with prog:
        last = None  # where the previous statement left its result: going on from there is what the compiler fuses
        for _ in range(steps):
            src = last if last is not None and rng.random() < 0.5 else sorted(held)[int(rng.integers(0, len(held)))]
            last = None
            # (two chunks at a time only without replication: msccl-tools gives instance k of a statement on s chunks at index x
            # the IR chunks [x * instances + k * s, + s), so statements of different sizes cut the same data differently between
            # the instances, and the dependencies it tracks instance by instance no longer cover what the instances touch)
            size = 2 if instances == 1 and (src[0], src[1], src[2] + 1) in held and rng.random() < 0.25 else 1
            if src[1] in names and src[2] + size > cf:
                size = 1
            dst_rank = int(rng.integers(0, ranks))
            if rng.random() < 0.4:  # reduce into slots that hold something
                # (not a local reduce of two slots nothing has written yet: msccl-tools' scheduler starts from the sends and
                # copies that follow the initial chunks, never reaches such a reduce, and silently leaves it out -- as does
                # this package's, which emits the same XML)
                touched = any((src[0], src[1], src[2] + k) in written for k in range(size))
                candidates = [d for d in sorted(held) if d[0] == dst_rank and d != src and all((d[0], d[1], d[2] + k) in held for k in range(size))
                              and not (d[0] == src[0] and d[1] == src[1] and abs(d[2] - src[2]) < size)
                              and (d[0] != src[0] or touched or any((d[0], d[1], d[2] + k) in written for k in range(size)))]
                if not candidates:
                    continue
                dst = candidates[int(rng.integers(0, len(candidates)))]
                ref = chunk(src[0], names.get(src[1], src[1]), src[2], size)
                chunk(dst[0], names.get(dst[1], dst[1]), dst[2], size).reduce(ref)
                statements.append(("reduce", src, dst, size))
                written.update((dst[0], dst[1], dst[2] + k) for k in range(size))
                last = dst
                continue
            kind = rng.random()
            if kind < 0.45:
                dst = (dst_rank, "o", int(rng.integers(0, cf - size + 1)))
            elif kind < 0.7:
                dst = (dst_rank, "i", int(rng.integers(0, cf - size + 1)))
            else:
                name = f"s{int(rng.integers(0, 2))}"
                dst = (dst_rank, name, scratch_len.get((dst_rank, name), 0))  # appended to the scratch buffer
            if dst[0] == src[0] and dst[1] == src[1] and abs(dst[2] - src[2]) < size:
                continue  # overlapping source and destination
            ref = chunk(src[0], names.get(src[1], src[1]), src[2], size)
            if dst[1] in names:
                ref.copy(dst[0], names[dst[1]], dst[2])
            else:
                ref.copy(dst[0], dst[1])
                scratch_len[(dst[0], dst[1])] = dst[2] + size
            for k in range(size):
                held.add((dst[0], dst[1], dst[2] + k))
                written.add((dst[0], dst[1], dst[2] + k))
            statements.append(("copy", src, dst, size))
            last = dst
        xml = prog.generate_xml()
    return xml, statements, ranks, cf, instances


def run_statements(statements, ranks, cf, instances, elems, inputs, outputs):
    """The statements one after the other: inputs/outputs are per-rank float32 arrays of cf * instances
    * elems elements (one program chunk = `instances` IR chunks of `elems` elements); returns the final
    (inputs, outputs)."""
    n = instances * elems
    mem = {}
    for r in range(ranks):
        mem[(r, "i")] = inputs[r].copy()
        mem[(r, "o")] = outputs[r].copy()
    for kind, src, dst, size in statements:
        s = mem[(src[0], src[1])][src[2] * n:(src[2] + size) * n]
        buf = mem.setdefault((dst[0], dst[1]), np.zeros(0, np.float32))
        if buf.size < (dst[2] + size) * n:
            buf = np.concatenate([buf, np.zeros((dst[2] + size) * n - buf.size, np.float32)])
            mem[(dst[0], dst[1])] = buf
        if kind == "copy":
            buf[dst[2] * n:(dst[2] + size) * n] = s
        else:
            buf[dst[2] * n:(dst[2] + size) * n] = buf[dst[2] * n:(dst[2] + size) * n] + s
    return [mem[(r, "i")] for r in range(ranks)], [mem[(r, "o")] for r in range(ranks)]
