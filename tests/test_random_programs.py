"""Random MSCCLang programs, end to end on the CPU: what this package's compiler emits for a random
sequence of copies and reduces, run by the interpreter, must leave in every rank's input and output
buffers exactly what the statements leave when they are executed one after the other -- a check of
the interpreter's step semantics (and of the compiler's hazard tracking, scheduling and replication)
against something that shares no code with either.  (The device takes the same programs in
tests/test_gpu_random_programs.py.)

Instruction fusion is off here: msccl-tools' fusion passes, which this package reproduces to the byte,
mis-handle programs outside the shapes its examples use -- about one random program in seven comes
out with unmatched connections or with a fused receive-and-forward that files its chunk at the
*destination's* scratch offset -- so fused programs are held to the weaker standards below."""
import re

import numpy as np
import pytest

import random_programs as rp
from msccl.executor import MscclxError, Plan, parse_algo_xml
from oracle import ir_interp as oi

SEEDS = list(range(80))
ELEMS = 37  # elements per IR chunk: not a multiple of anything


def initial(ranks, cf, instances, seed):
    rng = np.random.default_rng(1000 + seed)
    n = cf * instances * ELEMS
    return ([rng.standard_normal(n).astype(np.float32) for _ in range(ranks)], [rng.standard_normal(n).astype(np.float32) for _ in range(ranks)])


def interpret(xml, ins, outs):
    algo = oi.parse_xml(xml)
    bufs = [{"i": ins[r][:g.i_chunks * ELEMS].copy(), "o": outs[r][:g.o_chunks * ELEMS].copy(), "s": np.zeros(g.s_chunks * ELEMS, np.float32)}
            for r, g in enumerate(algo.gpus)]  # (the XML declares a buffer only as far as the program uses it)
    oi.Interpreter(algo).run(bufs, ELEMS, "float32")
    return algo, bufs


def means_its_statements(algo, bufs, want_i, want_o, ins, outs):
    for r, g in enumerate(algo.gpus):
        for b, want, before, used in (("i", want_i[r], ins[r], g.i_chunks * ELEMS), ("o", want_o[r], outs[r], g.o_chunks * ELEMS)):
            if not np.array_equal(bufs[r][b].view(np.uint32), want[:used].view(np.uint32)):
                return f"rank {r} buffer {b} differs"
            if not np.array_equal(want[used:].view(np.uint32), before[used:].view(np.uint32)):
                return f"rank {r} buffer {b}: the statements touch what the XML does not declare"
    return None


@pytest.mark.parametrize("seed", SEEDS)
def test_compiled_program_means_its_statements(seed):
    xml, statements, ranks, cf, instances = rp.random_program(seed, fusion=False)
    ins, outs = initial(ranks, cf, instances, seed)
    want_i, want_o = rp.run_statements(statements, ranks, cf, instances, ELEMS, ins, outs)
    algo, bufs = interpret(xml, ins, outs)
    assert means_its_statements(algo, bufs, want_i, want_o, ins, outs) is None


def test_fused_programs_mostly_mean_their_statements_and_cover_the_fused_step_types(mscclx_lib):
    """With fusion on: every step type of the IR turns up; what the host library accepts as well-formed
    and the interpreter can finish means its statements in at least nine cases out of ten."""
    seen, usable, right = set(), 0, 0
    for seed in range(120):
        xml, statements, ranks, cf, instances = rp.random_program(seed, fusion=True)
        try:
            Plan(parse_algo_xml(xml))
        except MscclxError:
            continue  # unmatched sends and receives: refused before anything runs
        ins, outs = initial(ranks, cf, instances, seed)
        try:
            algo, bufs = interpret(xml, ins, outs)
        except oi.Deadlock:
            continue
        usable += 1
        seen |= set(re.findall(r'type="(\w+)"', xml))
        want_i, want_o = rp.run_statements(statements, ranks, cf, instances, ELEMS, ins, outs)
        right += means_its_statements(algo, bufs, want_i, want_o, ins, outs) is None
    assert {"s", "r", "rcs", "rrc", "rrcs", "rrs", "cpy", "re", "nop"} <= seen, seen
    assert usable >= 90 and right >= 0.9 * usable, (usable, right)
