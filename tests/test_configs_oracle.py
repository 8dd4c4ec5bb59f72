"""The five benchmark algorithms and the other reference-emitted programs, executed by the NumPy
interpreter at small chunk sizes and compared with closed forms.  The IR comes from msccl-tools'
own compiler (tests/golden/reference_xml) and, for the five configurations, also from this
package's compiler."""
import numpy as np
import pytest

import golden_util
from msccl.executor.workloads import WORKLOADS, numpy_input
from oracle import collectives as oc
from oracle import ir_interp as oi

GOLDEN_OF = {"c1": "c1_allreduce_ring_8r_1ch_1inst", "c2": "c2_allgather_ring_8r_1ch_4inst", "c3": "c3_alltoall_two_step_2x8",
             "c4": "c4_hierarchical_allreduce_8x4_2inst_auto", "c5": "c5_allreduce_ring_64r_1ch_1inst", "c5_chain": "c5_allreduce_chain_64r"}
SMALL_BYTES = {"c1": 8 * 40, "c2": 4 * 4 * 24, "c3": 16 * 48, "c4": 64 * 2 * 24, "c5": 64 * 2 * 8, "c5_chain": 2 * 24}


def fold_orders(key):
    if key == "c1":
        return oc.ring_allreduce_orders(8)
    if key == "c5":
        return oc.ring_allreduce_orders(64)
    if key == "c4":
        return oc.two_level_allreduce_orders(8, 4, instances=2)
    if key == "c5_chain":
        return [list(range(64))]           # one chunk, summed from rank 0 to rank 63
    return None


def expected(w, x):
    if w.coll == "allgather":
        return oc.expected_allgather(x)
    if w.coll == "alltoall":
        return oc.expected_alltoall(x)
    return oc.expected_allreduce(x, w.nchunks, fold_orders(w.key), w.dtype)


def run_oracle(xml, w, x, **kw):
    algo = oi.parse_xml(xml)
    E = w.chunk_bytes // np.dtype(oi.DTYPES[w.dtype]).itemsize
    bufs = oc.place_inputs(algo, x, E, w.dtype)
    oi.Interpreter(algo, **kw).run(bufs, E, w.dtype)
    return oc.extract_outputs(algo, bufs, E)


@pytest.mark.parametrize("source", ["msccl-tools", "this-package"])
@pytest.mark.parametrize("key", sorted(WORKLOADS))
def test_config_matches_closed_form(key, source):
    w = WORKLOADS[key].scaled(SMALL_BYTES[key])
    xml = golden_util.load(GOLDEN_OF[key]) if source == "msccl-tools" else WORKLOADS[key].build()
    x = [numpy_input(w, r) for r in range(w.ranks)]
    outs = run_oracle(xml, w, x)
    want = expected(w, x)
    for r in range(w.ranks):
        assert np.array_equal(outs[r].view(np.uint8), want[r].view(np.uint8)), (key, r)


def test_two_level_order_matters():
    """bf16 sums in another association give other bits, so the closed form above really pins the
    reduction order the IR encodes."""
    w = WORKLOADS["c4"].scaled(64 * 2 * 512)
    x = [numpy_input(w, r) for r in range(w.ranks)]
    a = oc.expected_allreduce(x, 64, oc.two_level_allreduce_orders(8, 4, 2), "bfloat16")[0]
    b = oc.expected_allreduce(x, 64, [list(range(32))] * 64, "bfloat16")[0]
    assert not np.array_equal(a, b)


@pytest.mark.parametrize("seed", [0, 1])
def test_config_schedule_invariance(seed):
    for key in ("c3", "c4"):
        w = WORKLOADS[key].scaled(SMALL_BYTES[key])
        xml = golden_util.load(GOLDEN_OF[key])
        x = [numpy_input(w, r) for r in range(w.ranks)]
        base = run_oracle(xml, w, x)
        rnd = run_oracle(xml, w, x, schedule="random", seed=seed, fifo_depth=2)
        for r in range(w.ranks):
            assert np.array_equal(base[r].view(np.uint8), rnd[r].view(np.uint8))


REDUCE_SCATTERS = {
    # name of the fixture, this package's builder, input chunks per rank, chunks of the result per rank, fold orders
    "ring": ("reducescatter_ring_8r_1ch_4inst", lambda: _catalog().ring_reduce_scatter(8, 1, 4), 32, 4, lambda: oc.ring_reduce_scatter_orders(8, 4)),
    "allpairs": ("reducescatter_allpairs_8r", lambda: _catalog().allpairs_reduce_scatter(8), 64, 8, lambda: oc.allpairs_allreduce_orders(8)),
}


def _catalog():
    from msccl.programs import catalog
    return catalog


@pytest.mark.parametrize("source", ["msccl-tools", "this-package"])
@pytest.mark.parametrize("program", sorted(REDUCE_SCATTERS))
def test_reduce_scatter_matches_closed_form(program, source):
    """Reduce-scatter in place (msccl/language/collectives.py:172-225): rank r ends with
    out_r[c] = fold over ranks of in_i[r * cf + c] in its input chunks [r * cf, (r + 1) * cf), in the order the
    program's text fixes (ring: ranks k+1, k+2, ..., k; all-pairs: the owner, then its peers ascending) -- fp32,
    bit for bit, and another order gives other bits."""
    fixture, build, nchunks, per_rank, orders = REDUCE_SCATTERS[program]
    xml = golden_util.load(fixture) if source == "msccl-tools" else build()
    algo = oi.parse_xml(xml)
    assert algo.coll == "reduce_scatter" and algo.inplace and algo.gpus[0].i_chunks == nchunks and algo.gpus[0].o_chunks == 0
    E = 11
    rng = np.random.default_rng(31)
    x = [(rng.random(nchunks * E, dtype=np.float32) * 2 - 1) for _ in range(8)]
    bufs = oc.place_inputs(algo, x, E, "float32")
    oi.Interpreter(algo).run(bufs, E, "float32")
    got = oc.extract_outputs(algo, bufs, E)
    want = oc.expected_reduce_scatter(x, per_rank, orders(), "float32")
    other = oc.expected_reduce_scatter(x, per_rank, [list(range(8))[::-1]] * nchunks, "float32")
    for r in range(8):
        assert got[r].size == per_rank * E
        assert np.array_equal(got[r].view(np.uint32), want[r].view(np.uint32)), (program, source, r)
    assert any(not np.array_equal(want[r].view(np.uint32), other[r].view(np.uint32)) for r in range(8))


# every other reference-emitted program: integer data, where any summation order gives the same bits
OTHERS = {
    "allreduce_ring_8r_4ch_8inst": ("allreduce", 8, 64),
    "allreduce_allpairs_8r_2inst": ("allreduce", 8, 128),
    "allreduce_a100_allpairs_8r": ("allreduce", 8, None),
    "allreduce_recursive_doubling_halving_8r": ("allreduce", 8, None),
    "c4_hierarchical_allreduce_4x2_1inst_manual": ("allreduce", 8, None),
    "allgather_recursive_doubling_8r": ("allgather", 8, None),
    "allgather_allpairs_8r": ("allgather", 8, None),
    "alltoall_allpairs_4r": ("alltoall", 4, None),
    "alltoall_three_step_3x4": ("alltoall", 12, None),
    "c3_alltoall_registered_2x8": ("alltoall", 16, None),
    "simple_allgather_ring_4r_auto": ("allgather", 4, None),
    "simple_allreduce_ring_8r_2inst_auto": ("allreduce", 8, None),
    "allreduce_a100_allpairs_v2_8r": ("allreduce", 8, None),
    "alltoall_a100_three_step_3x4_example": ("alltoall", 12, None),
    "c5_allreduce_chain_64r": ("allreduce", 64, None),
}


@pytest.mark.parametrize("name", sorted(OTHERS))
def test_reference_emitted_programs_on_integers(name):
    coll, n, _ = OTHERS[name]
    algo = oi.parse_xml(golden_util.load(name))
    assert algo.coll == coll and algo.ngpus == n
    E = 6
    g0 = algo.gpus[0]
    if coll == "allgather":
        in_elems = (g0.o_chunks // n) * E if algo.inplace else g0.i_chunks * E
    else:
        in_elems = g0.i_chunks * E
    rng = np.random.default_rng(99)
    x = [rng.integers(-2 ** 31, 2 ** 31, in_elems, dtype=np.int64).astype(np.int32) for _ in range(n)]
    bufs = oc.place_inputs(algo, x, E, "int32")
    oi.Interpreter(algo).run(bufs, E, "int32")
    outs = oc.extract_outputs(algo, bufs, E)
    if coll == "allreduce":
        want = [np.sum(np.stack(x).astype(np.int64), axis=0).astype(np.int32)] * n  # wraps like int32 adds
    elif coll == "allgather":
        want = oc.expected_allgather(x)
    else:
        want = oc.expected_alltoall(x)
    for r in range(n):
        assert np.array_equal(outs[r][:want[r].size], want[r]), (name, r)


@pytest.mark.parametrize("name", ["simple_custom_collective_3r_fanout", "simple_custom_collective_3r_relay"])
def test_custom_collective_examples(name):
    """examples/mscclang/simple/custom_collective.py (coll="custom"): rank 0's input chunk ends up in the
    output buffers of ranks 1 and 2, sent to both (fan-out) or handed on by rank 1 (relay)."""
    algo = oi.parse_xml(golden_util.load(name))
    assert algo.coll == "custom" and algo.ngpus == 3
    E = 7
    x = [np.arange(g.i_chunks * E, dtype=np.int32) + 1000 for g in algo.gpus]
    bufs = oc.place_inputs(algo, x, E, "int32")
    oi.Interpreter(algo).run(bufs, E, "int32")
    for r in (1, 2):
        assert np.array_equal(bufs[r]["o"], x[0]), (name, r)


@pytest.mark.parametrize("n,instances", [(8, 1), (5, 2), (2, 1)])
def test_allpairs_allgather_is_a_concatenation(n, instances):
    """The all-pairs all-gather of the mi355x plans: every rank ends with every rank's input, in rank order;
    one hand-off deep (a threadblock per peer and instance: one send to it, one receive from it)."""
    from msccl.programs import catalog
    algo = oi.parse_xml(catalog.allpairs_allgather(n, instances))
    assert algo.coll == "allgather" and algo.inplace and algo.ngpus == n
    assert all(sorted(st.type for st in tb.steps) == ["r", "s"] for g in algo.gpus for tb in g.tbs)
    E = 3
    rng = np.random.default_rng(n)
    x = [rng.integers(-2 ** 31, 2 ** 31, instances * E, dtype=np.int64).astype(np.int32) for _ in range(n)]
    bufs = oc.place_inputs(algo, x, E, "int32")
    oi.Interpreter(algo).run(bufs, E, "int32")
    want = np.concatenate(x)
    for r in range(n):
        assert np.array_equal(bufs[r]["o"], want), r


def test_allpairs_fold_order_float():
    algo_xml = golden_util.load("allreduce_allpairs_8r_2inst")
    algo = oi.parse_xml(algo_xml)
    E = 5
    rng = np.random.default_rng(7)
    x = [(rng.random(128 * E, dtype=np.float32) * 2 - 1) for _ in range(8)]
    bufs = oc.place_inputs(algo, x, E, "float32")
    oi.Interpreter(algo).run(bufs, E, "float32")
    outs = oc.extract_outputs(algo, bufs, E)
    want = oc.expected_allreduce(x, 128, oc.allpairs_allreduce_orders(8, 2), "float32")
    for r in range(8):
        assert np.array_equal(outs[r].view(np.uint32), want[r].view(np.uint32))


# ---- documents emitted by msccl-tools' second emitter, ncclize (tests/golden/ncclize_xml) -----------------------
def _ncclize_case(name, E=5, seed=13):
    """(algo, per-rank int32 inputs filling every rank's 'i' buffer)."""
    algo = oi.parse_xml(golden_util.load(name))
    rng = np.random.default_rng(seed)
    x = [rng.integers(-2 ** 31, 2 ** 31, g.i_chunks * E, dtype=np.int64).astype(np.int32) for g in algo.gpus]
    return algo, x


def _ncclize_expected(name, algo, x, E):
    """What the hand-written send lists of tests/golden/make_ncclize_xml.py mean, on 32-bit integers
    (sums wrap, so the order of a reduction does not matter).  Returns {rank: (buffer, expected)}."""
    n = algo.ngpus
    inst = int(name.split("_")[-1][0]) if name.endswith("inst") else 1
    add = lambda *v: np.sum(np.stack(v).astype(np.int64), axis=0).astype(np.int32)
    if "allgather" in name:            # address a*inst + k sits at o[a*inst + k] everywhere
        return {r: ("o", np.concatenate(x)) for r in range(n)}
    if "alltoall" in name:             # chunk c goes from rank c % n (its i[c // n]) to rank c // n (o[c % n])
        return {r: ("o", np.concatenate([x[j][r * E:(r + 1) * E] for j in range(n)])) for r in range(n)}
    if "reduce_scatter" in name:       # rank a ends with the sum of everybody's addresses [a*chunks, (a+1)*chunks)
        per = algo.gpus[0].o_chunks * E
        return {a: ("o", add(*[x[r][a * per:(a + 1) * per] for r in range(n)])) for a in range(n)}
    if "reduce_tree" in name:
        return {0: ("o", add(*x))}
    if "scatter_line" in name:         # rank k ends with the root's chunk k
        return {k: ("o", x[0][k * E:(k + 1) * E]) for k in range(n)}
    if "allreduce_two_step" in name:
        # reduce-scatter then all-gather over buffers that every rank holds as INPUT: ncclize turns every
        # receive into an initialised slot into a reduction (msccl/ncclize.py:390-400), the second phase
        # included, so rank r ends with  own contribution + total  at every address it does not own
        total = add(*x)
        want = {}
        for r in range(n):
            w = total.copy()
            for a in range(n):
                if a != r:
                    sl = slice(a * inst * E, (a + 1) * inst * E)
                    w[sl] = add(x[r][sl], total[sl])
            want[r] = ("o", w)
        return want
    raise KeyError(name)


@pytest.mark.parametrize("name", golden_util.ncclize_names())
def test_ncclize_emitted_programs_match_their_send_lists(name):
    E = 5
    algo, x = _ncclize_case(name, E)
    assert algo.inplace == 0 and algo.proto == "Simple"
    types = {st.type for g in algo.gpus for tb in g.tbs for st in tb.steps}
    assert types <= {"s", "r", "rrc", "cpy", "nop"}                   # msccl/ncclize.py emits nothing else
    for sched in (dict(), dict(schedule="random", seed=3, fifo_depth=1)):
        bufs = oc.place_inputs(algo, x, E, "int32")
        oi.Interpreter(algo, **sched).run(bufs, E, "int32")
        for r, (buf, want) in _ncclize_expected(name, algo, x, E).items():
            assert np.array_equal(bufs[r][buf][:want.size], want), (name, r, sched)


def test_ncclize_scratch_behind_output_is_the_same_program():
    """use_scratch=False only renames scratch chunks to output chunks past o_chunks (ncclize.py:690-697)."""
    E = 4
    a, x = _ncclize_case("ncclize_scatter_line_4r", E)
    b, _ = _ncclize_case("ncclize_scatter_line_4r_noscratch", E)
    assert "dstoff=\"2\"" in golden_util.load("ncclize_scatter_line_4r_noscratch")   # o[2] with o_chunks = 1
    def local(st):   # the other rank's side of a message ('s': destination, receives: source) is informational
        src = (st.srcbuf, st.srcoff) if st.type in ("s", "cpy", "re") else None
        dst = (st.dstbuf, st.dstoff) if st.type != "s" else None
        return (st.s, st.type, src, dst, st.cnt, st.depid, st.deps, st.hasdep)
    flat = lambda algo: [(g.id, tb.id, local(st)) for g in algo.gpus for tb in g.tbs for st in tb.steps]
    assert flat(a) == flat(b)


def test_ncclize_reduce_tree_order_float():
    """rank 0 folds (x0 + x1) + (x2 + x3): rank 2 has added x3 before it sends."""
    E = 64
    algo = oi.parse_xml(golden_util.load("ncclize_reduce_tree_4r"))
    rng = np.random.default_rng(5)
    x = [((rng.random(E, dtype=np.float32) * 2 - 1) * np.float32(10.0 ** rng.integers(-3, 4))).astype(np.float32) for _ in range(4)]
    bufs = oc.place_inputs(algo, x, E, "float32")
    oi.Interpreter(algo).run(bufs, E, "float32")
    want = (x[0] + x[1]) + (x[2] + x[3])
    assert np.array_equal(bufs[0]["o"].view(np.uint32), want.view(np.uint32))
    assert not np.array_equal(want.view(np.uint32), (((x[0] + x[1]) + x[2]) + x[3]).view(np.uint32))
