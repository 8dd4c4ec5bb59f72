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
             "c4": "c4_hierarchical_allreduce_8x4_2inst_auto", "c5": "c5_allreduce_ring_64r_1ch_1inst"}
SMALL_BYTES = {"c1": 8 * 40, "c2": 4 * 4 * 24, "c3": 16 * 48, "c4": 64 * 2 * 24, "c5": 64 * 2 * 8}


def fold_orders(key):
    if key == "c1":
        return oc.ring_allreduce_orders(8)
    if key == "c5":
        return oc.ring_allreduce_orders(64)
    if key == "c4":
        return oc.two_level_allreduce_orders(8, 4, instances=2)
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
