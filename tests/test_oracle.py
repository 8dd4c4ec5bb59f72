"""Pins the NumPy IR interpreter (oracle/) against what the mathematics fixes.

The reference holds no execution vectors for IR, so each check here is chosen so that a plausible
mistake (dropped term, wrong operand, wrong chunk offset, wrong fold order) fails at least one.
"""
import numpy as np
import pytest
import torch

import ir_samples
from oracle import collectives as oc
from oracle import ir_interp as oi


def _inputs(n, elems, dtype, seed=0):
    rng = np.random.default_rng(seed)
    out = []
    for r in range(n):
        if dtype in ("float32", "float64"):
            out.append((rng.random(elems, dtype=np.float32) * 2 - 1).astype(oi.DTYPES[dtype]))
        elif dtype == "float16":
            out.append((rng.random(elems, dtype=np.float32) * 2 - 1).astype(np.float16))
        elif dtype == "bfloat16":
            out.append(oi.f32_to_bf16_bits(rng.standard_normal(elems, dtype=np.float32)))
        elif dtype == "uint8":
            out.append(rng.integers(0, 256, elems, dtype=np.uint8))
        else:
            info = np.iinfo(oi.DTYPES[dtype])
            out.append(rng.integers(info.min, info.max, elems, dtype=np.int64, endpoint=True).astype(oi.DTYPES[dtype]))
    return out


def _run(xml, inputs, chunk_elems, dtype, **kw):
    algo = oi.parse_xml(xml)
    bufs = oc.place_inputs(algo, inputs, chunk_elems, dtype)
    oi.Interpreter(algo, **kw).run(bufs, chunk_elems, dtype)
    return algo, oc.extract_outputs(algo, bufs, chunk_elems)


# ---- bf16 arithmetic against an independent implementation (torch CPU) ------------------------
def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(20000, dtype=np.float32) * 10.0 ** rng.integers(-20, 20, 20000),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 1.00390625, 1.01171875, 3.3895314e38], np.float32)])
    mine = oi.f32_to_bf16_bits(x)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(mine, ref)
    assert np.array_equal(oi.bf16_bits_to_f32(mine), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


@pytest.mark.parametrize("op", ["sum", "prod", "max", "min"])
def test_bf16_and_f16_reduce_match_torch(op):
    rng = np.random.default_rng(2)
    a32, b32 = rng.standard_normal(50000, dtype=np.float32), rng.standard_normal(50000, dtype=np.float32)
    top = {"sum": torch.add, "prod": torch.mul, "max": torch.maximum, "min": torch.minimum}[op]
    a, b = oi.f32_to_bf16_bits(a32), oi.f32_to_bf16_bits(b32)
    ta, tb = (torch.from_numpy(v.view(np.int16)).view(torch.bfloat16) for v in (a, b))
    assert np.array_equal(oi._reduce(a, b, "bfloat16", op), top(ta, tb).view(torch.int16).numpy().view(np.uint16))
    ha, hb = a32.astype(np.float16), b32.astype(np.float16)
    got = oi._reduce(ha, hb, "float16", op)
    # fp16: add in fp32 and round once == correctly rounded fp16 result
    f = {"sum": np.add, "prod": np.multiply, "max": np.maximum, "min": np.minimum}[op]
    assert np.array_equal(got.view(np.uint16), f(ha.astype(np.float32), hb.astype(np.float32)).astype(np.float16).view(np.uint16))


# ---- the reference's fusion example, executed ----------------------------------------------------
def test_fusion_chain_worked_example():
    E = 5
    x = _inputs(3, 3 * E, "float32", seed=3)
    algo, outs = _run(ir_samples.FUSION_CHAIN_XML, x, E, "float32")
    expect = x[2] + (x[1] + x[0])  # rank 1 forwards x1+x0 without storing, rank 2 stores and forwards
    for r in range(3):
        assert np.array_equal(outs[r].view(np.uint32), expect.view(np.uint32))
    assert oi.algorithmic_bytes(algo, E * 4) == 10 * 3 * E * 4


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "int32", "uint8", "float64", "int64"])
@pytest.mark.parametrize("n", [2, 3, 8])
def test_ring_allreduce_fold_order(n, dtype):
    E = 7
    x = _inputs(n, n * E, dtype, seed=10 + n)
    _, outs = _run(ir_samples.ring_allreduce_xml(n), x, E, dtype)
    expect = oc.expected_allreduce(x, n, oc.ring_allreduce_orders(n), dtype)
    for r in range(n):
        assert np.array_equal(outs[r].view(np.uint8), expect[r].view(np.uint8))


def test_fold_order_is_observable():
    """The bit-exact check above is not vacuous: another association gives other bits."""
    n, E = 8, 4096
    x = _inputs(n, n * E, "float32", seed=5)
    a = oc.expected_allreduce(x, n, oc.ring_allreduce_orders(n), "float32")[0]
    b = oc.expected_allreduce(x, n, [list(range(n))] * n, "float32")[0]
    assert not np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.allclose(a, b, rtol=1e-4, atol=1e-5)


def test_ring_allreduce_instances_interleaved():
    n, inst, E = 4, 3, 5
    x = _inputs(n, n * inst * E, "float32", seed=6)
    _, outs = _run(ir_samples.ring_allreduce_xml(n, inst), x, E, "float32")
    expect = oc.expected_allreduce(x, n * inst, oc.ring_allreduce_orders(n, instances=inst), "float32")
    for r in range(n):
        assert np.array_equal(outs[r].view(np.uint32), expect[r].view(np.uint32))


@pytest.mark.parametrize("n,inst", [(2, 1), (5, 1), (8, 4)])
def test_ring_allgather_is_concatenation(n, inst):
    E = 3
    x = _inputs(n, inst * E, "int32", seed=7)
    _, outs = _run(ir_samples.ring_allgather_xml(n, inst), x, E, "int32")
    expect = oc.expected_allgather(x)
    for r in range(n):
        assert np.array_equal(outs[r], expect[r])


@pytest.mark.parametrize("n", [2, 3, 6])
def test_allpairs_scratch_deps(n):
    E = 9
    x = _inputs(n, n * E, "float32", seed=8)
    _, outs = _run(ir_samples.allpairs_allreduce_xml(n), x, E, "float32")
    expect = oc.expected_allreduce(x, n, ir_samples.allpairs_orders(n), "float32")
    for r in range(n):
        assert np.array_equal(outs[r].view(np.uint32), expect[r].view(np.uint32))


def test_rrc_cpy_nop():
    E = 11
    x = _inputs(2, E, "int32", seed=9)
    algo = oi.parse_xml(ir_samples.RRC_CPY_NOP_XML)
    bufs = oc.place_inputs(algo, x, E, "int32")
    oi.Interpreter(algo).run(bufs, E, "int32")
    assert np.array_equal(bufs[1]["i"], x[1] + x[0])      # rrc: dst = dst + in
    assert np.array_equal(bufs[1]["o"], x[1] + x[0])      # cpy after the dependency
    assert np.array_equal(bufs[0]["i"], x[0])             # the sender keeps its data


# ---- brute force on one-element chunks with exactly representable values ------------------------
def test_brute_force_small_integers():
    for n in (2, 3, 4):
        x = [np.array([(r + 1) * 10 ** c for c in range(n)], dtype=np.int64) for r in range(n)]
        _, outs = _run(ir_samples.ring_allreduce_xml(n), x, 1, "int64")
        want = np.array([sum((r + 1) * 10 ** c for r in range(n)) for c in range(n)], dtype=np.int64)
        for r in range(n):
            assert np.array_equal(outs[r], want)


# ---- the result does not depend on the interleaving, nor on bounded connections ----------------
@pytest.mark.parametrize("seed", range(5))
def test_schedule_invariance(seed):
    n, E = 6, 4
    x = _inputs(n, n * E, "float32", seed=20)
    for xml in (ir_samples.ring_allreduce_xml(n), ir_samples.allpairs_allreduce_xml(n)):
        _, base = _run(xml, x, E, "float32")
        _, rnd = _run(xml, x, E, "float32", schedule="random", seed=seed)
        _, bounded = _run(xml, x, E, "float32", schedule="random", seed=seed, fifo_depth=2)
        for r in range(n):
            assert np.array_equal(base[r].view(np.uint32), rnd[r].view(np.uint32))
            assert np.array_equal(base[r].view(np.uint32), bounded[r].view(np.uint32))


def test_deadlock_is_reported():
    xml = ir_samples.RRC_CPY_NOP_XML.replace('type="s"', 'type="nop"')  # the receive is never fed
    with pytest.raises(oi.Deadlock):
        _run(xml, _inputs(2, 4, "int32"), 4, "int32")


def test_algorithmic_bytes_closed_forms():
    for n in (2, 4, 8):
        S = 1 << 20
        ar = oi.parse_xml(ir_samples.ring_allreduce_xml(n))
        assert oi.algorithmic_bytes(ar, S // n) * n == 5 * (n - 1) * S * n  # 5(n-1)S over all... per rank S
        ag = oi.parse_xml(ir_samples.ring_allgather_xml(n))
        assert oi.algorithmic_bytes(ag, S) == 2 * (n - 1) * n * S


# ---- the second emitter's schema (ncclize) ------------------------------------------------------
@pytest.mark.parametrize("n", [2, 3, 5])
def test_ncclize_style_allgather(n):
    x = _inputs(n, 6, "int32", seed=30)
    algo, outs = _run(ir_samples.ncclize_style_allgather_xml(n), x, 6, "int32")
    assert algo.inplace == 0
    for r in range(n):
        assert np.array_equal(outs[r], np.concatenate(x))


def test_ncclize_style_allreduce():
    x = _inputs(3, 64, "float32", seed=31)
    _, outs = _run(ir_samples.ncclize_style_allreduce_xml(), x, 64, "float32")
    want = (x[0] + x[1]) + x[2]
    for r in range(3):
        assert np.array_equal(outs[r].view(np.uint32), want.view(np.uint32))


def test_max_min_drop_nan_like_fmax():
    """max/min treat a NaN operand as missing (fmax/fmin), on every floating-point type; sum keeps it."""
    nan = np.float32(np.nan)
    a = np.array([1.0, nan, -2.0, nan], np.float32)
    b = np.array([nan, 3.0, -5.0, nan], np.float32)
    for dtype, conv, back in (("float32", lambda v: v, lambda v: v), ("float64", lambda v: v.astype(np.float64), lambda v: v),
                              ("float16", lambda v: v.astype(np.float16), lambda v: v),
                              ("bfloat16", oi.f32_to_bf16_bits, oi.bf16_bits_to_f32)):
        mx = back(oi._reduce(conv(a), conv(b), dtype, "max")).astype(np.float64)
        mn = back(oi._reduce(conv(a), conv(b), dtype, "min")).astype(np.float64)
        assert mx[:3].tolist() == [1.0, 3.0, -2.0] and np.isnan(mx[3]), dtype
        assert mn[:3].tolist() == [1.0, 3.0, -5.0] and np.isnan(mn[3]), dtype
        sm = back(oi._reduce(conv(a), conv(b), dtype, "sum")).astype(np.float64)
        assert np.isnan(sm[[0, 1, 3]]).all() and sm[2] == -7.0, dtype
