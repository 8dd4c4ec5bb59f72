"""HIP executor vs the NumPy interpreter on the same seeded inputs, through the C ABI."""
import numpy as np
import pytest
import torch

import golden_util
import ir_samples
from oracle import collectives as oc
from oracle import ir_interp as oi

pytestmark = pytest.mark.gpu

NP2TORCH = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16, "int32": torch.int32,
            "uint8": torch.uint8, "int8": torch.int8, "int64": torch.int64, "float64": torch.float64}


def make_inputs(n, elems, dtype, seed):
    out = []
    for r in range(n):
        rng = np.random.default_rng(1000 * seed + r)
        if dtype in ("float32", "float64"):
            out.append((rng.random(elems, dtype=np.float32) * 2 - 1).astype(oi.DTYPES[dtype]))
        elif dtype == "float16":
            out.append((rng.random(elems, dtype=np.float32) * 2 - 1).astype(np.float16))
        elif dtype == "bfloat16":
            out.append(oi.f32_to_bf16_bits(rng.standard_normal(elems, dtype=np.float32)))
        else:
            info = np.iinfo(oi.DTYPES[dtype])
            out.append(rng.integers(info.min, info.max, elems, dtype=oi.DTYPES[dtype], endpoint=True))
    return out


def to_torch(x, dtype):
    if dtype == "bfloat16":
        return torch.from_numpy(x.view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(x)


def to_numpy(t, dtype):
    t = t.cpu()
    if dtype == "bfloat16":
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def run_both(xml, chunk_elems, dtype, seed=1, redop="sum", in_elems=None, **knobs):
    """Returns (gpu buffers, oracle buffers) as lists over ranks of {'i','o'} numpy arrays."""
    from msccl.executor import Executor, collective_buffers, DTYPE_SIZES
    algo = oi.parse_xml(xml)
    n = algo.ngpus
    esz = DTYPE_SIZES[dtype]
    if in_elems is None:
        if algo.coll == "allgather" and algo.inplace:
            in_elems = algo.gpus[0].o_chunks * chunk_elems // n
        else:
            in_elems = algo.gpus[0].i_chunks * chunk_elems
    x = make_inputs(n, in_elems, dtype, seed)
    # oracle
    bufs = oc.place_inputs(algo, x, chunk_elems, dtype)
    oi.Interpreter(algo).run(bufs, chunk_elems, dtype, redop)
    # device
    ex = Executor(xml)
    print(f"case: {algo.name} n={n} dtype={dtype} chunk_elems={chunk_elems} knobs={knobs}", flush=True)
    info = ex.setup(chunk_elems * esz, dtype, redop, **knobs)
    ins, outs, _ = collective_buffers(ex.tables, chunk_elems * esz, dtype, inputs=[to_torch(v, dtype) for v in x])
    ex.run(ins, outs)
    torch.cuda.synchronize()
    got = [{"i": to_numpy(ins[r], dtype) if ins[r] is not None else np.zeros(0, oi.DTYPES[dtype]),
            "o": to_numpy(outs[r], dtype) if outs[r] is not None else np.zeros(0, oi.DTYPES[dtype])} for r in range(n)]
    return got, bufs, ex, info


def assert_same(got, want, keys=("i", "o")):
    for r, (g, w) in enumerate(zip(got, want)):
        for k in keys:
            gv, wv = g[k].view(np.uint8), w[k].view(np.uint8)
            assert gv.shape == wv.shape, (r, k, gv.shape, wv.shape)
            if not np.array_equal(gv, wv):
                bad = np.flatnonzero(gv != wv)
                raise AssertionError(f"rank {r} buffer {k}: {bad.size} bytes differ, first at byte {bad[0]}")


# How messages cross connections: counters with payloads read in place where that is safe, counters
# with every payload copied through a slot, flag-in-data lines.
MODES = {"in-place": dict(protocol="simple", staging=0), "staged": dict(protocol="simple", staging=1), "ll": dict(protocol="ll")}
PROTOCOLS = ["simple", "ll"]


@pytest.mark.parametrize("protocol", PROTOCOLS)
def test_fusion_chain_f32(protocol):
    got, want, _, info = run_both(ir_samples.FUSION_CHAIN_XML, 1024, "float32", protocol=protocol)
    assert info.protocol == PROTOCOLS.index(protocol) + 1
    assert_same(got, want)


@pytest.mark.parametrize("protocol", PROTOCOLS)
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "int32", "uint8", "float64", "int64", "int8", "uint32", "uint64"])
def test_ring_allreduce_dtypes(dtype, protocol):
    got, want, _, _ = run_both(ir_samples.ring_allreduce_xml(8), 4096, dtype, protocol=protocol)
    assert_same(got, want)


@pytest.mark.parametrize("protocol", PROTOCOLS)
@pytest.mark.parametrize("redop", ["prod", "max", "min"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16", "int32"])
def test_ring_allreduce_redops(dtype, redop, protocol):
    got, want, _, _ = run_both(ir_samples.ring_allreduce_xml(4), 2048, dtype, redop=redop, protocol=protocol)
    assert_same(got, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16", "float64"])
@pytest.mark.parametrize("redop", ["max", "min", "sum"])
def test_nan_operands(dtype, redop):
    """max and min drop a NaN operand (fmax / fmin, as the oracle does), sum propagates it: a quarter of
    every rank's elements are quiet NaNs, at places that differ from rank to rank, so chunks meet NaN
    against number, number against NaN and NaN against NaN along the ring."""
    from msccl.executor import Executor, collective_buffers
    n, E = 4, 2048
    xml = ir_samples.ring_allreduce_xml(n)
    algo = oi.parse_xml(xml)
    x = make_inputs(n, n * E, dtype, seed=90)
    rng = np.random.default_rng(91)
    for r in range(n):
        holes = rng.random(n * E) < 0.25
        if dtype == "bfloat16":
            x[r][holes] = 0x7FC0
        else:
            x[r][holes] = np.nan
    want = oc.place_inputs(algo, x, E, dtype)
    oi.Interpreter(algo).run(want, E, dtype, redop)
    ex = Executor(xml)
    print(f"case: NaN operands dtype={dtype} redop={redop}", flush=True)
    ex.setup(E * oi.DTYPES[dtype]().itemsize, dtype, redop)
    ins, outs, _ = collective_buffers(ex.tables, E * oi.DTYPES[dtype]().itemsize, dtype, inputs=[to_torch(v, dtype) for v in x])
    ex.run(ins, outs)
    torch.cuda.synchronize()
    as_float = (lambda v: oi.bf16_bits_to_f32(v)) if dtype == "bfloat16" else (lambda v: v)
    for r in range(n):
        got, ref = to_numpy(ins[r], dtype), want[r]["i"]
        gn, rn = np.isnan(as_float(got)), np.isnan(as_float(ref))
        assert np.array_equal(gn, rn), (r, int(gn.sum()), int(rn.sum()))           # NaN exactly where the oracle has NaN
        assert 0 < rn.sum() < rn.size
        assert np.array_equal(got[~rn].view(np.uint8), ref[~rn].view(np.uint8)), r  # and the same bits everywhere else


SIXTEEN_BIT_PARTNERS = {
    "bfloat16": [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x3F80, 0xBF80, 0x3F81, 0x3B80, 0x3B81, 0x3780, 0x3781, 0x4000,
                 0x40FF, 0x437F, 0x7F7F, 0xFF7F, 0x7F00, 0x7F80, 0xFF80, 0x7FC0, 0x0100, 0x8100, 0x3F00, 0x3EFF, 0x4B80, 0xCB80,
                 0x5F80, 0x1F80, 0x2F81, 0x6F7F],
    "float16": [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x3C00, 0xBC00, 0x3C01, 0x1400, 0x1401, 0x1000, 0x1001, 0x4000,
                0x47FF, 0x5BFF, 0x7BFF, 0xFBFF, 0x7800, 0x7C00, 0xFC00, 0x7E00, 0x0800, 0x8800, 0x3800, 0x37FF, 0x6400, 0xE400,
                0x6C00, 0x0C00, 0x2C01, 0x73FF],
}


@pytest.mark.parametrize("redop", ["sum", "prod"])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_every_16_bit_float_against_chosen_partners(dtype, redop):
    """Rounding of 16-bit results (the device uses the conversion instructions, the oracle the integer formula for bf16
    and NumPy's cast for fp16): every one of the 65536 bit patterns -- zeros, denormals, infinities, NaNs -- combined
    with 32 partners that lead to exact results, ties, carries into the exponent, overflow and underflow.  Bits equal
    wherever the oracle has a number, NaN exactly where it has a NaN."""
    from msccl.executor import Executor, collective_buffers
    partners = np.array(SIXTEEN_BIT_PARTNERS[dtype], np.uint16)
    every = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    bits = [np.tile(every, partners.size), np.repeat(partners, 65536)]
    x = bits if dtype == "bfloat16" else [v.view(np.float16) for v in bits]
    as_float = oi.bf16_bits_to_f32 if dtype == "bfloat16" else (lambda v: v.astype(np.float32))
    xml = ir_samples.ring_allreduce_xml(2)
    algo = oi.parse_xml(xml)
    E = x[0].size // 2
    want = oc.place_inputs(algo, x, E, dtype)
    oi.Interpreter(algo).run(want, E, dtype, redop)
    ex = Executor(xml)
    print(f"case: every {dtype} value, redop={redop}", flush=True)
    ex.setup(E * 2, dtype, redop)
    ins, outs, _ = collective_buffers(ex.tables, E * 2, dtype, inputs=[to_torch(v, dtype) for v in x])
    ex.run(ins, outs)
    torch.cuda.synchronize()
    for r in range(2):
        got, ref = to_numpy(ins[r], dtype), want[r]["i"]
        gn, rn = np.isnan(as_float(got)), np.isnan(as_float(ref))
        assert np.array_equal(gn, rn), (r, int(gn.sum()), int(rn.sum()))
        gb, rb = got.view(np.uint16), ref.view(np.uint16)
        assert np.array_equal(gb[~rn], rb[~rn]), (r, np.flatnonzero((gb != rb) & ~rn)[:8])


@pytest.mark.parametrize("protocol", PROTOCOLS)
@pytest.mark.parametrize("n,inst", [(2, 1), (8, 4), (5, 2)])
def test_ring_allgather(n, inst, protocol):
    got, want, _, _ = run_both(ir_samples.ring_allgather_xml(n, inst), 8192, "int32", protocol=protocol)
    assert_same(got, want)


@pytest.mark.parametrize("protocol", PROTOCOLS)
@pytest.mark.parametrize("n", [2, 4, 8])
def test_allpairs_scratch_and_deps(n, protocol):
    got, want, _, _ = run_both(ir_samples.allpairs_allreduce_xml(n), 4096, "float32", protocol=protocol)
    assert_same(got, want)


@pytest.mark.parametrize("mode", sorted(MODES))
def test_ncclize_schema(mode):
    """Documents shaped like msccl-tools' ncclize output: copy threadblocks, inplace=0, sender-side
    src on receives, rrc chains."""
    for n in (2, 3, 5):
        got, want, _, _ = run_both(ir_samples.ncclize_style_allgather_xml(n), 5000, "int32", in_elems=5000, **MODES[mode])
        assert_same(got, want)
    got, want, _, _ = run_both(ir_samples.ncclize_style_allreduce_xml(), 7000, "float32", **MODES[mode])
    assert_same(got, want)


@pytest.mark.parametrize("protocol", PROTOCOLS)
def test_rrc_cpy_nop(protocol):
    got, want, _, _ = run_both(ir_samples.RRC_CPY_NOP_XML, 1000 * 4, "int32", protocol=protocol)
    assert_same(got, want)


@pytest.mark.parametrize("knobs", [
    dict(slices=1, piece_bytes=256, fifo_depth=2),                  # 63 passes: every slot is reused 30 times
    dict(slices=3, piece_bytes=1024, fifo_depth=3, workgroups=4),   # many contexts per workgroup: the lane watches the last line
    dict(slices=2, piece_bytes=4096, fifo_depth=2, workgroups=64),  # one context per workgroup: threads go straight to the lines
    dict(slices=8, threads=64),
    dict(slices=1, threads=512),                                    # one big piece per step
])
def test_ll_geometry_and_relaunch(knobs):
    """Flag-in-data lines over many passes (slot reuse), both ways of noticing a message, and several
    launches on one binding: a launch must not take lines the previous launch left for its own."""
    from msccl.executor import Executor, collective_buffers
    xml = ir_samples.ring_allreduce_xml(8, 2)
    algo = oi.parse_xml(xml)
    E = 4000
    ex = Executor(xml)
    print(f"case: ll relaunch knobs={knobs}", flush=True)
    info = ex.setup(E * 4, "float32", protocol="ll", **knobs)
    assert info.protocol == 2 and info.zero_copy_messages == 0
    keep = None
    for it in range(4):
        x = make_inputs(8, 16 * E, "float32", seed=300 + it)
        if keep is None:
            keep = collective_buffers(ex.tables, E * 4, "float32", inputs=[torch.from_numpy(v) for v in x])
        else:
            for r in range(8):
                keep[0][r].copy_(torch.from_numpy(x[r]))
        ex.run(keep[0], keep[1])
        torch.cuda.synchronize()
        want = oc.place_inputs(algo, x, E, "float32")
        oi.Interpreter(algo).run(want, E, "float32")
        for r in range(8):
            assert np.array_equal(keep[0][r].cpu().numpy().view(np.uint32), want[r]["i"].view(np.uint32)), (it, r)


@pytest.mark.parametrize("chunk_elems,dtype", [(1, "float32"), (3, "float32"), (4, "float32"), (1001, "float16"),
                                               (7, "uint8"), (16, "uint8"), (100003, "int32")])
def test_ragged_chunk_sizes(chunk_elems, dtype):
    """Chunks that are not a multiple of 4 bytes take the element path, multiples of 4 the vector path with
    a partial last unit; tiny chunks leave most slices empty-handed, so the geometry must shrink."""
    got, want, _, info = run_both(ir_samples.ring_allreduce_xml(4), chunk_elems, dtype)
    assert_same(got, want)


# chunk sizes in bytes that are a multiple of 4 but not of 16: the vector path with a partial last unit
PARTIAL_UNIT_CASES = [(1001, "float32"), (1002, "float32"), (1003, "float32"), (5002, "bfloat16"), (1004, "uint8"), (1001, "float64"),
                      (3, "int32"), (40001, "float32"), (524289, "int32")]


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("chunk_elems,dtype", PARTIAL_UNIT_CASES)
def test_chunks_that_end_inside_a_unit(chunk_elems, dtype, mode):
    """A chunk of 4k bytes that is no multiple of 16 moves in 16-byte units all the same: rows start on
    4-byte boundaries and the last unit of every row is cut where the chunk ends.  Every byte of every
    buffer is compared, so a store that ran past a chunk's end would show in the chunk behind it.
    Ring (rrs/rrcs/rcs), all-pairs (folded nops, reduce chains as one step), multi-chunk steps."""
    from msccl.executor import DTYPE_SIZES
    assert (chunk_elems * DTYPE_SIZES[dtype]) % 4 == 0 and (chunk_elems * DTYPE_SIZES[dtype]) % 16 != 0
    for xml in (ir_samples.ring_allreduce_xml(8, 2), ir_samples.allpairs_allreduce_xml(5), ir_samples.RRC_CPY_NOP_XML):
        got, want, _, info = run_both(xml, chunk_elems, dtype, seed=chunk_elems % 97, **MODES[mode])
        assert info.vector_path == 1
        assert_same(got, want)


# chunk sizes that are no multiple of 4 bytes: rows start on odd 2-byte or 1-byte boundaries and end inside a dword
SUB_DWORD_CASES = [(1001, "float16"), (5001, "bfloat16"), (1003, "uint8"), (1001, "int8"), (1, "uint8"), (3, "bfloat16"), (40001, "float16"),
                   (262145, "bfloat16"), (1048579, "uint8")]


@pytest.mark.parametrize("mode", ["in-place", "staged"])
@pytest.mark.parametrize("chunk_elems,dtype", SUB_DWORD_CASES)
def test_chunks_that_end_inside_a_dword(chunk_elems, dtype, mode):
    """Chunks of 8- or 16-bit elements that are no multiple of 4 bytes move in 16-byte units too: whole dwords
    through descriptors that end with the row's last whole dword, the 1 to 3 bytes beyond it element by
    element -- at the row's end and, where a long row is moved from its destination's first cache line on,
    at the end of the head in front of that line.  (Flag-in-data lines carry whole dwords: refused.)"""
    from msccl.executor import DTYPE_SIZES, Executor, MscclxError
    assert (chunk_elems * DTYPE_SIZES[dtype]) % 4 != 0
    for xml in (ir_samples.ring_allreduce_xml(8, 2), ir_samples.allpairs_allreduce_xml(5), ir_samples.RRC_CPY_NOP_XML, ir_samples.ring_allgather_xml(8, 2)):
        got, want, _, info = run_both(xml, chunk_elems, dtype, seed=chunk_elems % 89, **MODES[mode])
        assert info.vector_path == 1
        assert_same(got, want)
    with pytest.raises(MscclxError):
        Executor(ir_samples.ring_allreduce_xml(8, 2)).setup(chunk_elems * DTYPE_SIZES[dtype], dtype, protocol="ll")


@pytest.mark.parametrize("knobs", [dict(slices=1, piece_bytes=4096), dict(slices=3, piece_bytes=16 * 7, threads=128), dict(slices=2, workgroups=1, threads=64),
                                   dict(slices=5, threads=512), dict(slices=16, threads=64), dict(slices=4, workgroups=3, threads=256)])
def test_sub_dword_tails_under_explicit_geometries(knobs):
    for xml, dtype, elems in ((ir_samples.ring_allreduce_xml(8, 2), "bfloat16", 20001), (ir_samples.allpairs_allreduce_xml(5), "float16", 20003),
                              (ir_samples.ring_allgather_xml(8, 2), "uint8", 40001)):
        got, want, _, info = run_both(xml, elems, dtype, seed=11, protocol="simple", **knobs)
        assert info.vector_path == 1 and info.slices == knobs["slices"]
        assert_same(got, want)


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("first_elem,chunk_elems", [(1, 1000), (3, 1001), (2, 40004), (1, 131075)])
def test_buffers_that_start_off_a_16_byte_boundary(first_elem, chunk_elems, mode):
    """Rank buffers need only start on a 4-byte boundary -- a view into a larger tensor, say: the units are
    laid out from the destination's cache lines, wherever the row starts.  The words around every
    view must come through untouched."""
    from msccl.executor import Executor
    for xml in (ir_samples.ring_allreduce_xml(8, 2), ir_samples.allpairs_allreduce_xml(5)):
        algo = oi.parse_xml(xml)
        n, elems = algo.ngpus, algo.gpus[0].i_chunks * chunk_elems
        x = make_inputs(n, elems, "float32", seed=first_elem + chunk_elems)
        want = oc.place_inputs(algo, x, chunk_elems, "float32")
        oi.Interpreter(algo).run(want, chunk_elems, "float32")
        guard = np.float32(-12345.5)
        whole = [torch.full((elems + 8,), float(guard), dtype=torch.float32, device="cuda:0") for _ in range(n)]
        views = [w[first_elem:first_elem + elems] for w in whole]
        for r in range(n):
            views[r].copy_(torch.from_numpy(x[r]))
        assert all(v.data_ptr() % 16 == 4 * first_elem for v in views)
        ex = Executor(xml)
        print(f"case: {algo.name} first_elem={first_elem} chunk_elems={chunk_elems} mode={mode}", flush=True)
        ex.setup(chunk_elems * 4, "float32", **MODES[mode])
        ex.run(views, [None] * n)
        torch.cuda.synchronize()
        for r in range(n):
            got = whole[r].cpu().numpy()
            assert np.array_equal(got[first_elem:first_elem + elems].view(np.uint32), want[r]["i"].view(np.uint32)), (algo.name, r)
            assert (got[:first_elem] == guard).all() and (got[first_elem + elems:] == guard).all(), (algo.name, r, "guard words")


@pytest.mark.parametrize("knobs", [dict(slices=1, piece_bytes=4096), dict(slices=3, piece_bytes=16 * 7, threads=128), dict(slices=2, workgroups=1, threads=64),
                                   dict(slices=5, threads=512), dict(slices=16, threads=64), dict(slices=4, workgroups=3, threads=256)])
@pytest.mark.parametrize("protocol", PROTOCOLS)
def test_partial_units_under_explicit_geometries(knobs, protocol):
    """The partial unit sits in the last pass of the last slice, whatever the passes, slices and hosting are;
    on one-wave workgroups with one context each the chain loops move it."""
    for xml, dtype in ((ir_samples.ring_allreduce_xml(8, 2), "float32"), (ir_samples.allpairs_allreduce_xml(5), "bfloat16"),
                       (ir_samples.ring_allgather_xml(8, 2), "int32")):
        elems = 10001 if dtype != "bfloat16" else 20002
        got, want, _, info = run_both(xml, elems, dtype, seed=7, protocol=protocol, **knobs)
        assert info.vector_path == 1 and info.slices == knobs["slices"]
        assert_same(got, want)


@pytest.mark.parametrize("knobs", [dict(), dict(slices=2, workgroups=40, threads=64), dict(threads=256, slices=3), dict(staging=1, slices=4, workgroups=300)])
def test_long_nop_runs_and_reduce_chains(knobs):
    """All-pairs over 16 ranks: every threadblock waits for 15 peers through runs of 14 nops, which one step stands for
    (its dependencies checked by the polling wave together, also where a workgroup hosts many contexts), and folds
    their 15 chunks with one step of 15 sources."""
    from msccl.programs import catalog
    xml = catalog.allpairs_allreduce(16, 1)
    for dtype, elems in (("float32", 33), ("bfloat16", 1001)):
        got, want, _, info = run_both(xml, elems, dtype, seed=5, protocol="simple", **knobs)
        assert_same(got, want)


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("chunk_elems,dtype,slices", [(4100, "float32", 16), (14001, "float16", 16), (2047, "uint8", 1), (261, "float32", 1),
                                                      (20000, "uint8", 16), (1025, "float64", 6), (509, "int32", 1)])
def test_slices_of_up_to_two_units_per_lane(chunk_elems, dtype, slices, mode):
    """One-wave workgroups whose slices are 65 to 128 units long move two units per lane in one round: whole rows,
    rows that end inside a unit and rows that end inside a dword, in copies, reduces and reduce chains."""
    from msccl.executor import DTYPE_SIZES
    nbytes = chunk_elems * DTYPE_SIZES[dtype]
    if mode == "ll" and nbytes % 4:
        pytest.skip("flag-in-data lines carry whole dwords")
    for xml in (ir_samples.ring_allreduce_xml(8, 2), ir_samples.allpairs_allreduce_xml(5), ir_samples.RRC_CPY_NOP_XML, ir_samples.ring_allgather_xml(8, 2)):
        got, want, _, info = run_both(xml, chunk_elems, dtype, seed=chunk_elems % 83, threads=64, slices=slices, **MODES[mode])
        assert info.threads == 64 and 64 * 16 < info.piece_bytes <= 128 * 16, (info.threads, info.piece_bytes)
        assert_same(got, want)


@pytest.mark.parametrize("knobs", [dict(), dict(slices=1, piece_bytes=4096), dict(threads=256, slices=2), dict(threads=64, slices=3)])
@pytest.mark.parametrize("dtype,redop", [("bfloat16", "sum"), ("float32", "sum"), ("int32", "max"), ("float16", "prod")])
@pytest.mark.parametrize("m,stride", [(7, 8), (11, 1), (2, 3), (31, 1), (17, 2)])
def test_reduce_chains_as_one_step(m, stride, dtype, redop, knobs):
    """Runs of reduce steps into one destination are done as one step with several sources (at most 8:
    11 in a row make two), in the order of the IR -- which the rounding of bfloat16 sums and fp16 products
    shows.  Sources in descending order are left step by step.  Several passes, several waves, ragged slices."""
    xml = ir_samples.reduce_chain_xml(m, stride)
    got, want, _, info = run_both(xml, 5000, dtype, seed=m * 10 + stride, redop=redop, **knobs)
    assert_same(got, want)


@pytest.mark.parametrize("knobs", [
    dict(slices=1, piece_bytes=4096, fifo_depth=2, threads=64),
    dict(slices=3, piece_bytes=16 * 7, fifo_depth=3, threads=128),
    dict(slices=16, piece_bytes=1 << 20, fifo_depth=8, threads=512),
    dict(slices=8, piece_bytes=65536, fifo_depth=2, threads=256),
    dict(slices=2, piece_bytes=8192, fifo_depth=2, threads=64, workgroups=1),    # one workgroup hosts every context
    dict(slices=6, piece_bytes=32768, fifo_depth=3, threads=128, workgroups=5),
    dict(slices=2, staging=1, workgroups=7),
])
def test_geometry_knobs(knobs):
    knobs = dict(protocol="simple", **knobs)
    got, want, _, info = run_both(ir_samples.ring_allreduce_xml(8, 2), 40000, "float32", **knobs)
    assert info.slices == knobs["slices"] and info.threads == knobs.get("threads", info.threads)
    assert_same(got, want)
    got, want, _, _ = run_both(ir_samples.allpairs_allreduce_xml(5), 40000, "bfloat16", **knobs)
    assert_same(got, want)


@pytest.mark.parametrize("batch", range(4))
def test_random_sizes_dtypes_and_geometries(batch):
    """Sixty random draws per batch of (program, element type, reduction, chunk size from 1 to 300 000 elements, message mode,
    geometry knobs) against the interpreter, every byte compared.  A draw the library refuses must be refused
    for a reason that the draw explains."""
    import random
    from msccl.executor import DTYPE_SIZES, MscclxError
    from msccl.executor import binding
    rnd = random.Random(1000 + batch)
    programs = [ir_samples.ring_allreduce_xml(8, 2), ir_samples.ring_allreduce_xml(4), ir_samples.allpairs_allreduce_xml(5), ir_samples.RRC_CPY_NOP_XML,
                ir_samples.ring_allgather_xml(8, 2), ir_samples.reduce_chain_xml(7, 8), golden_util.load("alltoall_three_step_3x4"),
                golden_util.load("c4_hierarchical_allreduce_4x2_1inst_manual"), golden_util.load("allreduce_a100_allpairs_v2_8r")]
    dtypes = ["float32", "bfloat16", "float16", "uint8", "int8", "int32", "float64", "int64"]
    ran = 0
    for case in range(60):
        xml, dtype = rnd.choice(programs), rnd.choice(dtypes)
        elems = rnd.choice([rnd.randint(1, 40), rnd.randint(41, 3000), rnd.randint(3001, 70000), rnd.randint(70001, 300000)])
        mode = rnd.choice(["in-place", "staged", "ll", "auto"])
        knobs = {} if mode == "auto" else dict(MODES[mode])
        g = rnd.random()
        if g < 0.25:
            knobs.update(slices=rnd.choice([1, 2, 3, 5, 8, 16]))
        elif g < 0.4:
            knobs.update(slices=rnd.choice([1, 2, 4]), threads=rnd.choice([64, 128, 256, 512]))
        elif g < 0.5:
            knobs.update(slices=2, workgroups=rnd.choice([1, 3, 7]), threads=rnd.choice([64, 256]))
        if rnd.random() < 0.2:
            knobs.update(piece_bytes=rnd.choice([112, 4096, 65536]))
        redop = rnd.choice(["sum", "sum", "max", "min", "prod"]) if dtype not in ("uint8", "int8") else rnd.choice(["sum", "max", "min"])
        try:
            got, want, _, info = run_both(xml, elems, dtype, seed=100 * batch + case, redop=redop, **knobs)
        except MscclxError as e:
            nbytes = elems * DTYPE_SIZES[dtype]
            explained = ((e.code == binding.ERR_UNSUPPORTED and mode == "ll" and nbytes % 4) or            # lines carry whole dwords
                         (e.code == binding.ERR_INVALID_ARG and knobs.get("slices", 0) > (nbytes + 15) // 16) or  # more slices than units
                         (e.code == binding.ERR_CAPACITY and "workgroups" in knobs))                       # too few workgroups for the contexts
            assert explained, (case, str(e), elems, dtype, knobs)
            continue
        assert_same(got, want)
        ran += 1
    assert ran >= 40


def test_relaunch_reuses_counters():
    """Launch several times on the same binding: the counter areas alternate and are re-armed."""
    from msccl.executor import Executor, collective_buffers
    xml = ir_samples.ring_allgather_xml(8, 2)
    algo = oi.parse_xml(xml)
    E = 5000
    ex = Executor(xml)
    ex.setup(E * 4, "int32")
    for it in range(5):
        x = make_inputs(8, 2 * E, "int32", seed=50 + it)
        ins, outs, res = collective_buffers(ex.tables, E * 4, "int32", inputs=[torch.from_numpy(v) for v in x])
        if it == 0:
            keep = (ins, outs, res)
        else:  # same device buffers, new contents
            for r in range(8):
                keep[1][r].copy_(outs[r])
        ex.run(keep[0], keep[1])
        want = np.concatenate(x)
        for r in range(8):
            assert np.array_equal(keep[2][r].cpu().numpy(), want), (it, r)


def test_hip_graph_replay():
    """A launch keeps no host-side state (the counter-area parity lives on the device), so it can be
    captured once and replayed; every replay, interleaved with eager work, must be right."""
    from msccl.executor import Executor, collective_buffers
    xml = ir_samples.ring_allreduce_xml(8, 2)
    E = 6000
    ex = Executor(xml)
    ex.setup(E * 4, "float32")
    base = make_inputs(8, 16 * E, "float32", seed=70)
    ins, outs, res = collective_buffers(ex.tables, E * 4, "float32", inputs=[torch.from_numpy(v) for v in base])
    ex.run(ins, outs)                                   # eager launch first (odd number of launches so far)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            ex.launch()
    algo = oi.parse_xml(xml)
    for it in range(4):
        x = make_inputs(8, 16 * E, "float32", seed=80 + it)
        for r in range(8):
            ins[r].copy_(torch.from_numpy(x[r]))        # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oc.place_inputs(algo, x, E, "float32")
        oi.Interpreter(algo).run(want, E, "float32")
        for r in range(8):
            assert np.array_equal(ins[r].cpu().numpy().view(np.uint32), want[r]["i"].view(np.uint32)), (it, r)
        if it == 1:                                     # an eager launch in between flips the parity once more
            ex.run(ins, outs)


def test_watchdog_reports_instead_of_hanging():
    """A 1 ms watchdog while a receive legitimately waits for tens of milliseconds: the waiting
    workgroup must give up cleanly (every wave exits, the producer still finishes), the error names
    the waiting step, and the next launch with the default limit works and is correct."""
    from msccl.executor import Executor, MscclxError, collective_buffers
    xml = ir_samples.slow_producer_xml(24)
    nbytes = 64 << 20
    ex = Executor(xml)
    ex.setup(nbytes, "uint8", timeout_ms=1, slices=1, piece_bytes=nbytes)  # one pass: the receive waits for all 24 copies
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    print("case: watchdog launch", flush=True)
    ex.launch()
    with pytest.raises(MscclxError) as e:
        ex.wait()
    assert "watchdog" in str(e.value) and "rank 1 tb 0 step 0" in str(e.value) and "incoming message" in str(e.value)
    torch.cuda.synchronize()
    # same plan, sane limit: completes and delivers
    ex2 = Executor(xml)
    ex2.setup(nbytes, "uint8", slices=4)
    ins, outs, _ = collective_buffers(ex2.tables, nbytes, "uint8", inputs=x)
    ex2.run(ins, outs)
    assert torch.equal(outs[1].cpu(), x[0]) and torch.equal(outs[0].cpu(), x[0])


def test_watchdog_names_the_ir_step_of_folded_nops():
    """Nop steps in front of a step are folded into it at bind; a watchdog report still counts steps
    as the IR does.  Threadblock 1's step 2 (behind two nops) waits for 24 copies of 64 MiB under a
    1 ms limit; with a sane limit the same program delivers."""
    from msccl.executor import Executor, MscclxError
    xml = ir_samples.slow_dependency_xml(24)
    nbytes = 64 << 20
    x = torch.arange(nbytes, dtype=torch.int32).to(torch.uint8).cuda()
    ex = Executor(xml)
    ex.setup(nbytes, "uint8", timeout_ms=1, slices=1, piece_bytes=nbytes)
    out = torch.zeros(2 * nbytes, dtype=torch.uint8, device="cuda")
    ex.bind([x], [out])
    print("case: watchdog on a step with folded nops", flush=True)
    ex.launch()
    with pytest.raises(MscclxError) as e:
        ex.wait()
    assert "watchdog" in str(e.value) and "rank 0 tb 1 step 2" in str(e.value) and "its dependency" in str(e.value)
    torch.cuda.synchronize()
    ex2 = Executor(xml)
    ex2.setup(nbytes, "uint8")
    out = torch.zeros(2 * nbytes, dtype=torch.uint8, device="cuda")
    ex2.run([x], [out])
    assert torch.equal(out[:nbytes], x) and torch.equal(out[nbytes:], x)


def test_poll_does_not_block():
    """mscclx_plan_poll: 'running' while the launch is under way, then the launch's result."""
    import time
    from msccl.executor import Executor, collective_buffers
    xml = ir_samples.slow_producer_xml(24)
    nbytes = 64 << 20
    ex = Executor(xml)
    ex.setup(nbytes, "uint8", slices=1, piece_bytes=nbytes)   # one workgroup makes the 24 copies: tens of milliseconds
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    torch.cuda.synchronize()
    print("case: poll", flush=True)
    ex.launch()
    t0 = time.perf_counter()
    first = ex.poll()
    dt_first = time.perf_counter() - t0
    polls = 1
    while ex.poll():
        polls += 1
        time.sleep(0.001)
        assert time.perf_counter() - t0 < 30
    assert first and dt_first < 0.005, (first, dt_first)         # came back at once, with the launch still running
    assert not ex.poll()                                         # finished: stays finished, no error
    assert torch.equal(outs[1].cpu(), x[0]) and torch.equal(outs[0].cpu(), x[0])
    print(f"polled {polls} times in {(time.perf_counter() - t0) * 1e3:.1f} ms", flush=True)


def test_abort_from_the_host():
    """mscclx_plan_abort ends a launch that still has a long way to go: every workgroup leaves by
    itself, wait() reports ABORTED well before the launch could have finished, and the same binding
    then runs to completion with the right result (the counters are re-armed)."""
    import time
    from msccl.executor import Executor, MscclxError, collective_buffers
    from msccl.executor.binding import ERR_ABORTED
    ncopies = 200
    xml = ir_samples.slow_producer_xml(ncopies)
    nbytes = 64 << 20
    ex = Executor(xml)
    ex.setup(nbytes, "uint8", slices=1, piece_bytes=nbytes)
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    torch.cuda.synchronize()
    print("case: full run for reference", flush=True)
    t0 = time.perf_counter()
    ex.launch()
    ex.wait()
    full = time.perf_counter() - t0
    assert torch.equal(outs[1].cpu(), x[0])
    outs[1].zero_()
    torch.cuda.synchronize()
    print(f"case: abort (a full run takes {full * 1e3:.1f} ms)", flush=True)
    t0 = time.perf_counter()
    ex.launch()
    assert ex.poll()
    ex.abort()
    with pytest.raises(MscclxError) as e:
        ex.wait()
    aborted = time.perf_counter() - t0
    assert e.value.code == ERR_ABORTED
    # the receiver gave up at once; the producer finishes the copy it is in (1/200 of the run) and leaves
    assert aborted < 0.5 * full, (aborted, full)
    assert not torch.equal(outs[1].cpu(), x[0])                  # the message never arrived
    print(f"aborted after {aborted * 1e3:.1f} ms; relaunching", flush=True)
    ex.launch()
    ex.wait()
    assert torch.equal(outs[1].cpu(), x[0]) and torch.equal(outs[0].cpu(), x[0])


def test_graph_replay_after_an_abort():
    """A launch captured in a HIP graph, replayed after mscclx_plan_abort ended a launch: the replay passes by the
    host code that re-arms the counters.  The first replay may still find the abort request on the device -- it
    then ends at once and the wait after it says ABORTED, never OK with a buffer that was not filled -- and the
    replay after that runs and delivers."""
    from msccl.executor import Executor, MscclxError, collective_buffers
    from msccl.executor.binding import ERR_ABORTED
    xml = ir_samples.slow_producer_xml(200)
    nbytes = 64 << 20
    ex = Executor(xml)
    ex.setup(nbytes, "uint8", slices=1, piece_bytes=nbytes)
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            ex.launch()
        print("case: replay before the abort", flush=True)
        graph.replay()
        ex.wait()
        assert torch.equal(outs[1].cpu(), x[0])
        outs[1].zero_()
        torch.cuda.synchronize()
        print("case: replay, aborted from the host", flush=True)
        graph.replay()
        assert ex.poll()
        ex.abort()
        with pytest.raises(MscclxError) as e:
            ex.wait()
        assert e.value.code == ERR_ABORTED
        assert not torch.equal(outs[1].cpu(), x[0])
        delivered = 0
        for attempt in range(3):
            outs[1].zero_()
            torch.cuda.synchronize()
            print(f"case: replay {attempt} after the abort", flush=True)
            graph.replay()
            try:
                ex.wait()
            except MscclxError as err:                        # only the first replay may be refused, and only this way
                assert err.code == ERR_ABORTED and attempt == 0 and delivered == 0, (attempt, err)
                continue
            assert torch.equal(outs[1].cpu(), x[0]) and torch.equal(outs[0].cpu(), x[0]), attempt
            delivered += 1
        assert delivered >= 2
    torch.cuda.synchronize()


@pytest.mark.parametrize("threads", [0, 64])
def test_watchdog_in_ll_mode(threads):
    """Flag-in-data lines, one context per workgroup (threads=64: a workgroup of one wave, which runs
    its context without a polling lane): the receiving threads themselves wait on the
    lines, so they carry the watchdog.  Same scenario as above; afterwards the same binding is launched
    again (the library clears counters and lines after a lost launch) -- it times out the same way,
    cleanly -- and a fresh plan with the default limit delivers."""
    from msccl.executor import Executor, MscclxError, collective_buffers
    xml = ir_samples.slow_producer_xml(24)
    nbytes = 64 << 20
    ex = Executor(xml)
    info = ex.setup(nbytes, "uint8", timeout_ms=1, slices=1, piece_bytes=nbytes, protocol="ll", threads=threads)
    assert info.protocol == 2 and info.max_hosted == 1
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    for attempt in range(2):
        print(f"case: ll watchdog launch {attempt}", flush=True)
        ex.launch()
        with pytest.raises(MscclxError) as e:
            ex.wait()
        assert "watchdog" in str(e.value) and "rank 1 tb 0 step 0" in str(e.value) and "incoming message" in str(e.value)
        torch.cuda.synchronize()
    ex2 = Executor(xml)
    ex2.setup(nbytes, "uint8", slices=4, protocol="ll")
    ins, outs, _ = collective_buffers(ex2.tables, nbytes, "uint8", inputs=x)
    ex2.run(ins, outs)
    assert torch.equal(outs[1].cpu(), x[0]) and torch.equal(outs[0].cpu(), x[0])


@pytest.mark.parametrize("knobs", [dict(threads=64), dict(threads=128, workgroups=2)])
def test_ll_launch_number_wraps(knobs):
    """The flag of an LL line carries the launch number in 10 bits.  1040 launches on one binding, each
    on the previous launch's results (in-place all-reduce of 3 ranks on 32-bit integers: after k launches every
    element is 3^(k-1) times the first sum, modulo 2^32, so every launch moves different bits and a line
    taken from an earlier launch would show): checked before, at and after the number wraps."""
    from msccl.executor import Executor, collective_buffers
    n, E = 3, 300
    xml = ir_samples.ring_allreduce_xml(n)
    ex = Executor(xml)
    info = ex.setup(E * 4, "int32", protocol="ll", slices=1, piece_bytes=512, **knobs)  # several passes: slots are reused inside a launch too
    assert info.protocol == 2 and info.passes >= 2
    rng = np.random.default_rng(11)
    x = [rng.integers(0, 2**32, n * E, dtype=np.uint64).astype(np.uint32) for _ in range(n)]
    ins, outs, _ = collective_buffers(ex.tables, E * 4, "int32", inputs=[torch.from_numpy(v.view(np.int32)).clone() for v in x])
    ex.bind(ins, outs)
    first = (x[0].astype(np.uint64) + x[1] + x[2]).astype(np.uint32)
    check_at = {1, 2, 3, 1022, 1023, 1024, 1025, 1026, 1040}
    print(f"case: ll launch-number wrap knobs={knobs}", flush=True)
    for k in range(1, 1041):
        ex.launch()
        if k in check_at:
            ex.wait()
            want = (first.astype(np.uint64) * pow(3, k - 1, 2**32) % 2**32).astype(np.uint32)
            for r in range(n):
                got = ins[r].cpu().numpy().view(np.uint32)
                assert np.array_equal(got, want), (k, r, int(np.flatnonzero(got != want)[0]))
    ex.wait()


def test_which_step_loop_runs():
    """mscclx_info.kernel_loop: the all-pairs family on small messages -- programs with folded nops, one-wave workgroups, one
    context each -- runs on exec_kernel_chain_fold (3); rings on the chain loops for counters (2) and for lines: with every
    step's slots and flags worked out at bind where a step is one row of at most 128 units in one pass (4), the general loop
    for lines where a slice takes several passes (1); a geometry that hosts several contexts on a workgroup on the hosting
    loop (0).  Every one bit-exact against the interpreter."""
    allpairs = golden_util.load("allreduce_a100_allpairs_8r")   # (as msccl-tools' compiler wrote it: runs of nops in front of the folds and the sends)
    cases = [(allpairs, 256, {}, 3), (allpairs, 256, dict(workgroups=8), 0),
             (ir_samples.ring_allreduce_xml(8), 4096, dict(protocol="simple"), 2), (ir_samples.ring_allreduce_xml(8), 256, dict(protocol="ll"), 4),
             (ir_samples.ring_allreduce_xml(8), 4096, dict(protocol="ll", slices=1, threads=64, piece_bytes=1024), 1),
             (ir_samples.reduce_chain_xml(5, 3), 700, {}, 3)]
    for xml, elems, knobs, loop in cases:
        got, ref, _, info = run_both(xml, elems, "float32", seed=91, **knobs)
        assert info.kernel_loop == loop, (knobs, info.kernel_loop, info.workgroups, info.threads, info.max_hosted)
        assert_same(got, ref)


@pytest.mark.parametrize("elems,slices", [(4, 1), (68, 1), (256, 1), (260, 1), (400, 1), (512, 1), (4096, 8), (4100, 8), (3000, 4), (8192, 32)])
def test_steps_worked_out_at_bind(elems, slices):
    """Rings on flag-in-data lines whose every step is one row of at most 128 units in one pass run with their steps' slots,
    flags and counter values worked out when the buffers are bound (mscclx_info.kernel_loop 4).  Rows of 1 to 128 units, one
    and two units per lane, slices of unequal length, connections whose ring of slots wraps many times (8, 16 and 64 ranks,
    up to 126 messages through two slots), all element widths that lines carry; launched three times on one binding (the
    flags carry the launch number); every byte against the interpreter."""
    from msccl.executor import Executor, collective_buffers, DTYPE_SIZES
    for xml, dtype in ((ir_samples.ring_allreduce_xml(8), "float32"), (golden_util.load("c5_allreduce_ring_64r_1ch_1inst"), "float16"),
                       (golden_util.load("c2_allgather_ring_8r_1ch_4inst"), "int32"), (golden_util.load("reducescatter_ring_8r_1ch_4inst"), "float64")):
        if elems * DTYPE_SIZES[dtype] % 16:
            continue  # (chunks that end inside a unit run on the general loop: covered elsewhere)
        got, ref, ex, info = run_both(xml, elems, dtype, seed=elems + slices, protocol="ll", slices=slices, threads=64)
        flat = info.passes == 1 and info.piece_bytes <= 2048 and info.max_hosted == 1  # (wider elements make longer rows: those take the general loop)
        assert info.kernel_loop == (4 if flat else 1 if info.max_hosted == 1 else 0), (info.kernel_loop, info.piece_bytes, info.passes, info.max_hosted)
        assert_same(got, ref)
    # the same binding launched again and again: an all-gather leaves its inputs alone, so every launch must leave the same bytes
    xml = golden_util.load("c2_allgather_ring_8r_1ch_4inst")
    algo = oi.parse_xml(xml)
    x = make_inputs(algo.ngpus, algo.gpus[0].o_chunks * elems // algo.ngpus, "int32", 5)
    ex = Executor(xml)
    info = ex.setup(elems * 4, "int32", protocol="ll", slices=slices, threads=64)
    ins, outs, res = collective_buffers(ex.tables, elems * 4, "int32", inputs=[to_torch(v, "int32") for v in x])
    ex.bind(ins, outs)
    want = np.concatenate(x)
    for launch in range(3):
        for r in range(algo.ngpus):
            others = torch.ones_like(res[r]) * 7
            others[r * x[r].size:(r + 1) * x[r].size] = res[r][r * x[r].size:(r + 1) * x[r].size]
            res[r].copy_(others)  # (everything but the rank's own contribution overwritten before each launch)
        ex.launch()
        ex.wait()
        for r in range(algo.ngpus):
            assert np.array_equal(to_numpy(res[r], "int32"), want), (launch, r)


def test_watchdog_and_abort_where_steps_are_worked_out_at_bind():
    """The loop for steps worked out at bind carries the watchdog and sees the host's abort like the others: rank 1's
    receive of one 2 KiB row waits while rank 0 makes 20 000 local copies of it first (tens of milliseconds) -- with a
    1 ms limit it gives up cleanly and names the step; with the default limit and an abort from the host the launch ends
    early with ABORTED; left alone it delivers."""
    import time
    from msccl.executor import Executor, MscclxError, collective_buffers
    from msccl.executor.binding import ERR_ABORTED
    xml = ir_samples.slow_producer_xml(20000)
    nbytes = 2048
    x = [torch.arange(nbytes, dtype=torch.int32).to(torch.uint8), torch.zeros(nbytes, dtype=torch.uint8)]
    ex = Executor(xml)
    info = ex.setup(nbytes, "uint8", timeout_ms=1, protocol="ll", slices=1, threads=64)
    assert info.kernel_loop == 4 and info.workgroups == 2
    ins, outs, _ = collective_buffers(ex.tables, nbytes, "uint8", inputs=x)
    ex.bind(ins, outs)
    print("case: watchdog where steps are worked out at bind", flush=True)
    ex.launch()
    with pytest.raises(MscclxError) as e:
        ex.wait()
    assert "watchdog" in str(e.value) and "rank 1 tb 0 step 0" in str(e.value) and "incoming message" in str(e.value)
    torch.cuda.synchronize()
    ex2 = Executor(xml)
    assert ex2.setup(nbytes, "uint8", protocol="ll", slices=1, threads=64).kernel_loop == 4
    ins, outs, _ = collective_buffers(ex2.tables, nbytes, "uint8", inputs=x)
    ex2.bind(ins, outs)
    print("case: full run for reference", flush=True)
    t0 = time.perf_counter()
    ex2.launch()
    ex2.wait()
    full = time.perf_counter() - t0
    assert torch.equal(outs[1].cpu(), x[0])
    outs[1].zero_()
    print("case: abort from the host", flush=True)
    ex2.launch()
    time.sleep(full / 20)
    ex2.abort()
    t0 = time.perf_counter()
    with pytest.raises(MscclxError) as e:
        ex2.wait()
    assert e.value.code == ERR_ABORTED
    assert time.perf_counter() - t0 < full / 2
    print("case: the same binding after the abort", flush=True)
    ex2.launch()
    ex2.wait()
    assert torch.equal(outs[1].cpu(), x[0])


def test_receives_that_take_over_their_senders_waits():
    """In exec_kernel_chain_fold a receive whose payload is read in place waits for its sender's dependencies itself instead
    of for the sender's announcement.  Programs in which such sends have dependencies of every kind -- their own, folded
    nops in front of them, steps in front of them in their threadblock -- in several passes over the step list, with
    ragged chunks, against the interpreter; every buffer of every rank compared."""
    import golden_util
    for name, elems, knobs in (("allreduce_a100_allpairs_8r", 333, {}), ("allreduce_a100_pcie_hierarchical_8r", 1001, {}),
                               ("pipeline_a100_allpairs_8r", 257, {}), ("c3_alltoall_two_step_2x8", 4000, dict(slices=2, threads=64, piece_bytes=2048)),
                               ("allreduce_a100_multinode_allpairs_16r", 129, {}), ("allreduce_a100_allpairs_8r", 3000, dict(slices=4, threads=64, piece_bytes=1024))):
        xml = golden_util.load(name)
        algo = oi.parse_xml(xml)
        rng = np.random.default_rng(17)
        init = [{b: (rng.random(n * elems, dtype=np.float32) * 2 - 1) for b, n in (("i", g.i_chunks), ("o", g.o_chunks), ("s", g.s_chunks))} for g in algo.gpus]
        want = [{b: v.copy() for b, v in d.items()} for d in init]
        oi.Interpreter(algo).run(want, elems, "float32")
        from msccl.executor import Executor
        ex = Executor(xml)
        print(f"case: takeover {name} elems={elems} knobs={knobs}", flush=True)
        info = ex.setup(elems * 4, "float32", **knobs)
        assert info.kernel_loop == 3 and (not knobs or info.passes > 1), (name, info.kernel_loop, info.passes)
        ins = [torch.from_numpy(d["i"]).cuda() if d["i"].size else None for d in init]
        outs = [torch.from_numpy(d["o"]).cuda() if d["o"].size else None for d in init]
        for r, d in enumerate(init):
            if d["s"].size:
                ex._scratch[r].view(torch.float32).copy_(torch.from_numpy(d["s"]))
        ex.run(ins, outs)
        torch.cuda.synchronize()
        for r in range(algo.ngpus):
            got = {"i": ins[r], "o": outs[r], "s": None if ex._scratch[r] is None else ex._scratch[r].view(torch.float32)}
            for b in "ios":
                if want[r][b].size:
                    assert np.array_equal(got[b].cpu().numpy().view(np.uint32), want[r][b].view(np.uint32)), (name, r, b)


def test_protocol_from_the_ir():
    """protocol="ir": the <algo proto=...> attribute picks the protocol (LL, LL128 -> lines)."""
    xml = ir_samples.ring_allreduce_xml(4)
    for proto, want in (("Simple", 1), ("LL", 2), ("LL128", 2)):
        doc = xml.replace('proto="Simple"', f'proto="{proto}"')
        assert f'proto="{proto}"' in doc
        got, ref, _, info = run_both(doc, 2048, "float32", protocol="ir")
        assert info.protocol == want
        assert_same(got, ref)
