"""The five benchmark configurations and every reference-emitted program on the GPU.

Reduced sizes: HIP executor vs the NumPy interpreter, bit for bit, on IR from msccl-tools' compiler
and from this package's compiler.  Full sizes: properties that need no CPU pass over the data --
all-gather = concatenation, all-to-all = block transpose, all-reduce = the closed-form fold evaluated
with torch's own bf16/fp16/fp32 arithmetic on the device, all compared bit for bit.
"""
import numpy as np
import pytest
import torch

import golden_util
import ir_samples
from msccl.executor.workloads import WORKLOADS, numpy_input, torch_input
from oracle import collectives as oc
from oracle import ir_interp as oi
from test_configs_oracle import GOLDEN_OF, OTHERS, fold_orders
from test_gpu_parity import to_numpy, to_torch

pytestmark = pytest.mark.gpu

REDUCED = {"c1": 8 * 4 * 5000, "c2": 4 * 4 * 30000, "c3": 16 * 70000, "c4": 64 * 2 * 3000, "c5": 64 * 2 * 2048, "c5_chain": 2 * 30000}


def device_run(xml, w, inputs_np, **knobs):
    from msccl.executor import Executor, collective_buffers
    ex = Executor(xml)
    print(f"case: {w.key} bytes/rank={w.bytes_per_rank} chunk_bytes={w.chunk_bytes} knobs={knobs}", flush=True)
    info = ex.setup(w.chunk_bytes, w.dtype, **knobs)
    ins, outs, res = collective_buffers(ex.tables, w.chunk_bytes, w.dtype, inputs=[to_torch(v, w.dtype) for v in inputs_np])
    ex.run(ins, outs)
    torch.cuda.synchronize()
    return [to_numpy(r, w.dtype) for r in res], info


def oracle_run(xml, w, inputs_np):
    algo = oi.parse_xml(xml)
    E = w.chunk_bytes // np.dtype(oi.DTYPES[w.dtype]).itemsize
    bufs = oc.place_inputs(algo, inputs_np, E, w.dtype)
    oi.Interpreter(algo).run(bufs, E, w.dtype)
    return oc.extract_outputs(algo, bufs, E)


# the three ways a message can cross a connection
MODES = {"in-place": dict(protocol="simple", staging=0), "staged": dict(protocol="simple", staging=1), "ll": dict(protocol="ll")}


@pytest.mark.parametrize("mode", sorted(MODES))
@pytest.mark.parametrize("source", ["msccl-tools", "this-package"])
@pytest.mark.parametrize("key", sorted(WORKLOADS))
def test_config_reduced_size_vs_oracle(key, source, mode):
    """in-place: payloads are read where the sender keeps them when the plan proved that safe;
    staged: every message is copied through a FIFO slot; ll: every message goes through a slot as
    flag-in-data lines.  All must give the interpreter's bits."""
    w = WORKLOADS[key].scaled(REDUCED[key])
    xml = golden_util.load(GOLDEN_OF[key]) if source == "msccl-tools" else WORKLOADS[key].build()
    x = [numpy_input(w, r) for r in range(w.ranks)]
    got, info = device_run(xml, w, x, **MODES[mode])
    assert (info.zero_copy_messages == 0) == (mode != "in-place")
    assert info.protocol == (2 if mode == "ll" else 1)
    want = oracle_run(xml, w, x)
    for r in range(w.ranks):
        assert np.array_equal(got[r].view(np.uint8), want[r].view(np.uint8)), (key, r)


@pytest.mark.parametrize("key", ["c1", "c2", "c3", "c4", "c5", "c5_chain"])
def test_config_full_size_vs_oracle_on_the_benchmark_inputs(key):
    """Every configuration at FULL size, on exactly the inputs the benchmark definition names (NumPy
    streams default_rng(1000 * cfg + rank)), under the automatic geometry -- what `bench.py` times --
    against the interpreter, bit for bit.  (The largest, 32 ranks x 128 MiB of bf16, takes the interpreter
    a few seconds and drawing its inputs most of a minute.)"""
    w = WORKLOADS[key]
    xml = w.build()
    x = [numpy_input(w, r) for r in range(w.ranks)]
    got, info = device_run(xml, w, x)
    print(f"{key}: {info.workgroups} workgroups x {info.threads} threads, {info.slices} slices, pieces of {info.piece_bytes} bytes, protocol {info.protocol}", flush=True)
    want = oracle_run(xml, w, x)
    for r in range(w.ranks):
        assert np.array_equal(got[r].view(np.uint8), want[r].view(np.uint8)), (key, r)


@pytest.mark.parametrize("mode", sorted(MODES))
@pytest.mark.parametrize("source", ["msccl-tools", "this-package"])
@pytest.mark.parametrize("program", ["ring", "allpairs"])
def test_reduce_scatter_in_place(program, source, mode):
    """Reduce-scatter programs, in place (rank r's result is its own input chunks [r * cf, (r + 1) * cf),
    msccl/language/collectives.py:220-225): collective_buffers' view of the result against the interpreter's,
    and against the closed form with the fold order the program's text fixes; bf16, so that the order shows."""
    from msccl.executor import Executor, collective_buffers
    from test_configs_oracle import REDUCE_SCATTERS
    fixture, build, nchunks, per_rank, orders = REDUCE_SCATTERS[program]
    xml = golden_util.load(fixture) if source == "msccl-tools" else build()
    algo = oi.parse_xml(xml)
    E = 2600 + (1 if mode == "in-place" else 0)           # chunks of 5200 or 5202 bytes (the latter end inside a dword)
    rng = np.random.default_rng(63)
    x = [oi.f32_to_bf16_bits(rng.standard_normal(nchunks * E, dtype=np.float32)) for _ in range(8)]
    ex = Executor(xml)
    print(f"case: reduce-scatter {program} from {source}, mode={mode}", flush=True)
    ex.setup(E * 2, "bfloat16", **MODES[mode])
    ins, outs, res = collective_buffers(ex.tables, E * 2, "bfloat16", inputs=[to_torch(v, "bfloat16") for v in x])
    assert all(o is None for o in outs) and all(res[r].data_ptr() == ins[r].data_ptr() + r * per_rank * E * 2 for r in range(8))
    ex.run(ins, outs)
    torch.cuda.synchronize()
    bufs = oc.place_inputs(algo, x, E, "bfloat16")
    oi.Interpreter(algo).run(bufs, E, "bfloat16")
    want = oc.extract_outputs(algo, bufs, E)
    closed = oc.expected_reduce_scatter(x, per_rank, orders(), "bfloat16")
    for r in range(8):
        got = to_numpy(res[r], "bfloat16")
        assert np.array_equal(got, want[r]) and np.array_equal(got, closed[r]), (program, source, mode, r)
        assert np.array_equal(to_numpy(ins[r], "bfloat16"), bufs[r]["i"]), (program, source, mode, r, "whole buffer")


@pytest.mark.parametrize("name", golden_util.names() + golden_util.ncclize_names())
def test_reference_emitted_programs_vs_oracle(name):
    """Every program msccl-tools' compiler (tests/golden/reference_xml) and its second emitter, ncclize
    (tests/golden/ncclize_xml), emitted for the fixtures, whatever its collective: all
    three buffers of every rank start from the same random bits on both sides and must end equal,
    with payloads read in place, with everything staged, and with flag-in-data lines."""
    from msccl.executor import Executor
    xml = golden_util.load(name)
    algo = oi.parse_xml(xml)
    E = 1536 if algo.ngpus * max(g.i_chunks + g.o_chunks + g.s_chunks for g in algo.gpus) > 4000 else 3000
    rng = np.random.default_rng(5)
    init = [{b: (rng.random(n * E, dtype=np.float32) * 2 - 1) for b, n in (("i", g.i_chunks), ("o", g.o_chunks), ("s", g.s_chunks))}
            for g in algo.gpus]
    want = [{b: v.copy() for b, v in d.items()} for d in init]
    oi.Interpreter(algo).run(want, E, "float32")
    for mode in sorted(MODES):
        ex = Executor(xml)
        print(f"case: {name} mode={mode}", flush=True)
        ex.setup(E * 4, "float32", **MODES[mode])
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
                    assert np.array_equal(got[b].cpu().numpy().view(np.uint32), want[r][b].view(np.uint32)), (name, r, b, mode)


@pytest.mark.parametrize("name", golden_util.ncclize_names())
def test_ncclize_emitted_programs_match_their_send_lists_on_device(name):
    """The documents ncclize emitted, on the device, against what their hand-written send lists mean
    (no interpreter in between): 32-bit integers, ragged chunks, automatic geometry."""
    from msccl.executor import Executor
    from test_configs_oracle import _ncclize_case, _ncclize_expected
    E = 2501
    algo, x = _ncclize_case(name, E, seed=21)
    ex = Executor(golden_util.load(name))
    print(f"case: {name} closed form", flush=True)
    ex.setup(E * 4, "int32")
    ins = [torch.from_numpy(v).cuda() if v.size else None for v in x]
    outs = [torch.zeros(g.o_chunks * E, dtype=torch.int32, device="cuda") if g.o_chunks else None for g in algo.gpus]
    ex.run(ins, outs)
    torch.cuda.synchronize()
    for r, (buf, want) in _ncclize_expected(name, algo, x, E).items():
        got = (outs if buf == "o" else ins)[r].cpu().numpy()
        assert np.array_equal(got[:want.size], want), (name, r)


def torch_fold(order, operands):
    if isinstance(order, int):
        return operands[order]
    acc = None
    for item in order:
        v = torch_fold(item, operands)
        acc = v if acc is None else acc + v   # torch adds bf16/fp16 in fp32 and rounds to nearest even
    return acc


@pytest.mark.parametrize("key", sorted(WORKLOADS))
def test_config_full_size_properties(key):
    from msccl.executor import Executor, collective_buffers
    w = WORKLOADS[key]
    dev = "cuda:0"
    xml = w.build()
    ex = Executor(xml)
    print(f"case: full-size {key}", flush=True)
    info = ex.setup(w.chunk_bytes, w.dtype)
    x = [torch_input(w, r, dev) for r in range(w.ranks)]
    ins, outs, res = collective_buffers(ex.tables, w.chunk_bytes, w.dtype, device=dev, inputs=x)
    ex.run(ins, outs)
    torch.cuda.synchronize()
    n = w.ranks
    if w.coll == "allgather":
        want = torch.cat(x)
        for r in range(n):
            assert torch.equal(res[r], want), r
    elif w.coll == "alltoall":
        blk = x[0].numel() // n
        for r in range(n):
            want = torch.cat([x[i][r * blk:(r + 1) * blk] for i in range(n)])
            assert torch.equal(res[r], want), r
    else:
        E = x[0].numel() // w.nchunks
        orders = fold_orders(key)
        itype = torch.int32 if x[0].element_size() == 4 else torch.int16
        for c in range(w.nchunks):
            want = torch_fold(orders[c], [x[i][c * E:(c + 1) * E] for i in range(n)])
            for r in range(n):
                assert torch.equal(res[r][c * E:(c + 1) * E].view(itype), want.view(itype)), (c, r)
    del x, ins, outs, res
    torch.cuda.empty_cache()


def test_chunks_beyond_4_gib():
    """Chunks larger than 4 GiB: every offset inside a rank buffer needs more than 32 bits.  A two-rank
    in-place all-gather of 5 GiB chunks (ragged against the slices) and a three-rank in-place all-reduce
    of 4.5 GiB per rank (its rrs results go through FIFO slots), both checked against closed forms on
    the device."""
    from msccl.executor import Executor, collective_buffers
    dev = "cuda:0"
    cb = (5 << 30) + 48
    ex = Executor(ir_samples.ring_allgather_xml(2, 1))
    print("case: 5 GiB chunks, all-gather", flush=True)
    info = ex.setup(cb, "uint8")
    x = [torch.randint(0, 256, (cb,), dtype=torch.uint8, device=dev) for _ in range(2)]
    ins, outs, res = collective_buffers(ex.tables, cb, "uint8", device=dev, inputs=x)
    ex.run(ins, outs)
    torch.cuda.synchronize()
    for r in range(2):
        assert torch.equal(res[r][:cb], x[0]) and torch.equal(res[r][cb:], x[1]), r
    del x, ins, outs, res, ex
    torch.cuda.empty_cache()

    cb = (3 << 29) + 64
    E = cb // 4
    ex = Executor(ir_samples.ring_allreduce_xml(3))
    print("case: 3 x 1.5 GiB chunks per rank, all-reduce", flush=True)
    info = ex.setup(cb, "int32")
    assert info.passes > 1 and info.staged_messages > 0
    x = [torch.randint(-2**31, 2**31 - 1, (3 * E,), dtype=torch.int32, device=dev) for _ in range(3)]
    want = x[0] + x[1] + x[2]
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", device=dev, inputs=x)
    ex.run(ins, outs)
    torch.cuda.synchronize()
    for r in range(3):
        assert torch.equal(res[r], want), r
    del x, ins, outs, res, want, ex
    torch.cuda.empty_cache()


def test_aliased_buffers_fall_back_to_staging():
    """An in-place call on an out-of-place algorithm aliases buffers the IR names separately: here every
    rank's 'i' is chunk r of its own 'o' (NCCL's in-place all-gather convention) on an out-of-place
    ring all-gather whose copy threadblock moves i[0] to o[r].  Reading payloads in place assumes
    distinct memory, so bind refuses with ALIASED, and so does the runner unless the caller passes
    allow_aliased=True; it then re-plans with every message staged, and this program (every write of a
    chunk writes its final value) must still deliver the concatenation.  On a program where aliasing
    makes a receive overwrite what a send of the same rank still has to read, nothing but the refusal is promised."""
    import ir_samples
    from msccl.executor import Executor, MscclxError
    from msccl.executor.binding import ERR_ALIASED
    n, E = 5, 3000
    xml = ir_samples.ncclize_style_allgather_xml(n)
    rng = np.random.default_rng(77)
    x = [rng.integers(-2 ** 31, 2 ** 31, E, dtype=np.int64).astype(np.int32) for _ in range(n)]
    want = np.concatenate(x)
    ex = Executor(xml)
    ex.setup(E * 4, "int32", protocol="simple")
    assert ex.info.zero_copy_messages > 0
    outs = [torch.zeros(n * E, dtype=torch.int32, device="cuda:0") for _ in range(n)]
    ins = [outs[r][r * E:(r + 1) * E] for r in range(n)]        # same memory as o[r]
    for r in range(n):
        ins[r].copy_(torch.from_numpy(x[r]))
    with pytest.raises(MscclxError) as e:                        # the C ABI itself refuses ...
        ex.plan.bind([t.data_ptr() for t in ins], [t.data_ptr() for t in outs], [0] * n, ex._workspace.data_ptr(), ex._workspace.numel())
    assert e.value.code == ERR_ALIASED
    with pytest.raises(MscclxError) as e:                        # ... and so does the runner, unless told otherwise
        ex.run(ins, outs)
    assert e.value.code == ERR_ALIASED
    print("case: aliased all-gather, staged", flush=True)
    ex.run(ins, outs, allow_aliased=True)                        # the caller vouches for the program: every message staged
    assert ex.info.zero_copy_messages == 0 and ex.info.staged_messages > 0
    torch.cuda.synchronize()
    for r in range(n):
        assert np.array_equal(outs[r].cpu().numpy(), want), r
    # buffers that do not overlap, on the same Executor: back to the knobs setup() was given
    outs3 = [torch.zeros(n * E, dtype=torch.int32, device="cuda:0") for _ in range(n)]
    ex.run([torch.from_numpy(v).cuda() for v in x], outs3, allow_aliased=True)
    assert ex.info.zero_copy_messages > 0
    for r in range(n):
        assert np.array_equal(outs3[r].cpu().numpy(), want), r
    # the same data out of place, payloads read in place: the same result
    ex2 = Executor(xml)
    ex2.setup(E * 4, "int32", protocol="simple")
    outs2 = [torch.zeros(n * E, dtype=torch.int32, device="cuda:0") for _ in range(n)]
    ex2.run([torch.from_numpy(v).cuda() for v in x], outs2)
    assert ex2.info.zero_copy_messages > 0
    for r in range(n):
        assert torch.equal(outs2[r], outs[r]), r


def test_workspace_handed_from_plan_to_plan_and_back():
    """One workspace, two plans with different layouts of it, bound in turn: A runs, B is bound to the same
    memory and runs, A is bound again -- same address, nothing it knows of has failed -- and must find that its
    counters are no longer its own (B's bind stamped the workspace) and clear them before it runs."""
    import ir_samples
    from msccl.executor import Executor, collective_buffers
    E = 3000
    plans = {}
    for name, xml in (("A", ir_samples.ring_allreduce_xml(8, 2)), ("B", ir_samples.allpairs_allreduce_xml(5))):
        ex = Executor(xml)
        ex.setup(E * 4, "float32", protocol="simple")
        plans[name] = (ex, oi.parse_xml(xml))
    shared = torch.empty(max(int(ex.info.workspace_bytes) for ex, _ in plans.values()), dtype=torch.uint8, device="cuda:0")
    for turn, name in enumerate("ABABBA"):
        ex, algo = plans[name]
        ex._workspace = shared
        ex._bound = None
        n = algo.ngpus
        rng = np.random.default_rng(900 + turn)
        x = [rng.random(algo.gpus[0].i_chunks * E, dtype=np.float32) * 2 - 1 for _ in range(n)]
        ins, outs, res = collective_buffers(ex.tables, E * 4, "float32", inputs=[torch.from_numpy(v) for v in x])
        print(f"case: shared workspace, turn {turn}, plan {name}", flush=True)
        for _ in range(1 + turn % 2):                       # (an odd and an even number of launches: both counter areas get used)
            for r in range(n):
                ins[r].copy_(torch.from_numpy(x[r]))
            ex.run(ins, outs)
            ex._bound = None
        torch.cuda.synchronize()
        want = oc.place_inputs(algo, x, E, "float32")
        oi.Interpreter(algo).run(want, E, "float32")
        for r in range(n):
            assert np.array_equal(res[r].cpu().numpy().view(np.uint32), want[r]["i"].view(np.uint32)), (turn, name, r)


def test_executor_cache_hands_back_a_working_executor():
    """msccl.executor.cache.executor_for: the same (document, chunk size, type, knobs) again gives the executor made the
    first time -- in microseconds -- and it still delivers on new buffers; another chunk size gets an executor of its own."""
    import time
    import ir_samples
    from msccl.executor import cache, collective_buffers
    cache.clear()
    xml = ir_samples.allpairs_allreduce_xml(6)
    algo = oi.parse_xml(xml)
    E = 2000
    first = cache.executor_for(xml, E * 4, "float32")
    t0 = time.perf_counter()
    again = cache.executor_for(xml, E * 4, "float32")
    lookup = time.perf_counter() - t0
    assert again is first and lookup < 2e-3
    assert cache.executor_for(cache.tables_for(xml), E * 4, torch.float32) is first            # by tables, dtype given as torch's
    other = cache.executor_for(xml, 2 * E * 4, "float32")
    assert other is not first and other.tables is first.tables
    for ex, elems, seed in ((first, E, 1), (other, 2 * E, 2), (again, E, 3)):
        rng = np.random.default_rng(seed)
        x = [rng.random(6 * elems, dtype=np.float32) * 2 - 1 for _ in range(6)]
        ins, outs, res = collective_buffers(ex.tables, elems * 4, "float32", inputs=[torch.from_numpy(v) for v in x])
        print(f"case: cached executor, chunks of {elems} floats", flush=True)
        ex.run(ins, outs)
        torch.cuda.synchronize()
        want = oc.place_inputs(algo, x, elems, "float32")
        oi.Interpreter(algo).run(want, elems, "float32")
        for r in range(6):
            assert np.array_equal(res[r].cpu().numpy().view(np.uint32), want[r]["i"].view(np.uint32)), (seed, r)
    cache.clear()


def test_rebind_new_buffers_same_plan():
    """Binding a second and third set of buffers to a configured plan re-uses the device-side state
    (one upload of the tables); every set must get its own, correct result, and going back to the
    first set must work too."""
    import ir_samples
    from msccl.executor import Executor, collective_buffers
    xml = ir_samples.allpairs_allreduce_xml(4)
    algo = oi.parse_xml(xml)
    E = 3000
    ex = Executor(xml)
    ex.setup(E * 4, "float32")
    sets = []
    for k in range(3):
        rng = np.random.default_rng(500 + k)
        x = [(rng.random(4 * E, dtype=np.float32) * 2 - 1) for _ in range(4)]
        ins, outs, res = collective_buffers(ex.tables, E * 4, "float32", inputs=[torch.from_numpy(v) for v in x])
        want = oc.place_inputs(algo, x, E, "float32")
        oi.Interpreter(algo).run(want, E, "float32")
        sets.append((x, ins, outs, res, want))
    print("case: rebind", flush=True)
    for k in (0, 1, 2, 0):
        x, ins, outs, res, want = sets[k]
        for r in range(4):
            ins[r].copy_(torch.from_numpy(x[r]))
        ex.run(ins, outs)
        torch.cuda.synchronize()
        for r in range(4):
            assert np.array_equal(res[r].cpu().numpy().view(np.uint32), want[r]["i"].view(np.uint32)), (k, r)


def test_init_to_run_alltoall_and_large_allgather(capsys):
    """The other mi355x plans of one group of 8: the one-step all-to-all (a block transpose) and, from 12 MB per
    rank on, the 4-instance ring all-gather -- at a size that is no multiple of 16 bytes per chunk."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    a2a_bytes, ag_bytes = 8 * 3001 * 4, 12000000 + 32 * 4     # per rank
    msccl.init('mi355x', 1, ('alltoall', a2a_bytes), ('allgather', ag_bytes))
    capsys.readouterr()
    algos = load_config()
    a2a, ag = select(algos, "alltoall", a2a_bytes), select(algos, "allgather", ag_bytes)
    assert a2a.tables.name == "mi355x_alltoall_allpairs" and ag.tables.name == "mi355x_ring_allgather"
    rng = np.random.default_rng(9)
    x = [rng.integers(-2 ** 31, 2 ** 31, a2a_bytes // 4, dtype=np.int64).astype(np.int32) for _ in range(8)]
    cb = a2a.bytes_per_rank_to_chunk_bytes(a2a_bytes)
    assert cb == 3001 * 4
    ex = Executor(a2a.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v) for v in x])
    ex.run(ins, outs)
    for r in range(8):
        want = np.concatenate([x[s][r * 3001:(r + 1) * 3001] for s in range(8)])
        assert np.array_equal(res[r].cpu().numpy(), want), r
    y = [rng.integers(-2 ** 31, 2 ** 31, ag_bytes // 4, dtype=np.int64).astype(np.int32) for _ in range(8)]
    cb = ag.bytes_per_rank_to_chunk_bytes(ag_bytes)
    ex = Executor(ag.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v) for v in y])
    ex.run(ins, outs)
    want = np.concatenate(y)
    assert all(np.array_equal(res[r].cpu().numpy(), want) for r in range(8))


@pytest.mark.parametrize("groups,elems", [(2, 251), (4, 65)])
def test_init_to_run_allpairs_over_groups(groups, elems, capsys):
    """16 and 32 virtual ranks in the middle sizes: msccl.init picks the all-pairs program over all ranks; int32 sums
    (exact in any order) of chunks that are no multiple of 16 bytes."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    n = 8 * groups
    nbytes = n * n * elems * 4                                # per rank
    msccl.init('mi355x', groups, ('allreduce', nbytes))
    capsys.readouterr()
    ar = select(load_config(), "allreduce", nbytes)
    assert ar.tables.name == f"mi355x_allpairs_allreduce_{groups}x8" and ar.tables.ngpus == n
    rng = np.random.default_rng(groups)
    x = [rng.integers(-2 ** 31, 2 ** 31, nbytes // 4, dtype=np.int64) for _ in range(n)]
    cb = ar.bytes_per_rank_to_chunk_bytes(nbytes)
    assert cb == elems * 4
    ex = Executor(ar.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v.astype(np.int32)) for v in x])
    ex.run(ins, outs)
    want = sum(x).astype(np.int32)                              # wraps like the device's 32-bit adds
    assert all(np.array_equal(res[r].cpu().numpy(), want) for r in range(n))


@pytest.mark.parametrize("groups,nbytes,plan", [(1, 8 * 8 * 501 * 4, "allpairs"), (1, 12000000 + 32, "ring"), (2, 16 * 16 * 33 * 4, "allpairs")])
def test_init_to_run_reduce_scatter(groups, nbytes, plan, capsys):
    """msccl.init -> MSCCL_CONFIG -> select -> run for reduce-scatter, in place: rank r ends with the sums of its own
    1/n of the buffer, where it lies in its input (int32: exact in any order)."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    n = 8 * groups
    msccl.init('mi355x', groups, ('reduce_scatter', nbytes))
    capsys.readouterr()
    rs = select(load_config(), "reduce_scatter", nbytes)
    assert rs.tables.name == f"mi355x_{plan}_reduce_scatter" and rs.tables.ngpus == n and rs.tables.inplace
    rng = np.random.default_rng(groups)
    x = [rng.integers(-2 ** 31, 2 ** 31, nbytes // 4, dtype=np.int64) for _ in range(n)]
    cb = rs.bytes_per_rank_to_chunk_bytes(nbytes)
    ex = Executor(rs.tables)
    print(f"case: reduce-scatter from msccl.init, {n} ranks, {nbytes} bytes per rank, chunks of {cb} bytes", flush=True)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v.astype(np.int32)) for v in x])
    ex.run(ins, outs)
    total = sum(x).astype(np.int32)                             # wraps like the device's 32-bit adds
    per = nbytes // 4 // n
    for r in range(n):
        assert np.array_equal(res[r].cpu().numpy(), total[r * per:(r + 1) * per]), r


def test_init_to_run_allreduce_over_eight_groups(capsys):
    """64 virtual ranks at 256 KiB per rank: msccl.init picks all-pairs inside the groups and across them (int32 sums, exact in any order)."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    n, nbytes = 64, 256 << 10
    msccl.init('mi355x', 8, ('allreduce', nbytes))
    capsys.readouterr()
    ar = select(load_config(), "allreduce", nbytes)
    assert ar.tables.name == "mi355x_allpairs_two_level_allreduce_8x8" and ar.tables.ngpus == n
    rng = np.random.default_rng(64)
    x = [rng.integers(-2 ** 31, 2 ** 31, nbytes // 4, dtype=np.int64) for _ in range(n)]
    cb = ar.bytes_per_rank_to_chunk_bytes(nbytes)
    ex = Executor(ar.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v.astype(np.int32)) for v in x])
    ex.run(ins, outs)
    want = sum(x).astype(np.int32)
    assert all(np.array_equal(res[r].cpu().numpy(), want) for r in range(n))


def test_init_to_run_allgather_over_two_groups(capsys):
    """16 virtual ranks: the all-pairs all-gather below 12 MB per rank -- every output is the concatenation of the inputs."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    n, e = 16, 2501
    nbytes = e * 4
    msccl.init('mi355x', 2, ('allgather', nbytes))
    capsys.readouterr()
    ag = select(load_config(), "allgather", nbytes)
    assert ag.tables.name == "mi355x_allpairs_allgather" and ag.tables.ngpus == n
    rng = np.random.default_rng(61)
    x = [rng.integers(-2 ** 31, 2 ** 31, e, dtype=np.int64).astype(np.int32) for _ in range(n)]
    cb = ag.bytes_per_rank_to_chunk_bytes(nbytes)
    ex = Executor(ag.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v) for v in x])
    ex.run(ins, outs)
    want = np.concatenate(x)
    assert all(np.array_equal(res[r].cpu().numpy(), want) for r in range(n))


def test_init_to_run_alltoall_over_two_groups(capsys):
    """16 virtual ranks: msccl.init picks the one-step all-to-all here too -- a block transpose, chunks of 1003 int32."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    n, e = 16, 1003
    nbytes = n * e * 4
    msccl.init('mi355x', 2, ('alltoall', nbytes))
    capsys.readouterr()
    a2a = select(load_config(), "alltoall", nbytes)
    assert a2a.tables.name == "mi355x_alltoall_allpairs" and a2a.tables.ngpus == n
    rng = np.random.default_rng(16)
    x = [rng.integers(-2 ** 31, 2 ** 31, n * e, dtype=np.int64).astype(np.int32) for _ in range(n)]
    cb = a2a.bytes_per_rank_to_chunk_bytes(nbytes)
    assert cb == e * 4
    ex = Executor(a2a.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v) for v in x])
    ex.run(ins, outs)
    for r in range(n):
        assert np.array_equal(res[r].cpu().numpy(), np.concatenate([x[s][r * e:(r + 1) * e] for s in range(n)])), r


def test_init_to_run_flow(capsys):
    """msccl.init -> MSCCL_CONFIG index -> select by size -> run: the drop-in path end to end."""
    import os
    import msccl
    from msccl.executor import Executor, collective_buffers, load_config, select
    for k in ("MSCCL_CONFIG", "NCCL_ALGO"):
        os.environ.pop(k, None)
    nbytes = 8 * 4 * 4 * 2500                                # bytes per rank
    msccl.init('mi355x', 1, ('allgather', nbytes), ('allreduce', nbytes))
    algos = load_config()
    ag = select(algos, "allgather", nbytes)
    ar = select(algos, "allreduce", nbytes)
    assert ag is not None and ar is not None and ar.tables.nchunksperloop == 64   # below 16 MB: all-pairs
    rng = np.random.default_rng(3)
    # all-gather
    x = [rng.integers(-2 ** 31, 2 ** 31, nbytes // 4, dtype=np.int64).astype(np.int32) for _ in range(8)]
    cb = ag.bytes_per_rank_to_chunk_bytes(nbytes)
    ex = Executor(ag.tables)
    ex.setup(cb, "int32")
    ins, outs, res = collective_buffers(ex.tables, cb, "int32", inputs=[torch.from_numpy(v) for v in x])
    ex.run(ins, outs)
    want = np.concatenate(x)
    assert all(np.array_equal(res[r].cpu().numpy(), want) for r in range(8))
    # all-reduce (all-pairs order: own value, then the peers' in ascending order)
    y = [(rng.random(nbytes // 4, dtype=np.float32) * 2 - 1) for _ in range(8)]
    cb = ar.bytes_per_rank_to_chunk_bytes(nbytes)
    ex = Executor(ar.tables)
    ex.setup(cb, "float32")
    ins, outs, res = collective_buffers(ex.tables, cb, "float32", inputs=[torch.from_numpy(v) for v in y])
    ex.run(ins, outs)
    want = oc.expected_allreduce(y, 64, oc.allpairs_allreduce_orders(8), "float32")
    assert all(np.array_equal(res[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32)) for r in range(8))


def test_bench_times_any_ir_file():
    """`bench.py --xml FILE --chunk-bytes A,B` times one MSCCL-IR document by itself: one JSON line per chunk size, with the
    geometry and the step loop it ran on; `bench.py --gpus 2` refuses (every rank is a virtual rank on one GPU)."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    fixture = os.path.join(root, "tests", "golden", "reference_xml", "allreduce_a100_allpairs_8r.xml.gz")
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--xml", fixture, "--chunk-bytes", "1024,65536", "--steps", "5", "--warmup", "1"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(l) for l in r.stdout.splitlines() if l.startswith("{")]
    assert [l["chunk_bytes"] for l in lines] == [1024, 65536]
    for l in lines:
        assert l["ranks"] == 8 and l["collective"] == "allreduce" and l["launches"] == 5
        assert 1.0 < l["us_per_launch_median"] < 10000.0 and l["algorithmic_bytes"] > 0
        assert set(l["geometry"]) >= {"workgroups", "threads", "slices", "piece_bytes", "passes"}
    assert lines[0]["step_loop"] == "chain, folded nops"   # (small chunks: one-wave workgroups, one context each)
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr
