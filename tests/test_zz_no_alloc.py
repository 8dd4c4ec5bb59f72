"""mscclx_plan_run_static -- a whole execution out of the library's static device array, for callers
that cannot allocate -- against mscclx_plan_bind + launch + wait and against the NumPy interpreter on the
same inputs, through the C ABI.  Bit-exact; several calls in a row share the array, each smaller than the
one before; the device's free memory is the same before and after a call."""
import numpy as np
import pytest
import torch

import ir_samples
from test_gpu_parity import make_inputs, to_numpy, to_torch

pytestmark = pytest.mark.gpu


def _both_ways(xml, chunk_elems, dtype, seed, **knobs):
    """The same plan and inputs through the existing entry points, through the static one and through
    the NumPy interpreter; returns the three lists of result buffers (every rank's 'i' and 'o' as raw bytes)."""
    from msccl.executor import DTYPE_SIZES, Executor, collective_buffers
    from oracle import collectives as oc
    from oracle import ir_interp as oi
    esz = DTYPE_SIZES[dtype]
    ex = Executor(xml)
    ex.setup(chunk_elems * esz, dtype, **knobs)
    n = ex.tables.ngpus
    x = make_inputs(n, int(ex.tables.rank_chunks[0, 0]) * chunk_elems, dtype, seed)
    results = []
    for way in ("bind+launch+wait", "run_static"):
        ins, outs, _ = collective_buffers(ex.tables, chunk_elems * esz, dtype, inputs=[to_torch(v, dtype) for v in x])
        print(f"case: {way} chunk_elems={chunk_elems} dtype={dtype} knobs={knobs}", flush=True)
        if way == "run_static":
            # Free device memory as the driver counts it (hipMemGetInfo): it sees a hipMalloc made inside the
            # library, which torch's own allocator statistics do not.  A first call on copies of the buffers takes
            # whatever the runtime sets up once per process (the code object's static array among it).
            warm_in, warm_out, _ = collective_buffers(ex.tables, chunk_elems * esz, dtype, inputs=[to_torch(v, dtype) for v in x])
            assert ex.run_static(warm_in, warm_out).code == 0
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            st = ex.run_static(ins, outs)
            assert st.code == 0
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "mscclx_plan_run_static changed the device's free memory"
        else:
            ex.run(ins, outs)
            first_binding = (ins, outs)
        torch.cuda.synchronize()
        results.append([to_numpy(b, dtype).view(np.uint8).copy() for pair in zip(ins, outs) for b in pair if b is not None])
    # the binding made by bind() is untouched by the static calls: launched again on fresh inputs, it still delivers
    ins, outs = first_binding
    fresh, _, _ = collective_buffers(ex.tables, chunk_elems * esz, dtype, inputs=[to_torch(v, dtype) for v in x])
    for b, f in zip(ins, fresh):
        if b is not None:
            b.copy_(f)
    for o in outs:
        if o is not None and not any(o is i for i in ins):
            o.zero_()
    ex.launch()
    ex.wait()
    torch.cuda.synchronize()
    results.append([to_numpy(b, dtype).view(np.uint8).copy() for pair in zip(ins, outs) for b in pair if b is not None])
    # the NumPy interpreter on the same inputs
    algo = oi.parse_xml(xml)
    want = oc.place_inputs(algo, x, chunk_elems, dtype)
    oi.Interpreter(algo).run(want, chunk_elems, dtype)
    oracle = []
    for r in range(n):
        for key, count in (("i", algo.gpus[r].i_chunks), ("o", algo.gpus[r].o_chunks)):
            if count:
                oracle.append(np.ascontiguousarray(want[r][key]).view(np.uint8).copy())
    results.append(oracle)
    return results


def _assert_equal(first, *others):
    for which, other in enumerate(others):
        assert len(first) == len(other), which
        for k, (u, v) in enumerate(zip(first, other)):
            assert u.shape == v.shape and np.array_equal(u, v), (which, k, int(np.flatnonzero(u != v)[0]) if u.shape == v.shape else (u.shape, v.shape))


def test_run_static_matches_bind_launch_wait_on_shrinking_inputs():
    # ring all-reduce, 8 ranks x 2 instances: rrs results go through FIFO slots in the array
    xml = ir_samples.ring_allreduce_xml(8, 2)
    for chunk_elems, seed in ((40000, 1), (3000, 2), (16, 3)):       # each call smaller than the one before
        _assert_equal(*_both_ways(xml, chunk_elems, "float32", seed))
    # all-pairs with rank scratch, dependencies and nops folded at bind (another kernel, other tables)
    _assert_equal(*_both_ways(ir_samples.allpairs_allreduce_xml(5), 2000, "bfloat16", 4))
    # flag-in-data lines: what the previous call's lines left in the slots must not be taken for this call's
    for chunk_elems, seed in ((8000, 5), (8000, 6), (512, 7)):
        _assert_equal(*_both_ways(xml, chunk_elems, "float32", seed, protocol="ll"))


def test_run_static_refuses_what_does_not_fit():
    from msccl.executor import Executor, MscclxError, collective_buffers
    from msccl.executor.binding import ERR_CAPACITY
    xml = ir_samples.ring_allreduce_xml(8, 2)
    ex = Executor(xml)
    E = 1 << 20                                                      # 4 MiB chunks: the staged rrs results alone need more than 32 MiB of slots
    ex.setup(E * 4, "float32", staging=1)
    ins, outs, _ = collective_buffers(ex.tables, E * 4, "float32")
    with pytest.raises(MscclxError) as e:
        ex.run_static(ins, outs)
    assert e.value.code == ERR_CAPACITY and "MSCCLX_STATIC_SCRATCH_BYTES" in e.value.message
    ex.run(ins, outs)                                                # the ordinary path takes it
