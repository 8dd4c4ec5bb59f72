"""mscclx_plan_run_static -- a whole execution out of the library's static device array, for callers
that cannot allocate -- against mscclx_plan_bind + launch + wait on the same inputs, through the C ABI.
Bit-exact; several calls in a row share the array, each smaller than the one before."""
import numpy as np
import pytest
import torch

import ir_samples
from test_gpu_parity import make_inputs, to_numpy, to_torch

pytestmark = pytest.mark.gpu


def _both_ways(xml, chunk_elems, dtype, seed, **knobs):
    """The same plan and inputs through the existing entry points and through the static one;
    returns the two lists of result buffers (every rank's 'i' and 'o' as raw bytes)."""
    from msccl.executor import DTYPE_SIZES, Executor, collective_buffers
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
            allocated = torch.cuda.memory_allocated()
            st = ex.run_static(ins, outs)
            assert st.code == 0
            assert torch.cuda.memory_allocated() == allocated
        else:
            ex.run(ins, outs)
        torch.cuda.synchronize()
        results.append([to_numpy(b, dtype).view(np.uint8).copy() for pair in zip(ins, outs) for b in pair if b is not None])
    return results


def _assert_equal(a, b):
    assert len(a) == len(b)
    for k, (u, v) in enumerate(zip(a, b)):
        assert np.array_equal(u, v), (k, int(np.flatnonzero(u != v)[0]))


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
