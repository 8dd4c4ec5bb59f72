"""MSCCLang front-end: the known answers msccl-tools' own tests hold for the compiler
(tests/test_language.py there), re-stated against this package's implementation."""
import pytest

from msccl.language import *
from msccl.language.collectives import *
from msccl.language.routines import *
from msccl.topologies import fully_connected, line


class Send(Collective):
    """chunk_factor chunks start on rank 0's input; they must reach rank 2's output."""

    def init_buffers(self):
        cf = self.chunk_factor
        return [{Buffer.input: [Chunk(r, c, 2, c) if r == 0 else None for c in range(cf)], Buffer.output: [None] * cf}
                for r in range(self.num_ranks)]

    def check(self, prog):
        out = prog.buffers[2][Buffer.output]
        return all(out[c] is not None and (out[c].origin_rank, out[c].origin_index) == (0, 0) for c in range(self.chunk_factor))


class Reduce(Collective):
    """every rank holds chunk 0; rank 2 must end with the sum of all of them."""

    def init_buffers(self):
        cf = self.chunk_factor
        return [{Buffer.input: [Chunk(r, c, -1, c) for c in range(cf)], Buffer.output: [None] * cf} for r in range(self.num_ranks)]

    def check(self, prog):
        want = ReduceChunk(-1, [])
        for r in range(self.num_ranks):
            want = want.reduce(-1, Chunk(r, 0))
        got = prog.buffers[2][Buffer.input][0]
        return got is not None and got == want


def test_send():
    with MSCCLProgram("send", line(3), Send(3, 1, inplace=False), 1):
        chunk(0, Buffer.input, 0).copy(1, 'scratch').copy(2, Buffer.output, 0)
        assert Check()


def test_reduce():
    with MSCCLProgram("reduce", line(3), Reduce(3, 1, inplace=True), 1):
        c10 = chunk(1, Buffer.input, 0).reduce(chunk(0, Buffer.input, 0))
        chunk(2, Buffer.input, 0).reduce(c10)
        assert Check()


def test_local_copy():
    with MSCCLProgram("cpy", fully_connected(3), Send(3, 1, inplace=False), 1):
        chunk(0, Buffer.input, 0).copy(2, 'scratch').copy(2, Buffer.output, 0)
        assert Check()


def test_local_reduce(capsys):
    with MSCCLProgram("local-reduce", line(3), Reduce(3, 1, inplace=True), 1):
        c = chunk(1, Buffer.input, 0).reduce(chunk(0, Buffer.input, 0))
        c = c.copy(2, 'scratch', 0)
        chunk(2, Buffer.input, 0).reduce(c)
        XML()
        assert Check()
    xml = capsys.readouterr().out
    assert 'type="re"' in xml and 'srcbuf="s"' in xml


def test_scratch_buffers():
    """explicit index 2, then an append lands at 3 (msccl-tools tests/test_language.py:119-132)."""
    with MSCCLProgram("test", fully_connected(3), AllReduce(3, 3, inplace=False), 1):
        chunk(0, Buffer.input, 0).copy(2, 'scratch', 2)
        c = chunk(2, 'scratch', 2)
        assert c.index == 2
        c = chunk(1, Buffer.input, 0).copy(2, 'scratch')
        assert c.index == 3
        XML()


def test_program_order():
    prgm = MSCCLProgram("test", fully_connected(2), AllReduce(2, 2, inplace=False), 1)
    with prgm:
        chunk(1, Buffer.input, 0).copy(0, 'sc', 1)
        # this receive overwrites what the send above reads: it must come after it
        chunk(0, Buffer.input, 0).copy(1, Buffer.input, 0)
    prgm.lower()
    op = prgm.instr_dag.operations[(1, Buffer.input, 0)]
    assert op.inst == Instruction.start
    assert op.next[0].inst == Instruction.send
    assert op.next[0].next[0].inst == Instruction.recv


def test_allgather():
    with MSCCLProgram("allgather", fully_connected(2), AllGather(2, 1, True), 1):
        chunk(0, Buffer.input, 0).copy(1, Buffer.output, 0)
        chunk(1, Buffer.input, 0).copy(0, Buffer.output, 1)
        assert Check()


def test_reducescatter():
    with MSCCLProgram("reducescatter", fully_connected(2), ReduceScatter(2, 1, True), 1):
        chunk(1, Buffer.input, 1).reduce(chunk(0, Buffer.input, 1))
        chunk(0, Buffer.input, 0).reduce(chunk(1, Buffer.input, 0))
        assert Check()


def test_alltoall():
    with MSCCLProgram("alltoall", fully_connected(2), AllToAll(2, 1, False), 1):
        chunk(0, Buffer.input, 0).copy(0, Buffer.output, 0)
        chunk(0, Buffer.input, 1).copy(1, Buffer.output, 0)
        chunk(1, Buffer.input, 0).copy(0, Buffer.output, 1)
        chunk(1, Buffer.input, 1).copy(1, Buffer.output, 1)
        assert Check()


def test_allreduce():
    with MSCCLProgram("allreduce", fully_connected(2), AllReduce(2, 2, True), 1):
        chunk(1, Buffer.output, 0).reduce(chunk(0, Buffer.input, 0)).copy(0, Buffer.input, 0)
        chunk(0, Buffer.input, 1).reduce(chunk(1, Buffer.input, 1)).copy(1, Buffer.input, 1)
        assert Check()


def test_check_detects_a_wrong_program():
    with MSCCLProgram("allgather", fully_connected(2), AllGather(2, 1, True), 1):
        chunk(0, Buffer.input, 0).copy(1, Buffer.output, 0)
        assert not Check()


def test_instruction_fusion():
    """3-rank chain: gpu0 [s, rcs], gpu1 [rrs, r], gpu2 [rrcs] (msccl-tools tests/test_language.py:188-202)."""
    prgm = MSCCLProgram("allreduce", fully_connected(3), AllReduce(3, 3, True), 1, threadblock_policy=ThreadblockPolicy.manual)
    with prgm:
        c01 = chunk(1, Buffer.input, 0, 3).reduce(chunk(0, Buffer.input, 0, 3), sendtb=0, recvtb=0, ch=0)
        c012 = chunk(2, Buffer.input, 0, 3).reduce(c01, sendtb=0, recvtb=0, ch=0)
        c012.copy(0, Buffer.input, 0, sendtb=0, recvtb=0, ch=0).copy(1, Buffer.input, 0, sendtb=0, recvtb=0, ch=0)
        assert Check()
    lowered = prgm.lower()
    assert lowered.gpus[0].threadblocks[0].ops[0].inst == Instruction.send
    assert lowered.gpus[0].threadblocks[0].ops[1].inst == Instruction.recv_copy_send
    assert lowered.gpus[1].threadblocks[0].ops[0].inst == Instruction.recv_reduce_send
    assert lowered.gpus[1].threadblocks[0].ops[1].inst == Instruction.recv
    assert lowered.gpus[2].threadblocks[0].ops[0].inst == Instruction.recv_reduce_copy_send


def test_fusion_can_be_switched_off():
    prgm = MSCCLProgram("allreduce", fully_connected(3), AllReduce(3, 3, True), 1, threadblock_policy=ThreadblockPolicy.manual,
                        instr_fusion=False)
    with prgm:
        c01 = chunk(1, Buffer.input, 0, 3).reduce(chunk(0, Buffer.input, 0, 3), sendtb=0, recvtb=0, ch=0)
        c01.copy(2, Buffer.input, 0, sendtb=0, recvtb=0, ch=0)
    insts = [op.inst for op in prgm.lower().gpus[1].threadblocks[0].ops]
    assert insts == [Instruction.recv_reduce_copy, Instruction.send]


def _alltoall_2(instances):
    prgm = MSCCLProgram("alltoall", fully_connected(2), AllToAll(2, 1, False), instances)
    with prgm:
        chunk(0, Buffer.input, 0).copy(0, Buffer.output, 0)
        chunk(0, Buffer.input, 1).copy(1, Buffer.output, 0)
        chunk(1, Buffer.input, 0).copy(0, Buffer.output, 1)
        chunk(1, Buffer.input, 1).copy(1, Buffer.output, 1)
    return prgm


def test_replication():
    instances = 2
    one, two = _alltoall_2(1).lower(), _alltoall_2(instances).lower()
    for gpu1, gpu2 in zip(one.gpus, two.gpus):
        assert len(gpu1.threadblocks) * instances == len(gpu2.threadblocks)


def test_replication_indices_and_channels():
    """interleaved: index*instances + i; channel: max_channels*i + ch (rank_dag.py:337-355)."""
    xml = _alltoall_2(3).generate_xml()
    from msccl.executor import parse_algo_xml
    t = parse_algo_xml(xml)
    assert t.rank_chunks.tolist() == [[6, 6, 0], [6, 6, 0]]
    sends = t.ops[t.ops[:, 0] == 1]
    assert sorted(sends[:, 2].tolist()) == [0, 1, 2, 3, 4, 5]  # rank0 sends input 3,4,5; rank1 sends input 0,1,2
    assert sorted(set(t.tbs[:, 3].tolist())) == [0, 1, 2]


def test_illegal_tb_assignment():
    prgm = MSCCLProgram("alltoall", fully_connected(3), AllToAll(3, 1, False), 1, threadblock_policy=ThreadblockPolicy.manual)
    with prgm:
        with pytest.raises(Exception):
            # one threadblock cannot send to two different ranks
            chunk(0, Buffer.input, 0).copy(1, Buffer.output, 0, sendtb=0, recvtb=1)
            chunk(0, Buffer.input, 1).copy(2, Buffer.output, 0, sendtb=0, recvtb=1)
            XML()


def test_no_link_is_rejected():
    with MSCCLProgram("send", line(3), Send(3, 1, inplace=False), 1):
        with pytest.raises(AssertionError):
            chunk(0, Buffer.input, 0).copy(2, Buffer.output, 0)


def test_only_one_program_in_context():
    with MSCCLProgram("a", fully_connected(2), AllGather(2, 1, True), 1):
        with pytest.raises(RuntimeError):
            MSCCLProgram("b", fully_connected(2), AllGather(2, 1, True), 1).__enter__()
    with pytest.raises(RuntimeError):
        chunk(0, Buffer.input, 0)


def test_routines_allgather_ring_inplace():
    with MSCCLProgram("allgather_ring", fully_connected(4), AllGather(4, 1, True), 1):
        allgather_ring_inplace(4)
        assert Check()


def test_routines_allgather_ring_nodes():
    size = 8
    with MSCCLProgram("allgather_multi", fully_connected(size), AllGather(size, 1, True), 1):
        allgather_ring_inplace(4, 0, 0)
        allgather_ring_inplace(4, 4, 4)
        for r in range(0, 8):
            peer = (r + 4) % size
            exchange_index = 0 if r < 4 else 4
            chunk(r, Buffer.output, exchange_index, 4).copy(peer, Buffer.output, exchange_index)
        assert Check()


def test_routines_allreduce_ring_inplace():
    with MSCCLProgram("allreduce_ring", fully_connected(4), AllReduce(4, 4, True), 1):
        allreduce_ring_inplace(4)
        assert Check()


def test_routines_allreduce_nodes(capsys):
    size = 8
    with MSCCLProgram("allreduce_multi", fully_connected(size), AllReduce(size, size, True), 1):
        allreduce_ring_inplace(4, 0, 0)
        allreduce_ring_inplace(4, 0, 4, ch=1)
        allreduce_ring_inplace(4, 4, 4)
        allreduce_ring_inplace(4, 4, 0, ch=1)
        for r in range(0, 8):
            peer = (r + 4) % size
            exchange_index = 0 if r < 4 else 4
            c = chunk(peer, Buffer.output, exchange_index, 4)
            c.reduce(chunk(r, Buffer.output, exchange_index, 4))
            c = c.copy(r, Buffer.output, exchange_index)
        XML()
        assert Check()
    assert "<algo" in capsys.readouterr().out


def test_dependency_cycle_is_rejected():
    from msccl.language.checks import ScheduleError, check_dependency_cycles
    a = Op(Instruction.copy, 0, ChunkRef(0, Buffer.input, 0, 1), ChunkRef(0, Buffer.output, 0, 1), tb=0, step=0)
    b = Op(Instruction.copy, 0, ChunkRef(0, Buffer.input, 1, 1), ChunkRef(0, Buffer.output, 1, 1), tb=1, step=0)
    a.depends, b.depends = [b], [a]
    with pytest.raises(ScheduleError):
        check_dependency_cycles([{0: Threadblock(ops=[a]), 1: Threadblock(ops=[b])}])
