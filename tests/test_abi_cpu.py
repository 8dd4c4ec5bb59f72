"""The C-ABI library without a GPU: it loads, exports every declared symbol, and its host half
(table validation, connection matching, dry run, geometry) behaves."""
import ctypes
import os
import re

import numpy as np
import pytest

import golden_util
import ir_samples
from msccl.executor import (EXPORTED_SYMBOLS, IRError, MscclxError, Plan, parse_algo_xml)
from msccl.executor import binding

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(mscclx_lib):
    header = open(os.path.join(ROOT, "include", "mscclx.h")).read()
    declared = set(re.findall(r"\b(mscclx_[a-z_]+)\s*\(", header))
    assert declared == set(EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(mscclx_lib, name), name
    assert mscclx_lib.mscclx_version() == 4


def test_struct_layouts_match_header():
    assert ctypes.sizeof(binding.Config) == 48
    assert ctypes.sizeof(binding.Info) == 80
    assert ctypes.sizeof(binding.Status) == 32


def test_tables_from_xml():
    t = parse_algo_xml(ir_samples.FUSION_CHAIN_XML)
    assert (t.ngpus, t.ntbs, t.nops, t.coll, t.inplace) == (3, 3, 5, "allreduce", True)
    assert t.rank_chunks.tolist() == [[3, 0, 0]] * 3
    assert t.tbs.tolist() == [[0, 1, 2, 0, 0, 2], [1, 2, 0, 0, 2, 4], [2, 0, 1, 0, 4, 5]]
    assert t.ops[:, 0].tolist() == [1, 3, 4, 2, 6]  # s rcs | rrs r | rrcs
    assert t.algorithmic_units() == 30


def test_xml_errors():
    with pytest.raises(IRError):
        parse_algo_xml("<nope/>")
    with pytest.raises(IRError):
        parse_algo_xml(ir_samples.FUSION_CHAIN_XML.replace('type="rcs"', 'type="xyz"'))
    with pytest.raises(IRError):
        parse_algo_xml(ir_samples.FUSION_CHAIN_XML.replace('<gpu id="2"', '<gpu id="5"'))


def test_plan_create_and_dry_run(mscclx_lib):
    p = Plan(parse_algo_xml(ir_samples.ring_allreduce_xml(8)))
    assert p.algorithmic_units() == 5 * 7 * 8  # 5(n-1) chunk moves per chunk index
    with pytest.raises(MscclxError) as e:
        p.simulate(1)  # fused ring: every rank holds one outgoing message and wants to push another
    assert e.value.code == binding.ERR_DEADLOCK and "rrs" in e.value.message
    assert p.simulate(2) == 0
    assert p.simulate(0) == 0
    assert p.min_fifo_depth() == 2
    assert Plan(parse_algo_xml(ir_samples.allpairs_allreduce_xml(4))).min_fifo_depth() == 1


def _mutated(xml, old, new, count=1):
    assert old in xml
    return parse_algo_xml(xml.replace(old, new, count))


@pytest.mark.parametrize("old,new,needle", [
    ('type="rcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3"', 'type="rcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="1" cnt="3"', "outside"),
    ('<tb id="0" send="1" recv="2"', '<tb id="0" send="-1" recv="2"', "without a send peer"),
    ('type="rrcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3"', 'type="rrcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="2"', "cnt"),
    ('type="rrcs"', 'type="rrc"', "receiver"),
    ('<step s="1" type="r" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1"', '<step s="1" type="r" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="4" deps="0"', "depid"),
])
def test_plan_create_rejects_bad_ir(mscclx_lib, old, new, needle):
    with pytest.raises(MscclxError) as e:
        Plan(_mutated(ir_samples.FUSION_CHAIN_XML, old, new))
    assert e.value.code == binding.ERR_BAD_IR
    assert needle in e.value.message


def test_output_offsets_out_of_range_are_not_taken_for_scratch(mscclx_lib):
    """Only a rank that declares scratch and never names buffer 's' -- what ncclize(use_scratch=False)
    writes -- has its output offsets past o_chunks read as scratch.  A document that names 's' keeps
    its out-of-range output offset and is refused; a step that straddles the output's end is refused
    in either style."""
    ok = parse_algo_xml(ir_samples.relay_through_scratch_xml(name_scratch=False))
    assert ok.ops[1:, [1, 2, 3, 4]].tolist() == [[0, 0, 2, 0], [2, 0, 1, 0]]   # r -> s[0..1]; cpy s[0] -> o[0]
    Plan(ok)
    Plan(parse_algo_xml(ir_samples.relay_through_scratch_xml()))
    t = parse_algo_xml(ir_samples.relay_through_scratch_xml(out_off=1))      # names 's': o[1] stays o[1], past the output's one chunk
    assert t.ops[2, [3, 4]].tolist() == [1, 1]
    with pytest.raises(MscclxError) as e:
        Plan(t)
    assert e.value.code == binding.ERR_BAD_IR and "outside" in e.value.message
    with pytest.raises(IRError) as e:
        parse_algo_xml(ir_samples.relay_through_scratch_xml(out_off=0, out_cnt=2, name_scratch=False))
    assert "straddle" in str(e.value)
    from oracle import ir_interp as oi
    with pytest.raises(ValueError):
        oi.parse_xml(ir_samples.relay_through_scratch_xml(out_off=0, out_cnt=2, name_scratch=False))
    a = oi.parse_xml(ir_samples.relay_through_scratch_xml(out_off=1))
    assert (a.gpus[1].tbs[1].steps[0].dstbuf, a.gpus[1].tbs[1].steps[0].dstoff) == ("o", 1)
    a = oi.parse_xml(ir_samples.relay_through_scratch_xml(name_scratch=False))
    assert (a.gpus[1].tbs[0].steps[0].dstbuf, a.gpus[1].tbs[0].steps[0].dstoff) == ("s", 0)


def test_two_senders_on_one_connection_rejected(mscclx_lib):
    xml = ir_samples.ring_allreduce_xml(4, instances=2).replace('chan="1"', 'chan="0"')
    with pytest.raises(MscclxError) as e:
        Plan(parse_algo_xml(xml))
    assert "both send" in e.value.message


def test_unfed_receive_is_a_bad_connection(mscclx_lib):
    with pytest.raises(MscclxError) as e:
        Plan(parse_algo_xml(ir_samples.RRC_CPY_NOP_XML.replace('type="s"', 'type="nop"')))
    assert "no sender" in e.value.message


def test_dependency_cycle_is_a_deadlock(mscclx_lib):
    # tb0 step0 waits for tb1 step1, tb1 step0 waits for tb0 step0
    xml = ir_samples.RRC_CPY_NOP_XML.replace('type="rrc" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="1" depid="-1" deps="-1"',
                                             'type="rrc" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="1" depid="1" deps="1"')
    p = Plan(parse_algo_xml(xml))
    with pytest.raises(MscclxError) as e:
        p.simulate(0)
    assert e.value.code == binding.ERR_DEADLOCK


def test_geometry_without_a_device(mscclx_lib):
    p = Plan(parse_algo_xml(ir_samples.ring_allgather_xml(8, 4)))  # 32 threadblocks
    info = p.configure(8 << 20, "int32", max_workgroups=2048)
    assert info.vector_path == 1
    # 128 KiB pieces: 64 slices of every 8 MiB chunk, each done in one pass by a 512-thread workgroup
    assert (info.slices, info.piece_bytes, info.passes, info.threads) == (64, 128 * 1024, 1, 512)
    # 32 x 64 contexts shared by 16 waves per CU of a 256-CU part
    assert (info.workgroups, info.max_hosted) == (512, 4)
    assert info.fifo_depth == 2 and info.connections == 32
    assert info.algorithmic_units * (8 << 20) == 2 * 7 * 8 * (32 << 20)   # 2(n-1) n S_in
    # every message of an all-gather can be read where the sender keeps it: no FIFO memory at all
    assert (info.zero_copy_messages, info.staged_messages) == (7 * 32, 0)
    assert info.workspace_bytes < 2 << 20
    # with staging forced: 32 connections x 64 slices x 2 slots x 128 KiB of FIFO
    staged = p.configure(8 << 20, "int32", max_workgroups=2048, staging=1)
    assert (staged.zero_copy_messages, staged.staged_messages) == (0, 7 * 32)
    assert staged.workspace_bytes >= 32 * 64 * 2 * 128 * 1024
    # a FIFO budget of 4 GiB splits bigger pieces into passes
    big = p.configure(1 << 30, "int32", max_workgroups=2048, staging=1)
    assert big.passes > 1 and big.workspace_bytes <= (4 << 30) + (8 << 20)
    # explicit knobs
    k = p.configure(8 << 20, "int32", max_workgroups=2048, slices=16, piece_bytes=65536, fifo_depth=4, threads=256, workgroups=128)
    assert (k.slices, k.piece_bytes, k.passes, k.fifo_depth, k.threads, k.workgroups, k.max_hosted) == (16, 65536, 8, 4, 256, 128, 4)
    # every chunk size moves in 16-byte units (the chunk's last unit may be partial, down to a single byte)
    info = p.configure(1000 * 4 + 4, "int32", max_workgroups=2048)
    assert info.vector_path == 1 and info.slices == 8   # tiny chunks: one slice per XCD
    assert p.configure(4, "int32", max_workgroups=2048).vector_path == 1
    q = Plan(parse_algo_xml(ir_samples.ring_allgather_xml(8, 4)))
    assert q.configure(1002, "float16", max_workgroups=2048).vector_path == 1
    assert q.configure(1001, "uint8", max_workgroups=2048).vector_path == 1
    assert q.configure(1, "uint8", max_workgroups=2048).vector_path == 1
    with pytest.raises(MscclxError):
        p.configure(6, "int32", max_workgroups=2048)              # not a multiple of the element
    # more threadblocks than workgroups is fine: a workgroup hosts up to 64 contexts ...
    few = p.configure(8 << 20, "int32", max_workgroups=16)
    assert few.workgroups == 16 and few.max_hosted * 16 >= few.slices * 32
    # ... but not more than that
    with pytest.raises(MscclxError) as e:
        p.configure(8 << 20, "int32", max_workgroups=16, slices=64)
    assert e.value.code == binding.ERR_CAPACITY
    with pytest.raises(MscclxError) as e:
        p.configure(8 << 20, "int32", max_workgroups=2048, fifo_depth=1)
    assert e.value.code == binding.ERR_DEADLOCK


def test_launch_before_bind_is_a_state_error(mscclx_lib):
    p = Plan(parse_algo_xml(ir_samples.FUSION_CHAIN_XML))
    with pytest.raises(MscclxError) as e:
        p.launch()
    assert e.value.code == binding.ERR_STATE


def test_zero_copy_analysis(mscclx_lib):
    """Which payloads may be read in place (plan.cpp: find_zero_copy_messages)."""
    def counts(xml):
        info = Plan(parse_algo_xml(xml)).configure(1 << 20, "float32", max_workgroups=4096, protocol="simple")
        return info.zero_copy_messages, info.staged_messages
    n = 8
    # ring all-reduce: per chunk the first 's' (its source is overwritten only by the final value,
    # which is causally after the receive), the 'rrcs' and the n-2 'rcs' keep their payload in
    # place; the n-2 'rrs' results exist nowhere but in the slot
    assert counts(ir_samples.ring_allreduce_xml(n)) == (n * (1 + 1 + (n - 2)), n * (n - 2))
    # the fusion chain: s, rrcs, rcs in place; rrs staged
    assert counts(ir_samples.FUSION_CHAIN_XML) == (3, 1)
    # a sender that overwrites its source right after sending, with nothing ordering the overwrite
    # after the receive, must stage
    xml = ir_samples.RRC_CPY_NOP_XML.replace(
        '<tb id="0" send="1" recv="-1" chan="0">\n' + ir_samples._step(0, "s", "i", 0, "i", 0, 1),
        '<tb id="0" send="1" recv="-1" chan="0">\n' + ir_samples._step(0, "s", "i", 0, "i", 0, 1) + "\n" +
        ir_samples._step(1, "cpy", "o", 0, "i", 0, 1)).replace('<gpu id="0" i_chunks="1" o_chunks="0"', '<gpu id="0" i_chunks="1" o_chunks="1"')
    assert counts(ir_samples.RRC_CPY_NOP_XML) == (1, 0)
    assert counts(xml) == (0, 1)


def test_protocol_choice(mscclx_lib):
    """Flag-in-data lines double the slot bytes and stage every message.  They are used on request, and
    by themselves only for a deep chain of hand-offs whose pieces can be cut to 1 KiB on at most two
    one-wave workgroups per compute unit, with every other knob automatic."""
    p = Plan(parse_algo_xml(ir_samples.ring_allreduce_xml(8)))
    for chunk in (8 << 20, 256 << 10):
        auto = p.configure(chunk, "float32", max_workgroups=2048)
        assert auto.protocol == binding.PROTOCOL_CODES["simple"] and auto.zero_copy_messages > 0
    auto = p.configure(64 << 10, "float32", max_workgroups=2048)
    assert auto.protocol == binding.PROTOCOL_CODES["ll"] and (auto.slices, auto.piece_bytes, auto.threads, auto.max_hosted) == (64, 1024, 64, 1)
    for knobs in (dict(threads=64), dict(piece_bytes=1024), dict(workgroups=512), dict(staging=1), dict(protocol="simple")):
        assert p.configure(64 << 10, "float32", max_workgroups=2048, **knobs).protocol == binding.PROTOCOL_CODES["simple"], knobs
    # nops that can be folded into the next step are worth more than the lines: such programs keep the counters
    allpairs = Plan(parse_algo_xml(golden_util.load("allreduce_a100_allpairs_8r")))
    assert allpairs.configure(1024, "float32", max_workgroups=2048).protocol == binding.PROTOCOL_CODES["simple"]
    small = p.configure(64 << 10, "float32", max_workgroups=2048, protocol="ll")
    assert small.protocol == binding.PROTOCOL_CODES["ll"]
    assert small.zero_copy_messages == 0 and small.staged_messages == 8 * 14
    # same geometry, every message staged: the LL workspace holds twice the slot bytes
    a = p.configure(8 << 20, "float32", max_workgroups=2048, protocol="ll", slices=16, piece_bytes=65536)
    b = p.configure(8 << 20, "float32", max_workgroups=2048, protocol="simple", staging=1, slices=16, piece_bytes=65536)
    assert a.protocol == binding.PROTOCOL_CODES["ll"] and a.staged_messages == b.staged_messages == 8 * 14
    slots = 8 * 2 * 65536 * 16  # connections x depth x piece x slices
    assert b.workspace_bytes - slots == a.workspace_bytes - 2 * slots  # what is left are the counters
    assert p.configure(1000 * 4 + 4, "int32", max_workgroups=2048, protocol="ll").protocol == binding.PROTOCOL_CODES["ll"]  # (a partial last unit travels as a whole line)
    with pytest.raises(MscclxError) as e:
        p.configure(1002, "float16", max_workgroups=2048, protocol="ll")  # lines carry whole dwords
    assert e.value.code == binding.ERR_UNSUPPORTED
    with pytest.raises(MscclxError) as e:
        p.configure(64 << 10, "float32", max_workgroups=2048, protocol=7)
    assert e.value.code == binding.ERR_INVALID_ARG


def test_geometry_of_the_benchmark_workloads(mscclx_lib):
    """The automatic geometry of the five benchmark workloads on a 256-CU part, as measured best on
    MI355X: (workgroups, threads, slices, piece bytes, passes, most contexts on a workgroup)."""
    from msccl.executor.workloads import WORKLOADS
    want = {
        "c1": (1024, 64, 128, 1024, 1, 1),      # latency bound: one workgroup of one wave per SIMD, one 16-byte unit per lane
        "c2": (512, 512, 64, 131072, 1, 4),     # a ring is always busy: 4 contexts per workgroup, one pass
        "c3": (256, 1024, 16, 131072, 2, 16),   # two thirds of its bytes are cold and its threadblocks wait half the time: a workgroup of 1024 threads per CU, 2 passes of 128 KiB
        "c4": (512, 512, 8, 65536, 4, 30),      # threadblocks mostly wait for each other: 30 per workgroup
        "c5": (512, 64, 8, 512, 1, 1),          # 126 hops: the smallest pieces allowed, flag-in-data lines
        "c5_chain": (4096, 64, 64, 4096, 1, 1),  # one buffer through 64 ranks: latency bound however big the chunk, one rank busy at a time: lines
    }
    for key, w in WORKLOADS.items():
        i = Plan(parse_algo_xml(w.build())).configure(w.chunk_bytes, w.dtype, max_workgroups=4096)
        assert (i.workgroups, i.threads, i.slices, i.piece_bytes, i.passes, i.max_hosted) == want[key], key
        assert i.protocol == binding.PROTOCOL_CODES["ll" if key in ("c1", "c5", "c5_chain") else "simple"], key  # (c1: lines at four one-wave workgroups per compute unit)
        # which step loop they run: the rings on lines have their steps worked out at bind (one pass, one row of at most 128 units per
        # step, no waits between a rank's threadblocks); the chain's rows of 256 units take the general loop for lines; the others host
        loop = {"c1": 4, "c5": 4, "c5_chain": 1}.get(key, 0)
        assert i.kernel_loop == loop, (key, i.kernel_loop, binding.LOOP_NAMES[i.kernel_loop])


def test_wide_workgroups_for_cold_traffic(mscclx_lib):
    """Programs whose bytes are mostly read once and written once (the share is reported) and whose threadblocks wait part of
    the time get one workgroup of 1024 threads per compute unit and pieces of 128 KiB, from slices of 96 KiB on, and at most
    eight passes where more slices can be had; rings and all-reduces never do.  (workgroups, threads, slices, piece bytes, passes)"""
    from msccl.executor.workloads import WORKLOADS
    c3 = parse_algo_xml(WORKLOADS["c3"].build())
    want = {1 << 20: (512, 512, 16, 65536, 1), 2 << 20: (256, 1024, 16, 131072, 1), 8 << 20: (256, 1024, 16, 131072, 4), 32 << 20: (256, 1024, 32, 131072, 8)}
    for chunk_bytes, expect in want.items():
        i = Plan(c3).configure(chunk_bytes, "uint8", max_workgroups=4096)
        assert (i.workgroups, i.threads, i.slices, i.piece_bytes, i.passes) == expect, (chunk_bytes, (i.workgroups, i.threads, i.slices, i.piece_bytes, i.passes))
        assert i.cold_traffic_x100 == 67 and 150 <= i.waiting_ratio_x100 <= 250
    for key, cold in (("c2", 14), ("c4", 0), ("c1", 0)):
        w = WORKLOADS[key].scaled(256 << 20)
        i = Plan(parse_algo_xml(w.build())).configure(w.chunk_bytes, w.dtype, max_workgroups=4096)
        assert i.cold_traffic_x100 == cold and i.threads == 512 and i.piece_bytes <= 131072, (key, i.cold_traffic_x100, i.threads, i.piece_bytes)
    i = Plan(parse_algo_xml(golden_util.load("allgather_allpairs_8r"))).configure(16 << 20, "int32", max_workgroups=4096)
    assert i.cold_traffic_x100 == 100 and i.waiting_ratio_x100 == 100 and i.threads == 512     # all cold, but always busy: as before


def test_geometry_between_the_benchmark_sizes(mscclx_lib):
    """Smaller messages of the same algorithms: (threads, slices, piece bytes) as measured best on MI355X."""
    from msccl.executor.workloads import WORKLOADS
    want = {
        # tiny chunks: 8 slices, so that workgroup w (XCD w mod 8) hosts slice w mod 8 and hand-offs stay inside an XCD
        ("c5", 64 << 10): (64, 8, 128),
        ("c1", 16 << 10): (64, 8, 256),
        # threadblocks that mostly wait: more slices than the plain latency model gives, pieces of 4 KiB or more
        ("c4", 512 << 10): (64, 2, 4096),
        # ... but a workgroup of one wave for every context where pieces of at most 8 KiB can be had that way
        ("c4", 1 << 20): (64, 2, 8192),
        ("c3", 512 << 10): (64, 4, 8192),
        ("c3", 1 << 20): (64, 8, 8192),
        ("c3", 2 << 20): (64, 16, 8192),
        ("c1", 16 << 20): (64, 256, 8192),
        # between latency and bandwidth: contexts are counted per compute unit, whatever the workgroup size
        ("c3", 4 << 20): (256, 8, 32768),
        ("c4", 4 << 20): (128, 4, 16384),
        ("c4", 8 << 20): (256, 4, 32768),
        # rings keep the largest pieces that still fill the chip
        ("c2", 4 << 20): (256, 32, 32768),
        ("c1", 32 << 20): (256, 128, 32768),
    }
    for (key, nbytes), expect in want.items():
        w = WORKLOADS[key].scaled(nbytes)
        i = Plan(parse_algo_xml(WORKLOADS[key].build())).configure(w.chunk_bytes, w.dtype, max_workgroups=4096)
        assert (i.threads, i.slices, i.piece_bytes) == expect, (key, nbytes, (i.threads, i.slices, i.piece_bytes))


def test_small_chunks_are_cut_one_unit_per_lane(mscclx_lib):
    """Chunks of up to 64 KiB: pieces of 1 KiB (one 16-byte unit per lane of a one-wave workgroup), else 2 KiB,
    where every context keeps a workgroup of its own and the busy ones are at most one per SIMD (two where some
    threadblocks wait); the slices are a power of two up to 8 and a multiple of 8 beyond;
    (workgroups, threads, slices, piece bytes, most contexts on a workgroup) on a 256-CU part."""
    want = {
        ("allreduce_a100_pcie_hierarchical_8r", 16 << 10): (2048, 64, 16, 1024, 1),   # 128 threadblocks that wait two thirds of the time
        ("pipeline_a100_allpairs_8r", 16 << 10): (2176, 64, 16, 1024, 1),
        ("allreduce_1step_4r", 64 << 10): (1024, 64, 64, 1024, 1),
        ("allreduce_allpairs_8r_2inst", 16 << 10): (2048, 64, 16, 1024, 1),            # some threadblocks wait: up to two busy contexts per SIMD
        ("allreduce_allpairs_8r_2inst", 64 << 10): (1024, 64, 8, 8192, 1),             # 8192 or 4096 contexts would be more: the latency model's 4, cut on down to 8 KiB, a wave each
        ("allreduce_a100_allpairs_8r", 20000): (1536, 64, 24, 928, 1),                  # 1250 units: 24 slices, a multiple of 8, not 32
        ("c5_allreduce_ring_64r_1ch_1inst", 16 << 10): (1024, 64, 16, 1024, 1),        # every threadblock busy: one context per SIMD ...
        ("c5_allreduce_ring_64r_1ch_1inst", 64 << 10): (512, 64, 8, 8192, 1),          # ... and no more
        ("c4_hierarchical_allreduce_8x4_2inst_auto", 4 << 10): (3840, 64, 2, 2048, 1),  # 1920 threadblocks: four slices would not get a workgroup each
        ("c1_allreduce_ring_8r_1ch_1inst", 128 << 10): (1024, 64, 128, 1024, 1),       # up to 128 KiB where ALL contexts are one per SIMD
        ("allgather_recursive_doubling_8r", 128 << 10): (768, 64, 32, 4096, 1),        # 3072 contexts would be three per SIMD: the latency model's 32
    }
    for (name, chunk_bytes), expect in want.items():
        i = Plan(parse_algo_xml(golden_util.load(name))).configure(chunk_bytes, "float32", max_workgroups=4096)
        assert (i.workgroups, i.threads, i.slices, i.piece_bytes, i.max_hosted) == expect, (name, chunk_bytes, (i.workgroups, i.threads, i.slices, i.piece_bytes, i.max_hosted))
    # a knob that fixes the workgroups keeps the latency model's slices
    i = Plan(parse_algo_xml(golden_util.load("allreduce_a100_pcie_hierarchical_8r"))).configure(16 << 10, "float32", max_workgroups=4096, threads=128)
    assert i.slices == 4
    # sizes that 256-byte groups do not divide: the slices are cut finer rather than let one of them run to a 65th unit
    # (piece_bytes is the longest slice)
    t = parse_algo_xml(golden_util.load("allreduce_a100_allpairs_8r"))
    for chunk_bytes, longest in ((16384, 1024), (15616, 1024), (15624, 1008), (16368, 1024), (16380, 1024)):
        i = Plan(t).configure(chunk_bytes, "float32", max_workgroups=4096)
        assert (i.threads, i.slices, i.piece_bytes) == (64, 16, longest), (chunk_bytes, i.threads, i.slices, i.piece_bytes)


def test_run_static_refuses_an_oversized_plan_before_touching_the_gpu(mscclx_lib):
    """The size check of mscclx_plan_run_static is host arithmetic: a plan whose tables, counters and
    FIFO slots exceed MSCCLX_STATIC_SCRATCH_BYTES is refused with CAPACITY before any HIP call."""
    t = parse_algo_xml(ir_samples.ring_allreduce_xml(8, 2))
    p = Plan(t)
    p.configure(4 << 20, "float32", staging=1, max_workgroups=512)
    fake = [0x10000000 + r * (1 << 28) for r in range(t.ngpus)]      # never dereferenced
    with pytest.raises(MscclxError) as e:
        p.run_static(fake, [0] * t.ngpus, [0] * t.ngpus)
    assert e.value.code == binding.ERR_CAPACITY and "MSCCLX_STATIC_SCRATCH_BYTES" in e.value.message


def test_documents_are_parsed_once(mscclx_lib):
    """Tables are kept by the hash of the document's text: the same text again (another Executor, another temporary file
    written by msccl.init for the same program) costs a hash, not a parse; another text gets tables of its own."""
    from msccl.executor import cache
    cache.clear()
    xml = ir_samples.ring_allreduce_xml(8)
    a = cache.tables_for(xml)
    assert cache.tables_for(xml) is a and a.document_key == cache.document_key(xml) and len(a.document_key) == 40
    other = cache.tables_for(xml.replace('name="', 'name="x'))
    assert other is not a and other.document_key != a.document_key and (other.ops == a.ops).all()
    for k in range(cache.MAX_DOCUMENTS + 3):                         # bounded: the entry unused for longest goes
        cache.tables_for(xml.replace('name="', f'name="{k}_'))
    assert len(cache._tables) == cache.MAX_DOCUMENTS and a.document_key not in cache._tables
    with pytest.raises(ValueError):
        cache.executor_for(parse_algo_xml(xml), 1024, "float32")     # tables that did not come from the cache carry no key
