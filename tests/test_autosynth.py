"""`msccl.init` and the plan registry: the observable behaviour msccl-tools' own tests assert
(tests/test_autosynth.py:10-45, tests/test_programs.py:61-86 there), plus the MI355X side reading
the index back."""
import math
import os

import pytest

import msccl
from msccl.autosynth import _select_plans
from msccl.autosynth.registry import register_ef_file, register_synthesis_plan, synthesis_plans
from msccl.autosynth.sizes import format_size, parse_size
from msccl.executor import load_config, select


@pytest.fixture(autouse=True)
def clean_env(monkeypatch):
    for k in ("MSCCL_CONFIG", "NCCL_ALGO", "NCCL_IB_AR_THRESHOLD", "NCCL_IB_PCI_RELAXED_ORDERING", "NCCL_TOPO_FILE", "CUDA_VISIBLE_DEVICES"):
        monkeypatch.delenv(k, raising=False)


def test_sizes():
    assert parse_size("512B") == 512 and parse_size("1KB") == 1000 and parse_size("1MB") == 10 ** 6
    assert parse_size("1GiB") == 2 ** 30 and parse_size("82944B") == 82944 and parse_size(7) == 7
    assert format_size(512) == "512 bytes" and format_size(82944) == "82.94 KB" and format_size(math.inf) == "infinity"
    with pytest.raises(ValueError):
        parse_size("12 parsecs")


def test_msccl_init(capsys):
    msccl.init('not_a_machine_type', 4, ('alltoall', 0))
    out, _ = capsys.readouterr()
    assert 'No plan found' in out
    assert 'MSCCL_CONFIG' not in os.environ
    assert 'NCCL_ALGO' not in os.environ

    msccl.init('mi355x', 2, ('alltoall', '1MB'))
    out, _ = capsys.readouterr()
    assert 'mi355x_alltoall_allpairs' in out
    assert 'MSCCL_CONFIG' in os.environ
    assert 'NCCL_IB_AR_THRESHOLD' not in os.environ
    assert os.environ['NCCL_ALGO'] == 'MSCCL,RING,TREE'

    os.environ['NCCL_ALGO'] = 'RING,FAKE_MSCCL'
    msccl.init('ndv4', 8, (msccl.Collective.alltoall, '2MB'))
    out, _ = capsys.readouterr()
    assert 'ndv4_alltoall' in out
    assert 'NCCL_IB_AR_THRESHOLD' in os.environ
    assert os.environ['NCCL_ALGO'] == 'MSCCL,RING,FAKE_MSCCL'

    os.environ['NCCL_ALGO'] = 'HELLO,MSCCL,WORLD'
    msccl.init('ndv4', 16, (msccl.Collective.alltoall, '35MB'))
    out, _ = capsys.readouterr()
    assert 'ndv4_alltoall' in out
    assert os.environ['NCCL_ALGO'] == 'HELLO,MSCCL,WORLD'


def test_register_plan():
    @register_synthesis_plan('allgather', 'fancy_machine', sizes=(0, '4MB'))
    def dummy_plan(m):
        return "<algo/>"

    @register_synthesis_plan('allgather', ['m1', 'm2'], sizes=('1GiB', None))
    def dummy_plan2(m):
        return "<algo/>"
    assert synthesis_plans[('allgather', 'fancy_machine')][-1][3] == (0, 4 * 10 ** 6)
    assert synthesis_plans[('allgather', 'm1')][-1][3] == (2 ** 30, math.inf)
    assert synthesis_plans[('allgather', 'm2')][-1][0] == 'call dummy_plan2'


def test_registered_ndv4_allreduce(capsys):
    msccl.init('ndv4', 1, (msccl.Collective.allreduce, (512, 1024)))
    assert 'ndv4_allpairs_allreduce_config1 with LL protocol' in capsys.readouterr().out
    msccl.init('ndv4', 1, (msccl.Collective.allreduce, (82944, 458752)))
    assert 'ndv4_allpairs_allreduce_config2 with LL protocol' in capsys.readouterr().out
    msccl.init('ndv4', 1, (msccl.Collective.allreduce, (458752, 2129920)))
    assert 'ndv4_ring_allreduce_config1 with LL protocol' in capsys.readouterr().out
    msccl.init('ndv4', 1, (msccl.Collective.allreduce, (2129920, 22806528)))
    assert 'ndv4_ring_allreduce_config2 with LL128 protocol' in capsys.readouterr().out


def test_registered_ndv4_alltoall(capsys):
    msccl.init('ndv4', 8, (msccl.Collective.alltoall, ('1MB', '32MB')))
    assert 'ndv4_alltoall_hierarchical_config1 with LL128 protocol' in capsys.readouterr().out
    msccl.init('ndv4', 8, (msccl.Collective.alltoall, ('32MB', '64MB')))
    assert 'ndv4_alltoall_hierarchical_config2 with Simple protocol' in capsys.readouterr().out


def test_interval_selection_by_priority(capsys):
    plan_a, plan_b = (lambda m: "a"), (lambda m: "b")
    cands = [("A", plan_a, lambda m: True, (0, 1000), "Simple", 0),
             ("B", plan_b, lambda m: True, (500, 2000), "LL", 1),
             ("C", plan_a, lambda m: m == 99, (0, math.inf), "Simple", 5)]
    res = _select_plans("allreduce", cands, 1, (0, 3000))
    assert [(p, v) for p, v in res] == [(plan_a, [0, 500, "Simple"]), (plan_b, [500, 1000, "LL"]), (plan_b, [1000, 2000, "LL"])]
    out = capsys.readouterr().out
    assert "No plan found for allreduce with sizes from 2 KB to infinity" in out


def test_index_roundtrip_and_selection(capsys):
    msccl.init('ndv4', 1, (msccl.Collective.allreduce, (512, 3000000)))
    capsys.readouterr()
    algos = load_config()
    assert [(a.min_bytes, a.max_bytes, a.proto) for a in algos] == [(512, 82944, 'LL'), (82944, 458752, 'LL'), (458752, 2129920, 'LL'),
                                                                   (2129920, 22806528, 'LL128')]
    assert all(a.tables.coll == "allreduce" and a.tables.ngpus == 8 for a in algos)
    assert select(algos, "allreduce", 1024) is algos[0]
    assert select(algos, "allreduce", 1 << 20) is algos[2]
    assert select(algos, "allreduce", 100) is None
    assert select(algos, "alltoall", 1024) is None
    # ring all-reduce, 8 chunks x 8 instances
    assert algos[2].tables.nchunksperloop == 64 and algos[2].bytes_per_rank_to_chunk_bytes(1 << 20) == (1 << 20) // 64


def test_selection_windows_are_half_open(capsys):
    """A size on the boundary two plans share belongs to the upper one: windows are [minBytes, maxBytes),
    the interval convention of msccl.init (msccl/autosynth/__init__.py:57-68,130-131)."""
    msccl.init('mi355x', 1, ('allreduce', (0, None)))
    capsys.readouterr()
    algos = load_config()
    windows = [(a.min_bytes, a.max_bytes, a.tables.nchunksperloop) for a in algos]
    assert windows == [(0, 16000000, 64), (16000000, float("inf"), 32)]       # all-pairs below 16 MB, the ring from there on
    assert select(algos, "allreduce", 15999999) is algos[0]
    assert select(algos, "allreduce", 16000000) is algos[1]
    # msccl.init treats a requested size the same way: exactly 16 MB asks for [16000000, 16000001), which only the ring's window meets
    msccl.init('mi355x', 1, ('allreduce', 16000000))
    capsys.readouterr()
    assert [(a.min_bytes, a.max_bytes, a.tables.nchunksperloop) for a in load_config()] == [(16000000, float("inf"), 32)]
    msccl.init('mi355x', 1, ('allreduce', 15999999))
    capsys.readouterr()
    assert [(a.min_bytes, a.max_bytes, a.tables.nchunksperloop) for a in load_config()] == [(0, 16000000, 64)]


def test_mi355x_allgather_windows(capsys):
    """All-pairs all-gather (one hand-off deep) below 12 MB per rank, the ring (4 instances) from there on."""
    msccl.init('mi355x', 1, ('allgather', (0, None)))
    capsys.readouterr()
    algos = load_config()
    assert [(a.min_bytes, a.max_bytes, a.tables.name) for a in algos] == [(0, 12000000, 'mi355x_allpairs_allgather'),
                                                                          (12000000, float("inf"), 'mi355x_ring_allgather')]
    small, large = algos
    assert small.tables.ntbs == 8 * 7 and small.tables.nops == 8 * 14 and small.tables.nchunksperloop == 8   # a threadblock per peer: one send, one receive
    assert large.tables.nchunksperloop == 32                                              # 8 chunks x 4 instances
    assert select(algos, "allgather", 1 << 20) is small and select(algos, "allgather", 64 << 20) is large
    # two groups: the same two programs over all 16 ranks
    msccl.init('mi355x', 2, ('allgather', (0, None)))
    capsys.readouterr()
    small, large = load_config()
    assert (small.tables.name, small.tables.ngpus, small.tables.ntbs) == ('mi355x_allpairs_allgather', 16, 16 * 15)
    assert (large.tables.name, large.tables.ngpus, large.tables.nchunksperloop) == ('mi355x_ring_allgather', 16, 64)
    # eight groups: 63 messages into every rank -- the ring from 160 KiB per rank on
    msccl.init('mi355x', 8, ('allgather', (0, None)))
    capsys.readouterr()
    small, large = load_config()
    assert (small.max_bytes, small.tables.name, small.tables.ngpus) == (160 << 10, 'mi355x_allpairs_allgather_8x8', 64)
    assert (large.min_bytes, large.tables.name, large.tables.ngpus) == (160 << 10, 'mi355x_ring_allgather_8x8', 64)


def test_mi355x_alltoall_plans(capsys):
    """The one-step all-to-all for any number of groups of 8 virtual ranks (between ranks of one GPU the hierarchical
    program's gathering step is a second pass over the data); the ndv4 machine type keeps msccl-tools' hierarchical plans."""
    msccl.init('mi355x', 1, ('alltoall', '1MB'))
    assert 'mi355x_alltoall_allpairs' in capsys.readouterr().out
    (a,) = load_config()
    assert a.tables.coll == "alltoall" and a.tables.ngpus == 8 and not a.tables.inplace
    assert a.tables.nops == 2 * 8 * 7 + 8      # a send and a receive for every pair, and every rank's copy of its own chunk
    msccl.init('mi355x', 2, ('alltoall', '1MB'))
    assert 'mi355x_alltoall_allpairs' in capsys.readouterr().out
    (a,) = load_config()
    assert a.tables.ngpus == 16 and a.tables.nops == 2 * 16 * 15 + 16
    msccl.init('ndv4', 8, ('alltoall', '2MB'))
    assert 'ndv4_alltoall_hierarchical' in capsys.readouterr().out


def test_mi355x_allreduce_windows_of_two_and_four_groups(capsys):
    """16 and 32 virtual ranks: all-pairs over all ranks from 4 KiB to 16 MiB per rank (16 ranks; one ring over all ranks
    above) or from 256 KiB to 8 MiB (32 ranks; the two-level program above), all-pairs inside the groups and across them
    below -- 16 or 32 chunks, so it also serves what is too small for the 256 or 1024 chunks of all-pairs over all ranks."""
    for groups, windows, chunks in ((2, [(0, 4 << 10, 'allpairs_two_level'), (4 << 10, 16 << 20, 'allpairs'), (16 << 20, float("inf"), 'ring')], 256),
                                    (4, [(0, 256 << 10, 'allpairs_two_level'), (256 << 10, 8 << 20, 'allpairs'), (8 << 20, float("inf"), 'two_level')], 1024)):
        msccl.init('mi355x', groups, ('allreduce', (0, None)))
        capsys.readouterr()
        algos = load_config()
        assert [(a.min_bytes, a.max_bytes, a.tables.name) for a in algos] == [(lo, hi, f'mi355x_{kind}_allreduce_{groups}x8') for lo, hi, kind in windows]
        mid = select(algos, "allreduce", 1 << 20)
        assert mid.tables.ngpus == 8 * groups and mid.tables.nchunksperloop == chunks and mid.tables.inplace
        assert select(algos, "allreduce", 64 << 20).tables.name == f'mi355x_{windows[-1][2]}_allreduce_{groups}x8'
        small = select(algos, "allreduce", 1 << 10)
        assert small.tables.nchunksperloop == 8 * groups and small.tables.rank_chunks[0].tolist() == [8 * groups, 0, 7 * groups + groups - 1]


def test_mi355x_allreduce_windows_of_eight_groups(capsys):
    """64 virtual ranks: all-pairs inside the groups and across them (seven moving steps deep) below 6 MiB per rank, the
    two-level program (28 hand-offs deep, two instances) up to 12 MiB, one ring over all ranks (126 deep) from there on."""
    msccl.init('mi355x', 8, ('allreduce', (0, None)))
    capsys.readouterr()
    algos = load_config()
    assert [(a.min_bytes, a.max_bytes, a.tables.name, a.tables.nchunksperloop) for a in algos] == [
        (0, 6 << 20, 'mi355x_allpairs_two_level_allreduce_8x8', 64), (6 << 20, 12 << 20, 'mi355x_two_level_allreduce_8x8', 128),
        (12 << 20, float("inf"), 'mi355x_ring_allreduce_8x8', 64)]
    assert all(a.tables.ngpus == 64 for a in algos)
    assert select(algos, "allreduce", 256 << 10) is algos[0]


def test_mi355x_reduce_scatter_plans(capsys):
    """Reduce-scatter, in place: all-pairs through scratch below 12 MB per rank (10 MiB on 64 ranks), the ring from there on;
    registered through msccl-tools' own decorator (msccl/autosynth/registry.py:65-99, collective 'reduce_scatter')."""
    from msccl.autosynth.registry import synthesis_plans
    windows = sorted((low, high) for _, _, machines, (low, high), _, _ in synthesis_plans[('reduce_scatter', 'mi355x')] if machines(8))
    assert windows == [(0, 10 << 20), (10 << 20, float("inf"))]      # (64 ranks: listed, not compiled here -- 4096 chunks a rank)
    for groups, switch in ((1, 12 * 10 ** 6), (2, 12 * 10 ** 6)):
        n = 8 * groups
        msccl.init('mi355x', groups, (msccl.Collective.reduce_scatter, (0, None)))
        out = capsys.readouterr().out
        assert 'mi355x_allpairs_reduce_scatter' in out and 'mi355x_ring_reduce_scatter' in out
        small, large = load_config()
        assert (small.min_bytes, small.max_bytes, small.tables.name) == (0, switch, 'mi355x_allpairs_reduce_scatter')
        assert (large.min_bytes, large.max_bytes, large.tables.name) == (switch, float("inf"), 'mi355x_ring_reduce_scatter')
        for a, chunks, scratch in ((small, n * n, n * (n - 1)), (large, n, 0)):
            assert a.tables.coll == "reduce_scatter" and a.tables.inplace and a.tables.ngpus == n
            assert a.tables.rank_chunks[0].tolist() == [chunks, 0, scratch]
        assert select(load_config(), "reduce_scatter", 1 << 20) is not None


def test_ef_file_plan(tmp_path, capsys):
    import ir_samples
    f = tmp_path / "ring.xml"
    f.write_text(ir_samples.ring_allgather_xml(4))
    register_ef_file(str(f), 'allgather', 'testbox', 1, sizes=('1KB', '1MB'))
    msccl.init('testbox', 1, ('allgather', '64KB'))
    assert f'load {f}' in capsys.readouterr().out
    a = select(load_config(), "allgather", 65536)
    assert a.path == str(f) and a.tables.ngpus == 4 and (a.min_bytes, a.max_bytes) == (1000, 10 ** 6)
