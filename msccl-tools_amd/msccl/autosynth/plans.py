"""Registered plans.  `ndv4`: the MSCCLang plans of msccl-tools' msccl/autosynth/ndv4_plans.py:12-48
(same programs, replication, protocols and size windows).  `mi355x`: plans for algorithms whose ranks
are all virtual ranks of one MI355X (machines = groups of 8 virtual ranks)."""
from msccl.autosynth.registry import register_msccl_program
from msccl.language.ir import ThreadblockPolicy
from msccl.programs.allgather_allpairs import allgather_allpairs
from msccl.programs.allgather_ring import allgather_ring
from msccl.programs.allreduce_a100_ring import allreduce_ring
from msccl.programs.allreduce_allpairs import allreduce_allpairs
from msccl.programs.allreduce_allpairs_two_level import allreduce_allpairs_two_level
from msccl.programs.reducescatter_allpairs import reducescatter_allpairs
from msccl.programs.reducescatter_ring import reducescatter_ring
from msccl.programs.alltoall_a100_8kp1 import alltoall_three_step
from msccl.programs.alltoall_allpairs import alltoall_allpairs
from msccl.programs.alltoall_a100_yifan import alltoall_hierarchical
from msccl.programs.hierarchical_allreduce import hierarchical_allreduce
from msccl.topologies import fully_connected


def register_ndv4_plans():
    one = lambda x: x == 1
    manual = ThreadblockPolicy.manual

    @register_msccl_program(fully_connected(8), 'allreduce', 'ndv4', chunk_factor=64, inplace=True, instances=2, protocol='LL',
                            sizes=('512B', '82944B'), threadblock_policy=manual, interleaved_replication=False,
                            dependence_nop=True, machines=one)
    def ndv4_allpairs_allreduce_config1(prog, nodes):
        allreduce_allpairs(8)

    @register_msccl_program(fully_connected(8), 'allreduce', 'ndv4', chunk_factor=64, inplace=True, instances=4, protocol='LL',
                            sizes=('82944B', '458752B'), threadblock_policy=manual, interleaved_replication=False,
                            dependence_nop=True, machines=one)
    def ndv4_allpairs_allreduce_config2(prog, nodes):
        allreduce_allpairs(8)

    @register_msccl_program(fully_connected(8), 'allreduce', 'ndv4', chunk_factor=8, inplace=True, instances=8, protocol='LL',
                            sizes=('458752B', '2129920B'), threadblock_policy=manual, machines=one)
    def ndv4_ring_allreduce_config1(prog, nodes):
        allreduce_ring(size=8, channels=4)

    @register_msccl_program(fully_connected(8), 'allreduce', 'ndv4', chunk_factor=8, inplace=True, instances=8, protocol='LL128',
                            sizes=('2129920B', '22806528B'), threadblock_policy=manual, machines=one)
    def ndv4_ring_allreduce_config2(prog, nodes):
        allreduce_ring(size=8, channels=4)

    @register_msccl_program(fully_connected(8), 'alltoall', 'ndv4', protocol='LL128', sizes=('1MB', '32MB'),
                            machines=lambda x: x in (8, 16, 32, 64))
    def ndv4_alltoall_hierarchical_config1(prog, nodes):
        alltoall_hierarchical(num_nodes=nodes, gpus_per_node=8)

    @register_msccl_program(fully_connected(8), 'alltoall', 'ndv4', protocol='Simple', sizes=('32MB', None),
                            machines=lambda x: x in (8, 16, 32))
    def ndv4_alltoall_hierarchical_config2(prog, nodes):
        alltoall_hierarchical(num_nodes=nodes, gpus_per_node=8)

    @register_msccl_program(fully_connected(8), 'alltoall', 'ndv4', protocol='Simple', sizes=('32MB', None), machines=lambda x: x == 64)
    def ndv4_alltoall_three_step(prog, nodes):
        alltoall_three_step(num_nodes=nodes, gpus_per_node=8)

    @register_msccl_program(fully_connected(8), 'alltoall', 'ndv4', protocol='Simple', sizes=('1KB', None), machines=lambda x: x in (2, 4))
    def ndv4_alltoall_hierarchical_config2(prog, nodes):  # noqa: F811 -- same name, other machine counts, as upstream
        alltoall_hierarchical(num_nodes=nodes, gpus_per_node=8)


def register_mi355x_plans():
    """Virtual-rank plans: `machines` counts groups of 8 virtual ranks held in one GPU's HBM."""
    one = lambda x: x == 1
    manual = ThreadblockPolicy.manual

    # Measured on MI355X, 8 virtual ranks, fp32 (microseconds, all-pairs / ring): 4 KiB to 512 KiB per
    # rank 17-18 / 25-26, 1 MiB 19 / 32, 2 MiB 24 / 35, 4 MiB 37 / 45, 8 MiB 54 / 63, 16 MiB 96 / 101,
    # 32 MiB 214 / 183, 64 MiB 372 / 348, 256 MiB 1774 / 1375.  All-pairs is three hand-offs deep, the ring fourteen; the ring moves
    # 5(n-1)/n chunks per chunk reduced, all-pairs about 4(n-1)/n + 2 on this executor.
    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=64, inplace=True, instances=1,
                            sizes=(0, '16MB'), threadblock_policy=manual, interleaved_replication=False,
                            dependence_nop=True, machines=one)
    def mi355x_allpairs_allreduce(prog, nodes):
        allreduce_allpairs(8)

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=8, inplace=True, instances=4,
                            sizes=('16MB', None), threadblock_policy=manual, machines=one)
    def mi355x_ring_allreduce_large(prog, nodes):
        allreduce_ring(size=8, channels=1)

    # All-gather, int32, microseconds by bytes per rank (all-pairs / ring x 4 instances): 1 MiB 18 / 31, 2 MB 26 / 51,
    # 4 MiB 67 / 78, 8 MiB 136 / 144, 12 MB 215 / 212, 16 MiB 287 / 276, 32 MB 570 / 529.  Both move the same bytes; all-pairs
    # is one hand-off deep, the ring seven, and the ring's pieces stream better at the large end.
    # Two and four groups, all 16 or 32 ranks in one all-pairs program or one ring, the same way -- 16 ranks: 64 KiB per rank
    # 12 / 33, 1 MiB 50 / 82, 4 MiB 271 / 294, 8 MiB 565 / 579, 16 MiB 1152 / 1150; 32 ranks: 64 KiB 19 / 70, 1 MiB 297 / 299,
    # 4 MiB 1145 / 1183, 8 MiB 2343 / 2359, 16 MiB 5038 / 4705.
    @register_msccl_program(fully_connected(8), 'allgather', 'mi355x', chunk_factor=1, inplace=True, instances=1,
                            sizes=(0, '12MB'), threadblock_policy=manual, machines=lambda x: x in (1, 2, 4))
    def mi355x_allpairs_allgather(prog, nodes):
        allgather_allpairs(8 * nodes)

    @register_msccl_program(fully_connected(8), 'allgather', 'mi355x', chunk_factor=1, inplace=True, instances=4,
                            sizes=('12MB', None), threadblock_policy=manual, machines=lambda x: x in (1, 2, 4))
    def mi355x_ring_allgather(prog, nodes):
        allgather_ring(size=8 * nodes, channels=1)

    # Eight groups (64 ranks, 63 messages into every rank): all-pairs / ring, 16 KiB per rank 20 / 114, 64 KiB 95 / 175,
    # 128 KiB 174 / 192, 192 KiB 256 / 244, 1 MiB 1251 / 1207, 4 MiB 5348 / 4769.
    @register_msccl_program(fully_connected(8), 'allgather', 'mi355x', chunk_factor=1, inplace=True, instances=1,
                            sizes=(0, '160KiB'), threadblock_policy=manual, machines=lambda x: x == 8)
    def mi355x_allpairs_allgather_8x8(prog, nodes):
        allgather_allpairs(64)

    @register_msccl_program(fully_connected(8), 'allgather', 'mi355x', chunk_factor=1, inplace=True, instances=1,
                            sizes=('160KiB', None), threadblock_policy=manual, machines=lambda x: x == 8)
    def mi355x_ring_allgather_8x8(prog, nodes):
        allgather_ring(size=64, channels=1)

    # The one-step all-to-all, every message read where its sender keeps it, for any number of groups: 8 ranks 8-10 us from
    # 8 KiB to 1 MiB per rank, 16 MiB 52 us, 64 MiB 204 us = 66 % of the HBM peak, 256 MiB 715 us = 75 % (instances make no
    # difference).  The hierarchical program gathers per destination group first, which pays on links between machines; between
    # virtual ranks of one GPU it is a second pass over the data.  uint8, microseconds, one-step / hierarchical -- 16 ranks:
    # 64 KiB per rank 9 / 15, 1 MiB 12 / 23, 16 MiB 116 / 135, 64 MiB 399 / 515; 32 ranks: 9 / 21, 19 / 38, 203 / 298, 793 / 1178;
    # 64 ranks: 12 / 38, 31 / 70, 407 / 720 (16 MiB).
    @register_msccl_program(fully_connected(8), 'alltoall', 'mi355x', machines=lambda x: 1 <= x <= 8)
    def mi355x_alltoall_allpairs(prog, nodes):
        alltoall_allpairs(8 * nodes)

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=16, inplace=True, instances=2,
                            interleaved_replication=False, machines=lambda x: x == 2)
    def mi355x_two_level_allreduce_2x8(prog, nodes):
        hierarchical_allreduce(8, 2, "auto")

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=32, inplace=True, instances=2,
                            interleaved_replication=False, machines=lambda x: x == 4)
    def mi355x_two_level_allreduce_4x8(prog, nodes):
        hierarchical_allreduce(8, 4, "auto")

    # All-pairs over all 16 or 32 ranks up to the sizes at which the two-level program's fewer and longer messages win; below
    # 4 / 16 KiB per rank its 256 / 1024 chunks would be smaller than an element.  fp32, microseconds, all-pairs / two-level --
    # 16 ranks: 16 KiB per rank 21 / 26, 1 MiB 28 / 47, 4 MiB 62 / 82, 16 MiB 202 / 228, 24 MiB 336 / 338, 32 MiB 427 / 420;
    # 32 ranks: 16 KiB 31 / 33, 64 KiB 30 / 35, 256 KiB 35 / 51, 1 MiB 42 / 70, 4 MiB 114 / 137, 6 MiB 174 / 180, 8 MiB 223 / 227,
    # 16 MiB 450 / 417.
    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=256, inplace=True, instances=1,
                            sizes=('4KiB', '16MiB'), threadblock_policy=manual, interleaved_replication=False,
                            dependence_nop=True, machines=lambda x: x == 2, priority=1)
    def mi355x_allpairs_allreduce_2x8(prog, nodes):
        allreduce_allpairs(16)

    # Eight groups (64 ranks), fp32, microseconds, all-pairs inside the groups and across them (seven moving steps deep) /
    # two-level program x 2 instances (28 hand-offs deep) / one ring over all ranks (126 deep): 16 KiB per rank 30 / 66 / 170,
    # 64 KiB 31 / 67 / 169, 256 KiB 42 / 73 / 172, 1 MiB 77 / 106 / 256, 2 MiB 123 / 159 / 299, 4 MiB 239 / 258 / 361,
    # 8 MiB 457 / 419 / 486, 12 MiB 746 / 604 / 628, 16 MiB 1025 / 794 / 767, 32 MiB 2092 / 1600 / 1524.  (One instance of the
    # two-level program on flag-in-data lines, the plan for the small sizes before: 47-49 us up to 64 KiB.)
    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=64, inplace=True, instances=1,
                            sizes=(0, '6MiB'), threadblock_policy=manual, dependence_nop=True, machines=lambda x: x == 8)
    def mi355x_allpairs_two_level_allreduce_8x8(prog, nodes):
        allreduce_allpairs_two_level(8, 8)

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=64, inplace=True, instances=2,
                            sizes=('6MiB', '12MiB'), interleaved_replication=False, machines=lambda x: x == 8)
    def mi355x_two_level_allreduce_8x8(prog, nodes):
        hierarchical_allreduce(8, 8, "auto")

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=64, inplace=True, instances=1,
                            sizes=('12MiB', None), threadblock_policy=manual, machines=lambda x: x == 8)
    def mi355x_ring_allreduce_8x8(prog, nodes):
        allreduce_ring(size=64, channels=1)

    # 16 ranks, large messages: one ring over all ranks (4 instances) against the two-level program, 16 MiB per rank 194 / 212,
    # 32 MiB 377 / 412, 128 MiB 1403 / 1498 (all-pairs: 202, 427).  On 32 ranks the two are level (128 MiB 2890 / 2917, 8 MiB 235 / 219).
    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=16, inplace=True, instances=4,
                            sizes=('16MiB', None), threadblock_policy=manual, machines=lambda x: x == 2, priority=1)
    def mi355x_ring_allreduce_2x8(prog, nodes):
        allreduce_ring(size=16, channels=1)

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=1024, inplace=True, instances=1,
                            sizes=('256KiB', '8MiB'), threadblock_policy=manual, interleaved_replication=False,
                            dependence_nop=True, machines=lambda x: x == 4, priority=1)
    def mi355x_allpairs_allreduce_4x8(prog, nodes):
        allreduce_allpairs(32)

    # Below that, all-pairs inside the groups and across them: 16 or 32 chunks where all-pairs over all ranks has 256 or 1024, so
    # it also serves the sizes at which those would be smaller than an element.  fp32, microseconds, this / all-pairs over all
    # ranks / two-level -- 32 ranks: 16 KiB per rank 26 / 31 / 34, 64 KiB 26 / 29 / 35, 256 KiB 30 / 30 / 49, 1 MiB 51 / 41 / 69;
    # 16 ranks: 4 KiB 24 / 22 / 26, 64 KiB 24 / 21 / 28 (all-pairs over all 16 ranks stays ahead wherever its chunks hold an element).
    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=32, inplace=True, instances=1,
                            sizes=(0, '256KiB'), threadblock_policy=manual, dependence_nop=True, machines=lambda x: x == 4, priority=1)
    def mi355x_allpairs_two_level_allreduce_4x8(prog, nodes):
        allreduce_allpairs_two_level(4, 8)

    @register_msccl_program(fully_connected(8), 'allreduce', 'mi355x', chunk_factor=16, inplace=True, instances=1,
                            sizes=(0, '4KiB'), threadblock_policy=manual, dependence_nop=True, machines=lambda x: x == 2, priority=1)
    def mi355x_allpairs_two_level_allreduce_2x8(prog, nodes):
        allreduce_allpairs_two_level(2, 8)

    # Reduce-scatter in place (rank r's result is its own input chunks [r * cf, (r + 1) * cf)): all-pairs through scratch, one
    # hand-off and one fold deep, below about 12 MB per rank, the ring from there on.  fp32, microseconds, all-pairs / ring --
    # 8 ranks: 8 KiB per rank 13 / 16, 1 MiB 15 / 19, 4 MiB 26 / 28, 8 MiB 37 / 42, 16 MiB 68 / 64, 64 MiB 246 / 209, 256 MiB 1099 / 825;
    # 16 ranks: 64 KiB 14 / 27, 4 MiB 40 / 61, 8 MiB 67 / 77, 16 MiB 132 / 123, 64 MiB 574 / 439; 32 ranks: 64 KiB 20 / 48, 4 MiB 67 / 119,
    # 8 MiB 134 / 152, 16 MiB 288 / 243; 64 ranks: 64 KiB 44 / 90, 4 MiB 130 / 238, 8 MiB 290 / 304, 16 MiB 615 / 499.
    def reduce_scatter_plans(groups, switch):
        n = 8 * groups

        @register_msccl_program(fully_connected(8), 'reduce_scatter', 'mi355x', chunk_factor=n, inplace=True, instances=1,
                                sizes=(0, switch), threadblock_policy=manual, dependence_nop=True, machines=lambda x: x == groups)
        def mi355x_allpairs_reduce_scatter(prog, nodes):
            reducescatter_allpairs(n)

        @register_msccl_program(fully_connected(8), 'reduce_scatter', 'mi355x', chunk_factor=1, inplace=True, instances=1,
                                sizes=(switch, None), threadblock_policy=manual, machines=lambda x: x == groups)
        def mi355x_ring_reduce_scatter(prog, nodes):
            reducescatter_ring(size=n, channels=1)

    for groups, switch in ((1, '12MB'), (2, '12MB'), (4, '12MB'), (8, '10MiB')):
        reduce_scatter_plans(groups, switch)
