"""`msccl.init`: pick plans for (machine type, machine count, collective, size range), compile them
to MSCCL-IR XML files, write the `<msccl_algos>` index and export MSCCL_CONFIG / NCCL_ALGO.

Behaviour follows msccl-tools' msccl/autosynth/__init__.py: size parsing (:50-68), interval
splitting and highest-priority choice per interval with the same log lines (:126-176), the index file
(:75-94) and the environment variables (:96-114).  SKU auto-detection needs nvidia-smi and is not
offered; name the machine type.  `msccl.executor.config` reads the index back on the MI355X side.
"""
import enum
import math
import os
import tempfile
import xml.etree.ElementTree as ET

from msccl.autosynth.plans import register_mi355x_plans, register_ndv4_plans
from msccl.autosynth.registry import synthesis_plans
from msccl.autosynth.sizes import format_size as _format_size
from msccl.autosynth.sizes import parse_size

register_ndv4_plans()
register_mi355x_plans()


class Collective(enum.Enum):
    allreduce = 'allreduce'
    allgather = 'allgather'
    reduce = 'reduce'
    broadcast = 'broadcast'
    alltoall = 'alltoall'
    reduce_scatter = 'reduce_scatter'

    def __str__(self):
        return self.value


def _requested_range(sizes):
    if isinstance(sizes, tuple):
        low, high = sizes
        low = parse_size(low) if isinstance(low, str) else low
        high = math.inf if high is None else parse_size(high) if isinstance(high, str) else high
        return (low, high)
    size = parse_size(sizes) if isinstance(sizes, str) else sizes
    return (size, size + 1)


def init(machine_type, num_machines, *collectives):
    if machine_type == "auto":
        print('Did not recognize the SKU type automatically. If you are sure about the SKU, try replacing "auto" with your '
              'explicit SKU name. Falling back to NCCL.')
        return
    selected = {}
    for name, sizes in collectives:
        name = str(name)
        plans = _select_plans(name, synthesis_plans[(name, machine_type)], num_machines, _requested_range(sizes))
        if plans:
            selected[name] = plans

    root = ET.Element('msccl_algos')
    for plans in selected.values():
        for plan, (low, high, proto) in plans:
            load = ET.SubElement(root, 'load')
            load.set('path', plan(num_machines))
            if low != 0:
                load.set('minBytes', str(low))
            if high != math.inf:
                load.set('maxBytes', str(high))
            load.set('proto', proto)
    if len(root) == 0:
        print('MSCCL: No algorithms were selected.')
        return
    ET.indent(root, space='  ')
    fd, path = tempfile.mkstemp(suffix=".xml")
    with os.fdopen(fd, 'w') as f:
        f.write(ET.tostring(root, encoding='unicode').replace(" />", "/>"))
    env = {'MSCCL_CONFIG': path}
    existing = os.environ.get('NCCL_ALGO', '')
    if existing:
        if 'MSCCL' not in existing.split(','):
            os.environ['NCCL_ALGO'] = 'MSCCL,' + existing
    else:
        env['NCCL_ALGO'] = 'MSCCL,RING,TREE'
    if machine_type == 'ndv4' and num_machines >= 8 and 'alltoall' in selected:
        print('MSCCL: Setting NCCL_IB_AR_THRESHOLD=0 (reason: alltoall and at least 16 ndv4 machines)')
        env['NCCL_IB_AR_THRESHOLD'] = '0'
    if machine_type == 'ndv4':
        print('MSCCL: Setting relaxed orderin, topo file and visible devices order')
        env['NCCL_IB_PCI_RELAXED_ORDERING'] = '1'
        env['NCCL_TOPO_FILE'] = '/opt/msft/topo.xml'
        env['CUDA_VISIBLE_DEVICES'] = '0,1,2,3,4,5,6,7'
    os.environ.update(env)


def _select_plans(name, candidates, num_machines, sizes):
    """Cut [0, inf) at every candidate's bounds; in each resulting interval that overlaps the request
    the candidate with the highest priority wins (the later registration on ties); neighbouring
    intervals won by the same plan and protocol are merged when they abut by one byte."""
    usable = [c for c in candidates if c[2](num_machines) and not (c[3][0] >= sizes[1] or sizes[0] >= c[3][1])]
    cuts = sorted({0, math.inf} | {b for c in usable for b in c[3]})
    results = []
    for low, high in zip(cuts, cuts[1:]):
        if low >= sizes[1] or sizes[0] >= high:
            continue
        covering = [c for c in usable if c[3][0] <= low and high <= c[3][1]]
        description = f'{name} with sizes from {_format_size(low)} to {_format_size(high)}'
        if not covering:
            print(f'MSCCL: No plan found for {description}. Falling back to NCCL baseline.')
            continue
        desc, plan, _, _, proto, _ = sorted(covering, key=lambda c: c[5])[-1]
        print(f'MSCCL: Plan for {description} is {desc} with {proto} protocol.')
        if results and plan == results[-1][0] and low == results[-1][1][1] + 1 and proto == results[-1][1][2]:
            results[-1][1][1] = high
        else:
            results.append((plan, [low, high, proto]))
    return results


def _describe_machines(machines, limit=2048):
    ranges, start = [], None
    for i in range(limit):
        if machines(i):
            start = i if start is None else start
        elif start is not None:
            ranges.append(str(start) if start == i - 1 else f'{start}-{i - 1}')
            start = None
    if start is not None:
        ranges.append(f'>={start}')
    return ','.join(ranges) if ranges else '???'


def _list_plan_parameters():
    headers = ['Machine', 'Collective', '# machines', 'From', 'To', 'Protocol', 'Priority', 'Plan name']
    rows = []
    for (collective, machine_type), plans in synthesis_plans.items():
        for name, _, machines, (low, high), protocol, priority in plans:
            rows.append(((machine_type, collective, low, high, protocol, priority, name),
                         (machine_type, collective, _describe_machines(machines), _format_size(low), _format_size(high), protocol,
                          priority, name)))
    return headers, [cols for _, cols in sorted(rows, key=lambda r: r[0])]


def tabulate_plans():
    from tabulate import tabulate
    headers, rows = _list_plan_parameters()
    return tabulate(rows, headers=headers, tablefmt='github')


def print_plans():
    print(tabulate_plans())
