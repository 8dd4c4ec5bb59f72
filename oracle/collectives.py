"""Closed forms of the collectives and buffer placement rules.  TEST INFRASTRUCTURE ONLY.

These are the expected results the reference's symbolic checkers assert, restated on numbers:

* all-gather:  out_r[i*cf + c] = in_i[c]                  msccl/language/collectives.py:92-107
* all-to-all:  out_r[i*cf + c] = in_i[r*cf + c]           msccl/language/collectives.py:47-60
* all-reduce:  out_r[c] = (+)_i in_i[c]                    msccl/language/collectives.py:144-163
* reduce-scatter: out_r[c] = (+)_i in_i[r*cf + c]          msccl/language/collectives.py:198-218

and the aliasing rules of in-place collectives (where the input lives inside the buffer the XML
names): all-reduce in place => every reference is 'i' (collectives.py:165-169); all-gather in
place => every reference is 'o' and rank r's input is output chunks [r*cf, (r+1)*cf)
(collectives.py:110-115); reduce-scatter in place => output of rank r is input chunks
[r*cf, (r+1)*cf) (collectives.py:220-225).

Floating-point sums are not associative, so the all-reduce closed form takes the fold order as
an argument: `fold_orders[c]` lists, for chunk c, a nested order description (see `fold`).
"""
from __future__ import annotations

import numpy as np

from .ir_interp import _reduce, DTYPES


def place_inputs(algo, inputs, chunk_elems, dtype):
    """Build the per-rank {'i','o','s'} buffers the XML addresses, with `inputs` where the
    collective's aliasing rule puts them.  inputs[r] is rank r's 1-D send buffer."""
    npdt = DTYPES[dtype]
    bufs = []
    n = algo.ngpus
    for g in algo.gpus:
        b = {"i": np.zeros(g.i_chunks * chunk_elems, npdt),
             "o": np.zeros(g.o_chunks * chunk_elems, npdt),
             "s": np.zeros(g.s_chunks * chunk_elems, npdt)}
        x = np.asarray(inputs[g.id], dtype=npdt).ravel()
        if algo.coll == "allgather" and algo.inplace:
            per = g.o_chunks * chunk_elems // n
            assert x.size == per, (x.size, per)
            b["o"][g.id * per:(g.id + 1) * per] = x
        else:
            assert x.size <= b["i"].size, (x.size, b["i"].size)
            b["i"][:x.size] = x
        bufs.append(b)
    return bufs


def extract_outputs(algo, bufs, chunk_elems):
    """The receive buffer of every rank after the run."""
    outs = []
    n = algo.ngpus
    for g in algo.gpus:
        b = bufs[g.id]
        if algo.coll == "allreduce" and algo.inplace:
            outs.append(b["i"])
        elif algo.coll == "reduce_scatter" and algo.inplace:
            per = g.i_chunks * chunk_elems // n
            outs.append(b["i"][g.id * per:(g.id + 1) * per])
        elif algo.coll == "alltoall" and algo.inplace and g.o_chunks == 0:
            outs.append(b["i"])
        else:
            outs.append(b["o"])
    return outs


def expected_allgather(inputs):
    cat = np.concatenate([np.asarray(x).ravel() for x in inputs])
    return [cat.copy() for _ in inputs]


def expected_alltoall(inputs):
    n = len(inputs)
    blk = np.asarray(inputs[0]).size // n
    return [np.concatenate([np.asarray(inputs[i]).ravel()[r * blk:(r + 1) * blk] for i in range(n)])
            for r in range(n)]


def fold(order, operands, dtype, redop="sum"):
    """Evaluate a nested fold description.  `order` is an int (operand index) or a list whose
    elements are folded left to right: [a, b, c] = ((a (+) b) (+) c); elements may themselves be
    lists (sub-expressions evaluated first)."""
    if isinstance(order, (int, np.integer)):
        return operands[int(order)]
    acc = None
    for item in order:
        v = fold(item, operands, dtype, redop)
        acc = v if acc is None else _reduce(acc, v, dtype, redop)
    return acc


def expected_allreduce(inputs, nchunks, fold_orders, dtype, redop="sum"):
    """All-reduce with an explicit fold order per chunk index."""
    n = len(inputs)
    E = np.asarray(inputs[0]).size // nchunks
    res = np.empty_like(np.asarray(inputs[0]).ravel())
    for c in range(nchunks):
        ops = [np.asarray(inputs[i]).ravel()[c * E:(c + 1) * E] for i in range(n)]
        res[c * E:(c + 1) * E] = fold(fold_orders[c], ops, dtype, redop)
    return [res.copy() for _ in range(n)]


def ring_allreduce_orders(n, nchunks=None, instances=1):
    """Fold order of the ring program msccl/programs/allreduce_a100_ring.py:12-18: chunk `index`
    starts on rank `index` and accumulates ranks index, index+1, ... (mod n), left to right.
    With instance replication (interleaved, rank_dag.py:337-338) chunk index*inst+i follows chunk
    `index`'s order."""
    nchunks = n if nchunks is None else nchunks
    orders = []
    for index in range(nchunks):
        base = [(index + k) % n for k in range(n)]
        orders.extend([base] * instances)
    return orders


def two_level_allreduce_orders(num_local, num_nodes, instances=1):
    """Fold order of msccl-tools' examples/mscclang/hierarchical_allreduce.py:13-19,38-44 with
    num_local*num_nodes chunks: chunk q (b = q // num_nodes, j = q % num_nodes) is first summed
    inside every node over local gpus b+1, b+2, ..., b (mod num_local), left to right, then the node
    partials are summed over nodes j+1, j+2, ..., j (mod num_nodes), left to right.  Replication is
    batched (rank_dag.py:339-340): chunk len*i + q of instance i follows chunk q."""
    n = num_local * num_nodes
    orders = []
    for q in range(n):
        b, j = q // num_nodes, q % num_nodes
        nodes = [(j + 1 + m) % num_nodes for m in range(num_nodes)]
        orders.append([[node * num_local + (b + 1 + k) % num_local for k in range(num_local)] for node in nodes])
    return orders * instances


def allpairs_allreduce_orders(n, instances=1):
    """msccl-tools' msccl/programs/allreduce_allpairs.py:6-28 with n*n chunks: chunk r*n + lane is
    folded on rank r as own value, then the peers' copies in ascending peer order (the order in
    which they were appended to rank r's scratch).  Batched replication."""
    orders = []
    for c in range(n * n):
        r = c // n
        orders.append([r] + [p for p in range(n) if p != r])
    return orders * instances


def expected_reduce_scatter(inputs, chunks_per_rank, fold_orders, dtype, redop="sum"):
    """Reduce-scatter (msccl/language/collectives.py:198-218): out_r[c] = fold over ranks of in_i[r*cf + c],
    cf = chunks_per_rank, with an explicit fold order per input chunk index r*cf + c."""
    n = len(inputs)
    E = np.asarray(inputs[0]).size // (n * chunks_per_rank)
    outs = []
    for r in range(n):
        res = np.empty(chunks_per_rank * E, np.asarray(inputs[0]).dtype)
        for c in range(chunks_per_rank):
            k = r * chunks_per_rank + c
            ops = [np.asarray(inputs[i]).ravel()[k * E:(k + 1) * E] for i in range(n)]
            res[c * E:(c + 1) * E] = fold(fold_orders[k], ops, dtype, redop)
        outs.append(res)
    return outs


def ring_reduce_scatter_orders(n, instances=1):
    """Fold order of the ring reduce-scatter whose chunk k walks k+1 -> k+2 -> ... -> k: ranks k+1, k+2, ...,
    k (mod n), left to right.  Interleaved replication: chunk k*inst + i follows chunk k."""
    orders = []
    for k in range(n):
        orders.extend([[(k + 1 + m) % n for m in range(n)]] * instances)
    return orders
