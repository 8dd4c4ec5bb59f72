"""NumPy interpreter of MSCCL-IR XML.  TEST INFRASTRUCTURE, NOT A PRODUCT PATH.

This file is the correctness oracle and the CPU baseline for the HIP executor.  Only the
test-suite, the smoke check and the benchmark's CPU-baseline leg may import it; the executor
package never does.

What it restates.  msccl-tools has no executor of its own: the IR it emits is consumed by an
external runtime.  The meaning of the IR is nevertheless fixed by the compiler that emits it,
and every rule below cites the reference text that fixes it (paths relative to the
msccl-tools checkout):

* XML schema (element/attribute names, units, -1 sentinels):  msccl/language/ir.py:320-391,
  second emitter msccl/ncclize.py:658-718.
* Buffers 'i'/'o'/'s', extents in chunks:                     msccl/language/ir.py:86-92,213-224,330-335.
* copy:   dst[...] = src[...]                                 msccl/language/__init__.py:65-71.
* reduce: dst[...] = dst[...] (+) src[...]                    msccl/language/__init__.py:74-82.
* send / recv / rrc creation (what each instruction moves):   msccl/language/rank_dag.py:99-154.
* fused rcs / rrs / rrcs (recv's local target == forwarded location): rank_dag.py:209-251.
* For recv-type ops the LOCAL operand/target is (dstbuf, dstoff); for 's', 'cpy', 're' the local
  source is (srcbuf, srcoff):                                  ir.py:203-208 (_local_src_insts/_local_dst_insts).
* depid/deps/hasdep: wait until threadblock `depid` of the same rank has finished its step
  `deps`:                                                       ir.py:235-262,380-391.
* Connections are FIFOs per (sender rank, receiver rank, channel); sends and matching receives
  occur in the same order:                                      msccl/language/passes.py:31-55.
* ncclize documents: on 's' the destination and on 'r'/'rrc' the source name the OTHER rank's
  location (msccl/ncclize.py:532-535) and take no part in execution; a receive into a slot that
  already holds data is an 'rrc' (ncclize.py:390-400); copies sit in a threadblock of their own,
  which may be empty (ncclize.py:621-626).

Parity pinning.  The reference holds no execution vectors for this path (its tests are
symbolic), so this interpreter is pinned by what the mathematics fixes: closed forms of the
collectives (all-gather = concatenation, all-to-all = block transpose, all-reduce = the fold
order read off the program text), brute force on one-element chunks, schedule invariance under
random interleavings, and the hand-derived worked example of the reference's fusion test
(tests/test_language.py:188-202).  Those checks live in tests/test_oracle.py.

Arithmetic.  Reductions are element-wise in the buffer's dtype.  fp16 uses numpy's float16
arithmetic (correctly rounded = fp32 add followed by one round-to-nearest-even); bf16 is carried
as uint16 bit patterns and reduced by widening to fp32, operating, and rounding to nearest even.
"""
from __future__ import annotations

import collections
import random
import xml.etree.ElementTree as ET

import numpy as np

RECV_TYPES = ("r", "rcs", "rrs", "rrc", "rrcs")
SEND_TYPES = ("s", "rcs", "rrs", "rrcs")
# algorithmic HBM traffic per op, in units of cnt*chunk_bytes: one read + one write per transfer
# edge (booked at the receiver), plus one operand read per reduction.
ALGO_BYTES_FACTOR = {"s": 0, "r": 2, "rcs": 2, "rrc": 3, "rrs": 3, "rrcs": 3, "cpy": 2, "re": 3, "nop": 0}

DTYPES = {
    "uint8": np.uint8, "int8": np.int8, "int32": np.int32, "uint32": np.uint32,
    "int64": np.int64, "uint64": np.uint64, "float16": np.float16, "float32": np.float32,
    "float64": np.float64, "bfloat16": np.uint16,  # bf16 carried as raw bits
}


# ----------------------------------------------------------------------------------------------
# bf16 helpers (bit patterns in uint16)
# ----------------------------------------------------------------------------------------------
def f32_to_bf16_bits(x):
    """Round fp32 -> bf16 (nearest even), return uint16 bit patterns. NaNs stay NaN (quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    r = ((u + bias) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def _reduce(a, b, dtype, redop):
    """Element-wise a (+) b in the buffer dtype.  max and min of floating-point data are C's
    fmax / fmin: a NaN operand counts as missing and the other operand is the result (NaN only if
    both are) -- the semantics of the fmaxf / fminf the collective runtimes of the NCCL family
    reduce with, and of the device code here; sum and prod propagate NaN as IEEE addition and
    multiplication do."""
    if dtype == "bfloat16":
        fa, fb = bf16_bits_to_f32(a), bf16_bits_to_f32(b)
        with np.errstate(all="ignore"):
            if redop == "sum":
                r = fa + fb
            elif redop == "prod":
                r = fa * fb
            elif redop == "max":
                r = np.fmax(fa, fb)
            elif redop == "min":
                r = np.fmin(fa, fb)
            else:
                raise ValueError(redop)
        return f32_to_bf16_bits(r)
    with np.errstate(all="ignore"):
        if redop == "sum":
            return a + b
        if redop == "prod":
            return a * b
        if redop == "max":
            return np.fmax(a, b)
        if redop == "min":
            return np.fmin(a, b)
    raise ValueError(redop)


# ----------------------------------------------------------------------------------------------
# XML -> plain Python structures (independent of the executor package's loader on purpose)
# ----------------------------------------------------------------------------------------------
Step = collections.namedtuple("Step", "s type srcbuf srcoff dstbuf dstoff cnt depid deps hasdep")


class Tb:
    __slots__ = ("id", "send", "recv", "chan", "steps")

    def __init__(self, id, send, recv, chan):
        self.id, self.send, self.recv, self.chan, self.steps = id, send, recv, chan, []


class Gpu:
    __slots__ = ("id", "i_chunks", "o_chunks", "s_chunks", "tbs")

    def __init__(self, id, i, o, s):
        self.id, self.i_chunks, self.o_chunks, self.s_chunks, self.tbs = id, i, o, s, []


class Algo:
    __slots__ = ("name", "proto", "nchannels", "nchunksperloop", "ngpus", "coll", "inplace", "gpus")


def _scratch_behind_output(gpu):
    """ncclize(use_scratch=False) addresses a rank's scratch as output chunks past o_chunks
    (msccl/ncclize.py:690-697, "scratch at the end of output") and then never names buffer 's':
    in a rank that declares scratch and names 's' nowhere, local references past the output's end
    mean scratch.  Any other out-of-range offset is left as written (and fails when executed)."""
    local_src, local_dst = ("s", "cpy", "re"), RECV_TYPES + ("cpy", "re")
    steps = [st for tb in gpu.tbs for st in tb.steps]
    if not gpu.s_chunks or any((st.type in local_src and st.srcbuf == "s") or (st.type in local_dst and st.dstbuf == "s") for st in steps):
        return
    for tb in gpu.tbs:
        for k, st in enumerate(tb.steps):
            for local, buf, off in ((st.type in local_src, "srcbuf", "srcoff"), (st.type in local_dst, "dstbuf", "dstoff")):
                at = getattr(st, off)
                if not (local and getattr(st, buf) == "o"):
                    continue
                if at < gpu.o_chunks < at + st.cnt:
                    raise ValueError(f"gpu {gpu.id}: a step's chunks [{at}, {at + st.cnt}) straddle the end of the output buffer")
                if at >= gpu.o_chunks:
                    st = st._replace(**{buf: "s", off: at - gpu.o_chunks})
            tb.steps[k] = st


def parse_xml(text):
    """Parse <algo> XML (ir.py:320-391 / ncclize.py:658-718) into Algo/Gpu/Tb/Step."""
    root = ET.fromstring(text)
    if root.tag != "algo":
        raise ValueError("root element must be <algo>")
    a = Algo()
    a.name = root.get("name", "")
    a.proto = root.get("proto", "Simple")
    a.nchannels = int(root.get("nchannels", "0"))
    a.nchunksperloop = int(root.get("nchunksperloop", "0"))
    a.ngpus = int(root.get("ngpus"))
    a.coll = root.get("coll", "custom")
    a.inplace = int(root.get("inplace", "0"))
    a.gpus = []
    for g in root.findall("gpu"):
        gpu = Gpu(int(g.get("id")), int(g.get("i_chunks")), int(g.get("o_chunks")), int(g.get("s_chunks")))
        for t in g.findall("tb"):
            tb = Tb(int(t.get("id")), int(t.get("send")), int(t.get("recv")), int(t.get("chan")))
            for st in t.findall("step"):
                ty = st.get("type")
                sb, so, db, do = st.get("srcbuf"), int(st.get("srcoff")), st.get("dstbuf"), int(st.get("dstoff"))
                tb.steps.append(Step(int(st.get("s")), ty, sb, so, db, do, int(st.get("cnt")),
                                     int(st.get("depid")), int(st.get("deps")), int(st.get("hasdep"))))
            gpu.tbs.append(tb)
        _scratch_behind_output(gpu)
        a.gpus.append(gpu)
    a.gpus.sort(key=lambda g: g.id)
    if [g.id for g in a.gpus] != list(range(a.ngpus)):
        raise ValueError("gpu ids must be 0..ngpus-1")
    return a


def algorithmic_bytes(algo, chunk_bytes):
    """chunk_bytes * sum over ops of cnt * a(type)."""
    total = 0
    for g in algo.gpus:
        for tb in g.tbs:
            for st in tb.steps:
                total += st.cnt * ALGO_BYTES_FACTOR[st.type]
    return total * chunk_bytes


class Deadlock(RuntimeError):
    pass


# ----------------------------------------------------------------------------------------------
# The interpreter
# ----------------------------------------------------------------------------------------------
class Interpreter:
    """Executes every rank's per-threadblock step list with a cooperative scheduler.

    schedule: 'fifo' (deterministic round-robin, each tb runs until it blocks) or 'random'
    (random tb order, random burst length; used to show that the result does not depend on the
    interleaving).  fifo_depth: None = unbounded connections, k = a send blocks while k messages
    are outstanding on its connection.
    """

    def __init__(self, algo, schedule="fifo", seed=0, fifo_depth=None):
        self.algo = algo if isinstance(algo, Algo) else parse_xml(algo)
        self.schedule = schedule
        self.rng = random.Random(seed)
        self.fifo_depth = fifo_depth

    def alloc(self, chunk_elems, dtype):
        npdt = DTYPES[dtype]
        bufs = []
        for g in self.algo.gpus:
            bufs.append({"i": np.zeros(g.i_chunks * chunk_elems, npdt),
                         "o": np.zeros(g.o_chunks * chunk_elems, npdt),
                         "s": np.zeros(g.s_chunks * chunk_elems, npdt)})
        return bufs

    def run(self, bufs, chunk_elems, dtype, redop="sum"):
        """bufs: list over ranks of {'i','o','s'} 1-D arrays sized extents*chunk_elems; updated in place."""
        algo = self.algo
        E = chunk_elems
        tbs = [(g.id, tb) for g in algo.gpus for tb in g.tbs]
        pc = {(r, tb.id): 0 for r, tb in tbs}
        fifos = collections.defaultdict(collections.deque)
        done_steps = pc  # a step index < pc is complete

        def view(rank, buf, off, cnt):
            arr = bufs[rank][buf]
            lo, hi = off * E, (off + cnt) * E
            if off < 0 or hi > arr.size:
                raise IndexError(f"rank {rank} buffer {buf}: chunks [{off},{off + cnt}) outside extent")
            return arr[lo:hi]

        def try_step(rank, tb):
            k = pc[(rank, tb.id)]
            if k >= len(tb.steps):
                return False
            st = tb.steps[k]
            if st.depid >= 0 and not (done_steps[(rank, st.depid)] > st.deps):
                return False
            t = st.type
            is_recv = t in RECV_TYPES
            is_send = t in SEND_TYPES
            if is_recv:
                q_in = fifos[(tb.recv, rank, tb.chan)]
                if not q_in:
                    return False
            if is_send:
                q_out = fifos[(rank, tb.send, tb.chan)]
                if self.fifo_depth is not None and len(q_out) >= self.fifo_depth:
                    return False
            if t == "nop":
                pass
            elif t == "s":
                q_out.append(view(rank, st.srcbuf, st.srcoff, st.cnt).copy())
            elif t == "cpy":
                view(rank, st.dstbuf, st.dstoff, st.cnt)[:] = view(rank, st.srcbuf, st.srcoff, st.cnt)
            elif t == "re":
                d = view(rank, st.dstbuf, st.dstoff, st.cnt)
                d[:] = _reduce(d, view(rank, st.srcbuf, st.srcoff, st.cnt), dtype, redop)
            else:
                msg = q_in.popleft()
                if msg.size != st.cnt * E:
                    raise ValueError(f"rank {rank} tb {tb.id} step {k}: message of {msg.size} elements, expected {st.cnt * E}")
                if t == "r":
                    view(rank, st.dstbuf, st.dstoff, st.cnt)[:] = msg
                elif t == "rcs":
                    view(rank, st.dstbuf, st.dstoff, st.cnt)[:] = msg
                    q_out.append(msg)
                elif t == "rrc":
                    d = view(rank, st.dstbuf, st.dstoff, st.cnt)
                    d[:] = _reduce(d, msg, dtype, redop)
                elif t == "rrs":
                    q_out.append(_reduce(view(rank, st.dstbuf, st.dstoff, st.cnt), msg, dtype, redop))
                elif t == "rrcs":
                    d = view(rank, st.dstbuf, st.dstoff, st.cnt)
                    d[:] = _reduce(d, msg, dtype, redop)
                    q_out.append(d.copy())
                else:
                    raise ValueError(f"unknown step type {t!r}")
            pc[(rank, tb.id)] = k + 1
            return True

        remaining = sum(len(tb.steps) for _, tb in tbs)
        while remaining:
            progressed = 0
            order = list(tbs)
            if self.schedule == "random":
                self.rng.shuffle(order)
            for rank, tb in order:
                burst = 1 << 30 if self.schedule == "fifo" else self.rng.randint(1, 3)
                while burst and try_step(rank, tb):
                    burst -= 1
                    progressed += 1
            remaining -= progressed
            if not progressed:
                stuck = [(r, tb.id, pc[(r, tb.id)], tb.steps[pc[(r, tb.id)]].type)
                         for r, tb in tbs if pc[(r, tb.id)] < len(tb.steps)]
                raise Deadlock(f"no threadblock can progress; blocked (rank, tb, step, type): {stuck[:8]}")
        leftovers = {k: len(q) for k, q in fifos.items() if q}
        if leftovers:
            raise ValueError(f"unconsumed messages left on connections {leftovers}")
        return bufs
