"""Runs a compiled MSCCL-IR algorithm on one MI355X with every rank held as a virtual rank.

PyTorch-ROCm is used for device memory and streams only.  Buffers follow the naming of the XML:
'i' = the rank's send buffer, 'o' = its receive buffer, 's' = scratch (allocated here).  In-place
algorithms alias them exactly as an in-place NCCL call would (msccl/language/collectives.py:
in-place all-reduce names only 'i'; in-place all-gather names only 'o', rank r's contribution being
output chunks [r*cf, (r+1)*cf)).
"""
from __future__ import annotations

import time

import torch

from .binding import DTYPE_SIZES, ERR_ALIASED, MscclxError, Plan
from .ir_tables import AlgoTables, parse_algo_xml

_TORCH_NAMES = {torch.uint8: "uint8", torch.int8: "int8", torch.int32: "int32", torch.int64: "int64",
                torch.float16: "float16", torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float64: "float64"}
for _n in ("uint32", "uint64"):
    if hasattr(torch, _n):
        _TORCH_NAMES[getattr(torch, _n)] = _n


def dtype_name(dtype):
    if isinstance(dtype, str):
        if dtype not in DTYPE_SIZES:
            raise ValueError(f"unsupported dtype {dtype!r}")
        return dtype
    if dtype in _TORCH_NAMES:
        return _TORCH_NAMES[dtype]
    raise ValueError(f"unsupported dtype {dtype!r}")


class Executor:
    """plan = Executor(xml_or_tables); plan.setup(chunk_bytes, dtype); plan.run(inputs, outputs)."""

    def __init__(self, algo, device="cuda:0"):
        if isinstance(algo, AlgoTables):
            self.tables = algo
        else:  # XML text: parsed once per distinct document
            from .cache import tables_for
            self.tables = tables_for(algo)
        self.device = torch.device(device)
        self.plan = Plan(self.tables)
        self.info = None
        self.chunk_bytes = None
        self.dtype = None
        self._scratch = None
        self._workspace = None
        self._bound = None
        self._staged_for_aliasing = False
        self.host_seconds = {}   # host time of the last configure / bind call into the library

    # -- geometry ---------------------------------------------------------------------------------
    def setup(self, chunk_bytes, dtype, redop="sum", **knobs):
        """Fix chunk size / element type / reduction and allocate scratch + workspace.

        protocol="ir" follows the algorithm's own `proto` attribute (msccl/language/ir.py:322):
        LL and LL128 run as flag-in-data lines, Simple as counters.  The default ignores the
        attribute and lets the library choose, as the attribute is a hint about another machine."""
        if not torch.cuda.is_available():
            raise RuntimeError("the MSCCL-IR executor needs a GPU; there is no CPU path")
        if knobs.get("protocol") == "ir":
            knobs = dict(knobs, protocol="ll" if self.tables.proto.upper().startswith("LL") else "simple")
        self.dtype = dtype_name(dtype)
        self.chunk_bytes = int(chunk_bytes)
        self._setup_args = (chunk_bytes, dtype, redop, dict(knobs))
        self._staged_for_aliasing = False
        with torch.cuda.device(self.device):
            t0 = time.perf_counter()
            self.info = self.plan.configure(self.chunk_bytes, self.dtype, redop, **knobs)
            self.host_seconds["configure"] = time.perf_counter() - t0
            t = self.tables
            self._scratch = [torch.empty(int(t.rank_chunks[r, 2]) * self.chunk_bytes, dtype=torch.uint8, device=self.device)
                             if t.rank_chunks[r, 2] else None for r in range(t.ngpus)]
            self._workspace = torch.empty(int(self.info.workspace_bytes), dtype=torch.uint8, device=self.device)
        self._bound = None
        return self.info

    def _check_buffers(self, bufs, col, what):
        t = self.tables
        ptrs = []
        bufs = bufs if bufs is not None else [None] * t.ngpus
        if len(bufs) != t.ngpus:
            raise ValueError(f"{what}: {len(bufs)} buffers for {t.ngpus} ranks")
        for r, b in enumerate(bufs):
            need = int(t.rank_chunks[r, col]) * self.chunk_bytes
            if need == 0:
                ptrs.append(b.data_ptr() if b is not None else 0)
                continue
            if b is None:
                raise ValueError(f"rank {r}: the algorithm uses the {what} buffer but none was given")
            if not b.is_cuda or not b.is_contiguous():
                raise ValueError(f"rank {r}: {what} buffer must be a contiguous device tensor")
            if b.numel() * b.element_size() < need:
                raise ValueError(f"rank {r}: {what} buffer holds {b.numel() * b.element_size()} bytes, the algorithm addresses {need}")
            ptrs.append(b.data_ptr())
        return ptrs

    def _spans_overlap(self, ins, outs):
        """Do any two rank buffers the algorithm addresses share memory?  (What mscclx_plan_bind refuses
        with ALIASED unless every message is staged.)"""
        t = self.tables
        spans = []
        for col, ptrs in ((0, ins), (1, outs), (2, [0 if s is None else s.data_ptr() for s in self._scratch])):
            for r, ptr in enumerate(ptrs):
                need = int(t.rank_chunks[r, col]) * self.chunk_bytes
                if need:
                    spans.append((ptr, ptr + need))
        spans.sort()
        return any(b[0] < a[1] for a, b in zip(spans, spans[1:]))

    def bind(self, inputs, outputs, allow_aliased=False):
        """Attach rank buffers.  Buffers that the IR names separately but that share memory (an in-place
        call on an out-of-place algorithm) are refused with MscclxError(ALIASED) unless
        allow_aliased=True: the plan is then configured again with every message copied through a FIFO
        slot.  That only takes away the executor's own reads of payloads where the sender keeps them; whether
        the *program* still computes the collective when two of its buffers are one is the caller's
        to know (it does for NCCL's in-place all-gather convention on an all-gather whose every write
        of a chunk writes that chunk's final value; it does not where a receive overwrites what a
        later step of the same rank still reads).  A later bind of buffers that do not overlap goes back
        to the knobs setup() was called with."""
        if self.info is None:
            raise RuntimeError("call setup() first")
        key = (tuple(0 if b is None else b.data_ptr() for b in (inputs or [])),
               tuple(0 if b is None else b.data_ptr() for b in (outputs or [])), bool(allow_aliased))
        if key == self._bound:
            return
        ins = self._check_buffers(inputs, 0, "input")
        outs = self._check_buffers(outputs, 1, "output")
        chunk_bytes, dtype, redop, knobs = self._setup_args
        if self._staged_for_aliasing and not self._spans_overlap(ins, outs):
            self.setup(chunk_bytes, dtype, redop, **knobs)
        scr = [0 if s is None else s.data_ptr() for s in self._scratch]
        try:
            with torch.cuda.device(self.device):
                t0 = time.perf_counter()
                self.plan.bind(ins, outs, scr, self._workspace.data_ptr(), self._workspace.numel())
                self.host_seconds["bind"] = time.perf_counter() - t0
        except MscclxError as e:
            if e.code != ERR_ALIASED or not allow_aliased:
                raise
            self.setup(chunk_bytes, dtype, redop, **dict(knobs, staging=1))
            self._setup_args = (chunk_bytes, dtype, redop, knobs)   # what the caller asked for, to go back to
            self._staged_for_aliasing = True
            scr = [0 if t is None else t.data_ptr() for t in self._scratch]
            with torch.cuda.device(self.device):
                self.plan.bind(ins, outs, scr, self._workspace.data_ptr(), self._workspace.numel())
        self._bound = key
        self._keepalive = (inputs, outputs)

    # -- execution --------------------------------------------------------------------------------
    def _stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    def launch(self):
        with torch.cuda.device(self.device):
            self.plan.launch(self._stream())

    def wait(self):
        with torch.cuda.device(self.device):
            return self.plan.wait(self._stream())

    def poll(self):
        """True while the launch is still running (non-blocking); raises like wait() once it has failed."""
        with torch.cuda.device(self.device):
            return self.plan.poll(self._stream())[0]

    def abort(self):
        """Ask the running launch to give up; wait() then raises MscclxError(ABORTED)."""
        with torch.cuda.device(self.device):
            self.plan.abort()

    def run(self, inputs, outputs, allow_aliased=False):
        self.bind(inputs, outputs, allow_aliased=allow_aliased)
        self.launch()
        self.wait()
        return outputs

    def run_static(self, inputs, outputs):
        """One whole execution that allocates nothing on the device: tables, counters and FIFO slots
        sit in the library's own static device array (mscclx_plan_run_static).  Refused with CAPACITY
        when the plan needs more than that array holds.  Leaves the binding of run()/launch() alone."""
        if self.info is None:
            raise RuntimeError("call setup() first")
        ins = self._check_buffers(inputs, 0, "input")
        outs = self._check_buffers(outputs, 1, "output")
        scr = [0 if s is None else s.data_ptr() for s in self._scratch]
        with torch.cuda.device(self.device):
            return self.plan.run_static(ins, outs, scr, self._stream())

    def time(self, iters):
        """Per-launch GPU time in ms (HIP events around each launch on the current stream)."""
        with torch.cuda.device(self.device):
            return self.plan.time(iters, self._stream())

    def algorithmic_bytes(self):
        return self.plan.algorithmic_units() * self.chunk_bytes


def collective_buffers(tables, chunk_bytes, dtype, device="cuda:0", inputs=None):
    """Allocate (inputs, outputs) tensors the way the collective's aliasing rule demands and, when
    `inputs` (one 1-D host or device tensor per rank, the rank's send data) is given, place it.

    Returns (in_bufs, out_bufs, results) where results[r] is the tensor view holding rank r's
    receive data after the run.
    """
    t = tables
    name = dtype_name(dtype)
    esz = DTYPE_SIZES[name]
    tdt = {v: k for k, v in _TORCH_NAMES.items()}[name]
    n = t.ngpus
    in_bufs, out_bufs, results = [], [], []
    for r in range(n):
        i_el = int(t.rank_chunks[r, 0]) * chunk_bytes // esz
        o_el = int(t.rank_chunks[r, 1]) * chunk_bytes // esz
        ib = torch.zeros(i_el, dtype=tdt, device=device) if i_el else None
        ob = torch.zeros(o_el, dtype=tdt, device=device) if o_el else None
        if t.inplace and t.coll == "alltoall" and ib is not None:
            ob = ib
        x = None if inputs is None else torch.as_tensor(inputs[r]).reshape(-1).to(device)
        if t.coll == "allgather" and t.inplace:
            per = o_el // n
            if x is not None:
                ob[r * per:(r + 1) * per].copy_(x)
            res = ob
        else:
            if x is not None:
                ib[:x.numel()].copy_(x)
            if t.coll == "allreduce" and t.inplace:
                res = ib
            elif t.coll == "reduce_scatter" and t.inplace:
                per = i_el // n
                res = ib[r * per:(r + 1) * per]
            else:
                res = ob
        in_bufs.append(ib)
        out_bufs.append(ob)
        results.append(res)
    return in_bufs, out_bufs, results
