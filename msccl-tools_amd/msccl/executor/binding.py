"""ctypes binding of libmscclx.so (C ABI in include/mscclx.h).

The library is the only execution path: if it cannot be loaded the import of this module's users
fails with ExecutorUnavailable; there is no CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "..", "csrc"))
LIB_PATH = os.path.join(CSRC_DIR, "libmscclx.so")

OK = 0
ERR_INVALID_ARG, ERR_BAD_IR, ERR_DEADLOCK, ERR_CAPACITY, ERR_HIP, ERR_TIMEOUT, ERR_STATE, ERR_UNSUPPORTED, ERR_ABORTED, ERR_ALIASED = range(-1, -11, -1)
ERROR_NAMES = {0: "OK", -1: "INVALID_ARG", -2: "BAD_IR", -3: "DEADLOCK", -4: "CAPACITY", -5: "HIP", -6: "TIMEOUT",
               -7: "STATE", -8: "UNSUPPORTED", -9: "ABORTED", -10: "ALIASED"}

DTYPE_CODES = {"uint8": 0, "int8": 1, "int32": 2, "uint32": 3, "int64": 4, "uint64": 5,
               "float16": 6, "bfloat16": 7, "float32": 8, "float64": 9}
DTYPE_SIZES = {"uint8": 1, "int8": 1, "int32": 4, "uint32": 4, "int64": 8, "uint64": 8,
               "float16": 2, "bfloat16": 2, "float32": 4, "float64": 8}
REDOP_CODES = {"sum": 0, "prod": 1, "max": 2, "min": 3}
LOOP_NAMES = {0: "hosted", 1: "chain, lines", 2: "chain, counters", 3: "chain, folded nops", 4: "chain, lines, steps worked out at bind"}  # mscclx_loop
PROTOCOL_CODES = {"auto": 0, "simple": 1, "ll": 2, "Simple": 1, "LL": 2}

# every symbol include/mscclx.h declares
EXPORTED_SYMBOLS = (
    "mscclx_version", "mscclx_last_error", "mscclx_plan_create", "mscclx_plan_destroy", "mscclx_plan_simulate",
    "mscclx_plan_min_fifo_depth", "mscclx_plan_algorithmic_units", "mscclx_plan_configure", "mscclx_plan_bind",
    "mscclx_plan_launch", "mscclx_plan_wait", "mscclx_plan_poll", "mscclx_plan_abort", "mscclx_plan_time",
    "mscclx_plan_run_static",
)


class ExecutorUnavailable(RuntimeError):
    pass


class MscclxError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"mscclx {ERROR_NAMES.get(code, code)}: {message}")
        self.code = code
        self.message = message


class PlanDesc(ctypes.Structure):
    _fields_ = [("nranks", ctypes.c_int32), ("ntbs", ctypes.c_int32), ("nops", ctypes.c_int32),
                ("rank_chunks", ctypes.POINTER(ctypes.c_int32)), ("tbs", ctypes.POINTER(ctypes.c_int32)),
                ("ops", ctypes.POINTER(ctypes.c_int32))]


class Config(ctypes.Structure):
    _fields_ = [("slices", ctypes.c_int32), ("piece_bytes", ctypes.c_int32), ("fifo_depth", ctypes.c_int32),
                ("threads", ctypes.c_int32), ("timeout_ms", ctypes.c_int32), ("max_workgroups", ctypes.c_int32),
                ("staging", ctypes.c_int32), ("workgroups", ctypes.c_int32),
                ("protocol", ctypes.c_int32), ("reserved", ctypes.c_int32 * 3)]


class Info(ctypes.Structure):
    _fields_ = [("workgroups", ctypes.c_int32), ("threads", ctypes.c_int32), ("slices", ctypes.c_int32),
                ("piece_bytes", ctypes.c_int32), ("fifo_depth", ctypes.c_int32), ("passes", ctypes.c_int32),
                ("connections", ctypes.c_int32), ("vector_path", ctypes.c_int32),
                ("zero_copy_messages", ctypes.c_int32), ("staged_messages", ctypes.c_int32),
                ("max_hosted", ctypes.c_int32), ("protocol", ctypes.c_int32),
                ("waiting_ratio_x100", ctypes.c_int32), ("dataflow_depth", ctypes.c_int32),
                ("kernel_loop", ctypes.c_int32), ("cold_traffic_x100", ctypes.c_int32),
                ("workspace_bytes", ctypes.c_uint64), ("algorithmic_units", ctypes.c_uint64)]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


class Status(ctypes.Structure):
    _fields_ = [("code", ctypes.c_int32), ("tb", ctypes.c_int32), ("step", ctypes.c_int32), ("slice", ctypes.c_int32),
                ("pass_", ctypes.c_int64), ("waiting_on", ctypes.c_int32), ("reserved", ctypes.c_int32)]


_lib = None


def load_library(path=None):
    """dlopen libmscclx.so and declare the prototypes.  Raises ExecutorUnavailable when it is not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or os.environ.get("MSCCLX_LIBRARY") or LIB_PATH
    if not os.path.exists(p):
        raise ExecutorUnavailable(f"{p} is not built; run `python {os.path.join(CSRC_DIR, 'build.py')}`")
    try:
        lib = ctypes.CDLL(p)
    except OSError as e:
        raise ExecutorUnavailable(f"cannot load {p}: {e}") from None
    vp, i32, u64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_uint64
    lib.mscclx_version.restype = ctypes.c_int
    lib.mscclx_last_error.restype = ctypes.c_char_p
    lib.mscclx_plan_create.argtypes = [ctypes.POINTER(PlanDesc), ctypes.POINTER(vp)]
    lib.mscclx_plan_destroy.argtypes = [vp]
    lib.mscclx_plan_simulate.argtypes = [vp, i32]
    lib.mscclx_plan_min_fifo_depth.argtypes = [vp]
    lib.mscclx_plan_algorithmic_units.argtypes = [vp]
    lib.mscclx_plan_algorithmic_units.restype = u64
    lib.mscclx_plan_configure.argtypes = [vp, ctypes.c_size_t, i32, i32, ctypes.POINTER(Config), ctypes.POINTER(Info)]
    lib.mscclx_plan_bind.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), vp, ctypes.c_size_t]
    lib.mscclx_plan_launch.argtypes = [vp, vp]
    lib.mscclx_plan_wait.argtypes = [vp, vp, ctypes.POINTER(Status)]
    lib.mscclx_plan_poll.argtypes = [vp, vp, ctypes.POINTER(Status)]
    lib.mscclx_plan_abort.argtypes = [vp]
    lib.mscclx_plan_time.argtypes = [vp, vp, i32, ctypes.POINTER(ctypes.c_float)]
    lib.mscclx_plan_run_static.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), vp, ctypes.POINTER(Status)]
    lib.mscclx_plan_run_static.restype = ctypes.c_int
    for name in ("mscclx_plan_create", "mscclx_plan_destroy", "mscclx_plan_simulate", "mscclx_plan_min_fifo_depth",
                 "mscclx_plan_configure", "mscclx_plan_bind", "mscclx_plan_launch", "mscclx_plan_wait", "mscclx_plan_poll",
                 "mscclx_plan_abort", "mscclx_plan_time"):
        getattr(lib, name).restype = ctypes.c_int
    if path is None:
        _lib = lib
    return lib


def _check(lib, rc):
    if rc < 0:
        raise MscclxError(rc, lib.mscclx_last_error().decode("utf-8", "replace"))
    return rc


class Plan:
    """Owns one mscclx_plan*."""

    def __init__(self, tables):
        self.lib = load_library()
        self.tables = tables
        self._rank_chunks = np.ascontiguousarray(tables.rank_chunks, np.int32)
        self._tbs = np.ascontiguousarray(tables.tbs, np.int32)
        self._ops = np.ascontiguousarray(tables.ops, np.int32)
        as_p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        desc = PlanDesc(tables.ngpus, self._tbs.shape[0], self._ops.shape[0], as_p(self._rank_chunks), as_p(self._tbs), as_p(self._ops))
        handle = ctypes.c_void_p()
        _check(self.lib, self.lib.mscclx_plan_create(ctypes.byref(desc), ctypes.byref(handle)))
        self.handle = handle
        self.info = None

    def close(self):
        if getattr(self, "handle", None):
            self.lib.mscclx_plan_destroy(self.handle)
            self.handle = None

    __del__ = close

    def simulate(self, fifo_depth):
        return _check(self.lib, self.lib.mscclx_plan_simulate(self.handle, fifo_depth))

    def min_fifo_depth(self):
        return _check(self.lib, self.lib.mscclx_plan_min_fifo_depth(self.handle))

    def algorithmic_units(self):
        return int(self.lib.mscclx_plan_algorithmic_units(self.handle))

    def configure(self, chunk_bytes, dtype, redop="sum", **knobs):
        cfg = Config()
        for k, v in knobs.items():
            if not hasattr(cfg, k):
                raise TypeError(f"unknown executor knob {k!r}")
            setattr(cfg, k, PROTOCOL_CODES[v] if k == "protocol" and isinstance(v, str) else int(v))
        info = Info()
        _check(self.lib, self.lib.mscclx_plan_configure(self.handle, chunk_bytes, DTYPE_CODES[dtype], REDOP_CODES[redop],
                                                       ctypes.byref(cfg), ctypes.byref(info)))
        self.info = info
        return info

    def bind(self, in_ptrs, out_ptrs, scratch_ptrs, workspace_ptr, workspace_bytes):
        n = self.tables.ngpus
        arr = lambda ptrs: (ctypes.c_void_p * n)(*[ctypes.c_void_p(p or None) for p in ptrs])
        _check(self.lib, self.lib.mscclx_plan_bind(self.handle, arr(in_ptrs), arr(out_ptrs), arr(scratch_ptrs),
                                                  ctypes.c_void_p(workspace_ptr), workspace_bytes))

    def run_static(self, in_ptrs, out_ptrs, scratch_ptrs, stream=0):
        """One whole execution out of the library's static device array (no allocation)."""
        n = self.tables.ngpus
        arr = lambda ptrs: (ctypes.c_void_p * n)(*[ctypes.c_void_p(p or None) for p in ptrs])
        st = Status()
        _check(self.lib, self.lib.mscclx_plan_run_static(self.handle, arr(in_ptrs), arr(out_ptrs), arr(scratch_ptrs),
                                                        ctypes.c_void_p(stream or None), ctypes.byref(st)))
        return st

    def launch(self, stream=0):
        _check(self.lib, self.lib.mscclx_plan_launch(self.handle, ctypes.c_void_p(stream or None)))

    def wait(self, stream=0):
        st = Status()
        _check(self.lib, self.lib.mscclx_plan_wait(self.handle, ctypes.c_void_p(stream or None), ctypes.byref(st)))
        return st

    def poll(self, stream=0):
        """(running, status): running is True while the launch stream still has work."""
        st = Status()
        rc = _check(self.lib, self.lib.mscclx_plan_poll(self.handle, ctypes.c_void_p(stream or None), ctypes.byref(st)))
        return rc == 1, st

    def abort(self):
        _check(self.lib, self.lib.mscclx_plan_abort(self.handle))

    def time(self, iters, stream=0):
        ms = (ctypes.c_float * iters)()
        _check(self.lib, self.lib.mscclx_plan_time(self.handle, ctypes.c_void_p(stream or None), iters, ms))
        return list(ms)
