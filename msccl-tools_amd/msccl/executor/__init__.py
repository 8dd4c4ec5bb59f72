"""MI355X executor for MSCCL-IR: XML -> flat tables -> libmscclx.so (HIP) through ctypes."""
from .ir_tables import AlgoTables, IRError, load_algo, parse_algo_xml, OP_CODES, BUF_CODES, ALGO_FACTOR
from .config import LoadedAlgo, load_config, select
from .binding import (ExecutorUnavailable, MscclxError, Plan, load_library, DTYPE_CODES, DTYPE_SIZES, REDOP_CODES,
                      EXPORTED_SYMBOLS, LIB_PATH)


def __getattr__(name):
    # torch is imported only when the device-facing classes are asked for
    if name in ("Executor", "collective_buffers", "dtype_name"):
        from . import runner
        return getattr(runner, name)
    if name in ("executor_for", "tables_for"):
        from . import cache
        return getattr(cache, name)
    raise AttributeError(name)
