"""What a caller pays for once per document, kept: the flat tables of an MSCCL-IR document by the hash of its
text, and whole executors -- tables, host plan, geometry, workspace, device tables -- by (document, chunk size,
element type, reduction, knobs, device).

Turning a compiled algorithm into something that can be launched costs milliseconds of host work (XML to
tables, validation and the analysis of which payloads may be read in place, the choice of a geometry, the first
bind), against microseconds for a launch.  A framework that issues the same collective on the same sizes again
and again -- every training step -- asks for the same executor every time; `executor_for` hands it back.
Both caches are bounded and evict the entry unused for longest.
"""
from __future__ import annotations

import collections
import hashlib

from .ir_tables import AlgoTables, parse_algo_xml

MAX_DOCUMENTS = 64
MAX_EXECUTORS = 32
_tables = collections.OrderedDict()     # sha1 of the text -> AlgoTables
_executors = collections.OrderedDict()  # (sha1, chunk_bytes, dtype, redop, knobs, device) -> Executor


def document_key(text):
    return hashlib.sha1(text.encode() if isinstance(text, str) else text).hexdigest()


def _touch(store, key, limit, make):
    if key in store:
        store.move_to_end(key)
        return store[key]
    value = store[key] = make()
    while len(store) > limit:
        store.popitem(last=False)
    return value


def tables_for(text):
    """AlgoTables of an <algo> document; parsed once per distinct text.  The tables are shared: treat them as read-only."""
    key = document_key(text)
    tables = _touch(_tables, key, MAX_DOCUMENTS, lambda: parse_algo_xml(text))
    tables.document_key = key
    return tables


def executor_for(algo, chunk_bytes, dtype, redop="sum", device="cuda:0", **knobs):
    """A set-up Executor for this document (XML text, or AlgoTables from tables_for) and configuration: the one handed
    out before for the same key, else a new one.  Its workspace and scratch are its own; callers that get the same
    executor share them, so their launches must not overlap (launches of one plan never may)."""
    from .runner import Executor, dtype_name
    if isinstance(algo, AlgoTables):
        tables, key = algo, algo.document_key
        if not key:
            raise ValueError("executor_for takes XML text or tables from tables_for (which carry the document's hash)")
    else:
        tables = tables_for(algo)
        key = tables.document_key
    full = (key, int(chunk_bytes), dtype_name(dtype), str(redop), tuple(sorted(knobs.items())), str(device))

    def make():
        ex = Executor(tables, device=device)
        ex.setup(chunk_bytes, dtype, redop, **knobs)
        return ex
    return _touch(_executors, full, MAX_EXECUTORS, make)


def clear():
    """Forget everything (tests; a caller that wants its device memory back)."""
    _tables.clear()
    _executors.clear()
