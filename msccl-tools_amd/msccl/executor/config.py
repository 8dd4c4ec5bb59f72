"""Consumer of what `msccl.init` leaves behind: the `<msccl_algos>` index named by $MSCCL_CONFIG
(msccl-tools' msccl/autosynth/__init__.py:75-99 writes it: one <load path= [minBytes=] [maxBytes=]
proto=/> per selected plan) and the algorithm XML files it lists."""
from __future__ import annotations

import dataclasses
import math
import os
import xml.etree.ElementTree as ET

from .ir_tables import AlgoTables, IRError


@dataclasses.dataclass
class LoadedAlgo:
    path: str
    min_bytes: int
    max_bytes: float
    proto: str
    tables: AlgoTables

    def bytes_per_rank_to_chunk_bytes(self, nbytes):
        """Bytes of one IR chunk when every rank's send buffer holds `nbytes`."""
        t = self.tables
        if t.coll == "allgather":
            chunks = int(t.rank_chunks[0, 1]) // t.ngpus if t.inplace or not t.rank_chunks[0, 0] else int(t.rank_chunks[0, 0])
        else:
            chunks = int(t.rank_chunks[0, 0])
        if chunks <= 0 or nbytes % chunks:
            raise ValueError(f"{nbytes} bytes per rank do not divide into the algorithm's {chunks} chunks")
        return nbytes // chunks


def _load(path):
    """The tables of the document at `path`: parsed once per distinct text (msccl.init writes a new temporary file for
    the same program every time it is called)."""
    from .cache import tables_for
    with open(path, "r") as f:
        return tables_for(f.read())


def load_config(path=None):
    """Parse the index at `path` (default: $MSCCL_CONFIG) and every algorithm it lists."""
    path = path or os.environ.get("MSCCL_CONFIG")
    if not path:
        raise IRError("MSCCL_CONFIG is not set; call msccl.init(...) first or pass a path")
    root = ET.parse(path).getroot()
    if root.tag != "msccl_algos":
        raise IRError(f"{path}: root element is <{root.tag}>, expected <msccl_algos>")
    algos = []
    for load in root.findall("load"):
        p = load.get("path")
        if p is None:
            raise IRError(f"{path}: <load> without path")
        algos.append(LoadedAlgo(p, int(load.get("minBytes", "0")), float(load.get("maxBytes", "inf")),
                                load.get("proto", "Simple"), _load(p)))
    return algos


def select(algos, coll, nbytes, ngpus=None):
    """First listed algorithm for collective `coll` whose window holds `nbytes`, optionally with
    `ngpus` ranks; None if there is none.  Windows are half-open, minBytes <= nbytes < maxBytes, the
    convention of the emitter: a single size n is written as (n, n + 1) and adjacent plans share
    their boundary value (msccl/autosynth/__init__.py:57-68)."""
    for a in algos:
        if a.tables.coll == str(coll) and a.min_bytes <= nbytes < a.max_bytes and (ngpus is None or a.tables.ngpus == ngpus):
            return a
    return None
