"""MSCCL-IR XML -> flat int32 tables of the C ABI (include/mscclx.h).

Reads what msccl/language/ir.py:320-391 and msccl/ncclize.py:658-718 of msccl-tools write: an
<algo> with <gpu>, <tb> and <step> children.  Uses only the standard library's ElementTree.
"""
from __future__ import annotations

import dataclasses
import xml.etree.ElementTree as ET

import numpy as np

OP_CODES = {"nop": 0, "s": 1, "r": 2, "rcs": 3, "rrs": 4, "rrc": 5, "rrcs": 6, "cpy": 7, "re": 8}
BUF_CODES = {"i": 0, "o": 1, "s": 2}
# algorithmic traffic of one step in units of cnt * chunk_bytes
ALGO_FACTOR = {"nop": 0, "s": 0, "r": 2, "rcs": 2, "rrs": 3, "rrc": 3, "rrcs": 3, "cpy": 2, "re": 3}


class IRError(ValueError):
    """The XML is not a well-formed MSCCL-IR algorithm."""


@dataclasses.dataclass
class AlgoTables:
    name: str
    proto: str
    coll: str
    inplace: bool
    nchannels: int
    nchunksperloop: int
    ngpus: int
    rank_chunks: np.ndarray  # [ngpus, 3] int32: i_chunks, o_chunks, s_chunks
    tbs: np.ndarray          # [ntbs, 6] int32: rank, send, recv, chan, op_begin, op_end
    ops: np.ndarray          # [nops, 9] int32: type, srcbuf, srcoff, dstbuf, dstoff, cnt, depid, deps, hasdep
    document_key: str = ""   # hash of the XML text these tables were parsed from (set by msccl.executor.cache.tables_for)

    @property
    def ntbs(self):
        return int(self.tbs.shape[0])

    @property
    def nops(self):
        return int(self.ops.shape[0])

    def algorithmic_units(self):
        factors = np.zeros(len(OP_CODES), np.int64)
        for k, v in OP_CODES.items():
            factors[v] = ALGO_FACTOR[k]
        return int((factors[self.ops[:, 0]] * self.ops[:, 5]).sum()) if self.nops else 0

    def has_reduction(self):
        red = [OP_CODES[k] for k in ("rrs", "rrc", "rrcs", "re")]
        return bool(np.isin(self.ops[:, 0], red).any()) if self.nops else False


def _int(elem, name, default=None):
    v = elem.get(name)
    if v is None:
        if default is None:
            raise IRError(f"<{elem.tag}> lacks attribute {name!r}")
        return default
    try:
        return int(v)
    except ValueError:
        raise IRError(f"<{elem.tag} {name}={v!r}> is not an integer") from None


_LOCAL_SRC = {OP_CODES[k] for k in ("s", "cpy", "re")}
_LOCAL_DST = {OP_CODES[k] for k in ("r", "rcs", "rrs", "rrc", "rrcs", "cpy", "re")}


def _scratch_behind_output(rows, o_chunks, where):
    """ncclize(use_scratch=False) writes a rank's scratch references as output offsets past the
    output's own chunks ("scratch at the end of output", msccl/ncclize.py:690-697) while still
    declaring o_chunks and s_chunks separately, and never names buffer 's'.  In such a rank -- one
    that declares scratch and none of whose steps names 's' -- a local reference past the output's
    end is taken back to the scratch buffer, so the caller's output buffer keeps the size the
    collective gives it.  (On 's' and receive steps the other side's location is informational and
    is left alone.)  Everywhere else an output offset out of range stays what it is: malformed,
    refused when the plan is made.  A step that straddles the output's end is refused here."""
    s_code, o_code = BUF_CODES["s"], BUF_CODES["o"]
    if any((row[0] in _LOCAL_SRC and row[1] == s_code) or (row[0] in _LOCAL_DST and row[3] == s_code) for row in rows):
        return rows
    out = []
    for k, (ty, sb, so, db, do, cnt, depid, deps, hasdep) in enumerate(rows):
        for is_local, buf, off in ((ty in _LOCAL_SRC, sb, so), (ty in _LOCAL_DST, db, do)):
            if is_local and buf == o_code and off < o_chunks < off + cnt:
                raise IRError(f"{where} step {k}: chunks [{off}, {off + cnt}) straddle the end of the output buffer ({o_chunks} chunks)")
        if ty in _LOCAL_SRC and sb == o_code and so >= o_chunks:
            sb, so = s_code, so - o_chunks
        if ty in _LOCAL_DST and db == o_code and do >= o_chunks:
            db, do = s_code, do - o_chunks
        out.append((ty, sb, so, db, do, cnt, depid, deps, hasdep))
    return out


def parse_algo_xml(text):
    """Parse one <algo> document into AlgoTables."""
    try:
        root = ET.fromstring(text)
    except ET.ParseError as e:
        raise IRError(f"not XML: {e}") from None
    if root.tag != "algo":
        raise IRError(f"root element is <{root.tag}>, expected <algo>")
    ngpus = _int(root, "ngpus")
    gpus = {}
    for g in root.findall("gpu"):
        gid = _int(g, "id")
        if gid in gpus:
            raise IRError(f"<gpu id={gid}> appears twice")
        gpus[gid] = g
    if sorted(gpus) != list(range(ngpus)):
        raise IRError(f"gpu ids {sorted(gpus)} do not cover 0..{ngpus - 1}")

    rank_chunks = np.zeros((ngpus, 3), np.int32)
    tb_rows, op_rows = [], []
    for r in range(ngpus):
        g = gpus[r]
        rank_chunks[r] = (_int(g, "i_chunks"), _int(g, "o_chunks"), _int(g, "s_chunks"))
        tbs = {}
        for t in g.findall("tb"):
            tid = _int(t, "id")
            if tid in tbs:
                raise IRError(f"gpu {r}: <tb id={tid}> appears twice")
            tbs[tid] = t
        if sorted(tbs) != list(range(len(tbs))):
            raise IRError(f"gpu {r}: tb ids {sorted(tbs)} are not 0..{len(tbs) - 1}")
        for tid in range(len(tbs)):
            t = tbs[tid]
            steps = t.findall("step")
            begin = len(op_rows)
            for k, st in enumerate(steps):
                if _int(st, "s") != k:
                    raise IRError(f"gpu {r} tb {tid}: step {k} carries s={st.get('s')}")
                ty = st.get("type")
                if ty not in OP_CODES:
                    raise IRError(f"gpu {r} tb {tid} step {k}: unknown type {ty!r}")
                sb, db = st.get("srcbuf", "i"), st.get("dstbuf", "o")
                if sb not in BUF_CODES or db not in BUF_CODES:
                    raise IRError(f"gpu {r} tb {tid} step {k}: unknown buffer {sb!r}/{db!r}")
                op_rows.append((OP_CODES[ty], BUF_CODES[sb], _int(st, "srcoff", -1), BUF_CODES[db], _int(st, "dstoff", -1),
                                _int(st, "cnt", 1 if ty != "nop" else 0), _int(st, "depid", -1), _int(st, "deps", -1),
                                _int(st, "hasdep", 0)))
            tb_rows.append((r, _int(t, "send"), _int(t, "recv"), _int(t, "chan"), begin, len(op_rows)))
        if rank_chunks[r, 2] > 0 and tb_rows and len(tbs):
            first = tb_rows[len(tb_rows) - len(tbs)][4]
            op_rows[first:] = _scratch_behind_output(op_rows[first:], int(rank_chunks[r, 1]), f"gpu {r}:")
    return AlgoTables(
        name=root.get("name", ""), proto=root.get("proto", "Simple"), coll=root.get("coll", "custom"),
        inplace=bool(_int(root, "inplace", 0)), nchannels=_int(root, "nchannels", 0),
        nchunksperloop=_int(root, "nchunksperloop", 0), ngpus=ngpus, rank_chunks=rank_chunks,
        tbs=np.asarray(tb_rows, np.int32).reshape(-1, 6), ops=np.asarray(op_rows, np.int32).reshape(-1, 9))


def load_algo(path):
    with open(path, "r") as f:
        return parse_algo_xml(f.read())
