"""Hand-built MSCCL-IR documents used by the tests (independent of the package's own compiler).

Each builder returns the XML text of one <algo> in the schema of msccl/language/ir.py:320-391.
"""


def _step(s, type, srcbuf="i", srcoff=-1, dstbuf="o", dstoff=-1, cnt=1, depid=-1, deps=-1, hasdep=0):
    return (f'<step s="{s}" type="{type}" srcbuf="{srcbuf}" srcoff="{srcoff}" dstbuf="{dstbuf}" dstoff="{dstoff}" '
            f'cnt="{cnt}" depid="{depid}" deps="{deps}" hasdep="{hasdep}"/>')


def _algo(name, coll, inplace, ngpus, nchannels, nchunksperloop, gpus):
    body = "\n".join(gpus)
    return (f'<algo name="{name}" proto="Simple" nchannels="{nchannels}" nchunksperloop="{nchunksperloop}" '
            f'ngpus="{ngpus}" coll="{coll}" inplace="{inplace}">\n{body}\n</algo>')


def _gpu(rank, i, o, s, tbs):
    return f'<gpu id="{rank}" i_chunks="{i}" o_chunks="{o}" s_chunks="{s}">\n' + "\n".join(tbs) + "\n</gpu>"


def _tb(id, send, recv, chan, steps):
    return f'<tb id="{id}" send="{send}" recv="{recv}" chan="{chan}">\n' + "\n".join(steps) + "\n</tb>"


# The worked example of the reference's fusion test (tests/test_language.py:188-202): 3 ranks, one
# 3-chunk message chained 0 -> 1 -> 2 -> 0 -> 1; op types gpu0 [s, rcs], gpu1 [rrs, r], gpu2 [rrcs].
FUSION_CHAIN_XML = """<algo name="allreduce" proto="Simple" nchannels="1" nchunksperloop="3" ngpus="3" coll="allreduce" inplace="1">
  <gpu id="0" i_chunks="3" o_chunks="0" s_chunks="0">
    <tb id="0" send="1" recv="2" chan="0">
      <step s="0" type="s" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1" hasdep="0"/>
      <step s="1" type="rcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1" hasdep="0"/>
    </tb>
  </gpu>
  <gpu id="1" i_chunks="3" o_chunks="0" s_chunks="0">
    <tb id="0" send="2" recv="0" chan="0">
      <step s="0" type="rrs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1" hasdep="0"/>
      <step s="1" type="r" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1" hasdep="0"/>
    </tb>
  </gpu>
  <gpu id="2" i_chunks="3" o_chunks="0" s_chunks="0">
    <tb id="0" send="0" recv="1" chan="0">
      <step s="0" type="rrcs" srcbuf="i" srcoff="0" dstbuf="i" dstoff="0" cnt="3" depid="-1" deps="-1" hasdep="0"/>
    </tb>
  </gpu>
</algo>"""


def ring_allreduce_xml(n, instances=1):
    """In-place ring all-reduce, one tb per instance and rank.  Instance k works on chunks
    index*instances + k (interleaved replication).  Chunk `index` accumulates ranks index, index+1, ..."""
    gpus = []
    for r in range(n):
        tbs = []
        for k in range(instances):
            def off(index):
                return (index % n) * instances + k
            steps = [("s", off(r))]
            steps += [("rrs", off(r - j)) for j in range(1, n - 1)]
            steps += [("rrcs", off(r + 1))]
            steps += [("rcs", off(r - j)) for j in range(0, n - 2)]
            steps += [("r", off(r - (n - 2)))]
            xml_steps = [_step(s, t, "i", o, "i", o) for s, (t, o) in enumerate(steps)]
            tbs.append(_tb(k, (r + 1) % n, (r - 1) % n, k, xml_steps))
        gpus.append(_gpu(r, n * instances, 0, 0, tbs))
    return _algo("ring_allreduce", "allreduce", 1, n, instances, n * instances, gpus)


def ring_allgather_xml(n, instances=1):
    """In-place ring all-gather ('o' references only); rank r contributes output chunks
    [r*instances, (r+1)*instances)."""
    gpus = []
    for r in range(n):
        tbs = []
        for k in range(instances):
            def off(index):
                return (index % n) * instances + k
            steps = [("s", off(r))] + [("rcs", off(r - j)) for j in range(1, n - 1)] + [("r", off(r - (n - 1)))]
            xml_steps = [_step(s, t, "o", o, "o", o) for s, (t, o) in enumerate(steps)]
            tbs.append(_tb(k, (r + 1) % n, (r - 1) % n, k, xml_steps))
        gpus.append(_gpu(r, 0, n * instances, 0, tbs))
    return _algo("ring_allgather", "allgather", 1, n, instances, n * instances, gpus)


def allpairs_allreduce_xml(n):
    """In-place all-pairs all-reduce over n chunks with scratch, local reductions, cross-threadblock
    dependencies and nops.  Rank r owns chunk r: every peer p sends its chunk r into r's scratch slot,
    r folds the slots into i[r] in ascending peer order, then sends the result to every peer.
    Threadblock p' (index of peer p among r's peers) talks to p both ways; the last tb reduces."""
    gpus = []
    for r in range(n):
        peers = [p for p in range(n) if p != r]
        red_tb = len(peers)
        tbs = []
        nred = len(peers)
        # the reducing tb: one 're' per peer, each waiting for that peer's tb step 1 (the receive)
        red_steps = []
        for k, p in enumerate(peers):
            red_steps.append(_step(k, "re", "s", k, "i", r, 1, depid=k, deps=1, hasdep=1 if k == nred - 1 else 0))
        for k, p in enumerate(peers):
            steps = [
                _step(0, "s", "i", p, "s", 0, 1),
                _step(1, "r", "i", r, "s", k, 1, hasdep=1),
                _step(2, "s", "i", r, "i", r, 1, depid=red_tb, deps=nred - 1),
                _step(3, "r", "i", p, "i", p, 1),
            ]
            tbs.append(_tb(k, p, p, 0, steps))
        tbs.append(_tb(red_tb, -1, -1, 0, red_steps))
        gpus.append(_gpu(r, n, 0, n - 1, tbs))
    return _algo("allpairs_allreduce", "allreduce", 1, n, 1, n, gpus)


def allpairs_orders(n):
    """Fold order of allpairs_allreduce_xml: chunk r = ((in_r + p0) + p1) + ... over peers ascending."""
    return [[r] + [p for p in range(n) if p != r] for r in range(n)]


# Two ranks: rank 0 sends chunk 0; rank 1 reduces it into its own chunk 0 (rrc), then a second
# threadblock copies the sum to the output buffer (cpy) after a nop that carries the dependency.
RRC_CPY_NOP_XML = _algo("rrc_cpy", "custom", 0, 2, 1, 1, [
    _gpu(0, 1, 0, 0, [_tb(0, 1, -1, 0, [_step(0, "s", "i", 0, "i", 0, 1)])]),
    _gpu(1, 1, 1, 0, [
        _tb(0, -1, 0, 0, [_step(0, "rrc", "i", 0, "i", 0, 1, hasdep=1)]),
        _tb(1, -1, -1, 0, [_step(0, "nop", "i", -1, "o", -1, 0, depid=0, deps=0),
                           _step(1, "cpy", "i", 0, "o", 0, 1)]),
    ]),
])


def slow_producer_xml(ncopies):
    """Rank 0 makes `ncopies` local copies of its chunk before it sends it; rank 1 only receives.
    Rank 1's receive therefore waits for as long as the copies take, without any deadlock."""
    steps = [_step(k, "cpy", "i", 0, "o", 0, 1) for k in range(ncopies)] + [_step(ncopies, "s", "i", 0, "o", 0, 1)]
    return _algo("slow_producer", "custom", 0, 2, 1, 1, [
        _gpu(0, 1, 1, 0, [_tb(0, 1, -1, 0, steps)]),
        _gpu(1, 1, 1, 0, [_tb(0, -1, 0, 0, [_step(0, "r", "i", 0, "o", 0, 1)])]),
    ])


def slow_dependency_xml(ncopies):
    """One rank.  Threadblock 0 makes `ncopies` copies of its chunk; threadblock 1 waits for the first
    and for the last of them through two nop steps (the way msccl-tools gives a step several
    dependencies, msccl/language/ir.py:296-311) and then copies the result on: its step 2 waits for as
    long as the copies take."""
    tb0 = [_step(k, "cpy", "i", 0, "o", 0, 1, hasdep=1 if k in (0, ncopies - 1) else 0) for k in range(ncopies)]
    tb1 = [_step(0, "nop", "i", -1, "o", -1, 0, depid=0, deps=0), _step(1, "nop", "i", -1, "o", -1, 0, depid=0, deps=ncopies - 1),
           _step(2, "cpy", "o", 0, "o", 1, 1)]
    return _algo("slow_dependency", "custom", 0, 1, 1, 2, [_gpu(0, 1, 2, 0, [_tb(0, -1, -1, 0, tb0), _tb(1, -1, -1, 0, tb1)])])


def reduce_chain_xml(m, stride):
    """One rank.  Threadblock 0 folds `m` chunks of its input, `stride` chunks apart, into chunk 0 with
    `m` reduce steps in a row (the shape of msccl-tools' msccl/programs/allreduce_allpairs.py:18-21),
    after a nop that waits for threadblock 1's first copy; threadblock 2 does the same into chunk 1 with
    its sources in descending order; threadblock 1 copies both results out when they are complete."""
    last = 2 + (m - 1) * stride
    up = [_step(0, "nop", "i", -1, "o", -1, 0, depid=1, deps=0)] + \
         [_step(1 + k, "re", "i", 2 + k * stride, "i", 0, 1, hasdep=1 if k == m - 1 else 0) for k in range(m)]
    down = [_step(0, "nop", "i", -1, "o", -1, 0, depid=1, deps=0)] + \
           [_step(1 + k, "re", "i", last - k * stride, "i", 1, 1, hasdep=1 if k == m - 1 else 0) for k in range(m)]
    out = [_step(0, "cpy", "i", 2, "o", 2, 1, hasdep=1), _step(1, "nop", "i", -1, "o", -1, 0, depid=0, deps=m),
           _step(2, "cpy", "i", 0, "o", 0, 1, depid=2, deps=m), _step(3, "cpy", "i", 1, "o", 1, 1)]
    return _algo("reduce_chain", "custom", 0, 1, 1, last + 1,
                 [_gpu(0, last + 1, 3, 0, [_tb(0, -1, -1, 0, up), _tb(1, -1, -1, 0, out), _tb(2, -1, -1, 0, down)])])


# ---- documents in the style of msccl-tools' second emitter (msccl/ncclize.py:658-718) ----------
# inplace="0", only s / r / rrc / cpy / nop, sending and receiving threadblocks separate, one extra
# threadblock per rank (send=recv=-1, chan 0) holding the pre/post copies, and on r / rrc steps
# srcbuf/srcoff naming the SENDER's location (ncclize.py:534-535).
def ncclize_style_allgather_xml(n=3):
    """Ring all-gather out of place: the copy threadblock puts i[0] into o[r]; chunk k travels
    k -> k+1 -> ...; forwarding sends wait for the receive that delivered the chunk."""
    gpus = []
    for r in range(n):
        nxt, prv = (r + 1) % n, (r - 1) % n
        send_steps, recv_steps = [], []
        for h in range(n - 1):
            c_out, c_in = (r - h) % n, (r - 1 - h) % n
            if h == 0:
                send_steps.append(_step(h, "s", "i", 0, "o", c_out, 1))
                recv_steps.append(_step(h, "r", "i", 0, "o", c_in, 1, hasdep=1 if n > 2 else 0))
            else:
                send_steps.append(_step(h, "s", "o", c_out, "o", c_out, 1, depid=1, deps=h - 1))
                recv_steps.append(_step(h, "r", "o", c_in, "o", c_in, 1, hasdep=1 if h < n - 2 else 0))
        gpus.append(_gpu(r, 1, n, 0, [_tb(0, nxt, -1, 0, send_steps), _tb(1, -1, prv, 0, recv_steps),
                                     _tb(2, -1, -1, 0, [_step(0, "cpy", "i", 0, "o", r, 1)])]))
    return _algo("ncclize_allgather", "allgather", 0, n, 1, n, gpus)


def ncclize_style_allreduce_xml():
    """3 ranks, 1 chunk, out of place: every rank copies i[0] to o[0]; ranks 1 and 2 send i[0] to rank
    0, which reduces them into o[0] in that order (rrc, the second waiting for the first); rank 0 then
    sends o[0] to both, whose receives wait for their own copy.  Result everywhere: (x0 + x1) + x2."""
    g0 = _gpu(0, 1, 1, 0, [
        _tb(0, 1, -1, 0, [_step(0, "s", "o", 0, "o", 0, 1, depid=3, deps=0)]),
        _tb(1, 2, -1, 0, [_step(0, "s", "o", 0, "o", 0, 1, depid=3, deps=0)]),
        _tb(2, -1, 1, 0, [_step(0, "rrc", "i", 0, "o", 0, 1, depid=4, deps=0, hasdep=1)]),
        _tb(3, -1, 2, 0, [_step(0, "rrc", "i", 0, "o", 0, 1, depid=2, deps=0, hasdep=1)]),
        _tb(4, -1, -1, 0, [_step(0, "cpy", "i", 0, "o", 0, 1, hasdep=1)]),
    ])
    def leaf(rank):
        return _gpu(rank, 1, 1, 0, [
            _tb(0, 0, -1, 0, [_step(0, "s", "i", 0, "o", 0, 1)]),
            _tb(1, -1, 0, 0, [_step(0, "r", "o", 0, "o", 0, 1, depid=2, deps=0)]),
            _tb(2, -1, -1, 0, [_step(0, "cpy", "i", 0, "o", 0, 1, hasdep=1)]),
        ])
    return _algo("ncclize_allreduce", "allreduce", 0, 3, 1, 1, [g0, leaf(1), leaf(2)])


def relay_through_scratch_xml(out_off=0, out_cnt=1, name_scratch=True):
    """2 ranks, out of place: rank 0 sends i[0..1] to rank 1, which receives them into scratch
    (name_scratch: as s[0..1], the way the MSCCLang emitter writes scratch; else as o[1..2], "scratch at
    the end of output", the way ncclize(use_scratch=False) does) and copies `out_cnt` of them to
    o[out_off..].  Rank 1 declares one output chunk and two scratch chunks."""
    sbuf, soff = ("s", 0) if name_scratch else ("o", 1)
    g0 = _gpu(0, 2, 0, 0, [_tb(0, 1, -1, 0, [_step(0, "s", "i", 0, sbuf, soff, 2)])])
    g1 = _gpu(1, 0, 1, 2, [_tb(0, -1, 0, 0, [_step(0, "r", "i", 0, sbuf, soff, 2, hasdep=1)]),
                           _tb(1, -1, -1, 0, [_step(0, "cpy", sbuf, soff, "o", out_off, out_cnt, depid=0, deps=0)])])
    return _algo("relay_through_scratch", "custom", 0, 2, 1, 2, [g0, g1])
