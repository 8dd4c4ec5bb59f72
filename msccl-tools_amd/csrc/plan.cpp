// Host side of the MSCCL-IR executor: table validation, connection matching, dry run, geometry.
// Nothing in this file touches the GPU, so it is exercised by CPU-only tests through the C ABI.
#include "plan.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <queue>
#include <sstream>
#include <tuple>

namespace mscclx {

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }
int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}

int dtype_size(int dtype) {
  switch (dtype) {
    case MSCCLX_U8: case MSCCLX_I8: return 1;
    case MSCCLX_F16: case MSCCLX_BF16: return 2;
    case MSCCLX_I32: case MSCCLX_U32: case MSCCLX_F32: return 4;
    case MSCCLX_I64: case MSCCLX_U64: case MSCCLX_F64: return 8;
    default: return 0;
  }
}

// algorithmic traffic factor per step type: one read + one write per transfer edge (booked at the
// receiving step) and one more operand read per reduction.
static int algo_factor(int type) {
  switch (type) {
    case MSCCLX_OP_RECV: case MSCCLX_OP_RCS: case MSCCLX_OP_COPY: return 2;
    case MSCCLX_OP_RRC: case MSCCLX_OP_RRS: case MSCCLX_OP_RRCS: case MSCCLX_OP_REDUCE: return 3;
    default: return 0;
  }
}

static const char* op_name(int t) {
  static const char* names[] = {"nop", "s", "r", "rcs", "rrs", "rrc", "rrcs", "cpy", "re"};
  return (t >= 0 && t <= 8) ? names[t] : "?";
}

static std::string where(const mscclx_plan& p, int tb_row, int step) {
  std::ostringstream os;
  os << "rank " << p.tbs[tb_row].rank << " tb " << p.tbs[tb_row].local_id << " step " << step;
  return os.str();
}

// One pass of all step lists with `depth` messages per connection (0 = unbounded).  The program is
// a deterministic dataflow network (FIFOs + monotone step counters), so whether it finishes does
// not depend on the order in which ready threadblocks are advanced.
int simulate(const mscclx_plan& plan, int depth) {
  const int ntb = (int)plan.tbs.size();
  std::vector<int> pc(ntb, 0);
  std::vector<int64_t> head(plan.conns.size(), 0), tail(plan.conns.size(), 0);
  size_t remaining = plan.ops.size();
  while (remaining) {
    size_t progressed = 0;
    for (int t = 0; t < ntb; ++t) {
      const Tb& tb = plan.tbs[t];
      const int n = tb.op_end - tb.op_begin;
      while (pc[t] < n) {
        const Op& op = plan.ops[tb.op_begin + pc[t]];
        if (op.depid >= 0) {
          const int dep_row = plan.rank_tb_begin[tb.rank] + op.depid;
          if (!(pc[dep_row] > op.deps)) break;
        }
        const bool rcv = is_recv_type(op.type), snd = is_send_type(op.type);
        if (rcv && head[tb.recv_conn] <= tail[tb.recv_conn]) break;
        if (snd && depth > 0 && head[tb.send_conn] - tail[tb.send_conn] >= depth) break;
        if (rcv) ++tail[tb.recv_conn];
        if (snd) ++head[tb.send_conn];
        ++pc[t];
        ++progressed;
      }
    }
    if (!progressed) {
      std::ostringstream os;
      os << "deadlock with connection depth " << depth << "; blocked:";
      int shown = 0;
      for (int t = 0; t < ntb && shown < 6; ++t) {
        const Tb& tb = plan.tbs[t];
        if (pc[t] < tb.op_end - tb.op_begin) {
          os << " [" << where(plan, t, pc[t]) << " " << op_name(plan.ops[tb.op_begin + pc[t]].type) << "]";
          ++shown;
        }
      }
      return fail(MSCCLX_ERR_DEADLOCK, os.str());
    }
    remaining -= progressed;
  }
  return MSCCLX_OK;
}

// Which messages need no FIFO slot.  The payload of a send-type step already sits at a fixed place on
// the sending rank: the source chunks of an 's', or the local destination an 'rcs'/'rrcs' has just
// written ('rrs' keeps no local copy, so its payload exists only in the slot).  The receiver may
// read it from there if no step of the sending rank can overwrite those chunks before the matching
// receive has run.  That is decided on the program's happens-before graph -- step order inside a
// threadblock, depid/deps waits, and send -> matching receive -- which holds in every execution:
// every later writer W of the chunks must be reachable from the matching receive R (then W cannot
// start before R has finished), and every other writer must be an ancestor of the send.
static void find_zero_copy_messages(mscclx_plan* p) {
  const int n = (int)p->ops.size();
  std::vector<int> tb_of(n), rank_of(n);
  for (int t = 0; t < (int)p->tbs.size(); ++t)
    for (int o = p->tbs[t].op_begin; o < p->tbs[t].op_end; ++o) { tb_of[o] = t; rank_of[o] = p->tbs[t].rank; }
  std::vector<std::vector<int>> succ(n), pred(n);
  auto edge = [&](int a, int b) { succ[a].push_back(b); pred[b].push_back(a); };
  for (int t = 0; t < (int)p->tbs.size(); ++t) {
    const Tb& tb = p->tbs[t];
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      if (o + 1 < tb.op_end) edge(o, o + 1);
      const Op& op = p->ops[o];
      if (op.depid >= 0) edge(p->tbs[p->rank_tb_begin[tb.rank] + op.depid].op_begin + op.deps, o);
      if (is_send_type(op.type)) edge(o, op.match_recv);
    }
  }
  // local writers per (rank, buffer)
  struct Writer { int op, lo, hi; };
  std::vector<std::vector<Writer>> writers((size_t)p->nranks * 3);
  for (int o = 0; o < n; ++o) {
    const Op& op = p->ops[o];
    if (touches_local_dst(op.type) && op.type != MSCCLX_OP_RRS)
      writers[(size_t)rank_of[o] * 3 + op.dstbuf].push_back({o, op.dstoff, op.dstoff + op.cnt});
  }
  std::vector<uint32_t> mark_back(n, 0), mark_fwd(n, 0);
  uint32_t epoch = 0;
  std::vector<int> stack;
  auto reach = [&](int from, const std::vector<std::vector<int>>& adj, std::vector<uint32_t>& mark) {
    stack.assign(1, from);
    mark[from] = epoch;
    while (!stack.empty()) {
      int v = stack.back();
      stack.pop_back();
      for (int w : adj[v])
        if (mark[w] != epoch) { mark[w] = epoch; stack.push_back(w); }
    }
  };
  std::vector<int> later;
  for (int s = 0; s < n; ++s) {
    Op& op = p->ops[s];
    if (!is_send_type(op.type) || op.type == MSCCLX_OP_RRS) continue;
    const bool from_src = op.type == MSCCLX_OP_SEND;
    const int buf = from_src ? op.srcbuf : op.dstbuf;
    const int lo = from_src ? op.srcoff : op.dstoff, hi = lo + op.cnt;
    later.clear();
    for (const Writer& w : writers[(size_t)rank_of[s] * 3 + buf])
      if (w.op != s && w.lo < hi && lo < w.hi) later.push_back(w.op);
    if (!later.empty()) {
      ++epoch;
      reach(s, pred, mark_back);  // ancestors of the send wrote before it read
      size_t k = 0;
      for (int w : later)
        if (mark_back[w] != epoch) later[k++] = w;
      later.resize(k);
    }
    if (!later.empty()) {
      reach(op.match_recv, succ, mark_fwd);
      bool safe = true;
      for (int w : later)
        if (mark_fwd[w] != epoch) { safe = false; break; }
      if (!safe) continue;
    }
    op.zero_copy = 1;
  }
}

// Local destinations nobody reads: not as a local source ('s', 'cpy', 're'), not as the accumulator
// of a reduction, not by a peer reading a forwarded payload in place.  Conservative: a read anywhere
// in the program, before or after the write, keeps the write cacheable.
static void find_final_writes(mscclx_plan* p) {
  typedef std::pair<int, int> Span;  // [lo, hi) in chunks
  std::vector<std::vector<Span>> reads((size_t)p->nranks * 3);
  for (const Tb& tb : p->tbs)
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const Op& op = p->ops[o];
      if (reads_local_src(op.type)) reads[(size_t)tb.rank * 3 + op.srcbuf].push_back({op.srcoff, op.srcoff + op.cnt});
      if (is_reduce_type(op.type) || op.type == MSCCLX_OP_RCS) reads[(size_t)tb.rank * 3 + op.dstbuf].push_back({op.dstoff, op.dstoff + op.cnt});
    }
  // merge into disjoint sorted spans
  for (auto& v : reads) {
    std::sort(v.begin(), v.end());
    size_t k = 0;
    for (const Span& s : v) {
      if (k && s.first <= v[k - 1].second) v[k - 1].second = std::max(v[k - 1].second, s.second);
      else v[k++] = s;
    }
    v.resize(k);
  }
  for (const Tb& tb : p->tbs)
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      Op& op = p->ops[o];
      if (!touches_local_dst(op.type) || op.type == MSCCLX_OP_RRS) continue;
      const std::vector<Span>& v = reads[(size_t)tb.rank * 3 + op.dstbuf];
      const int lo = op.dstoff, hi = op.dstoff + op.cnt;
      auto it = std::upper_bound(v.begin(), v.end(), Span{lo, 0x7fffffff});  // first span starting after lo
      bool any = it != v.end() && it->first < hi;
      if (it != v.begin() && std::prev(it)->second > lo) any = true;
      op.final_write = any ? 0 : 1;
    }
}

static int build_plan(const mscclx_plan_desc* d, mscclx_plan* p) {
  if (d->nranks <= 0 || d->ntbs < 0 || d->nops < 0) return fail(MSCCLX_ERR_INVALID_ARG, "negative table size");
  if (!d->rank_chunks || (d->ntbs && !d->tbs) || (d->nops && !d->ops)) return fail(MSCCLX_ERR_INVALID_ARG, "null table pointer");
  p->nranks = d->nranks;
  p->rank_chunks.assign(d->rank_chunks, d->rank_chunks + (size_t)d->nranks * 3);
  for (int32_t v : p->rank_chunks)
    if (v < 0) return fail(MSCCLX_ERR_BAD_IR, "negative buffer extent");

  p->tbs.resize(d->ntbs);
  p->ops.resize(d->nops);
  p->rank_tb_begin.assign(d->nranks + 1, 0);
  int prev_rank = 0, expect_begin = 0;
  for (int t = 0; t < d->ntbs; ++t) {
    const int32_t* r = d->tbs + (size_t)t * MSCCLX_TB_COLS;
    Tb& tb = p->tbs[t];
    tb.rank = r[0]; tb.send = r[1]; tb.recv = r[2]; tb.chan = r[3]; tb.op_begin = r[4]; tb.op_end = r[5];
    if (tb.rank < 0 || tb.rank >= d->nranks) return fail(MSCCLX_ERR_BAD_IR, "threadblock row " + std::to_string(t) + ": rank out of range");
    if (tb.rank < prev_rank) return fail(MSCCLX_ERR_BAD_IR, "threadblock rows must be grouped by ascending rank");
    if (tb.send < -1 || tb.send >= d->nranks || tb.recv < -1 || tb.recv >= d->nranks)
      return fail(MSCCLX_ERR_BAD_IR, "threadblock row " + std::to_string(t) + ": peer out of range");
    if (tb.send == tb.rank || tb.recv == tb.rank) return fail(MSCCLX_ERR_BAD_IR, "threadblock row " + std::to_string(t) + ": a rank cannot be its own peer");
    if (tb.chan < 0) return fail(MSCCLX_ERR_BAD_IR, "threadblock row " + std::to_string(t) + ": negative channel");
    if (tb.op_begin != expect_begin || tb.op_end < tb.op_begin || tb.op_end > d->nops)
      return fail(MSCCLX_ERR_BAD_IR, "threadblock row " + std::to_string(t) + ": step ranges must tile the op table in order");
    expect_begin = tb.op_end;
    prev_rank = tb.rank;
    p->rank_tb_begin[tb.rank + 1]++;
  }
  if (expect_begin != d->nops) return fail(MSCCLX_ERR_BAD_IR, "op table has rows no threadblock owns");
  for (int r = 0; r < d->nranks; ++r) p->rank_tb_begin[r + 1] += p->rank_tb_begin[r];
  for (int t = 0; t < d->ntbs; ++t) p->tbs[t].local_id = t - p->rank_tb_begin[p->tbs[t].rank];

  // steps
  for (int t = 0; t < d->ntbs; ++t) {
    Tb& tb = p->tbs[t];
    const int ntb_rank = p->rank_tb_begin[tb.rank + 1] - p->rank_tb_begin[tb.rank];
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const int32_t* r = d->ops + (size_t)o * MSCCLX_OP_COLS;
      Op& op = p->ops[o];
      op.type = r[0]; op.srcbuf = r[1]; op.srcoff = r[2]; op.dstbuf = r[3]; op.dstoff = r[4];
      op.cnt = r[5]; op.depid = r[6]; op.deps = r[7]; op.hasdep = r[8] ? 1 : 0;
      const std::string at = where(*p, t, o - tb.op_begin);
      if (op.type < MSCCLX_OP_NOP || op.type > MSCCLX_OP_REDUCE) return fail(MSCCLX_ERR_BAD_IR, at + ": unknown step type " + std::to_string(op.type));
      if (op.type != MSCCLX_OP_NOP && op.cnt < 1) return fail(MSCCLX_ERR_BAD_IR, at + ": cnt must be >= 1");
      if (op.cnt >= (1 << 24)) return fail(MSCCLX_ERR_BAD_IR, at + ": cnt must be below 2^24");
      auto check_ref = [&](int buf, int off, const char* what) -> int {
        if (buf < 0 || buf > 2) return fail(MSCCLX_ERR_BAD_IR, at + ": bad " + what + " buffer");
        const int extent = p->rank_chunks[(size_t)tb.rank * 3 + buf];
        if (off < 0 || (int64_t)off + op.cnt > extent)
          return fail(MSCCLX_ERR_BAD_IR, at + ": " + what + " chunks [" + std::to_string(off) + "," + std::to_string((int64_t)off + op.cnt) +
                                             ") outside the buffer's " + std::to_string(extent) + " chunks");
        return MSCCLX_OK;
      };
      int rc;
      if (reads_local_src(op.type) && (rc = check_ref(op.srcbuf, op.srcoff, "source"))) return rc;
      if (touches_local_dst(op.type) && (rc = check_ref(op.dstbuf, op.dstoff, "destination"))) return rc;
      if (is_send_type(op.type)) {
        if (tb.send < 0) return fail(MSCCLX_ERR_BAD_IR, at + ": sending step in a threadblock without a send peer");
        op.send_seq = tb.nsend++;
      }
      if (is_recv_type(op.type)) {
        if (tb.recv < 0) return fail(MSCCLX_ERR_BAD_IR, at + ": receiving step in a threadblock without a recv peer");
        op.recv_seq = tb.nrecv++;
      }
      if (is_reduce_type(op.type)) p->has_reduce = true;
      if ((op.depid < 0) != (op.deps < 0)) return fail(MSCCLX_ERR_BAD_IR, at + ": depid and deps must both be set or both be -1");
      if (op.depid >= 0) {
        if (op.depid >= ntb_rank) return fail(MSCCLX_ERR_BAD_IR, at + ": depid names no threadblock of this rank");
        const Tb& dep = p->tbs[p->rank_tb_begin[tb.rank] + op.depid];
        if (op.deps >= dep.op_end - dep.op_begin) return fail(MSCCLX_ERR_BAD_IR, at + ": deps beyond the last step of threadblock " + std::to_string(op.depid));
      }
      p->algorithmic_units += (uint64_t)op.cnt * algo_factor(op.type);
    }
  }
  // A step somebody waits for must publish its completion even if the emitter forgot hasdep.
  for (int t = 0; t < d->ntbs; ++t) {
    const Tb& tb = p->tbs[t];
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const Op& op = p->ops[o];
      if (op.depid >= 0) {
        const Tb& dep = p->tbs[p->rank_tb_begin[tb.rank] + op.depid];
        p->ops[dep.op_begin + op.deps].hasdep = 1;
      }
    }
  }

  // connections: exactly one producing and one consuming threadblock per (src, dst, chan)
  std::map<std::tuple<int, int, int>, int> conn_id;
  auto get_conn = [&](int src, int dst, int chan) {
    auto key = std::make_tuple(src, dst, chan);
    auto it = conn_id.find(key);
    if (it != conn_id.end()) return it->second;
    Conn c; c.src = src; c.dst = dst; c.chan = chan;
    p->conns.push_back(c);
    return conn_id[key] = (int)p->conns.size() - 1;
  };
  for (int t = 0; t < d->ntbs; ++t) {
    Tb& tb = p->tbs[t];
    if (tb.nsend) {
      const int c = get_conn(tb.rank, tb.send, tb.chan);
      if (p->conns[c].send_tb >= 0)
        return fail(MSCCLX_ERR_BAD_IR, "rank " + std::to_string(tb.rank) + ": threadblocks " + std::to_string(p->tbs[p->conns[c].send_tb].local_id) + " and " +
                                           std::to_string(tb.local_id) + " both send to rank " + std::to_string(tb.send) + " on channel " + std::to_string(tb.chan));
      p->conns[c].send_tb = t;
      tb.send_conn = c;
    }
    if (tb.nrecv) {
      const int c = get_conn(tb.recv, tb.rank, tb.chan);
      if (p->conns[c].recv_tb >= 0)
        return fail(MSCCLX_ERR_BAD_IR, "rank " + std::to_string(tb.rank) + ": threadblocks " + std::to_string(p->tbs[p->conns[c].recv_tb].local_id) + " and " +
                                           std::to_string(tb.local_id) + " both receive from rank " + std::to_string(tb.recv) + " on channel " + std::to_string(tb.chan));
      p->conns[c].recv_tb = t;
      tb.recv_conn = c;
    }
  }
  for (size_t c = 0; c < p->conns.size(); ++c) {
    Conn& cn = p->conns[c];
    std::ostringstream name;
    name << "connection " << cn.src << "->" << cn.dst << " channel " << cn.chan;
    if (cn.send_tb < 0) return fail(MSCCLX_ERR_BAD_IR, name.str() + " has a receiver but no sender");
    if (cn.recv_tb < 0) return fail(MSCCLX_ERR_BAD_IR, name.str() + " has a sender but no receiver");
    const Tb& s = p->tbs[cn.send_tb];
    const Tb& r = p->tbs[cn.recv_tb];
    if (s.nsend != r.nrecv)
      return fail(MSCCLX_ERR_BAD_IR, name.str() + ": " + std::to_string(s.nsend) + " sends but " + std::to_string(r.nrecv) + " receives");
    cn.nmsg = s.nsend;
    int ro = r.op_begin;
    for (int so = s.op_begin; so < s.op_end; ++so) {
      if (!is_send_type(p->ops[so].type)) continue;
      while (!is_recv_type(p->ops[ro].type)) ++ro;
      if (p->ops[so].cnt != p->ops[ro].cnt)
        return fail(MSCCLX_ERR_BAD_IR, name.str() + ": message " + std::to_string(p->ops[so].send_seq) + " is sent with cnt " + std::to_string(p->ops[so].cnt) +
                                           " but received with cnt " + std::to_string(p->ops[ro].cnt));
      cn.max_cnt = std::max(cn.max_cnt, p->ops[so].cnt);
      p->ops[so].match_recv = ro;
      p->ops[ro].match_send = so;
      ++ro;
    }
  }
  find_zero_copy_messages(p);
  find_final_writes(p);
  for (Conn& cn : p->conns) {
    const Tb& s = p->tbs[cn.send_tb];
    for (int so = s.op_begin; so < s.op_end; ++so)
      if (is_send_type(p->ops[so].type) && !p->ops[so].zero_copy) cn.max_staged_cnt = std::max(cn.max_staged_cnt, p->ops[so].cnt);
  }
  return MSCCLX_OK;
}

static int thread_index(int threads) {
  switch (threads) { case 64: return 0; case 128: return 1; case 256: return 2; case 512: return 3; case 1024: return 4; default: return -1; }
}

// bytes a threadblock moves per chunk-sized unit of its steps, given which payloads are staged
static uint64_t tb_work(const mscclx_plan& plan, const Tb& tb, bool staging) {
  uint64_t w = 0;
  for (int o = tb.op_begin; o < tb.op_end; ++o) {
    const Op& op = plan.ops[o];
    const bool staged_out = is_send_type(op.type) && (staging || !op.zero_copy);
    int units = 0;
    switch (op.type) {
      case MSCCLX_OP_SEND: units = staged_out ? 2 : 0; break;
      case MSCCLX_OP_RECV: case MSCCLX_OP_COPY: units = 2; break;
      case MSCCLX_OP_RCS: units = staged_out ? 3 : 2; break;
      case MSCCLX_OP_RRC: case MSCCLX_OP_RRS: case MSCCLX_OP_REDUCE: units = 3; break;
      case MSCCLX_OP_RRCS: units = staged_out ? 4 : 3; break;
      default: break;
    }
    w += (uint64_t)units * op.cnt;
  }
  return w;
}

constexpr uint64_t kWidePieceBytes = 96 * 1024;  // pieces from which a workgroup of 1024 threads pays, for the programs it pays for at all
// threads: enough to cover a piece with a few 16-byte loads per thread
static int threads_for_piece(uint64_t piece_bytes) {
  return piece_bytes >= 48 * 1024 ? 512 : piece_bytes >= 24 * 1024 ? 256 : piece_bytes >= 12 * 1024 ? 128 : 64;
}

// How many threadblocks there are for every threadblock that is busy, on average, while the program
// runs: threadblocks x depth of the dataflow / moving steps, where the depth is the longest chain of
// moving steps through step order, depid/deps and send -> matching receive (connections unbounded).
// 1 = every threadblock always has something to do (a ring); a program in phases, or one whose
// threadblocks mostly wait for each other, scores higher and needs more contexts per workgroup for a
// workgroup to find a ready one.
static double waiting_ratio(const mscclx_plan& plan, int32_t* depth_out = nullptr) {
  const int ntb = (int)plan.tbs.size();
  std::vector<int> pc(ntb, 0);
  std::vector<int32_t> level(plan.ops.size(), -1);
  size_t remaining = plan.ops.size();
  int64_t moving = 0;
  int32_t depth = 0;
  while (remaining) {
    size_t progressed = 0;
    for (int t = 0; t < ntb; ++t) {
      const Tb& tb = plan.tbs[t];
      while (tb.op_begin + pc[t] < tb.op_end) {
        const int o = tb.op_begin + pc[t];
        const Op& op = plan.ops[o];
        int32_t l = pc[t] ? level[o - 1] : 0;
        if (op.depid >= 0) {
          const Tb& dep = plan.tbs[plan.rank_tb_begin[tb.rank] + op.depid];
          const int32_t dl = level[dep.op_begin + op.deps];
          if (dl < 0) break;
          l = std::max(l, dl);
        }
        if (is_recv_type(op.type)) {
          const int32_t sl = level[op.match_send];
          if (sl < 0) break;
          l = std::max(l, sl);
        }
        const bool moves = op.type != MSCCLX_OP_NOP && !(op.type == MSCCLX_OP_SEND && op.zero_copy);
        level[o] = l + (moves ? 1 : 0);
        moving += moves ? 1 : 0;
        depth = std::max(depth, level[o]);
        ++pc[t];
        ++progressed;
      }
    }
    if (!progressed) { if (depth_out) *depth_out = 1; return 1.0; }  // (a program that cannot finish is refused elsewhere)
    remaining -= progressed;
  }
  if (depth_out) *depth_out = std::max<int32_t>(1, depth);
  return moving ? std::max(1.0, (double)ntb * (double)depth / (double)moving) : 1.0;
}

// How evenly longest-processing-time-first spreads `slices` copies of every threadblock over `wgs`
// workgroups of at most kMaxHosted contexts: mean load / largest load, 1 = perfectly even.
static double hosting_balance(const std::vector<uint64_t>& tb_works, int64_t slices, int64_t wgs) {
  std::vector<uint64_t> sorted(tb_works);
  std::sort(sorted.begin(), sorted.end(), std::greater<uint64_t>());
  typedef std::pair<uint64_t, int> Load;  // (work so far, contexts so far)
  std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
  for (int64_t w = 0; w < wgs; ++w) heap.push({0, 0});
  uint64_t total = 0, largest = 0;
  for (uint64_t work : sorted)
    for (int64_t j = 0; j < slices; ++j) {
      if (heap.empty()) return 0.0;
      Load l = heap.top();
      heap.pop();
      l.first += work + 1;  // the weights the hosting table itself is built with
      l.second += 1;
      total += work + 1;
      largest = std::max(largest, l.first);
      if (l.second < kMaxHosted) heap.push(l);
    }
  return largest ? (double)total / (double)wgs / (double)largest : 1.0;
}

// The share of a program's algorithmic bytes that memory sees once only: reads of chunks no step of the program writes
// (the collective's inputs) and writes of chunks no step reads again (its results).  Everything else is written by one step
// and read by another soon after, out of the memory-side cache.  A ring re-reads nearly all it writes (all-gather ring of 8
// ranks: 0.25); an all-to-all reads its input cold and writes its output for good (one-step: 1.0; hierarchical, a third of
// whose bytes pass through scratch: 0.67); the all-pairs programs lie between.
double cold_fraction(const mscclx_plan& plan) {
  typedef std::pair<int, int> Span;  // [lo, hi) in chunks
  std::vector<std::vector<Span>> written((size_t)plan.nranks * 3);
  for (const Tb& tb : plan.tbs)
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const Op& op = plan.ops[o];
      if (touches_local_dst(op.type) && op.type != MSCCLX_OP_RRS) written[(size_t)tb.rank * 3 + op.dstbuf].push_back({op.dstoff, op.dstoff + op.cnt});
    }
  for (auto& v : written) {
    std::sort(v.begin(), v.end());
    size_t k = 0;
    for (const Span& sp : v) {
      if (k && sp.first <= v[k - 1].second) v[k - 1].second = std::max(v[k - 1].second, sp.second);
      else v[k++] = sp;
    }
    v.resize(k);
  }
  auto never_written = [&](int rank, int buf, int lo, int cnt) {  // chunks of [lo, lo + cnt) outside every written span
    if (buf < 0 || buf > 2) return 0;
    int covered = 0;
    for (const Span& sp : written[(size_t)rank * 3 + buf]) covered += std::max(0, std::min(sp.second, lo + cnt) - std::max(sp.first, lo));
    return cnt - covered;
  };
  uint64_t total = 0, cold = 0;
  for (const Tb& tb : plan.tbs)
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const Op& op = plan.ops[o];
      if (op.cnt <= 0) continue;
      if (op.type == MSCCLX_OP_COPY || op.type == MSCCLX_OP_REDUCE) {  // the local source
        total += op.cnt;
        cold += never_written(tb.rank, op.srcbuf, op.srcoff, op.cnt);
      }
      if (is_recv_type(op.type) && op.match_send >= 0) {              // the payload, where the sender had it
        const Op& sender = plan.ops[op.match_send];
        const int sender_rank = plan.tbs[plan.conns[tb.recv_conn].send_tb].rank;
        total += op.cnt;
        if (sender.type == MSCCLX_OP_SEND) cold += never_written(sender_rank, sender.srcbuf, sender.srcoff, op.cnt);
      }
      if (is_reduce_type(op.type)) total += op.cnt;                     // the local operand: written by this very step, at the least
      if (touches_local_dst(op.type) && op.type != MSCCLX_OP_RRS) {     // the local destination
        total += op.cnt;
        if (op.final_write) cold += op.cnt;
      }
      if (op.type == MSCCLX_OP_RRS) total += op.cnt;                    // its result, handed on
    }
  return total ? (double)cold / (double)total : 0.0;
}

bool has_foldable_nops(const mscclx_plan& plan) {
  for (const Tb& tb : plan.tbs)
    for (int o = tb.op_begin; o + 1 < tb.op_end; ++o)
      if (plan.ops[o].type == MSCCLX_OP_NOP && !plan.ops[o].hasdep) return true;
  return false;
}

bool one_wave_each(const Geometry& g) {
  if (g.threads != 64 || g.wg_begin.size() != g.ctx_tb.size() + 1) return false;
  for (size_t w = 0; w < g.wg_begin.size(); ++w)
    if (g.wg_begin[w] != (int32_t)w) return false;
  return true;
}

int decide_geometry(mscclx_plan& plan, size_t chunk_bytes, int dtype, const mscclx_config& cfg,
                    int num_cus, const int capacity_by_threads[kThreadChoices], uint64_t fifo_budget_bytes, Geometry* out) {
  const int elem = dtype_size(dtype);
  if (!elem) return fail(MSCCLX_ERR_INVALID_ARG, "unknown dtype " + std::to_string(dtype));
  if (chunk_bytes == 0 || chunk_bytes % elem) return fail(MSCCLX_ERR_INVALID_ARG, "chunk_bytes must be a positive multiple of the element size");
  if (cfg.slices < 0 || cfg.piece_bytes < 0 || cfg.fifo_depth < 0 || cfg.workgroups < 0 || cfg.threads < 0)
    return fail(MSCCLX_ERR_INVALID_ARG, "geometry knobs must be >= 0");
  Geometry g;
  // Every chunk moves in 16-byte units, whatever its size: rows start wherever their chunk starts (multi-dword
  // accesses need no alignment), the last unit of a chunk may be partial -- down to a single byte.
  g.vector_path = 1;
  g.unit_bytes = 16;
  g.chunk_units = (chunk_bytes + g.unit_bytes - 1) / g.unit_bytes;
  if (cfg.protocol < 0 || cfg.protocol > MSCCLX_PROTO_LL) return fail(MSCCLX_ERR_INVALID_ARG, "unknown protocol");
  if (cfg.protocol == MSCCLX_PROTO_LL && chunk_bytes % 4) return fail(MSCCLX_ERR_UNSUPPORTED, "the LL protocol needs chunks that are a multiple of 4 bytes");
  g.staging = cfg.staging ? 1 : 0;
  const int64_t ntbs = (int64_t)plan.tbs.size();
  if (ntbs == 0) return fail(MSCCLX_ERR_BAD_IR, "the algorithm has no threadblocks");

  // connection depth: as asked (must not deadlock), else the smallest that works, at least 2
  int depth = cfg.fifo_depth;
  if (depth) {
    int rc = simulate(plan, depth);
    if (rc) return rc;
  } else {
    depth = 1;
    while (simulate(plan, depth) != MSCCLX_OK)
      if (++depth > 4096) return fail(MSCCLX_ERR_DEADLOCK, "the program does not finish with any connection depth up to 4096");
    depth = std::max(depth, 2);
  }
  g.depth = depth;
  g.waiting_ratio = waiting_ratio(plan, &g.dataflow_depth);
  g.cold_fraction = cold_fraction(plan);

  // Slices are independent copies of the program on 1/slices of every chunk; they are what keeps
  // the chip busy while one copy waits on its dependency chain.
  const int most_threads_capacity = *std::max_element(capacity_by_threads, capacity_by_threads + kThreadChoices);
  const int64_t host_limit = (int64_t)most_threads_capacity * kMaxHosted;
  if (ntbs > host_limit)
    return fail(MSCCLX_ERR_CAPACITY, std::to_string(ntbs) + " threadblocks but the device can host only " + std::to_string(host_limit) + " contexts");
  int64_t slices = cfg.slices;
  bool lines = cfg.protocol == MSCCLX_PROTO_LL;  // flag-in-data lines instead of counters
  bool wide = false;                             // one workgroup of 1024 threads per compute unit, pieces of 128 KiB
  if (!slices) {
    const int64_t finest = (int64_t)(chunk_bytes / (32 * 1024));       // most slices of at least 32 KiB
    const int64_t to_fill = ((int64_t)2 * num_cus + ntbs - 1) / ntbs;  // fewest slices that give every compute unit a context or two
    // A long chain of hand-offs with few bytes on each (a chain all-reduce passes one buffer through
    // every rank) is bound by latency however big its chunks: about 2 us a hop against the bytes at
    // 5 TB/s.  It goes the way of the small chunks below.
    bool chain_bound = false;
    {
      uint64_t moved = 0;  // in chunks
      for (const Tb& tb : plan.tbs) moved += tb_work(plan, tb, cfg.staging != 0 || cfg.protocol == MSCCLX_PROTO_LL);
      const double data_us = (double)moved * (double)chunk_bytes / 5e6, chain_us = 2.0 * (double)g.dataflow_depth;
      chain_bound = chain_us > 2.0 * data_us;
    }
    if (finest >= 2 && finest >= to_fill && !chain_bound) {
      // Slices of 32 KiB or more can give every compute unit a context.  Measured on MI355X (8 to 1920
      // threadblocks, 128 KiB to 64 MiB chunks), what matters is (1) that the contexts spread EVENLY
      // over the resident workgroups -- 7.5 contexts per workgroup on average means some host 8, and
      // the launch takes as long as those take -- (2) enough contexts to always find one ready --
      // per half compute unit, four for every threadblock that is busy at a time (waiting_ratio),
      // between 4 and 32 -- and (3) several passes of 64 KiB pieces over a big slice rather than one
      // big piece, so that the phases of a program overlap (pass k+1 of an early phase runs beside
      // pass k of a later one).  Candidates are scored on (1) and (2); (3) follows below.
      std::vector<uint64_t> works;
      for (const Tb& tb : plan.tbs) works.push_back(tb_work(plan, tb, cfg.staging != 0 || cfg.protocol == MSCCLX_PROTO_LL));
      const int most_capacity = *std::max_element(capacity_by_threads, capacity_by_threads + kThreadChoices);
      const int64_t lo = std::max<int64_t>(1, to_fill);
      const double wanted_per_wg = std::min(32.0, 4.0 * waiting_ratio(plan));
      // pieces of 16 KiB only where 32 KiB pieces leave less than a quarter of the contexts wanted in (2)
      const int64_t finer = (double)(finest * ntbs) / (2.0 * num_cus) < wanted_per_wg / 4 ? (int64_t)(chunk_bytes / (16 * 1024)) : finest;
      const int64_t hi = std::max<int64_t>(lo, std::min<int64_t>(finer, ((int64_t)most_capacity * kMaxHosted) / ntbs));
      // Programs whose traffic is mostly cold -- inputs read once, results written once, little re-read out of the
      // memory-side cache: the all-to-alls -- and whose threadblocks wait for each other part of the time do better with
      // one workgroup of 1024 threads per compute unit walking pieces of 128 KiB: nothing to share the compute unit with
      // (two workgroups of 512 threads do not share it evenly: the earlier one runs 2.4 times faster and then polls), and
      // half the hand-offs per byte.  Hierarchical all-to-all, 16 ranks, chunks of 2 / 4 / 8 / 32 MiB: 278 -> 253,
      // 510 -> 485, 998 -> 943, 4421 -> 4004 us; with pieces of 64 KiB or less the wide workgroups lose (1 MiB chunks
      // 134 -> 135 us, 512 KiB 76 -> 82 us), and so do rings, which re-read what they have just written.  More than
      // eight passes over a slice cost such a program too (32 MiB chunks: 16 slices x 16 passes 4168 us, 32 x 8 4004 us).
      wide = !cfg.threads && !cfg.piece_bytes && !cfg.workgroups && g.cold_fraction >= 0.6 && g.waiting_ratio >= 1.5 &&
             capacity_by_threads[thread_index(1024)] >= num_cus;
      std::vector<int64_t> candidates = {lo, hi};
      for (int64_t base = 1; base <= hi; base *= 2)
        for (int64_t c : {base, base * 3})
          if (c >= lo && c <= hi) candidates.push_back(c);
      double best_score = -1e9;
      for (int64_t c : candidates) {
        // the workgroups this choice would run on: threads follow the piece, workgroups the threads
        const uint64_t slice_bytes = chunk_bytes / (uint64_t)c;
        const uint64_t piece_bytes = slice_bytes > 128 * 1024 + 2048 ? 64 * 1024 : slice_bytes;
        int threads = cfg.threads && thread_index(cfg.threads) >= 0 ? cfg.threads : threads_for_piece(piece_bytes);
        while (threads > 64 && capacity_by_threads[thread_index(threads)] < 1) threads /= 2;
        int64_t wgs = cfg.workgroups ? cfg.workgroups : (int64_t)num_cus * 16 / (threads / 64);
        wgs = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(wgs, capacity_by_threads[thread_index(threads)]), c * ntbs));
        if (wgs * kMaxHosted < c * ntbs) continue;
        // (2) is about the compute unit, not the workgroup: smaller pieces run on smaller workgroups, more
        // of them to a compute unit, and contexts per workgroup would not tell candidates apart.  The
        // unit is half a compute unit -- one workgroup of 512 threads.
        const double per_wg = std::max(1.0, (double)(c * ntbs) / (2.0 * num_cus));
        // (the slices of a wide program are scored as everybody's -- on the workgroups they would get with pieces of
        // 64 KiB -- plus its passes of 128 KiB beyond eight; pieces and threads follow from the slices below)
        const double wide_passes = std::ceil((double)slice_bytes / (128.0 * 1024.0));
        const double score = hosting_balance(works, c, wgs) - 0.02 * std::fabs(std::log2(per_wg / wanted_per_wg)) -
                             (wide && wide_passes > 8.0 ? 0.03 * std::log2(wide_passes / 8.0) : 0.0);
        if (score > best_score + 1e-9 || (std::fabs(score - best_score) <= 1e-9 && c < slices)) { best_score = score; slices = c; }
      }
      if (!slices) slices = lo;
    } else {
      // Small chunks: the launch is bound by latency.  Its time is about
      //   a * contexts + depth * (h0 + b * piece bytes)
      // -- a fixed cost per workgroup launched, and one hand-off plus one small move for every step
      // on the longest chain of the program's dataflow.  More slices shrink the pieces but add
      // workgroups; the minimum is at slices = sqrt(b/a * depth * chunk / threadblocks).  With
      // b/a = 12.5 per KiB (fitted on MI355X, workgroups of one wave running the chain loops) an
      // 8-rank ring on 1 MiB comes out at 53 slices and a 64-rank ring on 256 KiB at 10; 64 and 8
      // measured best.  Threadblocks that
      // mostly wait for each other cost less than the fixed cost each: with waiting_ratio r the
      // minimum moves to sqrt(r) times as many slices (two-level all-reduce, r = 9.4, 16 KiB chunks:
      // 4 slices 78 us, 1 slice 86 us).
      // Never finer than a context or two per compute unit with pieces down to 512 bytes, nor than
      // r times that with pieces of 4 KiB or more.
      int32_t depth_of_dataflow = 1;
      const double ratio = waiting_ratio(plan, &depth_of_dataflow);
      const double best = std::sqrt(ratio * 12.5 * (double)depth_of_dataflow * ((double)chunk_bytes / 1024.0) / (double)ntbs);
      const int64_t fill = (int64_t)std::ceil((double)to_fill * ratio);
      const int64_t most = std::max<int64_t>(1, std::max(std::min<int64_t>(std::max(finest, to_fill), (int64_t)(chunk_bytes / 512)),
                                                         std::min<int64_t>(std::max(finest, fill), (int64_t)(chunk_bytes / 4096))));
      // a power of two (small chunks divide evenly only by those): the nearest one, not above `most`
      slices = 1;
      while (slices * 2 <= most && (double)(slices * 2) <= best * 1.41421356) slices *= 2;
      // hosting many contexts per workgroup is cheap, but polling them is not free: keep it to ~32
      const int64_t comfortable = std::max<int64_t>(1, ((int64_t)2 * num_cus * 32) / ntbs);
      slices = std::min(slices, comfortable);
      // Workgroup w runs on XCD w mod 8, and contexts are dealt out threadblock by threadblock: with
      // a multiple of 8 slices every slice's contexts -- the ones that hand data to each other -- sit
      // on one XCD, under one L2.  A hand-off inside an XCD takes about 10 % less than one across
      // (64-rank ring, 2 KiB chunks: 251 us with 8 slices of 256 bytes, 264 us with 4 of 512).
      // Only where that still is a workgroup or two per compute unit: more of them cost more than the hand-offs save.
      if (slices < 8 && chunk_bytes / 8 >= 128 && 8 * ntbs <= 2 * (int64_t)num_cus) slices = 8;
      // One unit per lane: a piece of at most 1 KiB is one 16-byte unit for each lane of a one-wave
      // workgroup, the cheapest move there is, and a workgroup that starts from its context's record costs
      // little.  Chunks of up to 64 KiB are cut that fine (else into pieces of 2 KiB) where every
      // context still gets a workgroup of its own and the contexts that are busy at a time -- contexts over
      // waiting_ratio -- are at most one per SIMD.  Measured over the programs msccl-tools ships, 4 to 64 KiB
      // chunks: 6 to 40 % off twenty-odd of them (PCIe-hierarchical all-reduce at 16 KiB chunks 56 -> 33 us,
      // pipelined all-pairs 33 -> 23 us), within 2 % for the rest.  Bigger chunks lose as often as they win, and
      // a ring whose every threadblock is busy all the time (64 ranks) loses beyond one context per SIMD.
      // Chunks of up to 128 KiB too where ALL contexts are at most one per SIMD (8-rank ring on 1 MiB: 33.3 -> 31.5 us).
      // Where some threadblocks wait (waiting_ratio above 1) two busy contexts per SIMD still pay, and the slices need
      // not be a power of two: over the same programs at 14 chunk sizes from 2 to 128 KiB, seven of them not powers of
      // two, that took 0.9 % off the geometric mean -- PCIe-hierarchical all-reduce at 20 000-byte chunks 57 -> 40 us,
      // all-pairs all-reduce 28 -> 23 us, two-node all-pairs at 4 KiB 73 -> 58 us; one program (the second all-pairs
      // variant) rose by 2 to 7 %.  With no waiting at all (64-rank ring) a second context per SIMD costs 8 to 15 %.
      if (chunk_bytes <= 128 * 1024 && !cfg.piece_bytes && !cfg.threads && !cfg.workgroups) {
        const double busy_share = chunk_bytes <= 64 * 1024 ? ratio : 1.0;
        const double per_cu = chunk_bytes <= 64 * 1024 && ratio > 1.0 ? 8.0 : 4.0;
        // pieces of at most 1 KiB, else 2 KiB: a power of two up to 8 slices, a multiple of 8 (whole XCD rounds) beyond
        auto slices_of = [&](uint64_t piece_units) {
          const int64_t least = (int64_t)((g.chunk_units + piece_units - 1) / piece_units);
          int64_t s = 1;
          while (s < least && s < 8) s *= 2;
          return s < least ? (least + 7) / 8 * 8 : s;
        };
        for (int64_t s : {slices_of(64), slices_of(128)}) {
          if (s <= slices || (uint64_t)s > g.chunk_units) continue;
          const int64_t contexts = s * ntbs;
          if (contexts > capacity_by_threads[thread_index(64)] || (double)contexts > busy_share * per_cu * (double)num_cus) continue;
          slices = s;
          break;
        }
      }
      // Flag-in-data lines by themselves, where they win: a chain of hand-offs (8 or more deep) whose
      // pieces can be cut down to 1 KiB -- one unit per lane of a one-wave workgroup, the shape the
      // kernel's chain loop is written for -- with at most two such workgroups per compute unit, one
      // context each.  There a hop takes 1.55 us against 2.1 us with counters (64-rank ring on
      // 256 KiB per rank 198 against 262 us, 8-rank ring on 8 to 512 KiB per rank 30 against 35-38 us);
      // with bigger pieces or more workgroups the doubled slot traffic and the staging of every
      // message cost more than the hand-off saves (8-rank ring on 1 MiB: 38 us either way; on 2 MiB
      // 59 against 40 us).  Programs whose nops can be folded keep the counters: folding, and chains
      // of local reduces done as one step, are worth more there.  Only when every knob is automatic.
      // Since a row of lines is laid out halves apart (plan.h, kLLUnitBytes) and the chain loop has one copy of a step's
      // instructions per step type, lines also win with four such workgroups per compute unit (8-rank ring on 1 MiB per
      // rank 30.5 -> 27.0 us, 16-rank ring on 1 MiB 57.7 -> 53.4 us), with pieces of 2 KiB where a ring is 32 hand-offs
      // or longer (32-rank ring on 2 MiB per rank 146 -> 130 us; the 8- and 16-rank rings tie there; the 64-rank chain, in
      // which one rank works at a time, loses 5 %), and for chains of
      // seven hand-offs (8-rank ring all-gather and reduce-scatter at 1 to 128 KiB chunks: 0.7 to 1.5 us off 15 to 18).
      if (cfg.protocol == MSCCLX_PROTO_AUTO && chunk_bytes % 4 == 0 && !cfg.staging && !cfg.piece_bytes && !cfg.threads && !cfg.workgroups &&
          depth_of_dataflow >= 7 && !has_foldable_nops(plan)) {
        int64_t s = slices;
        // Where the chain is long (12 hand-offs or more) the two per compute unit are taken among the contexts busy at a
        // time, contexts over 1.6 x waiting_ratio: 32-rank two-level all-reduce at 0.5 to 2 KiB chunks 42-45 -> 34-40 us,
        // pipelined ring at 12 to 32 KiB 29-32 -> 25-28 us, 64-rank chain at 12 to 64 KiB 172-181 -> 119-126 us.  (Over
        // 2 x waiting_ratio the pipelined ring lost 23 % at 64 KiB; a chain of 8 hand-offs lost 6 to 10 %.)
        const double lines_most = depth_of_dataflow >= 12 ? std::max(4.0, 1.6 * ratio) * (double)num_cus : 4.0 * (double)num_cus;
        const uint64_t lines_piece = depth_of_dataflow >= 32 && ratio < 2.0 ? 2048 : 1024;  // (a ring: every threadblock busy all the time)
        while (chunk_bytes / (uint64_t)s > lines_piece && (double)(s * 2 * ntbs) <= lines_most && (uint64_t)(s * 2) <= g.chunk_units) s *= 2;
        int64_t most_msgs = 0;
        for (const Conn& c : plan.conns) most_msgs = std::max<int64_t>(most_msgs, c.nmsg);
        if (chunk_bytes / (uint64_t)s <= lines_piece && (double)(s * ntbs) <= lines_most && s * ntbs <= capacity_by_threads[thread_index(64)] &&
            most_msgs < (1 << 22) - 1) {
          slices = s;
          lines = true;
        } else if (depth_of_dataflow >= 12 && most_msgs < (1 << 22) - 1) {
          // A long chain in which hardly anything is busy at a time -- a quarter of the compute units at most -- is all
          // hand-offs: the doubled slot traffic is free there, and lines win with pieces of up to 8 KiB too, on as many
          // slices as still give every context a workgroup
          // (64-rank reduce chain + broadcast chain on one 128 / 256 / 512 KiB chunk: 204 -> 154, 217 -> 171, 253 -> 143 us).
          const double few = std::min(ratio * 0.25 * (double)num_cus,
                                      (double)std::min<int64_t>(capacity_by_threads[thread_index(64)], (int64_t)num_cus * 16));  // a workgroup each
          int64_t fewer = slices;
          // (fewer slices only for a real chain, one rank at work at a time: a pipelined ring cut from 64 slices to 8 this
          // way took 43 us instead of 30)
          while (ratio >= 16.0 && fewer > 1 && (double)(fewer * ntbs) > few && chunk_bytes / (uint64_t)(fewer / 2) <= 8192) fewer /= 2;
          if (chunk_bytes / (uint64_t)fewer <= 8192 && (double)(fewer * ntbs) <= few) {
            slices = fewer;
            lines = true;
          }
        }
      }
    }
  }
  // A workgroup of one wave for every context -- the shape the kernels' chain loops are written for -- is worth more than
  // the slices chosen above where pieces of at most 8 KiB (one wave's worth) can be had that way: a context that is hosted
  // with others pays the hosting loop's hand-off (2 us against 1.4 to 1.7), one that has a workgroup of several waves pays
  // its barrier.  Where more contexts were asked for than there are workgroups to give them one each, take the most
  // slices that still do (two-level all-reduce of 32 ranks at 1 MiB per rank: 72 -> 66 us); where fewer were asked for,
  // cut on down to 8 KiB (hierarchical all-to-all of 16 ranks at 1 / 2 MiB per rank: 21 -> 17, 29 -> 27 us; all-pairs
  // all-gather at 128 / 256 KiB chunks 10.6 -> 8.6, 11.6 -> 9.6 us; over the programs msccl-tools ships at 64 KiB to 1 MiB
  // chunks it changed 38 cases, 34 of them for the better by 2 to 19 %, all-to-next at 256 KiB chunks for the worse
  // by 5 and 15 %).  Only where the launch is mostly hand-offs -- its bytes at 5 TB/s take at most six times its chain
  // at 2 us a hop -- and not for the longest chains (64-rank ring, 126 hops, 128 KiB chunks: 485 -> 520 us).  Pieces of
  // 16 KiB on one wave lose as often as they win (PCIe-hierarchical all-reduce at 256 KiB chunks 123 -> 140 us, chain
  // all-reduce of 64 ranks 284 -> 375 us): those keep two waves, or their hosted contexts.
  if (!cfg.slices && !cfg.piece_bytes && !cfg.threads && !cfg.workgroups && !lines && slices >= 1) {
    uint64_t moved = 0;  // in chunks
    for (const Tb& tb : plan.tbs) moved += tb_work(plan, tb, cfg.staging != 0);
    const double data_us = (double)moved * (double)chunk_bytes / 5e6, chain_us = 2.0 * (double)g.dataflow_depth;  // the bytes at 5 TB/s, 2 us a hop
    const int64_t one_each = std::min<int64_t>(capacity_by_threads[thread_index(64)], (int64_t)num_cus * 16) / ntbs;  // most slices with a workgroup each
    if (one_each >= 1) {
      int64_t s = 1;
      while (s * 2 <= one_each) s *= 2;
      if (slices > s) {
        if (chunk_bytes / (uint64_t)s <= 8 * 1024) slices = s;
      } else if (g.dataflow_depth <= 32 && data_us <= 6.0 * chain_us) {  // (a launch that is mostly hand-offs, not mostly bytes)
        int64_t finer = slices;
        while (finer * 2 <= s && chunk_bytes / (uint64_t)finer > 8 * 1024) finer *= 2;
        if (chunk_bytes / (uint64_t)finer <= 8 * 1024) slices = finer;
      }
    }
  }
  slices = std::min<int64_t>(slices, (int64_t)g.chunk_units);
  if (slices < 1 || (cfg.slices && (uint64_t)cfg.slices > g.chunk_units)) return fail(MSCCLX_ERR_INVALID_ARG, "more slices than units in a chunk");
  if (slices * ntbs > host_limit) {
    if (cfg.slices) return fail(MSCCLX_ERR_CAPACITY, std::to_string(slices * ntbs) + " contexts requested but the device can host only " + std::to_string(host_limit));
    slices = std::max<int64_t>(1, host_limit / ntbs);
  }
  g.slices = (int)slices;

  // piece: the whole slice in one pass unless the FIFO slots of staged messages would not fit the budget
  g.slice_grain = std::max<uint32_t>(1, 256 / g.unit_bytes);
  if (g.chunk_units / g.slice_grain < (uint64_t)slices) g.slice_grain = 1;
  // Slices of at most a kilobyte are moved one unit per lane by one wave: a 65th unit -- what the longer slices get
  // when groups of 256 bytes do not divide evenly -- would cost every step of such a slice a second round.  Take the
  // coarsest cut of 16, 8 ... 1 units that keeps every slice within 64 units: slices that start on cache lines are
  // worth 10 % even at this size, a second round costs 50 %.
  if ((g.chunk_units + (uint64_t)slices - 1) / (uint64_t)slices <= 64) {
    auto longest = [&](uint32_t grain) {
      uint64_t most_units = 0;
      for (int64_t j = 0; j < slices; ++j)
        most_units = std::max(most_units, slice_begin(g.chunk_units, grain, (int32_t)slices, (int32_t)j + 1) - slice_begin(g.chunk_units, grain, (int32_t)slices, (int32_t)j));
      return most_units;
    };
    while (g.slice_grain > 1 && (g.chunk_units / g.slice_grain < (uint64_t)slices || longest(g.slice_grain) > 64)) g.slice_grain /= 2;
  }
  uint64_t longest_slice = 0;
  for (int64_t j = 0; j < slices; ++j)
    longest_slice = std::max(longest_slice, slice_begin(g.chunk_units, g.slice_grain, (int32_t)slices, (int32_t)j + 1) -
                                                slice_begin(g.chunk_units, g.slice_grain, (int32_t)slices, (int32_t)j));
  uint64_t piece_units = cfg.piece_bytes ? std::max<uint64_t>(1, (uint64_t)cfg.piece_bytes / g.unit_bytes) : longest_slice;
  // (a slice a few units over -- a chunk that is no power of two -- is not worth a pass of its own: 2 KiB of slack)
  const uint64_t slack = 2048 / g.unit_bytes;
  if (!cfg.piece_bytes && longest_slice * g.unit_bytes > 128 * 1024 + 2048) {
    // equal passes of about 64 KiB (a short last pass costs as many hand-offs as a full one), on 256-byte boundaries
    const uint64_t target = (uint64_t)(wide ? 128 * 1024 : 64 * 1024) / g.unit_bytes;
    const uint64_t passes = (longest_slice - slack + target - 1) / target;
    piece_units = (longest_slice + passes - 1) / passes;
    piece_units = (piece_units + g.slice_grain - 1) / g.slice_grain * g.slice_grain;
  }
  piece_units = std::min(piece_units, longest_slice);
  // protocol: flag-in-data lines pay twice the slot traffic and stage every message to take the
  // counter round trip out of a hand-off.  On request, or where the rule for small chunks above
  // found them faster; everywhere else reading payloads in place (which LL gives up) wins.
  g.ll = lines ? 1 : 0;
  if (g.ll) g.staging = 1;
  const uint64_t fifo_unit_bytes = (uint64_t)g.unit_bytes * (g.ll ? 2 : 1);
  uint64_t slot_chunks = 0;  // FIFO units per slice per unit of piece
  for (const Conn& c : plan.conns) slot_chunks += (uint64_t)depth * (g.staging ? c.max_cnt : c.max_staged_cnt);
  if (!cfg.piece_bytes && slot_chunks) {
    const uint64_t cap = fifo_budget_bytes / (slot_chunks * (uint64_t)slices * fifo_unit_bytes);
    const uint64_t floor_units = std::max<uint64_t>(1, 16384 / g.unit_bytes);
    piece_units = std::min(piece_units, std::max(cap, std::min(floor_units, longest_slice)));
  }
  const uint64_t most_units = 0x3fffffffu / (g.ll ? 32 : 16);  // byte offsets inside a piece (a slot row, in LL lines) stay below 2^30
  if (piece_units > most_units) piece_units = most_units;
  g.piece_units = (uint32_t)piece_units;
  g.passes = (int)((longest_slice + piece_units - 1) / piece_units);
  for (const Conn& c : plan.conns) {  // the kernel addresses a connection's ring of slots with 32-bit byte offsets
    const uint64_t ring = (uint64_t)depth * (uint64_t)(g.staging ? c.max_cnt : c.max_staged_cnt) * piece_units * fifo_unit_bytes;
    if (ring >= (1ull << 32))
      return fail(MSCCLX_ERR_CAPACITY, "the slots of one connection would take 4 GiB or more; use a smaller piece_bytes or fifo_depth");
  }
  {  // the kernel keeps step and message numbers of one launch in 32 bits
    int64_t longest = 0;
    for (const Tb& tb : plan.tbs) longest = std::max<int64_t>(longest, tb.op_end - tb.op_begin);
    if (longest * g.passes >= (int64_t)1 << 31)
      return fail(MSCCLX_ERR_CAPACITY, "piece_bytes is so small that a threadblock would make more than 2^31 steps");
  }
  if (g.ll) {  // a message's flag carries its sequence number in 22 bits
    int64_t most = 0;
    for (const Conn& c : plan.conns) most = std::max<int64_t>(most, c.nmsg);
    if (most * g.passes >= (1 << 22) - 1)
      return fail(MSCCLX_ERR_UNSUPPORTED, "too many messages per connection for the LL protocol; use a larger piece_bytes");
  }

  // threads: enough to cover a piece with 8 16-byte loads per thread
  int threads = cfg.threads;
  if (threads) {
    if (thread_index(threads) < 0) return fail(MSCCLX_ERR_INVALID_ARG, "threads must be 64, 128, 256, 512 or 1024");
  } else {
    const uint64_t piece_bytes = piece_units * g.unit_bytes;
    threads = wide && piece_bytes >= kWidePieceBytes ? 1024 : threads_for_piece(piece_bytes);
    while (threads > 64 && capacity_by_threads[thread_index(threads)] < 1) threads /= 2;
  }
  const int capacity = capacity_by_threads[thread_index(threads)];
  if (capacity < 1) return fail(MSCCLX_ERR_CAPACITY, "no workgroup of " + std::to_string(threads) + " threads fits on the device");
  g.threads = threads;

  // resident workgroups: about 16 waves per compute unit, never more than contexts or capacity
  const int64_t contexts = slices * ntbs;
  int64_t wgs = cfg.workgroups ? cfg.workgroups : (int64_t)num_cus * 16 / (threads / 64);
  wgs = std::min<int64_t>(wgs, contexts);
  if (wgs > capacity) {
    if (cfg.workgroups) return fail(MSCCLX_ERR_CAPACITY, std::to_string(wgs) + " workgroups requested but only " + std::to_string(capacity) + " can be resident");
    wgs = capacity;
  }
  if (wgs * kMaxHosted < contexts) {
    if (cfg.workgroups || cfg.slices)
      return fail(MSCCLX_ERR_CAPACITY, std::to_string(contexts) + " contexts cannot be hosted by " + std::to_string(wgs) + " workgroups of " +
                                           std::to_string(kMaxHosted) + " contexts each");
    wgs = std::min<int64_t>(capacity, (contexts + kMaxHosted - 1) / kMaxHosted);
    if (wgs * kMaxHosted < contexts) return fail(MSCCLX_ERR_CAPACITY, "too many contexts for the resident workgroups");
  }
  g.workgroups = (int)wgs;

  // Hosting table: longest-processing-time first -- contexts by decreasing work onto the least
  // loaded workgroup that still has a free lane.
  struct Ctx { uint64_t work; int tb, slice; };
  std::vector<Ctx> ctxs;
  ctxs.reserve((size_t)contexts);
  for (int t = 0; t < (int)ntbs; ++t) {
    const uint64_t w = tb_work(plan, plan.tbs[t], g.staging != 0);
    for (int j = 0; j < (int)slices; ++j) ctxs.push_back({w, t, j});
  }
  std::stable_sort(ctxs.begin(), ctxs.end(), [](const Ctx& a, const Ctx& b) { return a.work > b.work; });
  std::vector<std::vector<int>> hosted((size_t)wgs);
  typedef std::pair<uint64_t, int> Load;  // (work so far, workgroup)
  std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
  for (int w = 0; w < (int)wgs; ++w) heap.push({0, w});
  for (size_t k = 0; k < ctxs.size(); ++k) {
    Load l = heap.top();
    heap.pop();
    hosted[l.second].push_back((int)k);
    // +1 so that contexts without data movement are spread too
    if ((int)hosted[l.second].size() < kMaxHosted) heap.push({l.first + ctxs[k].work + 1, l.second});
    if (heap.empty() && k + 1 < ctxs.size()) return fail(MSCCLX_ERR_CAPACITY, "hosting table overflow");
  }
  g.wg_begin.assign(1, 0);
  g.max_hosted = 0;
  for (int w = 0; w < (int)wgs; ++w) {
    // a workgroup polls its contexts lane by lane; keep slices of one threadblock in slice order
    std::sort(hosted[w].begin(), hosted[w].end(), [&](int a, int b) {
      return ctxs[a].slice != ctxs[b].slice ? ctxs[a].slice < ctxs[b].slice : ctxs[a].tb < ctxs[b].tb;
    });
    for (int k : hosted[w]) { g.ctx_tb.push_back(ctxs[k].tb); g.ctx_slice.push_back(ctxs[k].slice); }
    g.wg_begin.push_back((int32_t)g.ctx_tb.size());
    g.max_hosted = std::max<int32_t>(g.max_hosted, (int32_t)hosted[w].size());
  }

  g.slice_fifo_units = slot_chunks * g.piece_units;
  g.sync_slice_words = (uint64_t)(plan.tbs.size() + 2 * plan.conns.size()) * kSyncStrideWords;
  g.sync_words = kSyncHeaderWords + g.sync_slice_words * g.slices;
  const uint64_t sync_bytes = ((kControlWords + 2 * g.sync_words) * 8 + 255) / 256 * 256;  // control block + two areas
  g.fifo_byte_off = sync_bytes;
  {  // the kernel keeps slot positions as 32-bit offsets (16-byte steps) and counter positions as 32-bit word indices
    const uint64_t fifo_bytes = g.slice_fifo_units * g.slices * fifo_unit_bytes;
    if (fifo_bytes >= (1ull << 36) || g.sync_words >= (1ull << 31))
      return fail(MSCCLX_ERR_CAPACITY, "the FIFO slots or counters of this geometry exceed what the kernel can address; use fewer slices or a smaller piece_bytes");
  }
  g.workspace_bytes = sync_bytes + g.slice_fifo_units * g.slices * fifo_unit_bytes + 256;
  *out = std::move(g);
  return MSCCLX_OK;
}

}  // namespace mscclx

using namespace mscclx;

extern "C" {

int mscclx_version(void) { return MSCCLX_VERSION; }
const char* mscclx_last_error(void) { return g_last_error.c_str(); }

int mscclx_plan_create(const mscclx_plan_desc* desc, mscclx_plan** out) {
  if (!desc || !out) return fail(MSCCLX_ERR_INVALID_ARG, "null argument");
  *out = nullptr;
  mscclx_plan* p = new mscclx_plan();
  int rc = build_plan(desc, p);
  if (rc) {
    delete p;
    return rc;
  }
  *out = p;
  return MSCCLX_OK;
}

int mscclx_plan_destroy(mscclx_plan* plan) {
  if (!plan) return MSCCLX_OK;
  if (plan->dev) destroy_device_state(plan->dev);
  delete plan;
  return MSCCLX_OK;
}

int mscclx_plan_simulate(const mscclx_plan* plan, int32_t fifo_depth) {
  if (!plan || fifo_depth < 0) return fail(MSCCLX_ERR_INVALID_ARG, "bad argument");
  return simulate(*plan, fifo_depth);
}

int mscclx_plan_min_fifo_depth(const mscclx_plan* plan) {
  if (!plan) return fail(MSCCLX_ERR_INVALID_ARG, "null plan");
  int rc = simulate(*plan, 0);
  if (rc) return rc;  // not even unbounded connections help
  for (int d = 1; d <= 4096; ++d)
    if (simulate(*plan, d) == MSCCLX_OK) return d;
  return fail(MSCCLX_ERR_DEADLOCK, "needs a connection depth above 4096");
}

uint64_t mscclx_plan_algorithmic_units(const mscclx_plan* plan) { return plan ? plan->algorithmic_units : 0; }

}  // extern "C"
