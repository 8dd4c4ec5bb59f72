// Host half of the C ABI of the MI355X executor for MSCCL-IR: configure, bind, launch, wait.
// The kernels live in exec_device.h / exec_kernels.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <string>
#include <vector>

#include "plan.h"

namespace mscclx {

#define HIP_TRY(expr)                                                                              \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess)                                                                          \
      return fail(MSCCLX_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));              \
  } while (0)

// ------------------------------------------------------------------------------------------------
// host: kernel table, configure, bind, launch
// ------------------------------------------------------------------------------------------------
typedef void (*kernel_fn)(const KernelParams);
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// The kernels are compiled in five translation units, two element types each (exec_kernels.hip).
kernel_fn pick_kernel_group_0(int dtype, int op, bool ll, int fold, bool ragged);
kernel_fn pick_kernel_group_1(int dtype, int op, bool ll, int fold, bool ragged);
kernel_fn pick_kernel_group_2(int dtype, int op, bool ll, int fold, bool ragged);
kernel_fn pick_kernel_group_3(int dtype, int op, bool ll, int fold, bool ragged);
kernel_fn pick_kernel_group_4(int dtype, int op, bool ll, int fold, bool ragged);
static kernel_fn pick_kernel(int dtype, int op, bool ll, int fold, bool ragged) {
  switch (dtype / 2) {
    case 0: return pick_kernel_group_0(dtype, op, ll, fold, ragged);
    case 1: return pick_kernel_group_1(dtype, op, ll, fold, ragged);
    case 2: return pick_kernel_group_2(dtype, op, ll, fold, ragged);
    case 3: return pick_kernel_group_3(dtype, op, ll, fold, ragged);
    case 4: return pick_kernel_group_4(dtype, op, ll, fold, ragged);
    default: return nullptr;
  }
}

// Everything the kernel reads about the program, packed into one block of bytes that is uploaded in
// one copy: threadblocks | steps | folded dependencies | connections | hosting table | context records.
struct DeviceImage {
  std::vector<unsigned char> bytes;
  size_t off_tbs = 0, off_ops = 0, off_extras = 0, off_conns = 0, off_hosting = 0, off_ctxs = 0;
  bool one_each = false;              // workgroup w hosts context w and no other
  bool long_folds = false;            // some step stands for more folded nops than a lane checks by itself
  bool chain_fold = false;            // folded nops on one-wave workgroups with one context each: exec_kernel_chain_fold
  bool flat = false;                  // the step table holds FlatOp records: every step's slots and flags worked out here
  std::vector<int32_t> dev_op_begin;  // per threadblock: its first step in the device's list ...
  std::vector<int32_t> dev_ir_step;   // ... and, per device step, the IR step it stands for (runs of nops are folded)
  kernel_fn kernel = nullptr;
};

struct DeviceState {
  int device = -1;
  bool ready = false;                    // every table is uploaded and the workspace is armed
  unsigned char* tables = nullptr;       // device copy of DeviceImage::bytes
  size_t tables_capacity = 0;
  DeviceImage image;                     // (bytes are dropped after the upload)
  mscclx_status* host_status = nullptr;  // pinned, device-visible
  unsigned char* workspace = nullptr;
  unsigned long long stamp = 0;          // what this binding wrote into the workspace's stamp word when it armed it
  bool dirty = false;  // counters must be cleared before the next launch (after a failed or aborted launch)
  bool abort_requested = false;
  hipStream_t side = nullptr;            // for the host's abort request while the launch stream is busy
  unsigned long long* abort_word_host = nullptr;  // pinned source of that request
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  unsigned long long* prof = nullptr;  // MSCCLX_PROFILE builds: kProfWords words per workgroup
};

void destroy_device_state(DeviceState* d) {
  if (!d) return;
  if (d->tables) (void)hipFree(d->tables);
  if (d->prof) (void)hipFree(d->prof);
  if (d->host_status) (void)hipHostFree(d->host_status);
  if (d->abort_word_host) (void)hipHostFree(d->abort_word_host);
  if (d->side) (void)hipStreamDestroy(d->side);
  if (d->ev0) (void)hipEventDestroy(d->ev0);
  if (d->ev1) (void)hipEventDestroy(d->ev1);
  delete d;
}

// Resident workgroups of kernel k on the current device, per thread count.  Asked of the runtime once per (device, kernel):
// the answers never change, and the queries (device properties, five occupancy calculations) cost milliseconds.
static int query_capacity(kernel_fn k, int* num_cus, int capacity[kThreadChoices]) {
  struct Known { int num_cus; int capacity[kThreadChoices]; };
  static std::mutex mutex;
  static std::map<std::pair<int, const void*>, Known> known;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mutex);
  auto it = known.find({dev, (const void*)k});
  if (it == known.end()) {
    Known kn{};
    int cus = 0;
    HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    kn.num_cus = cus;
    const int threads[kThreadChoices] = {64, 128, 256, 512, 1024};
    for (int i = 0; i < kThreadChoices; ++i) {
      int per_cu = 0;
      HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k, threads[i], 0));
      kn.capacity[i] = per_cu * cus;
    }
    it = known.emplace(std::make_pair(dev, (const void*)k), kn).first;
  }
  *num_cus = it->second.num_cus;
  for (int i = 0; i < kThreadChoices; ++i) capacity[i] = it->second.capacity[i];
  return MSCCLX_OK;
}

// The caller's rank buffers as one table [rank][i, o, s]; refuses what the kernels cannot address.
static int collect_buffers(const mscclx_plan& plan, void* const* in, void* const* out, void* const* scratch, std::vector<void*>* bufs_out) {
  const Geometry& g = plan.geo;
  std::vector<void*> bufs((size_t)plan.nranks * 3, nullptr);
  void* const* tables[3] = {in, out, scratch};
  for (int r = 0; r < plan.nranks; ++r)
    for (int b = 0; b < 3; ++b) {
      void* ptr = tables[b] ? tables[b][r] : nullptr;
      if (plan.rank_chunks[(size_t)r * 3 + b] > 0) {
        if (!ptr) return fail(MSCCLX_ERR_INVALID_ARG, "rank " + std::to_string(r) + ": buffer " + "ios"[b] + " is used by the algorithm but NULL was given");
        if ((uintptr_t)ptr % dtype_size(plan.dtype)) return fail(MSCCLX_ERR_INVALID_ARG, "rank " + std::to_string(r) + ": buffer not aligned to its element type");
      }
      bufs[(size_t)r * 3 + b] = ptr;
    }
  if (!g.staging) {
    // reading payloads in place assumes that distinct buffers are distinct memory
    std::vector<std::pair<uintptr_t, uintptr_t>> spans;
    for (int r = 0; r < plan.nranks; ++r)
      for (int b = 0; b < 3; ++b) {
        const size_t len = (size_t)plan.rank_chunks[(size_t)r * 3 + b] * plan.chunk_bytes;
        if (len) spans.push_back({(uintptr_t)bufs[(size_t)r * 3 + b], (uintptr_t)bufs[(size_t)r * 3 + b] + len});
      }
    std::sort(spans.begin(), spans.end());
    for (size_t k = 1; k < spans.size(); ++k)
      if (spans[k].first < spans[k - 1].second)
        return fail(MSCCLX_ERR_ALIASED, "rank buffers overlap in memory; configure the plan with staging=1 for aliased buffers");
  }
  bufs_out->swap(bufs);
  return MSCCLX_OK;
}

template <typename T>
static size_t append_table(std::vector<unsigned char>& bytes, const std::vector<T>& v, size_t at_least = 1) {
  const size_t off = (bytes.size() + 255) / 256 * 256;
  const size_t n = std::max(v.size(), at_least);
  bytes.resize(off + n * sizeof(T), 0);
  if (!v.empty()) std::memcpy(bytes.data() + off, v.data(), v.size() * sizeof(T));
  return off;
}

// Whether a launch's step table can hold FlatOp records (plan.h): lines on one-wave workgroups, one pass, one row of at
// most 128 whole units per step, and no step that waits for, or is waited for by, another threadblock of its rank.
// (Not in profiling builds, whose clocks live in the general loop; -DMSCCLX_NO_FLAT_STEPS builds a library that always runs
// the general loop, to measure one against the other.)
static bool flat_steps(const mscclx_plan& plan, const Geometry& g) {
#if defined(MSCCLX_PROFILE) || defined(MSCCLX_NO_FLAT_STEPS)
  return false;
#endif
  if (!g.ll || !one_wave_each(g) || g.passes != 1 || g.piece_units > 128 || plan.chunk_bytes % 16 != 0) return false;
  uint64_t most_slot = 0;
  for (const Conn& c : plan.conns) most_slot = std::max<uint64_t>(most_slot, (uint64_t)c.max_cnt * g.piece_units * kLLUnitBytes);
  if (most_slot * (uint64_t)g.depth > 0xffffffffull) return false;
  for (const Op& op : plan.ops)
    if (op.type == MSCCLX_OP_NOP || op.cnt != 1 || op.depid >= 0 || op.hasdep) return false;
  return true;
}

// The device's tables for the configured geometry and these buffers.  Pure host work.
static int build_image(const mscclx_plan& plan_ref, const std::vector<void*>& bufs, DeviceImage* img) {
  const mscclx_plan* plan = &plan_ref;
  const Geometry& g = plan->geo;
  const bool fold = !g.ll && has_foldable_nops(*plan);
  DeviceImage* d = img;
  d->chain_fold = fold && one_wave_each(g);
  const size_t ntb = plan->tbs.size(), nop = plan->ops.size(), ncn = plan->conns.size();
  std::vector<DevTb> htb(ntb);
  std::vector<DevOp> hop(nop);
  std::vector<DevConn> hcn(ncn ? ncn : 1);
  uint64_t fifo_off = 0;
  for (size_t c = 0; c < ncn; ++c) {
    hcn[c].fifo_off = fifo_off;
    hcn[c].slot_units = (uint32_t)(g.staging ? plan->conns[c].max_cnt : plan->conns[c].max_staged_cnt) * g.piece_units;
    hcn[c].pad = 0;
    fifo_off += (uint64_t)g.depth * hcn[c].slot_units;
  }
  for (size_t t = 0; t < ntb; ++t) {
    const Tb& tb = plan->tbs[t];
    htb[t] = DevTb{tb.op_begin, tb.op_end - tb.op_begin, tb.send_conn, tb.recv_conn, tb.nsend, tb.nrecv, tb.rank, 0};
    for (int o = tb.op_begin; o < tb.op_end; ++o) {
      const Op& op = plan->ops[o];
      DevOp& dv = hop[o];
      dv = DevOp{};
      auto chunk_addr = [&](int buf, int off) -> uint64_t {
        if (buf < 0 || buf > 2 || off < 0) return 0;
        return (uint64_t)(uintptr_t)bufs[(size_t)tb.rank * 3 + buf] + (uint64_t)off * plan->chunk_bytes;
      };
      if (reads_local_src(op.type)) dv.src_addr = chunk_addr(op.srcbuf, op.srcoff);
      if (touches_local_dst(op.type)) dv.dst_addr = chunk_addr(op.dstbuf, op.dstoff);
      dv.dep_tb = -1; dv.dep_step = -1; dv.dep_nops = 0;
      if (op.depid >= 0) {
        dv.dep_tb = plan->rank_tb_begin[tb.rank] + op.depid;
        dv.dep_step = op.deps;
        dv.dep_nops = plan->tbs[dv.dep_tb].op_end - plan->tbs[dv.dep_tb].op_begin;
      }
      dv.extra = 0; dv.steps = 1;
      dv.word = (uint32_t)op.type | ((uint32_t)std::max(op.cnt, 0) << kOpCntShift);
      if (op.hasdep) dv.word |= kOpHasdep;
      if (op.final_write) dv.word |= kOpNtStore;
      if (is_send_type(op.type) && (g.staging || !op.zero_copy)) dv.word |= kOpOutStaged;
      if (is_recv_type(op.type) && !g.staging) {
        const Op& sender = plan->ops[op.match_send];
        if (sender.zero_copy) {  // read the payload where the sending rank keeps it
          const int sender_rank = plan->tbs[plan->conns[tb.recv_conn].send_tb].rank;
          const bool from_src = sender.type == MSCCLX_OP_SEND;
          dv.word |= kOpInPlace;
          dv.in_addr = (uint64_t)(uintptr_t)bufs[(size_t)sender_rank * 3 + (from_src ? sender.srcbuf : sender.dstbuf)] +
                       (uint64_t)(from_src ? sender.srcoff : sender.dstoff) * plan->chunk_bytes;
          const Tb& sender_tb = plan->tbs[plan->conns[tb.recv_conn].send_tb];
          if (from_src && op.match_send == sender_tb.op_begin && sender.depid < 0) dv.steps |= kStepsNoAnnouncement;
        }
      }
    }
  }
  // Fold runs of nop steps into the step that follows them: that step waits for all their
  // dependencies at once (one round of counter loads) instead of one hand-off per nop.  A nop that
  // somebody depends on stays a step of its own, as does the last step of a threadblock.
  std::vector<uint32_t> extras;
  {
    std::vector<DevOp> folded_ops;
    folded_ops.reserve(nop);
    d->dev_op_begin.assign(ntb, 0);
    d->dev_ir_step.clear();
    d->long_folds = false;
    // How many nops a step may stand for: as many as its context's own lane checks, or -- where the program has runs of
    // more than twice that (all-pairs over 16 or 32 ranks) -- as many as the polling wave checks together.  That check
    // runs on a kernel of its own, whose every step is some 4 % slower: a run of seven is not worth it.
    size_t longest_run = 0;
    for (size_t t = 0; fold && t < ntb; ++t) {
      size_t run = 0;
      for (int o = plan->tbs[t].op_begin; o < plan->tbs[t].op_end; ++o) {
        const bool foldable = (hop[o].word & 15u) == MSCCLX_OP_NOP && !(hop[o].word & kOpHasdep) && o + 1 < plan->tbs[t].op_end;
        run = foldable ? run + 1 : 0;
        longest_run = std::max(longest_run, run);
      }
    }
    // (exec_kernel_chain_fold checks a dependency per lane whatever their number: every run is folded, up to what its lanes hold)
    const size_t most_folded = d->chain_fold ? (size_t)kMaxChainFoldDeps - 1
                                             : longest_run > 2 * (size_t)kLaneExtraDeps ? (size_t)kMaxExtraDeps : (size_t)kLaneExtraDeps;
    for (size_t t = 0; t < ntb; ++t) {
      const Tb& tb = plan->tbs[t];
      d->dev_op_begin[t] = (int32_t)folded_ops.size();
      std::vector<uint32_t> pending;
      uint32_t folded = 0;
      for (int o = tb.op_begin; o < tb.op_end; ++o) {
        DevOp dv = hop[o];
        const bool nop_step = (dv.word & 15u) == MSCCLX_OP_NOP;
        if (fold && nop_step && !(dv.word & kOpHasdep) && o + 1 < tb.op_end && pending.size() / kExtraDepWords < most_folded &&
            dv.dep_nops < 65536 && folded < 255) {
          if (dv.dep_tb >= 0) {
            pending.push_back((uint32_t)dv.dep_tb * kSyncStrideWords);
            pending.push_back(((uint32_t)dv.dep_step + 1) | ((uint32_t)dv.dep_nops << 16));
          }
          ++folded;
          continue;
        }
        const size_t first = extras.size() / kExtraDepWords;
        if (first >= (1u << 24)) return fail(MSCCLX_ERR_CAPACITY, "too many folded dependencies");
        dv.extra = (uint32_t)(first << 8) | (uint32_t)(pending.size() / kExtraDepWords);
        if (pending.size() / kExtraDepWords > (size_t)kLaneExtraDeps) d->long_folds = true;
        dv.steps = (dv.steps & kStepsNoAnnouncement) | (1 + folded);
        extras.insert(extras.end(), pending.begin(), pending.end());
        pending.clear();
        folded = 0;
        folded_ops.push_back(dv);
        d->dev_ir_step.push_back(o - tb.op_begin);
      }
      htb[t].op_begin = d->dev_op_begin[t];
      htb[t].nops = (int32_t)folded_ops.size() - d->dev_op_begin[t];
    }
    hop.swap(folded_ops);
  }
  if (fold) {
    // A run of `re` steps of one chunk each into the same destination, from sources a fixed distance
    // apart (the local reduction of the all-pairs programs: msccl-tools' msccl/programs/allreduce_allpairs.py:18-21),
    // becomes one step with several sources.  Only the first of them may wait for anything, only
    // the last may be waited for.
    std::vector<DevOp> fused;
    std::vector<int32_t> fused_ir;
    fused.reserve(hop.size());
    for (size_t t = 0; t < ntb; ++t) {
      const int32_t begin = htb[t].op_begin, end = begin + htb[t].nops;
      const int32_t new_begin = (int32_t)fused.size();
      for (int32_t i = begin; i < end;) {
        DevOp dv = hop[(size_t)i];
        int32_t j = i + 1;
        auto plain_re = [&](const DevOp& o) { return (o.word & 15u) == MSCCLX_OP_REDUCE && (o.word >> kOpCntShift) == 1; };
        if (plain_re(dv) && !(dv.word & kOpHasdep)) {
          uint64_t stride = 0;
          int sources = 1;
          bool hasdep = false, nt = (dv.word & kOpNtStore) != 0;
          uint32_t steps = dv.steps;
          while (j < end && sources < kMaxReduceSources && !hasdep) {
            const DevOp& nx = hop[(size_t)j];
            if (!plain_re(nx) || nx.dst_addr != dv.dst_addr || nx.dep_tb >= 0 || (nx.extra & 255u) || nx.steps != 1) break;
            const uint64_t expect_stride = nx.src_addr - hop[(size_t)j - 1].src_addr;
            if (nx.src_addr <= hop[(size_t)j - 1].src_addr || (sources > 1 && expect_stride != stride)) break;
            // the sources must stay clear of the destination chunk
            const uint64_t cb = plan->chunk_bytes;
            if (!(nx.src_addr + cb <= dv.dst_addr || dv.dst_addr + cb <= nx.src_addr)) break;
            if ((uint64_t)sources * expect_stride + cb >= (1ull << 31)) break;  // one buffer descriptor spans all sources
            stride = expect_stride;
            hasdep = (nx.word & kOpHasdep) != 0;
            nt = (nx.word & kOpNtStore) != 0;
            ++sources; ++steps; ++j;
          }
          if (sources > 1 && (dv.src_addr + plan->chunk_bytes <= dv.dst_addr || dv.dst_addr + plan->chunk_bytes <= dv.src_addr)) {
            dv.word = (uint32_t)MSCCLX_OP_REDUCE | ((uint32_t)sources << kOpCntShift) | (hasdep ? kOpHasdep : 0u) | (nt ? kOpNtStore : 0u);
            dv.in_addr = stride;
            dv.steps = steps;
          } else {
            j = i + 1;
          }
        }
        fused.push_back(dv);
        fused_ir.push_back(d->dev_ir_step[(size_t)i]);
        i = j;
      }
      d->dev_op_begin[t] = new_begin;
      htb[t].op_begin = new_begin;
      htb[t].nops = (int32_t)fused.size() - new_begin;
    }
    hop.swap(fused);
    d->dev_ir_step.swap(fused_ir);
  }
  if (d->chain_fold && !g.staging) {
    // Receives take over the waits of sends that only announce.  S: an `s` whose payload is read in place; R: the receive
    // that reads it.  S moves nothing: it waits for its dependencies (its own and those of the nops folded into it) and
    // for the steps in front of it in its threadblock, then raises the connection's head -- one hand-off, which R spares
    // by waiting for the same counters itself.  Everything that happened before S still happens before R; every later
    // writer of the payload comes after R on the program's happens-before graph, or the payload would not be read in
    // place at all.  The step in front of S must publish its threadblock's flag for this.
    std::vector<int32_t> dev_of_ir(nop, -1);  // row of an IR step in plan->ops -> its step in the device's list
    for (size_t t = 0; t < ntb; ++t)
      for (int32_t i = htb[t].op_begin; i < htb[t].op_begin + htb[t].nops; ++i) dev_of_ir[(size_t)(plan->tbs[t].op_begin + d->dev_ir_step[(size_t)i])] = i;
    for (size_t t = 0; t < ntb; ++t) {
      const Tb& tb = plan->tbs[t];
      for (int32_t i = htb[t].op_begin; i < htb[t].op_begin + htb[t].nops; ++i) {
        DevOp& rv = hop[(size_t)i];
        if (!is_recv_type((int)(rv.word & 15u)) || !(rv.word & kOpInPlace) || (rv.steps & kStepsNoAnnouncement)) continue;
        const Op& rop = plan->ops[(size_t)(tb.op_begin + d->dev_ir_step[(size_t)i])];
        const int32_t si = rop.match_send >= 0 ? dev_of_ir[(size_t)rop.match_send] : -1;
        if (si < 0) continue;
        const DevOp& sv = hop[(size_t)si];
        if ((sv.word & 15u) != MSCCLX_OP_SEND || (sv.word & kOpOutStaged)) continue;  // (an rcs / rrcs writes its payload itself: it must have run)
        const size_t st = (size_t)plan->conns[(size_t)tb.recv_conn].send_tb;       // the sending threadblock's row
        const int32_t s_first = htb[st].op_begin, s_steps = htb[st].nops;
        const uint32_t s_ir_steps = (uint32_t)(plan->tbs[st].op_end - plan->tbs[st].op_begin);
        const uint32_t s_folded = (sv.steps & ~kStepsNoAnnouncement) - 1;                       // nops folded into S
        const uint32_t before_s = (uint32_t)d->dev_ir_step[(size_t)si] - s_folded;              // IR steps of the threadblock in front of S and its nops
        const bool waits_for_steps = before_s > 0 || g.passes > 1;
        const size_t mine = rv.extra & 255u, theirs = sv.extra & 255u;
        const size_t total = mine + theirs + (sv.dep_tb >= 0 ? 1 : 0) + (waits_for_steps ? 1 : 0);
        if (total > (size_t)kMaxChainFoldDeps || s_ir_steps >= 65536u || (sv.dep_tb >= 0 && sv.dep_nops >= 65536)) continue;
        const size_t first = extras.size() / kExtraDepWords;
        if (first + total >= (1u << 24)) continue;
        for (size_t k = 0; k < mine * kExtraDepWords; ++k) extras.push_back(extras[(size_t)(rv.extra >> 8) * kExtraDepWords + k]);
        for (size_t k = 0; k < theirs * kExtraDepWords; ++k) extras.push_back(extras[(size_t)(sv.extra >> 8) * kExtraDepWords + k]);
        if (sv.dep_tb >= 0) {
          extras.push_back((uint32_t)sv.dep_tb * kSyncStrideWords);
          extras.push_back(((uint32_t)sv.dep_step + 1) | ((uint32_t)sv.dep_nops << 16));
        }
        if (waits_for_steps) {
          extras.push_back((uint32_t)st * kSyncStrideWords);
          extras.push_back(before_s | (s_ir_steps << 16));
          hop[(size_t)(si > s_first ? si - 1 : s_first + s_steps - 1)].word |= kOpHasdep;  // the step in front of S (the last one, of the pass before, when S is the first)
        }
        rv.extra = (uint32_t)(first << 8) | (uint32_t)total;
        rv.steps |= kStepsNoAnnouncement;
      }
    }
  }
  // Lines on one-wave workgroups, one pass, one row of at most 128 units per step, no waits between the threadblocks of a
  // rank (the rings): which slot of its connections' rings a step uses, which flags it reads and writes, and what the
  // counters must show are then the same in every launch, and the step table says so (FlatOp) -- the chain loop's
  // bookkeeping, some hundred instructions per step of a lone wave, is done here instead, once.
  d->flat = flat_steps(*plan, g);
  for (size_t t = 0; d->flat && t < ntb; ++t) {
    const uint64_t in_slot = htb[t].recv_conn >= 0 ? (uint64_t)hcn[(size_t)htb[t].recv_conn].slot_units * kLLUnitBytes : 0;
    const uint64_t out_slot = htb[t].send_conn >= 0 ? (uint64_t)hcn[(size_t)htb[t].send_conn].slot_units * kLLUnitBytes : 0;
    uint64_t rseq = 0, sseq = 0;
    for (int32_t i = htb[t].op_begin; i < htb[t].op_begin + htb[t].nops; ++i) {
      const DevOp dv = hop[(size_t)i];
      const int type = (int)(dv.word & 15u);
      FlatOp f{};
      f.word = dv.word; f.src_addr = dv.src_addr; f.dst_addr = dv.dst_addr;
      if (is_recv_type(type)) {
        f.in_off = (uint32_t)((rseq % (uint64_t)g.depth) * in_slot);
        f.fin = (uint32_t)((rseq + 1) & 0x3fffffu);
        f.tail = ++rseq;
      }
      if (is_send_type(type)) {
        f.out_off = (uint32_t)((sseq % (uint64_t)g.depth) * out_slot);
        f.fout = (uint32_t)((sseq + 1) & 0x3fffffu);
        f.gate = sseq >= (uint64_t)g.depth ? (uint32_t)(sseq + 1 - (uint64_t)g.depth) : 0u;
        ++sseq;
      }
      std::memcpy(&hop[(size_t)i], &f, sizeof f);
    }
  }
  img->kernel = pick_kernel(plan->dtype, plan->redop, g.ll != 0, d->chain_fold ? 3 : fold ? (img->long_folds ? 2 : 1) : 0, plan->chunk_bytes % 16 != 0);
  if (!img->kernel) return fail(MSCCLX_ERR_UNSUPPORTED, "no kernel for this dtype/reduction");
  // One record per hosted context, in hosting order: where its counters and slots are, its slice's bounds.
  std::vector<DevCtx> ctxs(g.ctx_tb.size());
  {
    const uint64_t ub = g.unit_bytes, fb = g.ll ? (uint64_t)kLLUnitBytes : ub, slot_step = 16;
    for (size_t k = 0; k < ctxs.size(); ++k) {
      const int32_t tbi = g.ctx_tb[k], slice = g.ctx_slice[k];
      const DevTb& tb = htb[(size_t)tbi];
      DevCtx rec{};
      Hosted& h = rec.h;
      h.tb = tbi; h.slice = slice;
      h.nops = tb.nops; h.op_begin = tb.op_begin;
      const uint64_t u0 = slice_begin(g.chunk_units, g.slice_grain, g.slices, slice), u1 = slice_begin(g.chunk_units, g.slice_grain, g.slices, slice + 1);
      h.npasses = (unsigned)((u1 - u0 + g.piece_units - 1) / g.piece_units);
      const uint64_t slice_fifo = (uint64_t)slice * g.slice_fifo_units * fb;  // bytes from the start of the FIFO region (a multiple of 16)
      const uint64_t area = (uint64_t)kSyncHeaderWords + (uint64_t)slice * g.sync_slice_words;
      const uint64_t heads = area + (uint64_t)ntb * kSyncStrideWords, tails = heads + (uint64_t)ncn * kSyncStrideWords;
      if (tails + (uint64_t)ncn * kSyncStrideWords > 0xffffffffull) return fail(MSCCLX_ERR_CAPACITY, "counter area beyond 32-bit word indices");
      h.flags = (uint32_t)area;
      h.my_flag = (uint32_t)(area + (uint64_t)tbi * kSyncStrideWords);
      auto slots_of = [&](int conn, uint32_t* first, uint32_t* slot_bytes, uint32_t* wrap) -> bool {
        const uint64_t at = (slice_fifo + hcn[(size_t)conn].fifo_off * fb) / slot_step, bytes = (uint64_t)hcn[(size_t)conn].slot_units * fb;
        if (at > 0xffffffffull || bytes * (uint64_t)g.depth > 0xffffffffull) return false;
        *first = (uint32_t)at; *slot_bytes = (uint32_t)bytes; *wrap = (uint32_t)(bytes * (uint64_t)g.depth);
        return true;
      };
      if (tb.recv_conn >= 0) {
        if (!slots_of(tb.recv_conn, &h.in_slots, &h.in_slot_bytes, &h.in_wrap)) return fail(MSCCLX_ERR_CAPACITY, "FIFO region beyond 32-bit slot offsets");
        h.head_in = (uint32_t)(heads + (uint64_t)tb.recv_conn * kSyncStrideWords); h.tail_out = (uint32_t)(tails + (uint64_t)tb.recv_conn * kSyncStrideWords);
      }
      if (tb.send_conn >= 0) {
        if (!slots_of(tb.send_conn, &h.out_slots, &h.out_slot_bytes, &h.out_wrap)) return fail(MSCCLX_ERR_CAPACITY, "FIFO region beyond 32-bit slot offsets");
        h.head_out = (uint32_t)(heads + (uint64_t)tb.send_conn * kSyncStrideWords); h.tail_in = (uint32_t)(tails + (uint64_t)tb.send_conn * kSyncStrideWords);
      }
      h.clip = slice + 1 == g.slices ? (uint32_t)(g.chunk_units * ub - plan->chunk_bytes) : 0u;  // (0 unless the chunk ends inside its last unit)
      rec.left = (uint32_t)(u1 - u0);
      rec.off = u0 * ub;
      ctxs[k] = rec;
    }
  }
  img->one_each = g.wg_begin.size() == ctxs.size() + 1;  // (a workgroup hosts at least one context: then each hosts exactly one, in order)
  for (size_t w = 0; img->one_each && w < g.wg_begin.size(); ++w) img->one_each = g.wg_begin[w] == (int32_t)w;
  std::vector<int32_t> hosting(g.wg_begin);
  img->bytes.clear();
  img->off_tbs = append_table(img->bytes, htb);
  img->off_ops = append_table(img->bytes, hop);
  img->off_extras = append_table(img->bytes, extras, kExtraDepWords);
  img->off_conns = append_table(img->bytes, hcn);
  img->off_hosting = append_table(img->bytes, hosting);
  img->off_ctxs = append_table(img->bytes, ctxs);
  return MSCCLX_OK;
}

// Kernel arguments for tables at `tables` (a device copy of img.bytes) and a workspace.
static KernelParams make_params(const mscclx_plan& plan, const DeviceImage& img, const unsigned char* tables, unsigned char* workspace,
                                mscclx_status* status, unsigned long long* prof) {
  const Geometry& g = plan.geo;
  KernelParams kp;
  kp.tbs = (const DevTb*)(tables + img.off_tbs);
  kp.ops = (const DevOp*)(tables + img.off_ops);
  kp.conns = (const DevConn*)(tables + img.off_conns);
  kp.extra_deps = (const uint32_t*)(tables + img.off_extras);
  kp.sync_base = (unsigned long long*)workspace;
  kp.sync_cur = kp.sync_nxt = nullptr;
  kp.sync_words = g.sync_words;
  kp.fifo = workspace + g.fifo_byte_off;
  kp.host_status = status;
  kp.prof = prof;
  kp.chunk_units = g.chunk_units;
  kp.chunk_bytes = plan.chunk_bytes;
  kp.slice_fifo_units = g.slice_fifo_units;
  kp.sync_slice_words = g.sync_slice_words;
  kp.timeout_ticks = (uint64_t)plan.timeout_ms * 100000ull;  // wall_clock64 ticks at 100 MHz
  kp.piece_units = g.piece_units;
  kp.slice_grain = g.slice_grain;
  {  // as many counters of finished workgroups as there are workgroups, up to kFinishCounters; a power of two
    uint32_t counters = 1;
    while (counters * 2 <= (uint32_t)kFinishCounters && counters * 2 <= (uint32_t)g.workgroups) counters *= 2;
    auto magic = [](uint32_t divisor) -> uint64_t {
      return divisor <= 1 ? 0ull : (uint64_t)((((unsigned __int128)1 << 64) + divisor - 1) / divisor);
    };
    kp.finish_counters = counters;
    kp.finish_more = (uint32_t)g.workgroups % counters;
    kp.finish_magic_each = magic((uint32_t)g.workgroups / counters);
    kp.finish_magic_more = magic((uint32_t)g.workgroups / counters + 1);
  }
  kp.slices = g.slices; kp.depth = g.depth; kp.ntbs = (int)plan.tbs.size(); kp.nconns = (int)plan.conns.size();
  kp.wg_begin = (const int32_t*)(tables + img.off_hosting);
  kp.ctxs = (const DevCtx*)(tables + img.off_ctxs);
  kp.one_each = img.one_each ? 1u : 0u;
  kp.flat = img.flat ? 1u : 0u;
  return kp;
}

// Bytes of the workspace that must read zero before the first launch: both counter areas; LL: the
// slots too, so that no line of whatever the memory held carries a flag.
static size_t armed_bytes(const Geometry& g) { return g.ll ? g.workspace_bytes : g.fifo_byte_off; }

// How a finished launch ended, as the IR counts steps.
static int report_status(const mscclx_plan& plan, const DeviceImage& img, mscclx_status st, mscclx_status* status_out) {
  if (st.code != MSCCLX_OK && st.tb >= 0 && (size_t)st.tb < img.dev_op_begin.size()) {
    // the kernel counts the steps of its own list, in which runs of nops are folded: report the IR's step
    const size_t at = (size_t)img.dev_op_begin[(size_t)st.tb] + (size_t)std::max(st.step, 0);
    if (at < img.dev_ir_step.size()) st.step = img.dev_ir_step[at];
  }
  if (status_out) *status_out = st;
  if (st.code == MSCCLX_OK) return MSCCLX_OK;
  if (st.tb < 0 || (size_t)st.tb >= plan.tbs.size()) return fail(st.code, "the launch failed (no step was named)");
  const Tb& tb = plan.tbs[(size_t)st.tb];
  static const char* what[] = {"its dependency", "an incoming message", "a free slot on its outgoing connection", "?"};
  return fail(st.code, "watchdog: rank " + std::to_string(tb.rank) + " tb " + std::to_string(tb.local_id) + " step " + std::to_string(st.step) +
                           " (slice " + std::to_string(st.slice) + ", pass " + std::to_string(st.pass) + ") waited more than " +
                           std::to_string(plan.timeout_ms) + " ms for " + what[st.waiting_on & 3]);
}

// ------------------------------------------------------------------------------------------------
// mscclx_plan_run_static: one execution whose tables, counters and FIFO slots live in a device array
// of the library's own, so that the call allocates nothing.
// ------------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)MSCCLX_STATIC_SCRATCH_BYTES;
constexpr size_t kStaticStatusBytes = 256;  // the launch's mscclx_status sits in front of the tables
static_assert(sizeof(mscclx_status) <= kStaticStatusBytes, "status block");
// In host code this name only stands for the symbol; the array's device address (one per GPU, each
// GPU holds its own copy) comes from hipGetSymbolAddress and is kept in g_static_ptr.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static unsigned char* g_static_ptr[kMaxDevices] = {};
static std::mutex g_static_mutex;

// The calling thread's current device and the address of that device's copy of `scratch`.
static int static_scratch(unsigned char** ptr_out) {
  int device = -1;
  HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(MSCCLX_ERR_UNSUPPORTED, "device ordinal beyond " + std::to_string(kMaxDevices - 1));
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[device]) {
    unsigned char* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (!ptr || (uintptr_t)ptr % 256) return fail(MSCCLX_ERR_HIP, "hipGetSymbolAddress returned an unusable address for the static scratch array");
    g_static_ptr[device] = ptr;
  }
  *ptr_out = g_static_ptr[device];
  return MSCCLX_OK;
}

// (not hipMemsetAsync: a memset node recorded into a HIP graph has replayed wrongly on this platform)
__global__ void __launch_bounds__(256) zero_fill_kernel(u32x4* dst, size_t n16) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = zero;
}

}  // namespace mscclx

using namespace mscclx;

extern "C" {

int mscclx_plan_configure(mscclx_plan* plan, size_t chunk_bytes, int32_t dtype, int32_t redop, const mscclx_config* cfg_in, mscclx_info* info) {
  if (!plan) return fail(MSCCLX_ERR_INVALID_ARG, "null plan");
  mscclx_config cfg = {};
  if (cfg_in) cfg = *cfg_in;
  if (dtype < 0 || dtype >= MSCCLX_NUM_DTYPES) return fail(MSCCLX_ERR_INVALID_ARG, "unknown dtype");
  if (redop < 0 || redop >= MSCCLX_NUM_REDOPS) return fail(MSCCLX_ERR_INVALID_ARG, "unknown reduction");
  const int elem = dtype_size(dtype);
  if (chunk_bytes == 0 || chunk_bytes % elem) return fail(MSCCLX_ERR_INVALID_ARG, "chunk_bytes must be a positive multiple of the element size");
  int num_cus = 256;
  int capacity[kThreadChoices];
  if (cfg.max_workgroups > 0) {
    for (int i = 0; i < kThreadChoices; ++i) capacity[i] = cfg.max_workgroups;
  } else {
    const bool ll = cfg.protocol == MSCCLX_PROTO_LL;
    const bool fold = !ll && has_foldable_nops(*plan);
    const bool ragged = chunk_bytes % 16 != 0;  // rows may end inside a 16-byte unit: kernels of their own
    int rc = query_capacity(pick_kernel(dtype, redop, ll, fold ? 1 : 0, ragged), &num_cus, capacity);
    if (rc) return rc;
    if (fold) {  // long runs of folded nops run on a kernel of their own; which one it will be is known when the tables are built
      int other[kThreadChoices];
      rc = query_capacity(pick_kernel(dtype, redop, ll, 2, ragged), &num_cus, other);
      if (rc) return rc;
      for (int i = 0; i < kThreadChoices; ++i) capacity[i] = std::min(capacity[i], other[i]);
      rc = query_capacity(pick_kernel(dtype, redop, ll, 3, ragged), &num_cus, other);  // one-wave workgroups with one context each run on exec_kernel_chain_fold
      if (rc) return rc;
      capacity[0] = std::min(capacity[0], other[0]);
    }
    if (cfg.protocol == MSCCLX_PROTO_AUTO && !fold) {  // the geometry may choose LL lines by itself: what fits must fit either kernel
      int other[kThreadChoices];
      rc = query_capacity(pick_kernel(dtype, redop, true, 0, ragged), &num_cus, other);
      if (rc) return rc;
      for (int i = 0; i < kThreadChoices; ++i) capacity[i] = std::min(capacity[i], other[i]);
    }
  }
  Geometry g;
  const uint64_t fifo_budget = 4ull << 30;  // FIFO slots of staged messages; larger pieces are split into passes
  int rc = decide_geometry(*plan, chunk_bytes, dtype, cfg, num_cus, capacity, fifo_budget, &g);
  if (rc) return rc;
  plan->geo = std::move(g);
  const Geometry& gg = plan->geo;
  plan->chunk_bytes = chunk_bytes;
  plan->dtype = dtype;
  plan->redop = redop;
  plan->timeout_ms = cfg.timeout_ms > 0 ? cfg.timeout_ms : 10000;
  plan->configured = true;
  if (plan->dev) { destroy_device_state(plan->dev); plan->dev = nullptr; }
  if (info) {
    const Geometry& g = gg;
    info->workgroups = g.workgroups;
    info->max_hosted = g.max_hosted;
    info->protocol = g.ll ? MSCCLX_PROTO_LL : MSCCLX_PROTO_SIMPLE;
    info->waiting_ratio_x100 = (int32_t)std::min(2.0e9, g.waiting_ratio * 100.0 + 0.5);
    info->dataflow_depth = g.dataflow_depth;
    info->kernel_loop = !one_wave_each(g) ? MSCCLX_LOOP_HOSTED : g.ll ? (flat_steps(*plan, g) ? MSCCLX_LOOP_CHAIN_LINES_FLAT : MSCCLX_LOOP_CHAIN_LINES)
                        : has_foldable_nops(*plan) ? MSCCLX_LOOP_CHAIN_FOLD : MSCCLX_LOOP_CHAIN_COUNTERS;
    info->cold_traffic_x100 = (int32_t)(g.cold_fraction * 100.0 + 0.5);
    info->threads = g.threads;
    info->slices = g.slices;
    info->piece_bytes = (int32_t)(g.piece_units * g.unit_bytes);
    info->fifo_depth = g.depth;
    info->passes = g.passes;
    info->connections = (int32_t)plan->conns.size();
    info->vector_path = g.vector_path;
    info->zero_copy_messages = 0;
    info->staged_messages = 0;
    for (const Op& op : plan->ops)
      if (is_send_type(op.type)) ((!g.staging && op.zero_copy) ? info->zero_copy_messages : info->staged_messages)++;
    info->workspace_bytes = g.workspace_bytes;
    info->algorithmic_units = plan->algorithmic_units;
  }
  return MSCCLX_OK;
}

int mscclx_plan_bind(mscclx_plan* plan, void* const* in, void* const* out, void* const* scratch, void* workspace, size_t workspace_bytes) {
  if (!plan) return fail(MSCCLX_ERR_INVALID_ARG, "null plan");
  if (!plan->configured) return fail(MSCCLX_ERR_STATE, "configure the plan before binding buffers");
  const Geometry& g = plan->geo;
  if (!workspace || workspace_bytes < g.workspace_bytes)
    return fail(MSCCLX_ERR_CAPACITY, "workspace of " + std::to_string(workspace_bytes) + " bytes given, " + std::to_string(g.workspace_bytes) + " needed");
  if ((uintptr_t)workspace % 256) return fail(MSCCLX_ERR_INVALID_ARG, "workspace must be 256-byte aligned");
  std::vector<void*> bufs;
  int rc = collect_buffers(*plan, in, out, scratch, &bufs);
  if (rc) return rc;
  DeviceImage img;
  rc = build_image(*plan, bufs, &img);
  if (rc) return rc;

  // The plan keeps its device state across binds of the same geometry (configure drops it): a new
  // set of buffers then costs one upload of the tables.  The state is built aside and handed to the
  // plan only when every call has succeeded, so a failed bind leaves nothing a launch could use.
  int device = -1;
  HIP_TRY(hipGetDevice(&device));
  DeviceState* d = plan->dev;
  plan->dev = nullptr;
  if (d && (d->device != device || d->tables_capacity < img.bytes.size())) { destroy_device_state(d); d = nullptr; }
  struct Guard {  // frees the state unless it is handed over
    DeviceState* d;
    ~Guard() { if (d) destroy_device_state(d); }
  } guard{d};
  const bool fresh = d == nullptr;
  if (fresh) {
    d = guard.d = new DeviceState();
    d->device = device;
    HIP_TRY(hipMalloc((void**)&d->tables, img.bytes.size()));
    d->tables_capacity = img.bytes.size();
    HIP_TRY(hipHostMalloc((void**)&d->host_status, sizeof(mscclx_status), hipHostMallocDefault));
    HIP_TRY(hipHostMalloc((void**)&d->abort_word_host, sizeof(unsigned long long), hipHostMallocDefault));
    *d->abort_word_host = kAbortByHost;
    HIP_TRY(hipStreamCreateWithFlags(&d->side, hipStreamNonBlocking));
    HIP_TRY(hipEventCreate(&d->ev0));
    HIP_TRY(hipEventCreate(&d->ev1));
#ifdef MSCCLX_PROFILE
    HIP_TRY(hipMalloc((void**)&d->prof, sizeof(unsigned long long) * kProfWords * g.workgroups));
    HIP_TRY(hipMemset(d->prof, 0, sizeof(unsigned long long) * kProfWords * g.workgroups));
#endif
  }
  d->ready = false;
  HIP_TRY(hipMemcpy(d->tables, img.bytes.data(), img.bytes.size(), hipMemcpyHostToDevice));
  std::memset(d->host_status, 0, sizeof(mscclx_status));
  // The workspace is armed (counters zero; LL: slots too) when this plan first sees it, after a lost launch, and when
  // the stamp this plan left in it is gone: another plan's bind has cleared and stamped it in between, and its
  // counters and slots, laid out for that plan, mean nothing here.
  bool arm = fresh || d->dirty || d->workspace != (unsigned char*)workspace;
  if (!arm) {
    unsigned long long seen = 0;
    HIP_TRY(hipMemcpy(&seen, (unsigned long long*)workspace + kStampWord, sizeof seen, hipMemcpyDeviceToHost));
    arm = seen != d->stamp;
  }
  if (arm) {
    static std::atomic<unsigned long long> next_stamp{1};
    d->stamp = (next_stamp.fetch_add(1) << 20) | ((unsigned long long)(uintptr_t)d >> 4 & 0xfffffull) | 1ull;  // (never 0)
    HIP_TRY(hipMemset(workspace, 0, armed_bytes(g)));
    HIP_TRY(hipMemcpy((unsigned long long*)workspace + kStampWord, &d->stamp, sizeof d->stamp, hipMemcpyHostToDevice));
    HIP_TRY(hipDeviceSynchronize());
    d->dirty = false;
  }
  d->workspace = (unsigned char*)workspace;
  d->abort_requested = false;
  img.bytes.clear();
  img.bytes.shrink_to_fit();
  d->image = std::move(img);
  d->ready = true;
  plan->dev = d;
  guard.d = nullptr;
  return MSCCLX_OK;
}

int mscclx_plan_launch(mscclx_plan* plan, void* stream) {
  if (!plan || !plan->dev || !plan->dev->ready) return fail(MSCCLX_ERR_STATE, "bind buffers before launching");
  DeviceState* d = plan->dev;
  const Geometry& g = plan->geo;
  hipStream_t s = (hipStream_t)stream;
  if (d->dirty) {  // the previous launch gave up half-way: its counters mean nothing
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipStreamSynchronize(d->side));
    HIP_TRY(hipMemset(d->workspace, 0, armed_bytes(g)));  // LL: launches count from 0 again, old lines must go
    HIP_TRY(hipMemcpy((unsigned long long*)d->workspace + kStampWord, &d->stamp, sizeof d->stamp, hipMemcpyHostToDevice));
    HIP_TRY(hipDeviceSynchronize());
    std::memset(d->host_status, 0, sizeof(mscclx_status));
    d->dirty = false;
    d->abort_requested = false;
  }
  const KernelParams kp = make_params(*plan, d->image, d->tables, d->workspace, d->host_status, d->prof);
  hipLaunchKernelGGL(d->image.kernel, dim3((unsigned)g.workgroups), dim3(g.threads), 0, s, kp);
  HIP_TRY(hipGetLastError());
  return MSCCLX_OK;
}

// How the launches so far ended, once the stream has drained.
static int finish_wait(mscclx_plan* plan, mscclx_status* status) {
  DeviceState* d = plan->dev;
  mscclx_status st = *d->host_status;
#ifdef MSCCLX_PROFILE
  if (d->prof && getenv("MSCCLX_PROFILE_DUMP")) {
    const size_t nwg = plan->geo.workgroups;
    std::vector<unsigned long long> all(nwg * kProfWords), h(nwg * 8);
    (void)hipMemcpy(all.data(), d->prof, all.size() * 8, hipMemcpyDeviceToHost);
    for (size_t w = 0; w < nwg; ++w) std::copy(all.begin() + w * kProfWords, all.begin() + w * kProfWords + 8, h.begin() + w * 8);
    double sw = 0, sm = 0, sa = 0, sf = 0, st_ = 0; unsigned long long first = ~0ull, last = 0;
    for (size_t w = 0; w < nwg; ++w) {
      sw += h[w * 8]; sm += h[w * 8 + 1]; st_ += h[w * 8 + 2]; sa += h[w * 8 + 4]; sf += h[w * 8 + 5];
      if (h[w * 8 + 3] < first) first = h[w * 8 + 3];
      if (h[w * 8 + 3] + h[w * 8 + 2] > last) last = h[w * 8 + 3] + h[w * 8 + 2];
    }
    fprintf(stderr, "[prof] wgs=%zu span=%.1f us  mean per wg: poll %.1f us  move %.1f us  ack+barrier %.1f us  finish+describe %.1f us  total %.1f us\n",
            nwg, (last - first) / 100.0, sw / nwg / 100, sm / nwg / 100, sa / nwg / 100, sf / nwg / 100, st_ / nwg / 100);
    // When the workgroups ended, and how long each polled: deciles over the workgroups, in microseconds from the first start.
    std::vector<double> ends(nwg), polls(nwg), starts(nwg);
    for (size_t w = 0; w < nwg; ++w) {
      starts[w] = (h[w * 8 + 3] - first) / 100.0;
      ends[w] = (h[w * 8 + 3] + h[w * 8 + 2] - first) / 100.0;
      polls[w] = h[w * 8] / 100.0;
    }
    std::sort(ends.begin(), ends.end()); std::sort(polls.begin(), polls.end()); std::sort(starts.begin(), starts.end());
    std::string line = "[prof] deciles";
    for (const auto* v : {&starts, &ends, &polls}) {
      line += v == &starts ? "  start:" : v == &ends ? "  end:" : "  poll:";
      for (int q = 0; q <= 10; ++q) { char b[32]; snprintf(b, sizeof b, " %.0f", (*v)[std::min(nwg - 1, q * nwg / 10)]); line += b; }
    }
    fprintf(stderr, "%s\n", line.c_str());
    // MSCCLX_PROFILE_DUMP=<path ending in .csv>: one row per workgroup, in ticks of 10 ns.
    const char* path = getenv("MSCCLX_PROFILE_DUMP");
    if (std::strlen(path) > 4 && !std::strcmp(path + std::strlen(path) - 4, ".csv")) {
      if (FILE* f = fopen(path, "w")) {
        fprintf(f, "wg,start,total,poll,move,ack,finish,hw_id,xcc_id\n");
        for (size_t w = 0; w < nwg; ++w)
          fprintf(f, "%zu,%llu,%llu,%llu,%llu,%llu,%llu,%llu,%llu\n", w, h[w * 8 + 3] - first, h[w * 8 + 2], h[w * 8], h[w * 8 + 1], h[w * 8 + 4], h[w * 8 + 5], h[w * 8 + 6], h[w * 8 + 7]);
        fclose(f);
      }
      // <path>.moves: one row per logged move (the first kProfTrace of every workgroup)
      if (FILE* f = fopen((std::string(path) + ".moves").c_str(), "w")) {
        fprintf(f, "wg,index,tb,slice,start,duration\n");
        const Geometry& g = plan->geo;
        for (size_t w = 0; w < nwg; ++w)
          for (int i = 0; i < kProfTrace; ++i) {
            const unsigned long long e = all[w * kProfWords + 8 + i];
            if (!e) break;
            const int ctx = g.wg_begin[w] + (int)(e & 0xff);
            fprintf(f, "%zu,%d,%d,%d,%llu,%llu\n", w, i, g.ctx_tb[ctx], g.ctx_slice[ctx], (e >> 32) + h[w * 8 + 3] - first, (e >> 8) & 0xffffff);
          }
        fclose(f);
      }
    }
  }
#endif
  // (st.code is ABORTED when a launch found the request on the device by itself: one replayed from a HIP graph
  // after an abort, which passes by the re-arming in mscclx_plan_launch -- the replay after it runs normally,
  // because every launch, aborted or not, clears the counters of the area the next one uses)
  if (d->abort_requested || st.code == MSCCLX_ERR_ABORTED) {
    d->dirty = true;
    d->abort_requested = false;
    if (status) { *status = st; status->code = MSCCLX_ERR_ABORTED; }
    std::memset(d->host_status, 0, sizeof(mscclx_status));
    return fail(MSCCLX_ERR_ABORTED, "the launch was aborted by mscclx_plan_abort; the rank buffers hold partial results");
  }
  if (st.code != MSCCLX_OK) {
    d->dirty = true;
    std::memset(d->host_status, 0, sizeof(mscclx_status));
  }
  return report_status(*plan, d->image, st, status);
}

int mscclx_plan_wait(mscclx_plan* plan, void* stream, mscclx_status* status) {
  if (!plan || !plan->dev || !plan->dev->ready) return fail(MSCCLX_ERR_STATE, "nothing was launched");
  DeviceState* d = plan->dev;
  hipError_t e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) {
    d->dirty = true;
    return fail(MSCCLX_ERR_HIP, std::string("hipStreamSynchronize: ") + hipGetErrorString(e));
  }
  return finish_wait(plan, status);
}

int mscclx_plan_poll(mscclx_plan* plan, void* stream, mscclx_status* status) {
  if (!plan || !plan->dev || !plan->dev->ready) return fail(MSCCLX_ERR_STATE, "nothing was launched");
  DeviceState* d = plan->dev;
  hipError_t e = hipStreamQuery((hipStream_t)stream);
  if (e == hipErrorNotReady) {
    if (status) *status = *d->host_status;  // a watchdog report shows here before the kernel has drained
    return 1;
  }
  if (e != hipSuccess) {
    d->dirty = true;
    return fail(MSCCLX_ERR_HIP, std::string("hipStreamQuery: ") + hipGetErrorString(e));
  }
  return finish_wait(plan, status);
}

int mscclx_plan_abort(mscclx_plan* plan) {
  if (!plan || !plan->dev || !plan->dev->ready) return fail(MSCCLX_ERR_STATE, "nothing was launched");
  DeviceState* d = plan->dev;
  const Geometry& g = plan->geo;
  // Raise the abort word of both counter areas (which one the running launch uses is known to the
  // device only) from a stream of the library's own: the launch stream is busy with the kernel.
  d->abort_requested = true;
  unsigned long long* base = (unsigned long long*)d->workspace;
  for (int area = 0; area < 2; ++area)
    HIP_TRY(hipMemcpyAsync(base + kControlWords + (uint64_t)area * g.sync_words, d->abort_word_host, sizeof(unsigned long long),
                           hipMemcpyHostToDevice, d->side));
  HIP_TRY(hipStreamSynchronize(d->side));
  return MSCCLX_OK;
}

int mscclx_plan_run_static(mscclx_plan* plan, void* const* in, void* const* out, void* const* rank_scratch, void* stream, mscclx_status* status) {
  if (!plan) return fail(MSCCLX_ERR_INVALID_ARG, "null plan");
  if (!plan->configured) return fail(MSCCLX_ERR_STATE, "configure the plan before running it");
  const Geometry& g = plan->geo;
  std::vector<void*> bufs;
  int rc = collect_buffers(*plan, in, out, rank_scratch, &bufs);
  if (rc) return rc;
  DeviceImage img;
  rc = build_image(*plan, bufs, &img);
  if (rc) return rc;
  // layout inside the array: status | tables | workspace (control block, counters, FIFO slots)
  const size_t tables_off = kStaticStatusBytes;
  const size_t workspace_off = (tables_off + img.bytes.size() + 255) / 256 * 256;
  const size_t need = workspace_off + g.workspace_bytes;
  if (need > kStaticScratchBytes)
    return fail(MSCCLX_ERR_CAPACITY, "this plan needs " + std::to_string(need) + " bytes of tables, counters and FIFO slots; mscclx_plan_run_static has " +
                                         std::to_string(kStaticScratchBytes) + " (MSCCLX_STATIC_SCRATCH_BYTES): use mscclx_plan_bind with a workspace of the caller's");
  unsigned char* base = nullptr;
  rc = static_scratch(&base);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  // whatever the previous call left: the status, the counters (LL: the slots too) must read zero
  const size_t clear_to = workspace_off + armed_bytes(g);
  hipLaunchKernelGGL(zero_fill_kernel, dim3(256), dim3(256), 0, s, (u32x4*)base, kStaticStatusBytes / 16);
  hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, s, (u32x4*)(base + workspace_off), (clear_to - workspace_off + 15) / 16);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpyAsync(base + tables_off, img.bytes.data(), img.bytes.size(), hipMemcpyHostToDevice, s));
  const KernelParams kp = make_params(*plan, img, base + tables_off, base + workspace_off, (mscclx_status*)base, nullptr);
  hipLaunchKernelGGL(img.kernel, dim3((unsigned)g.workgroups), dim3(g.threads), 0, s, kp);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipStreamSynchronize(s));
  mscclx_status st;
  HIP_TRY(hipMemcpy(&st, base, sizeof st, hipMemcpyDeviceToHost));
  return report_status(*plan, img, st, status);
}

int mscclx_plan_time(mscclx_plan* plan, void* stream, int32_t iters, float* ms_out) {
  if (!plan || !plan->dev || !plan->dev->ready) return fail(MSCCLX_ERR_STATE, "bind buffers before timing");
  if (iters <= 0 || !ms_out) return fail(MSCCLX_ERR_INVALID_ARG, "bad argument");
  DeviceState* d = plan->dev;
  hipStream_t s = (hipStream_t)stream;
  for (int i = 0; i < iters; ++i) {
    HIP_TRY(hipEventRecord(d->ev0, s));
    int rc = mscclx_plan_launch(plan, stream);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(d->ev1, s));
    rc = mscclx_plan_wait(plan, stream, nullptr);
    if (rc) return rc;
    HIP_TRY(hipEventElapsedTime(&ms_out[i], d->ev0, d->ev1));
  }
  return MSCCLX_OK;
}

}  // extern "C"
