// Internal host/device structures of the MSCCL-IR executor (not part of the C ABI).
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "mscclx.h"

namespace mscclx {

constexpr int kThreadChoices = 5;  // workgroups of 64, 128, 256, 512 or 1024 threads

// One <step>, plus what plan_create derives for it.
struct Op {
  int32_t type, srcbuf, srcoff, dstbuf, dstoff, cnt, depid, deps, hasdep;
  int32_t send_seq = -1;  // position among this threadblock's send-type steps
  int32_t recv_seq = -1;  // position among this threadblock's recv-type steps
  int32_t match_recv = -1;  // send-type steps: op row of the receive that takes this step's message
  int32_t match_send = -1;  // recv-type steps: op row of the send whose message this step takes
  // Send-type steps whose payload stays readable where it already is (the source of an 's', the
  // local destination an 'rcs'/'rrcs' has just written) until the matching receive has consumed it:
  // the receiver reads it from there and no FIFO slot is filled.
  int32_t zero_copy = 0;
  // Steps whose local destination chunks no step of the program ever reads (neither this rank nor,
  // in place, a peer): their stores are marked non-temporal so they do not displace reusable lines.
  int32_t final_write = 0;
};

struct Tb {
  int32_t rank, send, recv, chan, op_begin, op_end;
  int32_t local_id = 0;    // <tb id>
  int32_t send_conn = -1;  // connection this threadblock produces into
  int32_t recv_conn = -1;  // connection this threadblock consumes from
  int32_t nsend = 0, nrecv = 0;
};

// FIFO (sender rank, receiver rank, channel).
struct Conn {
  int32_t src, dst, chan;
  int32_t send_tb = -1, recv_tb = -1;  // global threadblock rows
  int32_t nmsg = 0;                    // messages per pass
  int32_t max_cnt = 0;                 // largest message, in chunks
  int32_t max_staged_cnt = 0;          // largest message that must go through a FIFO slot
};

inline bool is_send_type(int t) { return t == MSCCLX_OP_SEND || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRCS; }
inline bool is_recv_type(int t) { return t == MSCCLX_OP_RECV || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRCS; }
inline bool is_reduce_type(int t) { return t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRCS || t == MSCCLX_OP_REDUCE; }
inline bool reads_local_src(int t) { return t == MSCCLX_OP_SEND || t == MSCCLX_OP_COPY || t == MSCCLX_OP_REDUCE; }
inline bool touches_local_dst(int t) { return is_recv_type(t) || t == MSCCLX_OP_COPY || t == MSCCLX_OP_REDUCE; }

// ---- device-side images (plain data, uploaded at bind) ----
struct DevOp {
  // bits 0-3 type, 4 hasdep, 5 out_staged (send-type: 1 = copy the payload into a FIFO slot, 0 = the
  // receiver reads it in place), 6 nt_store (the local destination is never read again: store it
  // non-temporally), 7 in_place (recv-type: the payload is read where the sender keeps it), 8-31 cnt
  uint32_t word;
  int32_t dep_tb, dep_step;  // global threadblock row / step, or -1
  int32_t dep_nops;          // number of steps of the threadblock depended on
  // A run of nop steps in front of this one is folded into it: their dependencies are entries
  // [extra >> 8, (extra >> 8) + (extra & 255)) of the extra-dependency table, and finishing this step
  // finishes `steps` steps of the IR (itself and the folded ones).
  uint32_t extra;
  uint32_t steps;
  // byte addresses of the first named chunk, resolved when buffers are bound (0 where the step has none)
  uint64_t src_addr;         // local source of s / cpy / re
  uint64_t dst_addr;         // local destination (and local reduction operand) of every step but s
  uint64_t in_addr;          // in_place: the chunk of the sending rank's buffer that holds the payload
};
static_assert(sizeof(DevOp) == 48, "three 16-byte loads fetch a step");
// The same 48 bytes for a launch whose every step's place in its connections' rings is known when buffers are bound
// (flag-in-data lines on one-wave workgroups, one pass, one row of at most 128 units per step, no step that waits for or is
// waited for by another threadblock of its rank: KernelParams::flat).  The device then works nothing out per step:
struct FlatOp {
  uint32_t word;          // as DevOp::word
  uint32_t in_off;        // byte offset of the step's slot in the incoming connection's ring (receiving steps)
  uint32_t out_off;       // the same for the outgoing connection (sending steps)
  uint32_t fin;           // low 22 bits of the flag its incoming lines carry
  uint32_t fout;          // ... and of the flag it writes
  uint32_t gate;          // what the outgoing connection's tail must have reached before the slot may be written; 0: nothing
  uint64_t src_addr;      // as DevOp
  uint64_t dst_addr;
  uint64_t tail;          // what the incoming connection's tail reads once this step has its lines (receiving steps)
};
static_assert(sizeof(FlatOp) == sizeof(DevOp) && offsetof(FlatOp, src_addr) == offsetof(DevOp, src_addr) && offsetof(FlatOp, dst_addr) == offsetof(DevOp, dst_addr),
              "a flat step lies where the step it was made from lay");
constexpr uint32_t kOpHasdep = 1u << 4, kOpOutStaged = 1u << 5, kOpNtStore = 1u << 6, kOpInPlace = 1u << 7;
constexpr int kOpCntShift = 8;
// Bit 31 of DevOp::steps, on a receive that reads its payload in place: the matching send is the first step of its
// threadblock and waits for nothing, so the payload is what the sender's buffer holds when the launch starts --
// there is no announcement to wait for.  (Every later writer of those chunks comes after this receive, or the
// payload would not be read in place at all; and a step without predecessors lies on no path between two steps.)
constexpr uint32_t kStepsNoAnnouncement = 1u << 31;
// The same bit, in programs that run on exec_kernel_chain_fold, on a receive that has TAKEN OVER the waits of its send: where
// the matching step is an `s` whose payload is read in place, that step does nothing but wait for its dependencies
// and announce -- a hand-off the receive can do without by waiting for those dependencies itself (they are counters of
// another rank's threadblocks, in the same area) and for the sending threadblock's steps in front of the send.
constexpr int kMaxChainFoldDeps = 61;     // counters a step of that kernel may wait for through its table: one per lane, three lanes kept for the step's own
// A run of `re` steps with one chunk each, the same destination and sources a fixed distance apart is
// done as one step on the device -- dst = (..((dst + src0) + src1)..) + src[m-1]: an `re` whose
// in_addr holds the distance between sources in bytes (0 for an ordinary `re`) and whose cnt holds m.
constexpr int kMaxReduceSources = 64;      // sources of one such step, at most ...
constexpr int kReduceSourcesAtOnce = 8;    // ... of which this many are in flight together
constexpr int kMaxExtraDeps = 64;        // nop steps folded into the step that follows them, at most: one for each lane of the polling wave
constexpr int kLaneExtraDeps = 6;        // up to this many a context's own lane checks; longer runs the wave checks together
constexpr int kExtraDepWords = 2;        // one folded dependency: counter word (from the slice's first flag); step + 1 | steps per pass of that threadblock << 16

struct DevTb {
  int32_t op_begin, nops;
  int32_t send_conn, recv_conn;
  int32_t nsend, nrecv;
  int32_t rank, pad;
};

struct DevConn {
  uint64_t fifo_off;    // offset of this connection's slots inside one slice's FIFO region, in units
  uint32_t slot_units;  // units per slot = max_cnt * piece_units
  uint32_t pad;
};

// One hosted context = (threadblock, slice), run by one lane of wave 0.  What never changes while it
// runs sits in LDS (one entry per lane, touched by that lane only), so that it occupies no registers
// while the workgroup moves data; what changes from step to step is the lane's Context.
struct Hosted {
  int nops, op_begin;
  unsigned npasses;
  // Slots: offsets from the start of the FIFO region, in 16-byte steps; counters: 64-bit word index
  // inside this launch's counter area.  32 bits each, so that the lot is read from LDS in one go.
  uint32_t in_slots, out_slots;    // first slot of the incoming / outgoing connection, in this slice
  uint32_t in_slot_bytes, out_slot_bytes;
  uint32_t in_wrap, out_wrap;      // depth * slot bytes: where the ring of slots starts over
  uint32_t flags;                  // flag of threadblock t of this slice is flags + t * kSyncStrideWords
  uint32_t my_flag;
  uint32_t head_out, tail_in;      // outgoing connection: the head this context advances, the tail it watches
  uint32_t head_in, tail_out;      // incoming connection: the head it watches, the tail it advances
  uint32_t clip;                   // bytes (0 to 15) that the slice's last unit lacks: the chunk's last slice, when a chunk is no multiple of 16 bytes
  int tb, slice;                   // for the watchdog's report only
};

// A context's record as the device reads it: everything about (threadblock, slice) that the geometry and
// the tables fix, worked out once when buffers are bound, so that a workgroup starts a context with
// one round of loads instead of a walk hosting table -> threadblock -> connections and a handful of
// 64-bit divisions for the slice's bounds.
struct DevCtx {
  Hosted h;
  uint32_t left;   // units of the slice (what the first pass has in front of it)
  uint64_t off;    // byte offset of the slice inside every chunk
};
static_assert(sizeof(DevCtx) == 88, "a context is fetched with six loads");

struct Geometry {
  uint64_t chunk_units = 0;   // units (16-byte vectors or elements) per chunk
  uint32_t unit_bytes = 0;
  uint32_t piece_units = 0;
  int32_t slices = 0, depth = 0, threads = 0, vector_path = 0;  // (vector_path: always 1, reported for callers of older versions)
  uint32_t slice_grain = 1;       // see slice_begin()
  int32_t staging = 0;            // 1: every message goes through a FIFO slot
  int32_t ll = 0;                 // 1: flag-in-data lines in the slots (implies staging); FIFO bytes double
  int32_t workgroups = 0;         // resident workgroups; each hosts up to kMaxHosted (threadblock, slice) contexts
  int32_t max_hosted = 0;
  std::vector<int32_t> wg_begin, ctx_tb, ctx_slice;  // the hosting table
  int32_t passes = 0;
  double waiting_ratio = 1.0;     // threadblocks x depth of the dataflow / moving steps
  double cold_fraction = 0.0;     // share of the algorithmic bytes that memory sees once only
  int32_t dataflow_depth = 1;
  uint64_t slice_fifo_units = 0;  // FIFO units one slice needs (all connections)
  uint64_t sync_words = 0;        // uint64 words of ONE synchronisation area (there are two)
  uint64_t sync_slice_words = 0;  // words per slice inside an area
  uint64_t workspace_bytes = 0;
  uint64_t fifo_byte_off = 0;     // where the FIFO region starts inside the workspace
};

struct KernelParams {
  const DevTb* tbs;
  const DevOp* ops;
  const DevConn* conns;
  const uint32_t* extra_deps;   // kExtraDepWords words per folded dependency
  unsigned long long* sync_base; // control block (kControlWords): counters of finished workgroups, from which a launch works out its number
  unsigned long long* sync_cur;  // this launch's counters   } both derived inside the kernel
  unsigned long long* sync_nxt;  // next launch's counters   } from the control block
  unsigned char* fifo;
  mscclx_status* host_status;   // pinned host memory
  unsigned long long* prof;     // per-workgroup tick counters of MSCCLX_PROFILE builds, else null
  uint64_t chunk_units;         // 16-byte units per chunk; the last one may be partial
  uint64_t chunk_bytes;         // rows of a rank buffer are this far apart
  uint64_t slice_fifo_units;
  uint64_t sync_slice_words;
  uint64_t sync_words;
  uint64_t timeout_ticks;
  uint32_t piece_units;
  uint32_t slice_grain;
  uint32_t finish_counters;     // counters of finished workgroups in use: a power of two, at most kFinishCounters; workgroup w counts in w mod that
  uint32_t finish_more;         // the first so many counters count one workgroup more than the others
  uint64_t finish_magic_each;   // ceil(2^64 / workgroups per counter), 0 if that is 1: a division as a multiplication ...
  uint64_t finish_magic_more;   // ... the same for the counters that count one more
  int32_t slices, depth, ntbs, nconns;
  const int32_t* wg_begin;      // [workgroups+1] first hosted context of each workgroup
  const DevCtx* ctxs;           // hosted contexts, grouped by workgroup
  uint32_t one_each;            // 1: workgroup w hosts context w and no other (wg_begin need not be read)
  uint32_t flat;                // 1: the step table holds FlatOp records (see there)
};

#ifdef __HIPCC__
#define MSCCLX_HOST_DEVICE __host__ __device__
#else
#define MSCCLX_HOST_DEVICE
#endif
// First unit of slice j of a chunk (j = slices: one past the chunk's last unit).  The chunk is dealt
// out in groups of `grain` units (256 bytes where a chunk has at least one such group per slice, so
// that no slice starts in the middle of a cache line; else 1); the last slice takes the remainder.
MSCCLX_HOST_DEVICE inline uint64_t slice_begin(uint64_t chunk_units, uint32_t grain, int32_t slices, int32_t j) {
  if (j >= slices) return chunk_units;
  return (chunk_units / grain) * (uint64_t)j / (uint64_t)slices * grain;
}

constexpr int kMaxHosted = 64;        // contexts per workgroup: one per lane of the polling wave
constexpr int kProfTrace = 248;       // MSCCLX_PROFILE builds: moves logged per workgroup ...
constexpr int kProfWords = 8 + kProfTrace;  // ... after its 8 words of totals
// A unit under the flag-in-data protocol: 16 bytes of payload travel as two 16-byte halves (word flag word flag), 32 bytes
// in all.  A row of n units is laid out as the n first halves followed by the n second halves, so that each of the two
// store instructions that write a row covers whole cache lines (unit by unit, each would write half of every 32 bytes:
// twice the write transactions, and a step of a 64-rank ring 5 to 19 % longer).
constexpr int kLLUnitBytes = 32;
constexpr int kSyncStrideWords = 8;   // every counter sits alone in 64 bytes
constexpr int kSyncHeaderWords = 8;   // word 0 of an area = abort flag
// The control block in front of the two counter areas: word 2 = the stamp of the binding that armed the workspace, then
// from word 8 the counters of finished workgroups, each alone in 128 bytes (exec_device.h: begin_launch).
constexpr int kStampWord = 2;
// Values of an area's abort word: raised by a workgroup whose watchdog expired (which then reports the step it
// waited for), or by mscclx_plan_abort from the host (reported by the workgroups that leave on seeing it, so that a launch
// replayed from a HIP graph onto a raised word still tells the host that it did not run).
constexpr unsigned long long kAbortByWatchdog = 1, kAbortByHost = 2;
constexpr int kFinishCounters = 64;
constexpr int kFinishStrideWords = 16;
constexpr int kControlWords = 8 + kFinishCounters * kFinishStrideWords;

struct DeviceState;  // defined in exec.hip (host half of the ABI)

}  // namespace mscclx

struct mscclx_plan {
  int32_t nranks = 0;
  std::vector<int32_t> rank_chunks;  // [nranks*3]
  std::vector<mscclx::Tb> tbs;
  std::vector<mscclx::Op> ops;
  std::vector<mscclx::Conn> conns;
  std::vector<int32_t> rank_tb_begin;  // [nranks+1] first global tb row of each rank
  bool has_reduce = false;
  uint64_t algorithmic_units = 0;

  // set by configure
  bool configured = false;
  size_t chunk_bytes = 0;
  int32_t dtype = 0, redop = 0;
  int32_t timeout_ms = 10000;
  mscclx::Geometry geo;

  // set by bind
  mscclx::DeviceState* dev = nullptr;
};

namespace mscclx {
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);
int dtype_size(int dtype);
// Host dry run of one pass; returns MSCCLX_OK or MSCCLX_ERR_DEADLOCK (error text names a blocked step).
int simulate(const mscclx_plan& plan, int depth);
// Pure geometry decision (no HIP): max_wgs = resident workgroup capacity per thread count.
// A nop that nobody depends on and that is not its threadblock's last step can be folded into the
// step after it when the device tables are built; programs with such nops run on kernels of their own.
bool has_foldable_nops(const mscclx_plan& plan);
// Share of the program's algorithmic bytes that are read or written once only (inputs read, results written).
double cold_fraction(const mscclx_plan& plan);
// Does this geometry give every context a one-wave workgroup of its own (workgroup w hosts context w)?
bool one_wave_each(const Geometry& g);
int decide_geometry(mscclx_plan& plan, size_t chunk_bytes, int dtype, const mscclx_config& cfg,
                    int num_cus, const int capacity_by_threads[kThreadChoices], uint64_t fifo_budget_bytes, Geometry* out);
void destroy_device_state(DeviceState* d);
}  // namespace mscclx
