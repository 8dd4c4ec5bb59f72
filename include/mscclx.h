/*
 * mscclx — C ABI of the MI355X executor for MSCCL-IR.
 *
 * msccl-tools hands a compiled algorithm to "the runtime" as files and environment variables, not
 * through an FFI: an <algo> XML per algorithm (msccl/language/ir.py:320-391, second emitter
 * msccl/ncclize.py:658-718) listed in an <msccl_algos> index exported as MSCCL_CONFIG
 * (msccl/autosynth/__init__.py:75-99).  The entry points below are what a Python backend module of
 * msccl-tools binds with ctypes to *run* such an algorithm on one MI355X, with all ranks of the
 * algorithm held as virtual ranks in one GPU's HBM.  Every table is a flat int32 array, every
 * buffer a plain device pointer; no C++ or torch types cross this boundary.
 *
 * Ownership: the caller owns the rank buffers and the workspace; the library owns the plan (host
 * tables and their device copies) and never frees caller memory.  Between a bind and the last wait
 * on that binding the workspace's contents belong to the plan: nobody else may write there.  A
 * workspace may be handed from plan to plan (every bind stamps it, and a plan that finds another
 * plan's stamp clears it again), but whoever writes into it by other means must clear its first
 * 64 bytes too, or the next bind of the plan that armed it will trust what it holds.
 * Errors: 0 on success, a negative mscclx_error otherwise; mscclx_last_error() returns the text of
 * the calling thread's last failure.  No exception crosses the ABI.
 * Threading: a plan is not thread-safe; launches are stream-ordered; launches of one plan must all
 * go to the same stream, and bind/configure only while none is in flight.
 * Residency: a launch is one grid of workgroups that wait for each other, sized at configure time to
 * what an otherwise idle GPU keeps resident.  The stream must therefore have the GPU to itself for
 * the duration of a launch: a kernel of another stream that occupies compute units can keep part of
 * the grid from starting, and the part that runs then waits until the in-kernel watchdog ends the
 * launch with MSCCLX_ERR_TIMEOUT (never a hang).  mscclx_config.workgroups caps the grid for callers
 * that share the GPU on purpose.
 */
#ifndef MSCCLX_H
#define MSCCLX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSCCLX_VERSION 4

typedef enum {
  MSCCLX_OK = 0,
  MSCCLX_ERR_INVALID_ARG = -1, /* null pointer, bad enum, size not a multiple of the element ... */
  MSCCLX_ERR_BAD_IR = -2,      /* the tables do not describe a valid MSCCL-IR program            */
  MSCCLX_ERR_DEADLOCK = -3,    /* the program cannot finish with the chosen connection depth     */
  MSCCLX_ERR_CAPACITY = -4,    /* more threadblocks than can be resident / workspace too small   */
  MSCCLX_ERR_HIP = -5,         /* a HIP runtime call failed                                      */
  MSCCLX_ERR_TIMEOUT = -6,     /* the in-kernel watchdog expired while a step was waiting        */
  MSCCLX_ERR_STATE = -7,       /* call order violated (launch before bind, ...)                  */
  MSCCLX_ERR_UNSUPPORTED = -8,
  MSCCLX_ERR_ABORTED = -9,     /* mscclx_plan_abort ended the launch                              */
  MSCCLX_ERR_ALIASED = -10     /* rank buffers overlap in memory but the plan reads payloads in place */
} mscclx_error;

/* <step type=...>: msccl/language/ir.py:69-83 (the 'd' and 'st' members are never emitted). */
typedef enum {
  MSCCLX_OP_NOP = 0,  /* nop  */
  MSCCLX_OP_SEND = 1, /* s    */
  MSCCLX_OP_RECV = 2, /* r    */
  MSCCLX_OP_RCS = 3,  /* rcs  */
  MSCCLX_OP_RRS = 4,  /* rrs  */
  MSCCLX_OP_RRC = 5,  /* rrc  */
  MSCCLX_OP_RRCS = 6, /* rrcs */
  MSCCLX_OP_COPY = 7, /* cpy  */
  MSCCLX_OP_REDUCE = 8 /* re  */
} mscclx_op;

/* srcbuf/dstbuf: msccl/language/ir.py:86-92. */
typedef enum { MSCCLX_BUF_INPUT = 0, MSCCLX_BUF_OUTPUT = 1, MSCCLX_BUF_SCRATCH = 2 } mscclx_buf;

typedef enum {
  MSCCLX_U8 = 0, MSCCLX_I8 = 1, MSCCLX_I32 = 2, MSCCLX_U32 = 3, MSCCLX_I64 = 4, MSCCLX_U64 = 5,
  MSCCLX_F16 = 6, MSCCLX_BF16 = 7, MSCCLX_F32 = 8, MSCCLX_F64 = 9, MSCCLX_NUM_DTYPES = 10
} mscclx_dtype;

/* How a message crosses a connection.  SIMPLE: payload, then (after the stores are acknowledged) a
 * counter; payloads that may be read in place are not copied at all.  LL: every message is written
 * into its FIFO slot as 16-byte lines of two (data, flag) pairs and the receiver polls the flags in
 * the data itself -- twice the slot traffic, about half the latency per hop; meant for small pieces
 * (the trade msccl-tools names with proto="LL", msccl/language/__init__.py:38-39). */
typedef enum { MSCCLX_PROTO_AUTO = 0, MSCCLX_PROTO_SIMPLE = 1, MSCCLX_PROTO_LL = 2 } mscclx_protocol;

/* The step loop a launch runs (reported, not chosen: it follows from the geometry).  HOSTED: workgroups of any size that
 * host several (threadblock, slice) contexts each and poll for all of them.  The CHAIN loops serve one-wave workgroups
 * with one context each -- the shape of latency-bound launches: LINES for flag-in-data lines, COUNTERS for counters,
 * FOLD for counters in programs whose nop steps are folded into the steps behind them (msccl/language/ir.py:296-311
 * gives a step one dependency and puts a nop in front of it for every other: the all-pairs family); LINES_FLAT for lines
 * where every step's slots, flags and counter values could be worked out when the buffers were bound (one pass, one row
 * of at most 128 units per step, no waits between the threadblocks of a rank: the rings on small messages). */
typedef enum { MSCCLX_LOOP_HOSTED = 0, MSCCLX_LOOP_CHAIN_LINES = 1, MSCCLX_LOOP_CHAIN_COUNTERS = 2, MSCCLX_LOOP_CHAIN_FOLD = 3, MSCCLX_LOOP_CHAIN_LINES_FLAT = 4 } mscclx_loop;

typedef enum { MSCCLX_SUM = 0, MSCCLX_PROD = 1, MSCCLX_MAX = 2, MSCCLX_MIN = 3, MSCCLX_NUM_REDOPS = 4 } mscclx_redop;

#define MSCCLX_TB_COLS 6 /* rank, send, recv, chan, op_begin, op_end */
#define MSCCLX_OP_COLS 9 /* type, srcbuf, srcoff, dstbuf, dstoff, cnt, depid, deps, hasdep */

/*
 * Flat image of one <algo>.  Replaces the XML attributes of msccl/language/ir.py:330-391:
 *   rank_chunks[r*3 + {0,1,2}] = i_chunks, o_chunks, s_chunks of <gpu id=r>            (ir.py:330-335)
 *   tbs[t*6 + ..]  = rank, send, recv, chan of a <tb>, and the [op_begin, op_end) range of its
 *                    <step>s in `ops`.  Rows are grouped by rank in ascending order and, within a
 *                    rank, row k is the <tb> with id=k (depid refers to that id)         (ir.py:336-341)
 *   ops[o*9 + ..]  = type (mscclx_op), srcbuf, srcoff, dstbuf, dstoff (chunks; -1 when absent),
 *                    cnt, depid, deps (-1/-1 when absent), hasdep                        (ir.py:342-391)
 */
typedef struct {
  int32_t nranks;
  int32_t ntbs;
  int32_t nops;
  const int32_t* rank_chunks;
  const int32_t* tbs;
  const int32_t* ops;
} mscclx_plan_desc;

/* Launch geometry knobs; a zero field means "choose automatically". */
typedef struct {
  int32_t slices;      /* independent copies of the program, each on a 1/slices part of every chunk */
  int32_t piece_bytes; /* bytes of one chunk moved per step per pass of the step list            */
  int32_t fifo_depth;  /* messages a connection can hold                                         */
  int32_t threads;     /* threads per workgroup: 64, 128, 256, 512 or 1024                       */
  int32_t timeout_ms;  /* in-kernel watchdog; default 10000                                      */
  int32_t max_workgroups; /* cap on resident workgroups assumed when no device is queried (tests) */
  int32_t staging;     /* 0: a receiver reads a payload in place where that is provably safe; 1: always stage in FIFO slots */
  int32_t workgroups;  /* resident workgroups that share the (threadblock, slice) contexts       */
  int32_t protocol;    /* 0 automatic, MSCCLX_PROTO_SIMPLE, MSCCLX_PROTO_LL                       */
  int32_t reserved[3];
} mscclx_config;

typedef struct {
  int32_t workgroups;  /* resident workgroups; threadblocks * slices contexts are spread over them */
  int32_t threads;
  int32_t slices;
  int32_t piece_bytes;
  int32_t fifo_depth;
  int32_t passes;      /* passes of the step list the longest slice makes          */
  int32_t connections;
  int32_t vector_path; /* always 1: every chunk size moves in 16-byte units            */
  int32_t zero_copy_messages; /* messages per pass read in place instead of staged  */
  int32_t staged_messages;
  int32_t max_hosted;  /* most contexts any workgroup hosts                         */
  int32_t protocol;    /* MSCCLX_PROTO_SIMPLE or MSCCLX_PROTO_LL                    */
  int32_t waiting_ratio_x100; /* 100 * threadblocks * depth of the dataflow / moving steps: 100 = every threadblock always has work (a ring) */
  int32_t dataflow_depth;     /* moving steps on the longest chain through step order, dependencies and messages */
  int32_t kernel_loop; /* mscclx_loop: which of the kernels' step loops this geometry runs */
  int32_t cold_traffic_x100; /* 100 * share of the algorithmic bytes that memory sees once only: inputs read, results written */
  uint64_t workspace_bytes;
  uint64_t algorithmic_units; /* sum over ops of cnt * a(type); times chunk_bytes = algorithmic bytes */
} mscclx_info;

typedef struct {
  int32_t code;   /* mscclx_error of the last finished launch */
  int32_t tb;     /* global threadblock row that gave up      */
  int32_t step;
  int32_t slice;
  int64_t pass;
  int32_t waiting_on; /* 0 dependency flag, 1 incoming message, 2 free slot on the outgoing connection */
  int32_t reserved;
} mscclx_status;

typedef struct mscclx_plan mscclx_plan;

int mscclx_version(void);
const char* mscclx_last_error(void);

/* Validates the tables (ranges, one sending and one receiving threadblock per connection
 * (rank, peer, chan), sends matched by receives in order with equal cnt —
 * msccl/language/passes.py:31-55, tb_assignment.py:12-19) and builds the host plan.  Uses no GPU. */
int mscclx_plan_create(const mscclx_plan_desc* desc, mscclx_plan** out);
int mscclx_plan_destroy(mscclx_plan* plan);

/* Dry-runs one pass of the step lists on the host with `fifo_depth` messages per connection
 * (0 = unbounded).  MSCCLX_OK or MSCCLX_ERR_DEADLOCK.  Uses no GPU. */
int mscclx_plan_simulate(const mscclx_plan* plan, int32_t fifo_depth);
/* Smallest connection depth with which the program finishes; negative error if none does. */
int mscclx_plan_min_fifo_depth(const mscclx_plan* plan);
/* sum over ops of cnt * a(type), a = {s:0, r:2, rcs:2, rrc:3, rrs:3, rrcs:3, cpy:2, re:3, nop:0}. */
uint64_t mscclx_plan_algorithmic_units(const mscclx_plan* plan);

/* Fixes the geometry for chunks of `chunk_bytes` bytes of `dtype` and reports it, including the
 * workspace the caller must provide.  Queries the current device unless cfg->max_workgroups > 0.
 * Any positive multiple of the element size is accepted (fastest when chunks start on cache
 * lines: multiples of 128 bytes). */
int mscclx_plan_configure(mscclx_plan* plan, size_t chunk_bytes, int32_t dtype, int32_t redop,
                          const mscclx_config* cfg, mscclx_info* info);

/* Attaches device memory: in/out/scratch[r] are rank r's buffers of i/o/s_chunks * chunk_bytes
 * bytes (may be NULL where the extent is 0; in == out aliasing is the caller's choice, as with an
 * in-place NCCL call; buffers that overlap in memory need a plan configured with staging=1, else
 * MSCCLX_ERR_ALIASED).  A buffer must start on a boundary of its element type; a view into a
 * larger tensor is fine.
 * Uploads the plan tables to the current device and arms the workspace (counters zero, the plan's
 * stamp in control word 2).  Binding again after a launch has been waited for (new buffers, same
 * geometry) re-uses the device-side allocations -- one upload of the tables, no allocation -- and
 * clears the workspace again only if it must: another address, a lost launch before, or a stamp
 * that is no longer this plan's because another plan was bound to the same memory in between. */
int mscclx_plan_bind(mscclx_plan* plan, void* const* in, void* const* out, void* const* scratch,
                     void* workspace, size_t workspace_bytes);

/* Enqueues one execution of the whole algorithm on `stream` (a hipStream_t; NULL = default). */
int mscclx_plan_launch(mscclx_plan* plan, void* stream);
/* Waits for `stream` and reports how the last launch ended. */
int mscclx_plan_wait(mscclx_plan* plan, void* stream, mscclx_status* status);
/* The same without blocking: 1 while work is still queued or running on `stream` (a watchdog report
 * that has already arrived is copied to `status`), else what mscclx_plan_wait would return. */
int mscclx_plan_poll(mscclx_plan* plan, void* stream, mscclx_status* status);
/* Asks the running launch (and any launch of this plan queued behind it) to give up: every
 * workgroup sees the request while it polls and leaves, every wave exits normally.  Returns once
 * the request is on the device; mscclx_plan_wait then returns MSCCLX_ERR_ABORTED, the rank buffers
 * hold partial results, and the next mscclx_plan_launch re-arms the counters.  A launch replayed from
 * a HIP graph passes by that re-arming: the first replay after an abort may still find the request,
 * ends at once and is reported as MSCCLX_ERR_ABORTED by the wait that follows it; the replay after
 * that runs normally (every launch clears the counters the next one uses). */
int mscclx_plan_abort(mscclx_plan* plan);
/* Bytes of the device array behind mscclx_plan_run_static (one copy per GPU, held until the process ends). */
#define MSCCLX_STATIC_SCRATCH_BYTES (32u << 20)
/* No counterpart in msccl-tools.  For callers that cannot allocate device memory (tight serving
 * loops, harnesses that forbid hipMalloc): one whole execution of a configured plan -- bind, launch,
 * wait -- that calls no hipMalloc, hipFree or other allocating routine.  The plan tables, the
 * counters and the FIFO slots, which mscclx_plan_bind keeps in memory it allocates and in the
 * caller's workspace, live in a device array that is part of the library; the caller passes only
 * the rank buffers (as to mscclx_plan_bind).  A plan that needs more than
 * MSCCLX_STATIC_SCRATCH_BYTES for them is refused with MSCCLX_ERR_CAPACITY.  Returns when the
 * launch has finished, with mscclx_plan_wait's result.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (from several threads or streams) race, and a call must
 * not overlap a launch of the same plan made through mscclx_plan_launch either.  The plan's own
 * binding (mscclx_plan_bind) is left untouched. */
int mscclx_plan_run_static(mscclx_plan* plan, void* const* in, void* const* out, void* const* rank_scratch,
                           void* stream, mscclx_status* status);
/* Times `iters` back-to-back launches with HIP events on `stream`; ms_out[i] = duration of launch i. */
int mscclx_plan_time(mscclx_plan* plan, void* stream, int32_t iters, float* ms_out);

#ifdef __cplusplus
}
#endif
#endif /* MSCCLX_H */
