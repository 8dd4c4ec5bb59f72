// MI355X (gfx950) executor kernels for MSCCL-IR and the device half of the C ABI.
//
// Execution model.  All ranks of the algorithm are virtual ranks whose buffers live in this GPU's
// HBM.  Every <tb> of every rank is run by `slices` persistent workgroups; workgroup (tb, j) owns
// the j-th 1/slices part of EVERY chunk, which is legal because every IR step is element-wise, and
// makes the parts fully independent (own FIFOs, own counters).  A workgroup walks its step list once
// per "pass"; a pass moves one piece (piece_units) of each chunk its steps name, so a connection's
// message is cnt pieces and fits a bounded FIFO slot in HBM whatever the chunk size.
//
// Synchronisation (all counters monotone, 64-bit, one per 64 bytes, agent scope):
//   flag[tb]   = pass*nsteps + step + 1 of the last finished step with hasdep=1     (depid/deps wait)
//   head[conn] = messages produced;  tail[conn] = messages consumed                  (FIFO hand-off)
// Wave 0 polls up to three conditions at once, one per lane; a barrier releases the other waves.
// Payload is read and written with device-scope (sc1) accesses only, so a producer publishes by
// waiting for its stores to be acknowledged, a workgroup barrier, and a counter store; a consumer
// reads the payload after its poll succeeds.  No cache-wide write-back or invalidate is issued.
// Two counter areas alternate between launches: a launch clears the area the next launch will
// use, so no memset sits between launches.
//
// Every wait is bounded by a wall-clock watchdog; on expiry the workgroup raises the area's abort
// word, all other workgroups see it in their own waits, and every wave leaves the kernel.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <utility>
#include <string>
#include <vector>

#include "plan.h"

namespace mscclx {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

#define HIP_TRY(expr)                                                                              \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess)                                                                          \
      return fail(MSCCLX_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));              \
  } while (0)

// ------------------------------------------------------------------------------------------------
// element-wise reducers.  Reducer<DT, OP>::combine<S>(a, b) reduces two storage words of type S
// (one element of 1/2/4/8 bytes, or 16 bytes of elements) element by element.
// ------------------------------------------------------------------------------------------------
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

template <int OP, typename T>
__device__ __forceinline__ T red_int(T a, T b) {
  if (OP == MSCCLX_SUM) return (T)(a + b);
  if (OP == MSCCLX_PROD) return (T)(a * b);
  if (OP == MSCCLX_MAX) return a > b ? a : b;
  return a < b ? a : b;
}
template <int OP>
__device__ __forceinline__ float red_float(float a, float b) {
  if (OP == MSCCLX_SUM) return a + b;
  if (OP == MSCCLX_PROD) return a * b;
  if (OP == MSCCLX_MAX) return fmaxf(a, b);
  return fminf(a, b);
}
template <int OP>
__device__ __forceinline__ double red_double(double a, double b) {
  if (OP == MSCCLX_SUM) return a + b;
  if (OP == MSCCLX_PROD) return a * b;
  if (OP == MSCCLX_MAX) return fmax(a, b);
  return fmin(a, b);
}

__device__ __forceinline__ float bf16_to_f32(unsigned short h) { return __uint_as_float((unsigned)h << 16); }
__device__ __forceinline__ unsigned short f32_to_bf16(float f) {  // round to nearest even, quiet NaN
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x0040u);
  return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float f16_to_f32(unsigned short h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ unsigned short f32_to_f16(float f) { return __builtin_bit_cast(unsigned short, (_Float16)f); }

// Element arithmetic per dtype on raw element storage E (unsigned type of the element's size).
// 16-bit floats: widen to fp32, operate, round to nearest even once.  For sum this equals the
// correctly rounded 16-bit result (24 >= 2p+2 for p = 11 and p = 8); products of two 16-bit values
// are exact in fp32, so they too are rounded once.
template <int DT, int OP> struct ElemOp;
#define MSCCLX_INT_ELEM(DT, T, E)                                                                  \
  template <int OP> struct ElemOp<DT, OP> {                                                        \
    typedef E store;                                                                               \
    static __device__ __forceinline__ E op(E a, E b) { return (E)red_int<OP, T>((T)a, (T)b); }     \
  };
MSCCLX_INT_ELEM(MSCCLX_U8, unsigned char, unsigned char)
MSCCLX_INT_ELEM(MSCCLX_I8, signed char, unsigned char)
MSCCLX_INT_ELEM(MSCCLX_I32, int, unsigned int)
MSCCLX_INT_ELEM(MSCCLX_U32, unsigned int, unsigned int)
MSCCLX_INT_ELEM(MSCCLX_I64, long long, unsigned long long)
MSCCLX_INT_ELEM(MSCCLX_U64, unsigned long long, unsigned long long)
template <int OP> struct ElemOp<MSCCLX_F16, OP> {
  typedef unsigned short store;
  static __device__ __forceinline__ unsigned short op(unsigned short a, unsigned short b) { return f32_to_f16(red_float<OP>(f16_to_f32(a), f16_to_f32(b))); }
};
template <int OP> struct ElemOp<MSCCLX_BF16, OP> {
  typedef unsigned short store;
  static __device__ __forceinline__ unsigned short op(unsigned short a, unsigned short b) { return f32_to_bf16(red_float<OP>(bf16_to_f32(a), bf16_to_f32(b))); }
};
template <int OP> struct ElemOp<MSCCLX_F32, OP> {
  typedef unsigned int store;
  static __device__ __forceinline__ unsigned int op(unsigned int a, unsigned int b) { return __float_as_uint(red_float<OP>(__uint_as_float(a), __uint_as_float(b))); }
};
template <int OP> struct ElemOp<MSCCLX_F64, OP> {
  typedef unsigned long long store;
  static __device__ __forceinline__ unsigned long long op(unsigned long long a, unsigned long long b) {
    return __builtin_bit_cast(unsigned long long, red_double<OP>(__builtin_bit_cast(double, a), __builtin_bit_cast(double, b)));
  }
};

template <int DT, int OP> struct Reducer {
  typedef ElemOp<DT, OP> E;
  typedef typename E::store store;
  static constexpr int kElemBytes = sizeof(store);
  // 16 bytes of elements
  static __device__ __forceinline__ u32x4 combine(u32x4 a, u32x4 b) {
    typedef store vt __attribute__((ext_vector_type(16 / sizeof(store))));
    vt x = __builtin_bit_cast(vt, a), y = __builtin_bit_cast(vt, b), r;
#pragma unroll
    for (int i = 0; i < (int)(16 / sizeof(store)); ++i) r[i] = E::op(x[i], y[i]);
    return __builtin_bit_cast(u32x4, r);
  }
  // one element held in the word a buffer access of its size returns
  static __device__ __forceinline__ unsigned char combine(unsigned char a, unsigned char b) { return (unsigned char)E::op((store)a, (store)b); }
  static __device__ __forceinline__ unsigned short combine(unsigned short a, unsigned short b) { return (unsigned short)E::op((store)a, (store)b); }
  static __device__ __forceinline__ unsigned int combine(unsigned int a, unsigned int b) { return (unsigned int)E::op((store)a, (store)b); }
  static __device__ __forceinline__ u32x2 combine(u32x2 a, u32x2 b) {
    return __builtin_bit_cast(u32x2, (unsigned long long)E::op((store)__builtin_bit_cast(unsigned long long, a), (store)__builtin_bit_cast(unsigned long long, b)));
  }
};

// ------------------------------------------------------------------------------------------------
// memory access.  Every load and store of payload goes through a raw buffer descriptor with the
// device-scope cache policy (sc1): stores are written through this XCD's L2 and loads do not hit
// lines the L2 may hold from before, so data handed from one workgroup to another (possibly on
// another XCD, with its own L2) needs no cache-wide write-back or invalidate -- only
// "my stores are acknowledged" (s_waitcnt vmcnt(0)) before the counter that announces them.
// The descriptor also bounds every access: lanes past the end of a piece load 0 and store nothing.
// ------------------------------------------------------------------------------------------------
#ifndef MSCCLX_AUX
#define MSCCLX_AUX 16 /* sc1 = device scope */
#endif
constexpr int kBufferFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family dword 3)

template <int W> struct Access;
template <> struct Access<16> {
  typedef u32x4 word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, AUX); }
};
template <> struct Access<8> {
  typedef u32x2 word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b64(v, r, off, 0, AUX); }
};
template <> struct Access<4> {
  typedef unsigned int word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, off, 0, AUX); }
};
template <> struct Access<2> {
  typedef unsigned short word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b16(v, r, off, 0, AUX); }
};
template <> struct Access<1> {
  typedef unsigned char word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b8(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b8(v, r, off, 0, AUX); }
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kBufferFlags);
}

#ifndef MSCCLX_UNROLL
#define MSCCLX_UNROLL 4
#endif
constexpr int kUnroll = MSCCLX_UNROLL;

// out1[, out2] = a [(+) b] over n units of W bytes.
template <class R, int W, bool HAS_B, bool HAS_O2>
__device__ __forceinline__ void move_units(unsigned char* o1, unsigned char* o2, const unsigned char* a, const unsigned char* b, uint32_t n) {
  typedef Access<W> A;
  typedef typename A::word word;
  constexpr int X = MSCCLX_AUX;
  const uint32_t bytes = n * W;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, bytes), r1 = make_rsrc(o1, bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(HAS_B ? b : a, bytes), r2 = make_rsrc(HAS_O2 ? o2 : o1, bytes);
  const uint32_t T = blockDim.x;
  for (uint32_t i = threadIdx.x; i < n; i += kUnroll * T) {
    word x[kUnroll], y[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) x[u] = A::template ld<X>(ra, (int)((i + u * T) * W));
    if (HAS_B) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) y[u] = A::template ld<X>(rb, (int)((i + u * T) * W));
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) x[u] = R::combine(y[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) A::template st<X>(r1, (int)((i + u * T) * W), x[u]);
    if (HAS_O2) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) A::template st<X>(r2, (int)((i + u * T) * W), x[u]);
    }
  }
}

// rows x n units.  Consecutive rows of an operand are `stride_*` units apart: a chunk for rank
// buffers, n for the packed rows of a FIFO slot.  b (the local reduction operand) is always a rank
// buffer, o2 (the forwarded copy) always a FIFO slot.
template <class R, bool VEC, bool HAS_B, bool HAS_O2>
__device__ __forceinline__ void move_rows(unsigned char* o1, uint64_t stride_o1, unsigned char* o2, const unsigned char* a, uint64_t stride_a,
                                          const unsigned char* b, uint64_t stride_b, int rows, uint32_t n) {
  constexpr int W = VEC ? 16 : R::kElemBytes;
  for (int r = 0; r < rows; ++r)
    move_units<R, W, HAS_B, HAS_O2>(o1 + (uint64_t)r * stride_o1 * W, HAS_O2 ? o2 + (uint64_t)r * n * W : nullptr,
                                    a + (uint64_t)r * stride_a * W, HAS_B ? b + (uint64_t)r * stride_b * W : nullptr, n);
}

// ------------------------------------------------------------------------------------------------
// waiting
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ u64 load_counter(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void publish(u64* p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Called by the 64 lanes of wave 0.  Lane l < 3 waits for *addr[l] >= target[l] (null = nothing to
// wait for).  Returns -1 when all conditions hold, else the index of a condition that timed out (or 3
// when another workgroup raised the abort word).
__device__ __forceinline__ int wait_conditions(const u64* a0, u64 t0, const u64* a1, u64 t1, const u64* a2, u64 t2,
                                               const u64* abort_word, u64 deadline) {
  const int lane = threadIdx.x;
  const u64* addr = lane == 0 ? a0 : lane == 1 ? a1 : lane == 2 ? a2 : nullptr;
  const u64 target = lane == 0 ? t0 : lane == 1 ? t1 : t2;
  int result = -1;
  unsigned spins = 0;
  for (;;) {
    bool ok = true;
    if (addr) ok = load_counter(addr) >= target;
    if (__all(ok)) break;
    __builtin_amdgcn_s_sleep(1);
    if ((++spins & 0xffu) == 0) {
      bool stop = false;
      if (lane == 0) stop = load_counter(abort_word) != 0;
      if (__any(stop)) { result = 3; break; }
      if (wall_clock64() > deadline) {
        const u64 bad = __ballot(!ok);
        result = bad ? __ffsll((long long)bad) - 1 : 3;
        break;
      }
    }
  }
  return result;
}

// ------------------------------------------------------------------------------------------------
// the executor kernel
// ------------------------------------------------------------------------------------------------
template <class R, bool VEC>
__global__ void __launch_bounds__(512) exec_kernel(const KernelParams p) {
  constexpr uint64_t UB = VEC ? 16 : R::kElemBytes;
  __shared__ int sh_fail;
  const int tbi = blockIdx.x / p.slices;
  const int j = blockIdx.x % p.slices;
  const DevTb tb = p.tbs[tbi];

  u64* const area = p.sync_cur + kSyncHeaderWords + (uint64_t)j * p.sync_slice_words;
  u64* const flags = area;
  u64* const heads = area + (uint64_t)p.ntbs * kSyncStrideWords;
  u64* const tails = heads + (uint64_t)p.nconns * kSyncStrideWords;
  const u64* const abort_word = p.sync_cur;

  if (threadIdx.x == 0) {
    sh_fail = 0;
    // clear, for the next launch, the counters this workgroup is the only writer of
    u64* nxt = p.sync_nxt + kSyncHeaderWords + (uint64_t)j * p.sync_slice_words;
    nxt[(uint64_t)tbi * kSyncStrideWords] = 0;
    if (tb.send_conn >= 0) nxt[((uint64_t)p.ntbs + tb.send_conn) * kSyncStrideWords] = 0;
    if (tb.recv_conn >= 0) nxt[((uint64_t)p.ntbs + p.nconns + tb.recv_conn) * kSyncStrideWords] = 0;
    if (blockIdx.x == 0) p.sync_nxt[0] = 0;
  }
  __syncthreads();

  // this slice's part of every chunk: units [u0, u1)
  const uint64_t u0 = p.chunk_units * (uint64_t)j / p.slices;
  const uint64_t u1 = p.chunk_units * (uint64_t)(j + 1) / p.slices;
  unsigned char* const fifo_slice = p.fifo + (uint64_t)j * p.slice_fifo_units * UB;
  unsigned char* fifo_out = nullptr;
  const unsigned char* fifo_in = nullptr;
  uint32_t slot_out = 0, slot_in = 0;
  if (tb.send_conn >= 0) { fifo_out = fifo_slice + p.conns[tb.send_conn].fifo_off * UB; slot_out = p.conns[tb.send_conn].slot_units; }
  if (tb.recv_conn >= 0) { fifo_in = fifo_slice + p.conns[tb.recv_conn].fifo_off * UB; slot_in = p.conns[tb.recv_conn].slot_units; }
  u64* const my_flag = flags + (uint64_t)tbi * kSyncStrideWords;
  u64* const my_head = tb.send_conn >= 0 ? heads + (uint64_t)tb.send_conn * kSyncStrideWords : nullptr;
  u64* const my_tail = tb.recv_conn >= 0 ? tails + (uint64_t)tb.recv_conn * kSyncStrideWords : nullptr;
  const u64* const peer_tail = tb.send_conn >= 0 ? tails + (uint64_t)tb.send_conn * kSyncStrideWords : nullptr;
  const u64* const peer_head = tb.recv_conn >= 0 ? heads + (uint64_t)tb.recv_conn * kSyncStrideWords : nullptr;
  const u64 deadline = wall_clock64() + p.timeout_ticks;

  u64 pass = 0;
  for (uint64_t off = u0; off < u1; off += p.piece_units, ++pass) {
    const uint32_t n = (uint32_t)((u1 - off) < (uint64_t)p.piece_units ? (u1 - off) : (uint64_t)p.piece_units);
    for (int s = 0; s < tb.nops; ++s) {
      const DevOp op = p.ops[tb.op_begin + s];
      const int t = op.type;
      const bool rcv = t == MSCCLX_OP_RECV || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRCS;
      const bool snd = t == MSCCLX_OP_SEND || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRCS;
      const u64 sseq = snd ? pass * (u64)tb.nsend + (u64)op.send_seq : 0;
      const u64 rseq = rcv ? pass * (u64)tb.nrecv + (u64)op.recv_seq : 0;

      // ---- wait: dependency, incoming message, free outgoing slot ----
      const u64* a0 = nullptr; u64 t0 = 0;
      const u64* a1 = nullptr; u64 t1 = 0;
      const u64* a2 = nullptr; u64 t2 = 0;
      if (op.dep_tb >= 0) { a0 = flags + (uint64_t)op.dep_tb * kSyncStrideWords; t0 = pass * (u64)op.dep_nops + (u64)op.dep_step + 1; }
      if (rcv) { a1 = peer_head; t1 = rseq + 1; }
      if (snd && sseq >= (u64)p.depth) { a2 = peer_tail; t2 = sseq + 1 - (u64)p.depth; }
      if (a0 || a1 || a2) {
        if (threadIdx.x < 64) {
          const int w = wait_conditions(a0, t0, a1, t1, a2, t2, abort_word, deadline);
          if (w >= 0 && threadIdx.x == 0) {
            sh_fail = 1;
            if (w < 3 && atomicCAS((u64*)abort_word, 0ull, 1ull) == 0ull) {
              mscclx_status* hs = p.host_status;
              hs->tb = tbi; hs->step = s; hs->slice = j; hs->pass = (int64_t)pass; hs->waiting_on = w;
              __threadfence_system();
              __hip_atomic_store(&hs->code, (int)MSCCLX_ERR_TIMEOUT, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            }
          }
        }
        __syncthreads();
        if (sh_fail) return;
      }

      // ---- move data ----
      // in: the incoming payload -- packed in a FIFO slot, or still where the sender has it (then
      // rows are a chunk apart, like any rank buffer).  out: the FIFO slot to fill, or null when the
      // receiver will read this step's payload in place.
      if (t != MSCCLX_OP_NOP) {
        const uint64_t cs = p.chunk_units;
        const unsigned char* lsrc = nullptr;
        unsigned char* ldst = nullptr;
        if (t == MSCCLX_OP_SEND || t == MSCCLX_OP_COPY || t == MSCCLX_OP_REDUCE)
          lsrc = (const unsigned char*)p.bufs[op.src_slot] + ((uint64_t)op.srcoff * cs + off) * UB;
        if (t != MSCCLX_OP_SEND)
          ldst = (unsigned char*)p.bufs[op.dst_slot] + ((uint64_t)op.dstoff * cs + off) * UB;
        unsigned char* out = (snd && op.out_staged) ? fifo_out + (sseq % (u64)p.depth) * slot_out * UB : nullptr;
        const unsigned char* in = nullptr;
        uint64_t in_stride = n;
        if (rcv) {
          if (op.in_slot >= 0) {
            in = (const unsigned char*)p.bufs[op.in_slot] + ((uint64_t)op.in_off * cs + off) * UB;
            in_stride = cs;
          } else {
            in = fifo_in + (rseq % (u64)p.depth) * slot_in * UB;
          }
        }
        switch (t) {
          case MSCCLX_OP_SEND:
            if (out) move_rows<R, VEC, false, false>(out, n, nullptr, lsrc, cs, nullptr, 0, op.cnt, n);
            break;
          case MSCCLX_OP_RECV: move_rows<R, VEC, false, false>(ldst, cs, nullptr, in, in_stride, nullptr, 0, op.cnt, n); break;
          case MSCCLX_OP_RCS:
            if (out) move_rows<R, VEC, false, true>(ldst, cs, out, in, in_stride, nullptr, 0, op.cnt, n);
            else     move_rows<R, VEC, false, false>(ldst, cs, nullptr, in, in_stride, nullptr, 0, op.cnt, n);
            break;
          case MSCCLX_OP_RRC: move_rows<R, VEC, true, false>(ldst, cs, nullptr, in, in_stride, ldst, cs, op.cnt, n); break;
          case MSCCLX_OP_RRS: move_rows<R, VEC, true, false>(out, n, nullptr, in, in_stride, ldst, cs, op.cnt, n); break;
          case MSCCLX_OP_RRCS:
            if (out) move_rows<R, VEC, true, true>(ldst, cs, out, in, in_stride, ldst, cs, op.cnt, n);
            else     move_rows<R, VEC, true, false>(ldst, cs, nullptr, in, in_stride, ldst, cs, op.cnt, n);
            break;
          case MSCCLX_OP_COPY:   move_rows<R, VEC, false, false>(ldst, cs, nullptr, lsrc, cs, nullptr, 0, op.cnt, n); break;
          case MSCCLX_OP_REDUCE: move_rows<R, VEC, true, false>(ldst, cs, nullptr, lsrc, cs, ldst, cs, op.cnt, n); break;
          default: break;
        }
      }

      // ---- publish ----
      if (rcv || snd || op.hasdep) {
        // each wave waits until its own device-scope stores are acknowledged; after the barrier
        // thread 0 may therefore announce the whole workgroup's data with plain counter stores
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (threadIdx.x == 0) {
          if (snd) publish(my_head, sseq + 1);
          if (rcv) publish(my_tail, rseq + 1);
          if (op.hasdep) publish(my_flag, pass * (u64)tb.nops + (u64)s + 1);
        }
      } else if (t != MSCCLX_OP_NOP) {
        __syncthreads();  // a later step of this threadblock may read what this one wrote
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// host: kernel table, configure, bind, launch
// ------------------------------------------------------------------------------------------------
typedef void (*kernel_fn)(const KernelParams);

template <int DT, int OP> static kernel_fn pick_vec(bool vec) {
  return vec ? (kernel_fn)exec_kernel<Reducer<DT, OP>, true> : (kernel_fn)exec_kernel<Reducer<DT, OP>, false>;
}
template <int DT> static kernel_fn pick_op(int op, bool vec) {
  switch (op) {
    case MSCCLX_SUM: return pick_vec<DT, MSCCLX_SUM>(vec);
    case MSCCLX_PROD: return pick_vec<DT, MSCCLX_PROD>(vec);
    case MSCCLX_MAX: return pick_vec<DT, MSCCLX_MAX>(vec);
    case MSCCLX_MIN: return pick_vec<DT, MSCCLX_MIN>(vec);
    default: return nullptr;
  }
}
static kernel_fn pick_kernel(int dtype, int op, bool vec) {
  switch (dtype) {
    case MSCCLX_U8: return pick_op<MSCCLX_U8>(op, vec);
    case MSCCLX_I8: return pick_op<MSCCLX_I8>(op, vec);
    case MSCCLX_I32: return pick_op<MSCCLX_I32>(op, vec);
    case MSCCLX_U32: return pick_op<MSCCLX_U32>(op, vec);
    case MSCCLX_I64: return pick_op<MSCCLX_I64>(op, vec);
    case MSCCLX_U64: return pick_op<MSCCLX_U64>(op, vec);
    case MSCCLX_F16: return pick_op<MSCCLX_F16>(op, vec);
    case MSCCLX_BF16: return pick_op<MSCCLX_BF16>(op, vec);
    case MSCCLX_F32: return pick_op<MSCCLX_F32>(op, vec);
    case MSCCLX_F64: return pick_op<MSCCLX_F64>(op, vec);
    default: return nullptr;
  }
}

struct DeviceState {
  int device = -1;
  DevTb* tbs = nullptr;
  DevOp* ops = nullptr;
  DevConn* conns = nullptr;
  void** bufs = nullptr;
  mscclx_status* host_status = nullptr;  // pinned, device-visible
  unsigned char* workspace = nullptr;
  kernel_fn kernel = nullptr;
  unsigned launches = 0;
  bool dirty = false;  // counters must be cleared before the next launch (after a failed launch)
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

void destroy_device_state(DeviceState* d) {
  if (!d) return;
  if (d->tbs) (void)hipFree(d->tbs);
  if (d->ops) (void)hipFree(d->ops);
  if (d->conns) (void)hipFree(d->conns);
  if (d->bufs) (void)hipFree(d->bufs);
  if (d->host_status) (void)hipHostFree(d->host_status);
  if (d->ev0) (void)hipEventDestroy(d->ev0);
  if (d->ev1) (void)hipEventDestroy(d->ev1);
  delete d;
}

static int query_capacity(kernel_fn k, int* num_cus, int capacity[4]) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, dev));
  *num_cus = prop.multiProcessorCount;
  const int threads[4] = {64, 128, 256, 512};
  for (int i = 0; i < 4; ++i) {
    int per_cu = 0;
    HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k, threads[i], 0));
    capacity[i] = per_cu * prop.multiProcessorCount;
  }
  return MSCCLX_OK;
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
  const bool vec = chunk_bytes % 16 == 0;
  int num_cus = 256;
  int capacity[4];
  if (cfg.max_workgroups > 0) {
    for (int i = 0; i < 4; ++i) capacity[i] = cfg.max_workgroups;
  } else {
    kernel_fn k = pick_kernel(dtype, redop, vec);
    int rc = query_capacity(k, &num_cus, capacity);
    if (rc) return rc;
  }
  Geometry g;
  int rc = decide_geometry(*plan, chunk_bytes, dtype, cfg, num_cus, capacity, &g);
  if (rc) return rc;
  plan->geo = g;
  plan->chunk_bytes = chunk_bytes;
  plan->dtype = dtype;
  plan->redop = redop;
  plan->timeout_ms = cfg.timeout_ms > 0 ? cfg.timeout_ms : 10000;
  plan->configured = true;
  if (plan->dev) { destroy_device_state(plan->dev); plan->dev = nullptr; }
  if (info) {
    info->workgroups = (int32_t)plan->tbs.size() * g.slices;
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
  std::vector<void*> bufs((size_t)plan->nranks * 3, nullptr);
  void* const* tables[3] = {in, out, scratch};
  for (int r = 0; r < plan->nranks; ++r)
    for (int b = 0; b < 3; ++b) {
      void* ptr = tables[b] ? tables[b][r] : nullptr;
      if (plan->rank_chunks[(size_t)r * 3 + b] > 0) {
        if (!ptr) return fail(MSCCLX_ERR_INVALID_ARG, "rank " + std::to_string(r) + ": buffer " + "ios"[b] + " is used by the algorithm but NULL was given");
        if (g.vector_path && (uintptr_t)ptr % 16) return fail(MSCCLX_ERR_INVALID_ARG, "rank " + std::to_string(r) + ": buffers must be 16-byte aligned");
        if ((uintptr_t)ptr % dtype_size(plan->dtype)) return fail(MSCCLX_ERR_INVALID_ARG, "rank " + std::to_string(r) + ": buffer not aligned to its element type");
      }
      bufs[(size_t)r * 3 + b] = ptr;
    }

  if (!g.staging) {
    // reading payloads in place assumes that distinct buffers are distinct memory
    std::vector<std::pair<uintptr_t, uintptr_t>> spans;
    for (int r = 0; r < plan->nranks; ++r)
      for (int b = 0; b < 3; ++b) {
        const size_t len = (size_t)plan->rank_chunks[(size_t)r * 3 + b] * plan->chunk_bytes;
        if (len) spans.push_back({(uintptr_t)bufs[(size_t)r * 3 + b], (uintptr_t)bufs[(size_t)r * 3 + b] + len});
      }
    std::sort(spans.begin(), spans.end());
    for (size_t k = 1; k < spans.size(); ++k)
      if (spans[k].first < spans[k - 1].second)
        return fail(MSCCLX_ERR_INVALID_ARG, "rank buffers overlap in memory; configure the plan with staging=1 for aliased buffers");
  }
  if (plan->dev) { destroy_device_state(plan->dev); plan->dev = nullptr; }
  DeviceState* d = new DeviceState();
  plan->dev = d;
  HIP_TRY(hipGetDevice(&d->device));
  d->kernel = pick_kernel(plan->dtype, plan->redop, g.vector_path != 0);
  if (!d->kernel) return fail(MSCCLX_ERR_UNSUPPORTED, "no kernel for this dtype/reduction");

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
      dv.type = op.type; dv.cnt = op.cnt;
      dv.src_slot = tb.rank * 3 + (op.srcbuf >= 0 && op.srcbuf <= 2 ? op.srcbuf : 0); dv.srcoff = op.srcoff;
      dv.dst_slot = tb.rank * 3 + (op.dstbuf >= 0 && op.dstbuf <= 2 ? op.dstbuf : 0); dv.dstoff = op.dstoff;
      dv.dep_tb = -1; dv.dep_step = -1; dv.dep_nops = 0;
      if (op.depid >= 0) {
        dv.dep_tb = plan->rank_tb_begin[tb.rank] + op.depid;
        dv.dep_step = op.deps;
        dv.dep_nops = plan->tbs[dv.dep_tb].op_end - plan->tbs[dv.dep_tb].op_begin;
      }
      dv.hasdep = op.hasdep; dv.send_seq = op.send_seq; dv.recv_seq = op.recv_seq;
      dv.in_slot = -1; dv.in_off = -1; dv.pad = 0;
      dv.out_staged = is_send_type(op.type) && (g.staging || !op.zero_copy) ? 1 : 0;
      if (is_recv_type(op.type) && !g.staging) {
        const Op& sender = plan->ops[op.match_send];
        if (sender.zero_copy) {  // read the payload where the sending rank keeps it
          const int sender_rank = plan->tbs[plan->conns[tb.recv_conn].send_tb].rank;
          const bool from_src = sender.type == MSCCLX_OP_SEND;
          dv.in_slot = sender_rank * 3 + (from_src ? sender.srcbuf : sender.dstbuf);
          dv.in_off = from_src ? sender.srcoff : sender.dstoff;
        }
      }
    }
  }
  HIP_TRY(hipMalloc((void**)&d->tbs, sizeof(DevTb) * (ntb ? ntb : 1)));
  HIP_TRY(hipMalloc((void**)&d->ops, sizeof(DevOp) * (nop ? nop : 1)));
  HIP_TRY(hipMalloc((void**)&d->conns, sizeof(DevConn) * hcn.size()));
  HIP_TRY(hipMalloc((void**)&d->bufs, sizeof(void*) * bufs.size()));
  HIP_TRY(hipMemcpy(d->tbs, htb.data(), sizeof(DevTb) * ntb, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d->ops, hop.data(), sizeof(DevOp) * nop, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d->conns, hcn.data(), sizeof(DevConn) * hcn.size(), hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d->bufs, bufs.data(), sizeof(void*) * bufs.size(), hipMemcpyHostToDevice));
  HIP_TRY(hipHostMalloc((void**)&d->host_status, sizeof(mscclx_status), hipHostMallocDefault));
  std::memset(d->host_status, 0, sizeof(mscclx_status));
  d->workspace = (unsigned char*)workspace;
  HIP_TRY(hipMemset(d->workspace, 0, g.fifo_byte_off));  // both counter areas
  HIP_TRY(hipDeviceSynchronize());
  HIP_TRY(hipEventCreate(&d->ev0));
  HIP_TRY(hipEventCreate(&d->ev1));
  return MSCCLX_OK;
}

int mscclx_plan_launch(mscclx_plan* plan, void* stream) {
  if (!plan || !plan->dev || !plan->dev->kernel) return fail(MSCCLX_ERR_STATE, "bind buffers before launching");
  DeviceState* d = plan->dev;
  const Geometry& g = plan->geo;
  hipStream_t s = (hipStream_t)stream;
  if (d->dirty) {  // the previous launch gave up half-way: its counters mean nothing
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipMemset(d->workspace, 0, g.fifo_byte_off));
    HIP_TRY(hipDeviceSynchronize());
    d->dirty = false;
    d->launches = 0;
  }
  KernelParams kp;
  kp.tbs = d->tbs; kp.ops = d->ops; kp.conns = d->conns; kp.bufs = d->bufs;
  unsigned long long* sync = (unsigned long long*)d->workspace;
  const unsigned parity = d->launches & 1u;
  kp.sync_cur = sync + (uint64_t)parity * g.sync_words;
  kp.sync_nxt = sync + (uint64_t)(parity ^ 1u) * g.sync_words;
  kp.fifo = d->workspace + g.fifo_byte_off;
  kp.host_status = d->host_status;
  kp.chunk_units = g.chunk_units;
  kp.slice_fifo_units = g.slice_fifo_units;
  kp.sync_slice_words = g.sync_slice_words;
  kp.timeout_ticks = (uint64_t)plan->timeout_ms * 100000ull;  // wall_clock64 ticks at 100 MHz
  kp.piece_units = g.piece_units;
  kp.slices = g.slices; kp.depth = g.depth; kp.ntbs = (int)plan->tbs.size(); kp.nconns = (int)plan->conns.size();
  const unsigned grid = (unsigned)plan->tbs.size() * (unsigned)g.slices;
  hipLaunchKernelGGL(d->kernel, dim3(grid), dim3(g.threads), 0, s, kp);
  HIP_TRY(hipGetLastError());
  d->launches++;
  return MSCCLX_OK;
}

int mscclx_plan_wait(mscclx_plan* plan, void* stream, mscclx_status* status) {
  if (!plan || !plan->dev) return fail(MSCCLX_ERR_STATE, "nothing was launched");
  DeviceState* d = plan->dev;
  hipError_t e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) {
    d->dirty = true;
    return fail(MSCCLX_ERR_HIP, std::string("hipStreamSynchronize: ") + hipGetErrorString(e));
  }
  mscclx_status st = *d->host_status;
  if (status) *status = st;
  if (st.code != MSCCLX_OK) {
    d->dirty = true;
    const Tb& tb = plan->tbs[st.tb];
    static const char* what[] = {"its dependency", "an incoming message", "a free slot on its outgoing connection", "?"};
    std::string msg = "watchdog: rank " + std::to_string(tb.rank) + " tb " + std::to_string(tb.local_id) + " step " + std::to_string(st.step) +
                      " (slice " + std::to_string(st.slice) + ", pass " + std::to_string(st.pass) + ") waited more than " +
                      std::to_string(plan->timeout_ms) + " ms for " + what[st.waiting_on & 3];
    std::memset(d->host_status, 0, sizeof(mscclx_status));
    return fail(st.code, msg);
  }
  return MSCCLX_OK;
}

int mscclx_plan_time(mscclx_plan* plan, void* stream, int32_t iters, float* ms_out) {
  if (!plan || !plan->dev) return fail(MSCCLX_ERR_STATE, "bind buffers before timing");
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
