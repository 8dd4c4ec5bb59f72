// MI355X (gfx950) executor kernels for MSCCL-IR (device code; included by exec_kernels.hip).
//
// Execution model.  All ranks of the algorithm are virtual ranks whose buffers live in this GPU's
// HBM.  The program is run as `slices` independent copies, copy j on the j-th 1/slices part of
// EVERY chunk -- legal because every IR step is element-wise -- each with its own FIFOs and counters.
// A context is one <tb> in one slice; it walks its step list once per "pass", a pass moving one piece
// (piece_units) of each chunk its steps name.  Contexts are spread over a fixed number of resident
// workgroups; a workgroup hosts up to 64 of them, polls what all of them wait for in one round of
// loads (one lane of wave 0 per context), and runs whichever is ready, so it never blocks on one
// context and the number of threadblocks is not tied to what fits on the chip.
//
// Synchronisation (all counters monotone, 64-bit, one per 64 bytes, agent scope, per slice):
//   flag[tb]   = pass*nsteps + step + 1 of the last finished step with hasdep=1     (depid/deps wait)
//   head[conn] = messages produced;  tail[conn] = messages consumed                  (FIFO hand-off)
// Payload is read and written with device-scope (sc1) accesses only, so a producer publishes by
// waiting for its stores to be acknowledged, a workgroup barrier, and a counter store; a consumer
// reads the payload after its poll succeeds.  No cache-wide write-back or invalidate is issued.
// A receiver reads a payload where the sender keeps it when the plan proved that safe; only the
// other messages are copied through FIFO slots in HBM.
// Two counter areas alternate between launches: a launch clears the area the next launch will
// use, so no memset sits between launches.
//
// LL variant (flag-in-data, for small pieces): every message is written into its FIFO slot as 16-byte
// lines {d0, flag, d1, flag}, two lines per 16 bytes of payload.  The flag names the launch and the
// message, so a receiver needs no counter: its threads load the lines and retry the ones whose flags
// do not match yet.  The sender's "stores acknowledged -> barrier -> counter store" and the receiver's
// counter poll drop out of the hand-off.  Each 8-byte half of a line carries its own flag, so the
// scheme only relies on 8-byte accesses being indivisible.  Free slots are still granted through the
// tail counters.
//
// Chain loops.  A workgroup of one wave that hosts one context -- the geometry of every latency-bound
// launch -- leaves the hosting machinery: the wave runs its context with all its lanes in a loop
// written for that case (run_chain for lines, run_chain_counters for counters), with the bookkeeping
// in scalar registers.  Same steps, same counters, same slots: such a workgroup talks to workgroups
// that run the general loop.
//
// A workgroup that makes no progress for the watchdog period raises the area's abort word; all
// other workgroups see it while they poll, and every wave leaves the kernel.
#pragma once
#include <hip/hip_runtime.h>

#include "plan.h"

namespace mscclx {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;


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
// Round to nearest even, NaNs quieted with the top of their payload kept: the conversion instruction of gfx950
// (v_cvt_pk_bf16_f32), which gives, for every one of the 2^32 inputs, the bits of the usual integer formula --
// NaN: (u >> 16) | 0x40, else (u + 0x7fff + ((u >> 16) & 1)) >> 16 -- in one operation for two values instead of ten.
__device__ __forceinline__ unsigned short f32_to_bf16(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }
template <int OP>
__device__ __forceinline__ unsigned bf16_pair(unsigned a, unsigned b) {  // two bf16 elements in a dword
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const f32x2 r = {red_float<OP>(__uint_as_float(a << 16), __uint_as_float(b << 16)),
                   red_float<OP>(__uint_as_float(a & 0xffff0000u), __uint_as_float(b & 0xffff0000u))};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(r, bf16x2));
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
    if constexpr (DT == MSCCLX_BF16) return u32x4{bf16_pair<OP>(a.x, b.x), bf16_pair<OP>(a.y, b.y), bf16_pair<OP>(a.z, b.z), bf16_pair<OP>(a.w, b.w)};
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
// Loads are marked non-temporal: every payload byte is read exactly once by the step that loads it.
// Stores stay cacheable (a peer or a later step reads most of them soon, and the memory-side cache
// then serves that read) except the ones the plan proved are never read again.
#ifndef MSCCLX_AUX_LD
#define MSCCLX_AUX_LD (MSCCLX_AUX | 2)
#endif
#ifndef MSCCLX_AUX_ST
#define MSCCLX_AUX_ST MSCCLX_AUX
#endif
#ifndef MSCCLX_AUX_ST_FINAL
#define MSCCLX_AUX_ST_FINAL (MSCCLX_AUX | 2)
#endif
constexpr int kBufferFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family dword 3)

template <int W> struct Access;
template <> struct Access<16> {
  typedef u32x4 word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ word lds(__amdgpu_buffer_rsrc_t r, int off, int soff) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, AUX); }
};
template <> struct Access<8> {
  typedef u32x2 word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ word lds(__amdgpu_buffer_rsrc_t r, int off, int soff) { return __builtin_amdgcn_raw_buffer_load_b64(r, off, soff, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b64(v, r, off, 0, AUX); }
};
template <> struct Access<4> {
  typedef unsigned int word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ word lds(__amdgpu_buffer_rsrc_t r, int off, int soff) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, soff, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, off, 0, AUX); }
};
template <> struct Access<2> {
  typedef unsigned short word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ word lds(__amdgpu_buffer_rsrc_t r, int off, int soff) { return __builtin_amdgcn_raw_buffer_load_b16(r, off, soff, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b16(v, r, off, 0, AUX); }
};
template <> struct Access<1> {
  typedef unsigned char word;
  template <int AUX> static __device__ __forceinline__ word ld(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b8(r, off, 0, AUX); }
  template <int AUX> static __device__ __forceinline__ word lds(__amdgpu_buffer_rsrc_t r, int off, int soff) { return __builtin_amdgcn_raw_buffer_load_b8(r, off, soff, AUX); }
  template <int AUX> static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, int off, word v) { __builtin_amdgcn_raw_buffer_store_b8(v, r, off, 0, AUX); }
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kBufferFlags);
}

#ifndef MSCCLX_UNROLL
#define MSCCLX_UNROLL 8
#endif
constexpr int kUnroll = MSCCLX_UNROLL;

// The last 1 to 3 bytes of a row that is no whole number of dwords (chunks of 8- or 16-bit elements that are no
// multiple of 4 bytes), moved element by element by the first lanes: out1[, out2] = a [(+) b].  In two halves, so
// that the loads travel with the row's other loads and the stores with its other stores -- a round trip of its own
// per row would show in every step of a latency-bound program.
template <class R, bool HAS_B>
struct SubDword {
  static constexpr int E = R::kElemBytes < 4 ? R::kElemBytes : 1;  // (wider elements have no such rows; nothing below runs for them)
  typedef Access<E> A;
  typedef typename A::word word;
  word x, y;
  __device__ __forceinline__ void load(const unsigned char* a, const unsigned char* b, uint32_t bytes) {
    if constexpr (R::kElemBytes < 4) {
      const uint32_t i = threadIdx.x * E;
      if (i < bytes) {
        x = A::template ld<MSCCLX_AUX_LD>(make_rsrc(a, bytes), (int)i);
        if (HAS_B) y = A::template ld<MSCCLX_AUX_LD>(make_rsrc(b, bytes), (int)i);
      }
    }
  }
  template <bool HAS_O2, bool NT1>
  __device__ __forceinline__ void store(unsigned char* o1, unsigned char* o2, uint32_t bytes) {
    if constexpr (R::kElemBytes < 4) {
      const uint32_t i = threadIdx.x * E;
      if (i < bytes) {
        if (HAS_B) x = R::combine(y, x);
        A::template st<NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST>(make_rsrc(o1, bytes), (int)i, x);
        if (HAS_O2) A::template st<MSCCLX_AUX_ST>(make_rsrc(o2, bytes), (int)i, x);
      }
    }
  }
};

#ifdef MSCCLX_LDS_STAGING
// (one area for every instantiation of the movers: 64 KiB, so that two workgroups of 512 threads still share a compute unit)
__device__ __noinline__ u32x4* lds_stage_area() {
  __shared__ u32x4 area[(kUnroll / 2 > 0 ? kUnroll / 2 : 1) * 1024];
  return area;
}
#endif

// o1 = a [(+) b] over `bytes` bytes in units of W, UA units in flight per thread and operand: the loop of
// move_units, for the part of a row that starts on a line of its destination.
template <class R, bool HAS_B, bool NT1, int UA>
__device__ __forceinline__ void move_units_body(unsigned char* o1, const unsigned char* a, const unsigned char* b, uint32_t bytes) {
  constexpr int W = 16;
  typedef Access<W> A;
  typedef typename A::word word;
  constexpr int XL = MSCCLX_AUX_LD, X1 = NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, bytes), r1 = make_rsrc(o1, bytes), rb = make_rsrc(HAS_B ? b : a, bytes);
  const uint32_t T = blockDim.x, n = (bytes + W - 1) / W;
  for (uint32_t i = threadIdx.x; i < n; i += UA * T) {
    word x[UA], y[UA];
#pragma unroll
    for (int u = 0; u < UA; ++u) x[u] = A::template ld<XL>(ra, (int)((i + u * T) * W));
    if (HAS_B) {
#pragma unroll
      for (int u = 0; u < UA; ++u) y[u] = A::template ld<XL>(rb, (int)((i + u * T) * W));
#pragma unroll
      for (int u = 0; u < UA; ++u) x[u] = R::combine(y[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < UA; ++u) A::template st<X1>(r1, (int)((i + u * T) * W), x[u]);
  }
}

// out1[, out2] = a [(+) b] over n units of 16 bytes, the last of which lacks `clip` bytes (the end of a chunk that is
// no multiple of 16 bytes: the descriptors end there, so the missing dwords read as zero and are not written --
// the range check is per dword, so descriptors end on whole dwords and what is left of the row, 1 to 3 bytes when a
// chunk is no multiple of 4, goes element by element).
template <class R, bool HAS_B, bool HAS_O2, bool NT1>
__device__ __forceinline__ void move_units(unsigned char* o1, unsigned char* o2, const unsigned char* a, const unsigned char* b, uint32_t n, uint32_t clip) {
  constexpr int W = 16;
  typedef Access<W> A;
  typedef typename A::word word;
  constexpr int XL = MSCCLX_AUX_LD, XS = MSCCLX_AUX_ST, X1 = NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST;
  const uint32_t total = n * W - clip;                       // the row's bytes
  const uint32_t bytes = total & ~3u;                        // what whole dwords cover, counted from the row's start
  const uint32_t odd = total - bytes;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, bytes), r1 = make_rsrc(o1, bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(HAS_B ? b : a, bytes), r2 = make_rsrc(HAS_O2 ? o2 : o1, bytes);
  const uint32_t T = blockDim.x;
  if (n <= T) {
    // A small piece (latency-bound programs): at most one unit per thread.  The loads a big piece
    // needs in flight would only be instructions in the way here (measured: 4 % of a 64-rank ring
    // all-reduce on 512-byte pieces).
    const uint32_t i = threadIdx.x;
    SubDword<R, HAS_B> tail;
    if (odd) tail.load(a + bytes, HAS_B ? b + bytes : nullptr, odd);
    if (i < n) {
      word x = A::template ld<XL>(ra, (int)(i * W));
      if (HAS_B) x = R::combine(A::template ld<XL>(rb, (int)(i * W)), x);
      A::template st<X1>(r1, (int)(i * W), x);
      if (HAS_O2) A::template st<XS>(r2, (int)(i * W), x);
    }
    if (odd) tail.template store<HAS_O2, NT1>(o1 + bytes, HAS_O2 ? o2 + bytes : nullptr, odd);
    return;
  }
  if (n <= 2 * T) {
    // Two units per thread at most: a slice a few units over a workgroup's width (chunks that do not divide evenly).  The
    // loop below would issue its eight loads and stores per thread for them, nearly all beyond the row's end.
    const uint32_t i = threadIdx.x, j = i + T;
    SubDword<R, HAS_B> tail;
    if (odd) tail.load(a + bytes, HAS_B ? b + bytes : nullptr, odd);
    word x0 = A::template ld<XL>(ra, (int)(i * W)), x1 = A::template ld<XL>(ra, (int)(j * W));
    if (HAS_B) {
      const word y0 = A::template ld<XL>(rb, (int)(i * W)), y1 = A::template ld<XL>(rb, (int)(j * W));
      x0 = R::combine(y0, x0); x1 = R::combine(y1, x1);
    }
    A::template st<X1>(r1, (int)(i * W), x0); A::template st<X1>(r1, (int)(j * W), x1);
    if (HAS_O2) { A::template st<XS>(r2, (int)(i * W), x0); A::template st<XS>(r2, (int)(j * W), x1); }
    if (odd) tail.template store<HAS_O2, NT1>(o1 + bytes, HAS_O2 ? o2 + bytes : nullptr, odd);
    return;
  }
  // kUnroll loads are in flight per thread either way: all of a, or half of a and half of b
  constexpr int UA = HAS_B ? (kUnroll / 2 > 0 ? kUnroll / 2 : 1) : kUnroll;
  if (!HAS_O2) {
    // A destination that does not start on a 128-byte line (chunks that are no multiple of 128 bytes) costs a
    // sixth of the memory system's rate when every wave's kilobyte of stores straddles nine lines instead of
    // covering eight; where the source starts does not matter (measured with a plain streaming kernel:
    // 72 % of peak aligned, 60 % with the destination 4 to 64 bytes off, 69 % with the units laid out from
    // the destination's first line boundary).  So the row is moved in two parts: the body, whose units start
    // at that boundary, and the head in front of it -- at most 8 units, the last one cut by descriptors that
    // end where the body begins -- by the first lanes, loaded here and stored after the body.
    // (rows of 8 KiB and more: below that a move is a matter of round trips, not of the memory system's rate, and the head is one more)
    const uint32_t head = (128u - ((uint32_t)(uintptr_t)o1 & 127u)) & 127u;
    if (head != 0 && total >= 8192) {
      // (head and body each count their dwords from their own start: a row that starts on an odd 2-byte
      // boundary has a head of 4k + 2 bytes, and the body's dwords then sit on the destination's)
      const uint32_t hv = head & ~3u, hodd = head - hv, body = (total - head) & ~3u, bodd = total - head - body;
      const __amdgpu_buffer_rsrc_t hra = make_rsrc(a, hv), hr1 = make_rsrc(o1, hv), hrb = make_rsrc(HAS_B ? b : a, hv);
      const uint32_t h = threadIdx.x * W;
      word hx = A::template ld<XL>(hra, (int)(h < hv ? h : 0x7ffffff0u));
      word hy = hx;
      if (HAS_B) hy = A::template ld<XL>(hrb, (int)(h < hv ? h : 0x7ffffff0u));
      SubDword<R, HAS_B> head_tail, body_tail;
      if (hodd) head_tail.load(a + hv, HAS_B ? b + hv : nullptr, hodd);
      if (bodd) body_tail.load(a + head + body, HAS_B ? b + head + body : nullptr, bodd);
      move_units_body<R, HAS_B, NT1, UA>(o1 + head, a + head, HAS_B ? b + head : nullptr, body);
      if (HAS_B) hx = R::combine(hy, hx);
      if (h < hv) A::template st<X1>(hr1, (int)h, hx);
      if (hodd) head_tail.template store<false, NT1>(o1 + hv, nullptr, hodd);
      if (bodd) body_tail.template store<false, NT1>(o1 + head + body, nullptr, bodd);
      return;
    }
  }
  SubDword<R, HAS_B> tail;
  if (odd) tail.load(a + bytes, HAS_B ? b + bytes : nullptr, odd);
  for (uint32_t i = threadIdx.x; i < n; i += UA * T) {
    word x[UA], y[UA];
#pragma unroll
    for (int u = 0; u < UA; ++u) x[u] = A::template ld<XL>(ra, (int)((i + u * T) * W));
    if (HAS_B) {
#ifdef MSCCLX_LDS_STAGING
      // Experiment, off by default: the local operand of a reduction goes from memory straight into LDS (16 bytes per
      // lane, a wave's 1 KiB at a time) and is read from there when the payload has arrived, instead of waiting in
      // vector registers.  Measured slower everywhere (the registers are there, and LDS adds a trip): kept for the record.
      u32x4* const lds_stage = lds_stage_area();
#pragma unroll
      for (int u = 0; u < UA; ++u)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)&lds_stage[u * T + (threadIdx.x & ~63u)], 16,
                                             (int)((i + u * T) * W), 0, 0, XL);
      __builtin_amdgcn_s_waitcnt(0);
#pragma unroll
      for (int u = 0; u < UA; ++u) y[u] = i + u * T < n ? lds_stage[u * T + threadIdx.x] : word{0, 0, 0, 0};
#else
#pragma unroll
      for (int u = 0; u < UA; ++u) y[u] = A::template ld<XL>(rb, (int)((i + u * T) * W));
#endif
#pragma unroll
      for (int u = 0; u < UA; ++u) x[u] = R::combine(y[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < UA; ++u) A::template st<X1>(r1, (int)((i + u * T) * W), x[u]);
    if (HAS_O2) {
#pragma unroll
      for (int u = 0; u < UA; ++u) A::template st<XS>(r2, (int)((i + u * T) * W), x[u]);
    }
  }
  if (odd) tail.template store<HAS_O2, NT1>(o1 + bytes, HAS_O2 ? o2 + bytes : nullptr, odd);
}

// rows x n units.  Consecutive rows of an operand are `stride_*` BYTES apart: a chunk for rank
// buffers, n units for the packed rows of a FIFO slot.  b (the local reduction operand) is always a rank
// buffer, o2 (the forwarded copy) always a FIFO slot.  clip: see move_units.
template <class R, bool HAS_B, bool HAS_O2, bool NT1 = false, int RB = 4>
__device__ __forceinline__ void move_rows(unsigned char* o1, uint64_t stride_o1, unsigned char* o2, const unsigned char* a, uint64_t stride_a,
                                          const unsigned char* b, uint64_t stride_b, int rows, uint32_t n, uint32_t clip) {
  constexpr int W = 16;
  if (!HAS_B && !HAS_O2 && __builtin_expect(rows > 1 && n <= blockDim.x && ((n * W - clip) & 3u) == 0, 0)) {  // (plain copies only: the scatter and gather steps of all-pairs and all-to-all programs)
    // Several short rows (a multi-chunk step of a latency-bound program): one unit per thread and
    // row.  Four rows are loaded before the first is stored -- row by row, every row would wait
    // for its own round trip to memory.
    typedef Access<W> A;
    typedef typename A::word word;
    constexpr int XL = MSCCLX_AUX_LD, XS = MSCCLX_AUX_ST, X1 = NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST;
    const uint32_t i = threadIdx.x;  // (RB rows at a time: four, or eight where the kernel has the registers for them)
    if (i >= n) return;
    const uint32_t bytes = n * W - clip;
    for (int r0 = 0; r0 < rows; r0 += RB) {
      word x[RB], y[RB];
#pragma unroll
      for (int k = 0; k < RB; ++k)
        if (r0 + k < rows) x[k] = A::template ld<XL>(make_rsrc(a + (uint64_t)(r0 + k) * stride_a, bytes), (int)(i * W));
      if (HAS_B) {
#pragma unroll
        for (int k = 0; k < RB; ++k)
          if (r0 + k < rows) y[k] = A::template ld<XL>(make_rsrc(b + (uint64_t)(r0 + k) * stride_b, bytes), (int)(i * W));
#pragma unroll
        for (int k = 0; k < RB; ++k)
          if (r0 + k < rows) x[k] = R::combine(y[k], x[k]);
      }
#pragma unroll
      for (int k = 0; k < RB; ++k)
        if (r0 + k < rows) {
          A::template st<X1>(make_rsrc(o1 + (uint64_t)(r0 + k) * stride_o1, bytes), (int)(i * W), x[k]);
          if (HAS_O2) A::template st<XS>(make_rsrc(o2 + (uint64_t)(r0 + k) * n * W, bytes), (int)(i * W), x[k]);
        }
    }
    return;
  }
  for (int r = 0; r < rows; ++r)
    move_units<R, HAS_B, HAS_O2, NT1>(o1 + (uint64_t)r * stride_o1, HAS_O2 ? o2 + (uint64_t)r * n * W : nullptr,
                                    a + (uint64_t)r * stride_a, HAS_B ? b + (uint64_t)r * stride_b : nullptr, n, clip);
}

// dst = ((dst (+) a0) (+) a1) ... (+) a[m-1] over n units of W bytes; source k starts `stride` bytes
// after source k-1.  The sources of a unit are in flight together, eight at a time, and folded in order, so the
// result is bit for bit that of m reduce steps -- which would read and write dst m times.
template <class R, int W, bool NT1>
__device__ __forceinline__ void move_reduce_many(unsigned char* dst, const unsigned char* a, uint32_t stride, int m, uint32_t n, uint32_t clip) {
  typedef Access<W> A;
  typedef typename A::word word;
  constexpr int XL = MSCCLX_AUX_LD, X1 = NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST;
  const uint32_t bytes = n * W - clip;
  const __amdgpu_buffer_rsrc_t rd = make_rsrc(dst, bytes);
  // one descriptor for all sources (the host keeps their span below 2 GiB); source k is reached
  // through the scalar offset of the load, so that the sources cost one scalar register each
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(a, (uint32_t)(m - 1) * stride + bytes);
  for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
    word acc = A::template ld<XL>(rd, (int)(i * W));
    for (int first = 0; first < m; first += kReduceSourcesAtOnce) {  // (one round for the 7 peers of an 8-rank all-pairs program)
      word s[kReduceSourcesAtOnce];
#pragma unroll
      for (int k = 0; k < kReduceSourcesAtOnce; ++k)
        if (first + k < m) s[k] = A::template lds<XL>(rs, (int)(i * W), (int)((uint32_t)(first + k) * stride));
#pragma unroll
      for (int k = 0; k < kReduceSourcesAtOnce; ++k)
        if (first + k < m) acc = R::combine(acc, s[k]);
    }
    A::template st<X1>(rd, (int)(i * W), acc);
  }
}

// ------------------------------------------------------------------------------------------------
// the executor kernel
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ u64 load_counter(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void publish(u64* p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ u64 first_lane(u64 v) {  // the first lane's value, as a value the compiler knows to be the same in all lanes
  // (the builtin returns int: each half goes through uint32_t, or a low half with its top bit set would
  // sign-extend over the high half -- harmless for counters, fatal for addresses)
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32)), lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  return ((u64)hi << 32) | (u64)lo;
}

__device__ __forceinline__ uint32_t lane_value(uint32_t v, int l) { return (uint32_t)__builtin_amdgcn_readlane((int)v, l); }  // l: the same in all lanes
__device__ __forceinline__ u64 lane_value(u64 v, int l) { return ((u64)lane_value((uint32_t)(v >> 32), l) << 32) | (u64)lane_value((uint32_t)v, l); }

// Values that are the same in all lanes but that the compiler holds in vector registers (anything
// loaded from memory the kernel also writes): taken into scalar registers, so that addresses and
// buffer descriptors built from them are scalar too -- a descriptor in vector registers costs a
// loop of a dozen instructions around every load and store that uses it.
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t uniform(uint64_t v) { return (uint64_t)first_lane((u64)v); }
__device__ __forceinline__ DevOp uniform(const DevOp& o) {
  DevOp r;
  r.word = uniform(o.word); r.dep_tb = uniform(o.dep_tb); r.dep_step = uniform(o.dep_step); r.dep_nops = uniform(o.dep_nops);
  r.extra = uniform(o.extra); r.steps = uniform(o.steps);
  r.src_addr = uniform(o.src_addr); r.dst_addr = uniform(o.dst_addr); r.in_addr = uniform(o.in_addr);
  return r;
}

__device__ __forceinline__ bool is_recv(int t) { return t == MSCCLX_OP_RECV || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRCS; }
__device__ __forceinline__ bool is_send(int t) { return t == MSCCLX_OP_SEND || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRCS; }

// Between two polls of the same address.  It is more than a courtesy to the memory system: the
// compiler treats a buffer load as a function of its arguments and takes a re-load with unchanged
// arguments out of a loop that has nothing with a side effect in it -- the loop would then spin on
// a register.  The pause is such a side effect.
#define MSCCLX_POLL_PAUSE() __builtin_amdgcn_s_sleep(1)

// ------------------------------------------------------------------------------------------------
// LL lines.  One unit (16 payload bytes d0..d3) occupies 32 bytes of a slot: {d0,f,d1,f}{d2,f,d3,f}.
// f = launch number (10 bits) | message number + 1 (22 bits): never 0, so a cleared slot matches
// nothing, and what an earlier message or launch left in a line cannot be taken for this message.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t ll_flag(uint32_t epoch, u64 seq) { return ((epoch & 0x3ffu) << 22) | (uint32_t)((seq + 1) & 0x3fffffu); }
__device__ __forceinline__ bool ll_valid(u32x4 l0, u32x4 l1, uint32_t f) { return l0.y == f && l0.w == f && l1.y == f && l1.w == f; }
// The same question in integers, nonzero while a flag is missing (no `&&` whose early exits a lane would have to branch around).
__device__ __forceinline__ uint32_t ll_stale(u32x4 l0, u32x4 l1, uint32_t f) { return (l0.y ^ f) | (l0.w ^ f) | (l1.y ^ f) | (l1.w ^ f); }

// The area's abort word is raised.  If it was the host that raised it (mscclx_plan_abort), whoever sees it says so in the
// launch's status: a launch replayed from a HIP graph passes by the host code that would have re-armed the counters, and
// the caller must still learn from the wait that follows that this launch did not run.  (Out of line: the rare path.)
__device__ __forceinline__ void note_abort_here(const u64* abort_word, mscclx_status* hs) {
  if (load_counter(abort_word) == kAbortByHost && __hip_atomic_load(&hs->code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == (int)MSCCLX_OK)
    __hip_atomic_store(&hs->code, (int)MSCCLX_ERR_ABORTED, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
// (out of line for the chain loops, which call their slow checks anyway; in line for the hosting loop, which calls nothing:
// a single call would cost that whole kernel the registers a callee may clobber)
__device__ __noinline__ void note_abort(const u64* abort_word, mscclx_status* hs) { note_abort_here(abort_word, hs); }

// What a thread needs to give up on a message that never arrives.
struct LLWatch {
  u64* abort_word;
  mscclx_status* host_status;
  u64 timeout_ticks;
  int tb, step, slice;
  u64 pass;
};

// (arguments by value: a struct handed to a function that is not inlined would have to live in memory)
__device__ __noinline__ void ll_give_up(u64* abort_word, mscclx_status* hs, int tb, int step, int slice, u64 pass, int waiting_on = 1) {
  if (atomicCAS(abort_word, 0ull, kAbortByWatchdog) == 0ull) {
    hs->tb = tb; hs->step = step; hs->slice = slice; hs->pass = (int64_t)pass; hs->waiting_on = waiting_on;
    __threadfence_system();
    __hip_atomic_store(&hs->code, (int)MSCCLX_ERR_TIMEOUT, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// o1 (rank buffer) [and llo (LL slot)] = a [(+) b] over n units of 16 bytes.  a is an LL slot row when
// IN_LL (its lines are retried until they carry `fin`), a rank buffer otherwise; b is a rank buffer.
template <class R, bool IN_LL, bool HAS_B, bool HAS_O1, bool OUT_LL, bool NT1>
__device__ __forceinline__ void move_units_ll(unsigned char* o1, unsigned char* llo, const unsigned char* a, const unsigned char* b, uint32_t n,
                                              uint32_t clip, uint32_t fin, uint32_t fout, const LLWatch& watch) {
  typedef Access<16> A;
  // XV: the retried loads must really be issued again each time round the loop (bit 31 = volatile, for the compiler only)
  constexpr int XL = MSCCLX_AUX_LD, XF = MSCCLX_AUX, XV = (int)(0x80000000u | MSCCLX_AUX), X1 = NT1 ? MSCCLX_AUX_ST_FINAL : MSCCLX_AUX_ST;
  // (rank buffers end `clip` bytes inside their last unit; lines are always whole: their flags must arrive)
  const uint32_t local_bytes = n * 16 - clip;
  // (a row of lines: the first halves of its n units, then the second halves -- see kLLUnitBytes; one descriptor per half,
  // so that lanes past the row's end load zeros and store nothing in either)
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(a, IN_LL ? n * 16 : local_bytes);
  const __amdgpu_buffer_rsrc_t ra2 = make_rsrc(a + (IN_LL ? n * 16 : 0), IN_LL ? n * 16 : 0);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(HAS_B ? b : a, HAS_B ? local_bytes : (IN_LL ? n * 16 : local_bytes));
  const __amdgpu_buffer_rsrc_t r1 = make_rsrc(HAS_O1 ? o1 : const_cast<unsigned char*>(a), HAS_O1 ? local_bytes : 0);
  const __amdgpu_buffer_rsrc_t rl = make_rsrc(OUT_LL ? llo : const_cast<unsigned char*>(a), OUT_LL ? n * 16 : 0);
  const __amdgpu_buffer_rsrc_t rl2 = make_rsrc(OUT_LL ? llo + n * 16 : const_cast<unsigned char*>(a), OUT_LL ? n * 16 : 0);
  const uint32_t T = blockDim.x;
  constexpr int UA = 2;  // small pieces: few lines per thread, few registers
  for (uint32_t i = threadIdx.x; i < n; i += UA * T) {
    u32x4 x[UA], y[UA];
    if (IN_LL) {
      static_assert(UA == 2, "the retry below names its two units");
      const uint32_t ia = i, ib = i + T;
      u32x4 a0 = A::template ld<XV>(ra, (int)(ia * 16)), a1 = A::template ld<XV>(ra2, (int)(ia * 16));
      u32x4 b0 = A::template ld<XV>(ra, (int)(ib * 16)), b1 = A::template ld<XV>(ra2, (int)(ib * 16));
      if (HAS_B) {
#pragma unroll
        for (int u = 0; u < UA; ++u) y[u] = A::template ld<XL>(rb, (int)((i + u * T) * 16));
      }
      unsigned spins = 0;
      u64 since = 0;
      for (;;) {
        const bool ok_a = ll_valid(a0, a1, fin), ok_b = ib >= n || ll_valid(b0, b1, fin);
        if (ok_a && ok_b) break;
        MSCCLX_POLL_PAUSE();
        if (!ok_a) { a0 = A::template ld<XV>(ra, (int)(ia * 16)); a1 = A::template ld<XV>(ra2, (int)(ia * 16)); }
        if (!ok_b) { b0 = A::template ld<XV>(ra, (int)(ib * 16)); b1 = A::template ld<XV>(ra2, (int)(ib * 16)); }
        if ((++spins & 0x7fu) == 0) {
          const u64 now = wall_clock64();
          if (!since) since = now;
          const bool expired = now - since > watch.timeout_ticks;
          if (expired) ll_give_up(watch.abort_word, watch.host_status, watch.tb, watch.step, watch.slice, watch.pass);
          if (expired || load_counter(watch.abort_word) != 0) break;  // the launch is lost; leave with what is there
        }
      }
      x[0] = u32x4{a0.x, a0.z, a1.x, a1.z};
      x[1] = u32x4{b0.x, b0.z, b1.x, b1.z};
    } else {
#pragma unroll
      for (int u = 0; u < UA; ++u) x[u] = A::template ld<XL>(ra, (int)((i + u * T) * 16));
      if (HAS_B) {
#pragma unroll
        for (int u = 0; u < UA; ++u) y[u] = A::template ld<XL>(rb, (int)((i + u * T) * 16));
      }
    }
    if (HAS_B) {
#pragma unroll
      for (int u = 0; u < UA; ++u) x[u] = R::combine(y[u], x[u]);
    }
    if (OUT_LL) {  // the forwarded lines first: the next rank is waiting for them
#pragma unroll
      for (int u = 0; u < UA; ++u) {
        A::template st<XF>(rl, (int)((i + u * T) * 16), u32x4{x[u].x, fout, x[u].y, fout});
        A::template st<XF>(rl2, (int)((i + u * T) * 16), u32x4{x[u].z, fout, x[u].w, fout});
      }
    }
    if (HAS_O1) {
#pragma unroll
      for (int u = 0; u < UA; ++u) A::template st<X1>(r1, (int)((i + u * T) * 16), x[u]);
    }
  }
}

// rows x n units; rank-buffer rows are `stride_*` bytes apart, slot rows are packed.
template <class R, bool IN_LL, bool HAS_B, bool HAS_O1, bool OUT_LL, bool NT1 = false>
__device__ __forceinline__ void move_rows_ll(unsigned char* o1, uint64_t stride_o1, unsigned char* llo, const unsigned char* a, uint64_t stride_a,
                                             const unsigned char* b, uint64_t stride_b, int rows, uint32_t n, uint32_t clip, uint32_t fin, uint32_t fout,
                                             const LLWatch& watch) {
  for (int r = 0; r < rows; ++r)
    move_units_ll<R, IN_LL, HAS_B, HAS_O1, OUT_LL, NT1>(HAS_O1 ? o1 + (uint64_t)r * stride_o1 : nullptr,
                                                       OUT_LL ? llo + (uint64_t)r * n * kLLUnitBytes : nullptr,
                                                       a + (uint64_t)r * (IN_LL ? (uint64_t)n * kLLUnitBytes : stride_a),
                                                       HAS_B ? b + (uint64_t)r * stride_b : nullptr, n, clip, fin, fout, watch);
}

// What the workgroup does for one step of one context: operands as byte addresses, filled in by the
// context's lane when the context arrives at the step and handed to the other threads through LDS.
struct Move {
  u64 a;      // source: the incoming payload (slot, or the sender's buffer) or the local source
  u64 dst;    // local destination, which is also the local operand of a reduction
  u64 out;    // slot to fill
  uint32_t n; // units per row
  int rows, kind;
};
// kind: how the operands are used.  Rows of a rank buffer are a chunk apart, rows in a slot are packed.
enum {
  kHasB = 1,     // reduce: a (+) dst
  kHasO2 = 2,    // also forward the result into `out`
  kNt1 = 4,      // the first destination is never read again
  kLLKind = 8,   // flag-in-data lines: bits 0-2 then say which movement (kLL* below)
  kAPacked = 16, // a is a slot
  kToSlot = 32,  // the first (only) destination is `out` instead of dst
  kMany = 64,    // dst = ((dst (+) a[0]) (+) a[1]) ...: `rows` sources, `out` bytes apart
  kClipShift = 8, kClipMask = 15 << 8,  // bits 8-11: bytes that the last unit of a rank-buffer row lacks (see move_units)
};
enum { kLLSend = 0, kLLRecv, kLLRecvNt, kLLRcs, kLLRrc, kLLRrs, kLLRrcs };

// The changing part.  Everything that depends on the pass or on how many messages went by is kept
// as a running value, advanced when a step finishes: the lane's instructions between two moves are
// on the critical path of a latency-bound program, and multiplications and divisions dominate them.
struct Context {
  int step;
  unsigned pass;
  bool active;
  uint32_t count;           // steps finished so far in this launch (all passes)
  uint32_t sseq, rseq;      // messages sent / received so far = number of the next message on its connection
  uint32_t sslot, rslot;    // byte offset of that message's slot inside the connection's ring
  uint32_t left;            // units of the slice not yet covered before this pass
  u64 off;                  // byte offset of this pass's piece inside any chunk
  // the step the context stands at
  bool moves;  // false: nop or a send whose payload is read in place -- nothing to copy
  int type, hasdep;         // hasdep: bit 0 = others wait for this step; bits 8.. = IR steps this step stands for (itself and folded nops)
  uint32_t extra;           // folded dependencies: first entry << 8 | how many
  const u64 *w0, *w1, *w2;  // counters to wait for (null = none) ...
  uint32_t t0, t1, t2;      // ... until they reach these values (every counter of a launch stays below 2^32)
  Move m;
};

// The dependencies of the nop steps folded into the step `c` stands at: all their counters are
// loaded in one round, after one round for the table entries.
__device__ __forceinline__ bool extras_ready(const Context& c, const Hosted& h, const KernelParams& p) {
  const uint32_t n = c.extra & 255u;
  const uint2* const e = (const uint2*)p.extra_deps + (c.extra >> 8);
  const u64* const flags = p.sync_cur + h.flags;
  uint2 entry[kLaneExtraDeps];
#pragma unroll
  for (int k = 0; k < kLaneExtraDeps; ++k)
    if ((uint32_t)k < n) entry[k] = e[k];
  u64 v[kLaneExtraDeps];
#pragma unroll
  for (int k = 0; k < kLaneExtraDeps; ++k)
    if ((uint32_t)k < n) v[k] = load_counter(flags + entry[k].x);
  bool ok = true;
#pragma unroll
  for (int k = 0; k < kLaneExtraDeps; ++k)
    if ((uint32_t)k < n) ok = ok && v[k] >= (u64)(c.pass * (entry[k].y >> 16) + (entry[k].y & 0xffffu));
  return ok;
}

// The same for a context with more folded dependencies than that (up to kMaxExtraDeps = the wave's width): the whole
// polling wave checks them, a dependency per lane -- still two rounds of loads.  Called by all 64 lanes; `owner` is the
// lane whose context it is, and every lane gets the answer.
__device__ __forceinline__ bool extras_ready_together(const Context& c, const Hosted& h, const KernelParams& p, int owner, int lane) {
  const uint32_t extra = (uint32_t)__shfl((int)c.extra, owner), first_flag = (uint32_t)__shfl((int)h.flags, owner);
  const unsigned pass = (unsigned)__shfl((int)c.pass, owner);
  bool ok = true;
  if ((uint32_t)lane < (extra & 255u)) {
    const uint2 entry = ((const uint2*)p.extra_deps)[(extra >> 8) + (uint32_t)lane];
    ok = load_counter(p.sync_cur + first_flag + entry.x) >= (u64)(pass * (entry.y >> 16) + (entry.y & 0xffffu));
  }
  return __ballot(!ok) == 0;
}

// FOLD kernels: an `re` with several sources (in_addr = their distance in bytes, cnt = how many).
__device__ __forceinline__ void mark_many_sources(Context& c, const DevOp& op) {
  if ((op.word & 15u) == MSCCLX_OP_REDUCE && op.in_addr) {
    c.m.out = op.in_addr;
    c.m.kind = kMany | ((op.word & kOpNtStore) ? (int)kNt1 : 0) | (c.m.kind & kClipMask);
  }
}

// Describe the step `c` stands at: what it must wait for, whether it moves data, and from where to
// where.  LL: an incoming message is not announced by a counter; the lane watches the flag in the
// last 8 bytes of the message instead (w1 = that word, t1 = the flag).  Lines may land in any order,
// so this is a hint that the message is about to be complete; the threads that read it check every line.
template <bool LL, bool RAGGED>
__device__ __forceinline__ void describe_step(Context& c, const Hosted& h, const KernelParams& p, uint32_t epoch, const DevOp& op) {
  const int t = (int)(op.word & 15u);
  const int cnt = (int)(op.word >> kOpCntShift);
  const bool out_staged = op.word & kOpOutStaged, in_place = op.word & kOpInPlace;
  c.type = t;
  c.hasdep = ((op.word & kOpHasdep) ? 1 : 0) | (int)(op.steps << 8);
  c.extra = op.extra;
  const bool rcv = is_recv(t), snd = is_send(t);
  c.w0 = c.w1 = c.w2 = nullptr;
  c.t0 = c.t1 = c.t2 = 0;
  if (op.dep_tb >= 0) { c.w0 = p.sync_cur + (h.flags + (uint32_t)op.dep_tb * kSyncStrideWords); c.t0 = c.pass * (uint32_t)op.dep_nops + (uint32_t)op.dep_step + 1; }
  if (snd && c.sseq >= (uint32_t)p.depth) { c.w2 = p.sync_cur + h.tail_in; c.t2 = c.sseq + 1 - (uint32_t)p.depth; }
  c.moves = !(t == MSCCLX_OP_NOP || (t == MSCCLX_OP_SEND && !out_staged));

  const uint32_t n = c.left < p.piece_units ? c.left : p.piece_units;
  // out: the slot to fill, or 0 when the receiver will read this step's payload in place
  const u64 out = (snd && out_staged) ? (u64)p.fifo + (u64)h.out_slots * 16 + c.sslot : 0;
  // in: the incoming payload -- packed in a slot, or still where the sender has it (then its rows are
  // a chunk apart, like any rank buffer)
  u64 in = 0;
  int in_packed = kAPacked;
  if (rcv) {
    if (in_place) { in = op.in_addr + c.off; in_packed = 0; }
    else in = (u64)p.fifo + (u64)h.in_slots * 16 + c.rslot;
    if (LL) {
      c.w1 = (const u64*)(in + (uint64_t)((uint32_t)cnt * n) * kLLUnitBytes - 8);  // the last word and flag of the last row's last unit
      c.t1 = ll_flag(epoch, c.rseq);
    } else if (!(in_place && (op.steps & kStepsNoAnnouncement))) {
      c.w1 = p.sync_cur + h.head_in;
      c.t1 = c.rseq + 1;
    }
  }
  Move& m = c.m;
  m.n = n; m.rows = cnt;
  m.a = in; m.dst = op.dst_addr + c.off; m.out = out;
  const int nt = (op.word & kOpNtStore) ? kNt1 : 0;
  int kind = 0;
  switch (t) {
    case MSCCLX_OP_SEND: m.a = op.src_addr + c.off; kind = LL ? kLLKind | kLLSend : (int)kToSlot; break;
    case MSCCLX_OP_RECV: kind = LL ? kLLKind | (nt ? kLLRecvNt : kLLRecv) : in_packed | nt; break;
    case MSCCLX_OP_RCS: kind = LL ? kLLKind | kLLRcs : in_packed | (out ? (int)kHasO2 : 0); break;
    case MSCCLX_OP_RRC: kind = LL ? kLLKind | kLLRrc : in_packed | kHasB; break;
    case MSCCLX_OP_RRS: kind = LL ? kLLKind | kLLRrs : in_packed | kHasB | kToSlot; break;
    case MSCCLX_OP_RRCS: kind = LL ? kLLKind | kLLRrcs : in_packed | kHasB | (out ? (int)kHasO2 : 0); break;
    case MSCCLX_OP_COPY: m.a = op.src_addr + c.off; kind = nt; break;
    case MSCCLX_OP_REDUCE: m.a = op.src_addr + c.off; kind = kHasB; break;
    default: break;
  }
  m.kind = kind;
  // RAGGED (chunks that are no multiple of 16 bytes): in the pass that reaches the end of the slice, rows may end inside their last unit
  if constexpr (RAGGED) m.kind = kind | (c.left <= p.piece_units ? (int)h.clip << kClipShift : 0);
}

// The description of the step after the one `c` stands at.  It is fetched before the counters of
// the finished step are stored: a load issued after those stores would come back only after they
// are acknowledged, and the context could not look for its next message any earlier.
__device__ __forceinline__ DevOp fetch_next_op(const Context& c, const Hosted& h, const KernelParams& p) {
  const int next = c.step + 1 == h.nops ? 0 : c.step + 1;
  return p.ops[h.op_begin + next];
}

// Announce the completed step and move the context to its next one, described by `next`.
// `writer`: this thread stores the counters (the context's lane; one thread of a wave that runs a
// context with all its lanes).
template <bool LL, bool RAGGED>
__device__ __forceinline__ void finish_step(Context& c, const Hosted& entry, const KernelParams& p, uint32_t epoch, const DevOp& next, bool writer = true) {
  const Hosted h = entry;  // one batch of LDS reads, one wait -- not one wait per field as they are needed
  if (is_send(c.type)) {
    if (!LL && writer) publish(p.sync_cur + h.head_out, (u64)c.sseq + 1);  // LL: the lines announce themselves
    ++c.sseq;
    c.sslot += h.out_slot_bytes;
    if (c.sslot == h.out_wrap) c.sslot = 0;
  }
  if (is_recv(c.type)) {
    if (writer) publish(p.sync_cur + h.tail_out, (u64)c.rseq + 1);
    ++c.rseq;
    c.rslot += h.in_slot_bytes;
    if (c.rslot == h.in_wrap) c.rslot = 0;
  }
  c.count += (uint32_t)c.hasdep >> 8;
  if ((c.hasdep & 1) && writer) publish(p.sync_cur + h.my_flag, (u64)c.count);  // = pass * steps of the IR + IR step + 1
  if (++c.step == h.nops) {
    c.step = 0;
    ++c.pass;
    c.left -= c.left < p.piece_units ? c.left : p.piece_units;
    c.off += (u64)p.piece_units * 16;
  }
  if (c.pass >= h.npasses) c.active = false;
  else describe_step<LL, RAGGED>(c, h, p, epoch, next);
}

// Set up hosted context number `ctx`: its constants in `h` (the record worked out when the buffers were
// bound), its state in `c`, standing at its first step.  `writer` also clears, for the next launch,
// the counters this context alone writes.
template <bool LL, bool RAGGED>
__device__ __forceinline__ void init_context(Hosted& h, Context& c, const KernelParams& p, uint32_t epoch, int ctx, bool writer, const DevCtx* given = nullptr) {
  const DevCtx rec = given ? *given : p.ctxs[ctx];  // (given: a record that the caller asked for earlier)
  h = rec.h;
  c.step = 0; c.pass = 0; c.count = 0; c.sseq = c.rseq = 0; c.sslot = c.rslot = 0;
  c.left = rec.left;
  c.off = rec.off;
  c.active = h.nops > 0 && h.npasses > 0;
  if (writer) {  // (word 0 of an area is the abort word: no head or tail has index 0, which therefore says "no such connection")
    p.sync_nxt[h.my_flag] = 0;
    if (h.head_out) p.sync_nxt[h.head_out] = 0;
    if (h.tail_out) p.sync_nxt[h.tail_out] = 0;
  }
  if (c.active) describe_step<LL, RAGGED>(c, h, p, epoch, p.ops[h.op_begin]);
}

// The whole workgroup (or wave) copies / reduces one piece as `m` says.  rseq, sseq: numbers of the
// incoming / outgoing message (LL flags); tb, step, slice, pass: for the LL watchdog's report.
template <class R, bool LL, int FOLD, bool RAGGED, int ROWS_AT_ONCE = 4>
__device__ __forceinline__ void do_move(const Move& m, const KernelParams& p, uint32_t epoch, uint32_t rseq, uint32_t sseq,
                                        int tb, int step, int slice, unsigned pass) {
  constexpr int W = 16;
  const u64 cs = p.chunk_bytes;                   // rows of a rank buffer are a chunk apart ...
  const u64 packed = (u64)m.n * W;                // ... rows in a slot are packed
  const uint32_t clip = RAGGED ? ((uint32_t)m.kind & kClipMask) >> kClipShift : 0u;  // (a constant 0 folds every cut and tail below away)
  unsigned char* const dst = (unsigned char*)m.dst;
  unsigned char* const out = (unsigned char*)m.out;
  const unsigned char* const a = (const unsigned char*)m.a;
  if (FOLD && __builtin_expect((m.kind & kMany) != 0, 0)) {  // (only the bind of a FOLD kernel makes such steps)
    // (whole dwords in 16-byte units; what is left of a row that is no whole number of dwords, element by element)
    const uint32_t total = m.n * W - clip, odd = total & 3u;
    if (m.kind & kNt1) move_reduce_many<R, W, true>(dst, a, (uint32_t)m.out, m.rows, m.n, clip + odd);
    else move_reduce_many<R, W, false>(dst, a, (uint32_t)m.out, m.rows, m.n, clip + odd);
    if (odd) {
      constexpr int E = R::kElemBytes;
      if (m.kind & kNt1) move_reduce_many<R, E, true>(dst + (total - odd), a + (total - odd), (uint32_t)m.out, m.rows, odd / E, 0);
      else move_reduce_many<R, E, false>(dst + (total - odd), a + (total - odd), (uint32_t)m.out, m.rows, odd / E, 0);
    }
    return;
  }
  if (LL && (m.kind & kLLKind)) {
    const uint32_t fin = ll_flag(epoch, rseq), fout = ll_flag(epoch, sseq);
    const LLWatch watch{p.sync_cur, p.host_status, p.timeout_ticks, tb, step, slice, (u64)pass};
    switch (m.kind & 7) {
      case kLLSend: move_rows_ll<R, false, false, false, true>(nullptr, 0, out, a, cs, nullptr, 0, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRecv: move_rows_ll<R, true, false, true, false>(dst, cs, nullptr, a, 0, nullptr, 0, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRecvNt: move_rows_ll<R, true, false, true, false, true>(dst, cs, nullptr, a, 0, nullptr, 0, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRcs: move_rows_ll<R, true, false, true, true>(dst, cs, out, a, 0, nullptr, 0, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRrc: move_rows_ll<R, true, true, true, false>(dst, cs, nullptr, a, 0, dst, cs, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRrs: move_rows_ll<R, true, true, false, true>(nullptr, 0, out, a, 0, dst, cs, m.rows, m.n, clip, fin, fout, watch); break;
      case kLLRrcs: move_rows_ll<R, true, true, true, true>(dst, cs, out, a, 0, dst, cs, m.rows, m.n, clip, fin, fout, watch); break;
      default: break;
    }
  } else {
    const u64 stride_a = (m.kind & kAPacked) ? packed : cs;
    unsigned char* const o1 = (m.kind & kToSlot) ? out : dst;
    const u64 stride_o1 = (m.kind & kToSlot) ? packed : cs;
    switch (m.kind & 7) {
      case 0: move_rows<R, false, false, false, ROWS_AT_ONCE>(o1, stride_o1, nullptr, a, stride_a, nullptr, 0, m.rows, m.n, clip); break;
      case kNt1: move_rows<R, false, false, true, ROWS_AT_ONCE>(o1, stride_o1, nullptr, a, stride_a, nullptr, 0, m.rows, m.n, clip); break;
      case kHasO2: move_rows<R, false, true>(o1, stride_o1, out, a, stride_a, nullptr, 0, m.rows, m.n, clip); break;
      case kHasB: move_rows<R, true, false>(o1, stride_o1, nullptr, a, stride_a, dst, cs, m.rows, m.n, clip); break;
      case kHasB | kHasO2: move_rows<R, true, true>(o1, stride_o1, out, a, stride_a, dst, cs, m.rows, m.n, clip); break;
      default: break;
    }
  }
}

// What a wait of run_chain does once in 64 polls: look at the abort word and at the clock.  Returns
// the time the wait began (to be handed in again), or ~0 when the wait must be abandoned -- the
// launch is lost, by this wait's own expiry (which it reports) or by somebody else's.
__device__ __noinline__ u64 chain_slow_check(u64* abort_word, mscclx_status* hs, u64 timeout_ticks, u64 since, int tb, int step, int slice, u64 pass, int waiting_on) {
  if (load_counter(abort_word) != 0) {
    note_abort(abort_word, hs);
    return ~0ull;
  }
  const u64 now = wall_clock64();
  if (!since) return now;
  if (now - since > timeout_ticks) {
    ll_give_up(abort_word, hs, tb, step, slice, pass, waiting_on);
    return ~0ull;
  }
  return since;
}

// LL, one context on a workgroup of one wave: the wave runs the context with all its lanes.  This is
// the shape of latency-bound programs (small pieces, as many workgroups as contexts), where a launch
// takes as long as the instructions and round trips of the longest chain of steps: a ring of one-wave
// workgroups that does nothing but poll lines, add and store lines makes a round in 0.7 to 1.1 us
// on MI355X (512 workgroups, 512-byte messages), and every instruction added to the loop shows.  So
// this loop is written for that case and nothing else: every value of the bookkeeping is the same
// in all lanes and is kept in scalar registers (`uniform`), so that addresses and buffer descriptors
// are scalar; a step's state is a handful of running numbers; the table entry of the step after is
// asked for before the wait for this step's message; the local operand and the outgoing
// connection's tail are loaded together with the message's lines and looked at when the lines are
// there; stores are waited for only where a flag announces them (lines announce themselves, and the
// counter that frees the incoming slot only says that its lines were read).
#ifdef MSCCLX_PROFILE
#define MSCCLX_CHAIN_CLOCK(var) const u64 var = __builtin_amdgcn_s_memtime()
#define MSCCLX_CHAIN_ADD(k, a, b) (prof_acc[k] += (b) - (a))
#else
#define MSCCLX_CHAIN_CLOCK(var)
#define MSCCLX_CHAIN_ADD(k, a, b)
#endif
// What run_chain's waits need in order to give up, kept together so that a wait passes one reference.
struct ChainWatch {
  u64* abort_word;
  mscclx_status* host_status;
  u64 timeout_ticks;
  int tb, slice;
};

// A step's table entry asked for ahead of time.  Scalar loads would bring it straight to scalar registers, but
// they complete out of order, so the first wait for any scalar value -- a spilled register is enough -- waits
// for the entry as well, and an entry is used once per pass: most of these loads miss the scalar cache.  Asked
// for with vector loads (every lane the same address), the entry arrives behind the loads issued before it and
// ahead of the lines that the wave polls for; twelve moves then carry it to scalar registers.
struct StepAhead {
  u32x4 a, b, c;  // a: word dep_tb dep_step dep_nops, b: extra steps src_addr, c: dst_addr in_addr
};
static_assert(offsetof(DevOp, extra) == 16 && offsetof(DevOp, dst_addr) == 32, "StepAhead names DevOp's fields by their place");
__device__ __forceinline__ StepAhead ask_step(const __amdgpu_buffer_rsrc_t table, uint32_t index) {
  StepAhead r;
  const int at = (int)(index * (uint32_t)sizeof(DevOp));
  r.a = Access<16>::template lds<0>(table, 0, at);
  r.b = Access<16>::template lds<0>(table, 16, at);
  r.c = Access<16>::template lds<0>(table, 32, at);
  return r;
}
__device__ __forceinline__ DevOp take_step(const StepAhead& e) {
  DevOp r;
  r.word = uniform(e.a.x); r.dep_tb = (int32_t)uniform(e.a.y); r.dep_step = (int32_t)uniform(e.a.z); r.dep_nops = (int32_t)uniform(e.a.w);
  r.extra = uniform(e.b.x); r.steps = uniform(e.b.y);
  r.src_addr = (u64)uniform(e.b.z) | (u64)uniform(e.b.w) << 32;
  r.dst_addr = (u64)uniform(e.c.x) | (u64)uniform(e.c.y) << 32;
  r.in_addr = (u64)uniform(e.c.z) | (u64)uniform(e.c.w) << 32;
  return r;
}

__device__ __forceinline__ FlatOp take_flat_step(const StepAhead& e) {
  FlatOp r;
  r.word = uniform(e.a.x); r.in_off = uniform(e.a.y); r.out_off = uniform(e.a.z); r.fin = uniform(e.a.w);
  r.fout = uniform(e.b.x); r.gate = uniform(e.b.y);
  r.src_addr = (u64)uniform(e.b.z) | (u64)uniform(e.b.w) << 32;
  r.dst_addr = (u64)uniform(e.c.x) | (u64)uniform(e.c.y) << 32;
  r.tail = (u64)uniform(e.c.z);  // (message numbers stay below 2^22)
  return r;
}

// One round of a step of run_chain: units i0, i0 + 64, ... (U of them per lane) of one row of n units.
// Returns false when the launch is lost (the same answer in all lanes).  gate: the counter that must
// reach gate_target before the outgoing slot may be written, or null.  The polling is uniform: all
// lanes ask again until every lane has its lines (a line that is there stays until this context frees
// the slot) -- no per-lane masks to keep, a fifth less time per hop than lane-by-lane retries.
template <class R, int U, int T>
__device__ __forceinline__ bool chain_round(const __amdgpu_buffer_rsrc_t rin, const __amdgpu_buffer_rsrc_t rin2, const __amdgpu_buffer_rsrc_t rout,
                                            const __amdgpu_buffer_rsrc_t rout2, const __amdgpu_buffer_rsrc_t rsrc, const __amdgpu_buffer_rsrc_t rdst, const uint32_t i0, const uint32_t n, const bool nt, const uint32_t fin,
                                            const uint32_t fout, const u64* gate, const u64 gate_target, const ChainWatch& watch, const int step,
                                            const uint32_t pass, const __amdgpu_buffer_rsrc_t table, const uint32_t ask_index, StepAhead& asked, u64* prof_acc,
                                            u64& prof_mark, const u64 prof_floor) {
  // what a step of type T does, known where the code is generated: one straight run of instructions per type
  constexpr bool rcv = ((0x7cu >> T) & 1u) != 0, snd = ((0x5au >> T) & 1u) != 0;
  constexpr bool from_src = T == MSCCLX_OP_SEND || T == MSCCLX_OP_COPY || T == MSCCLX_OP_REDUCE;
  constexpr bool has_b = T == MSCCLX_OP_RRC || T == MSCCLX_OP_RRS || T == MSCCLX_OP_RRCS || T == MSCCLX_OP_REDUCE;
  constexpr bool to_local = T == MSCCLX_OP_RECV || T == MSCCLX_OP_RCS || T == MSCCLX_OP_RRC || T == MSCCLX_OP_RRCS || T == MSCCLX_OP_COPY || T == MSCCLX_OP_REDUCE;
  typedef Access<16> A;
  constexpr int XL = MSCCLX_AUX_LD, XP = (int)(0x80000000u | MSCCLX_AUX), XF = MSCCLX_AUX, XS = MSCCLX_AUX_ST, XN = MSCCLX_AUX_ST_FINAL;
  u32x4 lo[U], hi[U], x[U], y[U];
  MSCCLX_CHAIN_CLOCK(prof_ld);
#ifdef MSCCLX_PROFILE
  prof_acc[3] += prof_ld - (prof_mark > prof_floor ? prof_mark : prof_floor);
#endif
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t i = i0 + 64u * (uint32_t)u;
    lo[u] = hi[u] = x[u] = y[u] = u32x4{0, 0, 0, 0};
    if constexpr (rcv) {
      lo[u] = A::template ld<XP>(rin, (int)(i * 16));
      hi[u] = A::template ld<XP>(rin2, (int)(i * 16));
    } else if constexpr (from_src) {
      x[u] = A::template ld<XL>(rsrc, (int)(i * 16));
    }
  }
  if constexpr (has_b) {
#pragma unroll
    for (int u = 0; u < U; ++u) y[u] = A::template ld<XL>(rdst, (int)((i0 + 64u * (uint32_t)u) * 16));
  }
  u64 gate_seen = snd && gate ? load_counter(gate) : ~0ull;
  // run_chain_flat asks for the table entry of the step after next here, behind the step's own loads: answers come back in
  // the order of the requests, so the wait for the lines leaves this request outstanding, and it has a whole step to arrive.
  // (That loop measured 188 us on the 64-rank ring with the request at its top, one step ahead, and 147 with it here; the
  // general loop 178 at its top and 206 here.  Each keeps what it measured best with.)
  if (ask_index != ~0u) asked = ask_step(table, ask_index);
  bool lost = false;
  if constexpr (rcv) {
    auto all_there = [&]() {
      uint32_t missing = 0;
#pragma unroll
      for (int u = 0; u < U; ++u) missing |= i0 + 64u * (uint32_t)u < n ? ll_stale(lo[u], hi[u], fin) : 0u;
      return __builtin_amdgcn_ballot_w64(missing != 0) == 0;
    };
    unsigned spins = 0;
    u64 since = 0;
    while (!all_there()) {
      MSCCLX_POLL_PAUSE();
      if (spins >= 2) {
        // A long wait (the start of a pipeline, a rank far down a chain): asking for every line again
        // and again costs memory traffic that the ranks at work pay for -- 4096 waiting waves ask for
        // 16 MiB a round.  Watch the round's last line alone until it is there, then ask for all.
        const uint32_t round_end = i0 - threadIdx.x + 64u * (uint32_t)U;
        const int watched = (int)(((round_end < n ? round_end : n) - 1u) * 16u);  // (its second half)
        for (;;) {
          const u32x4 w = A::template ld<XP>(rin2, watched);
          if (uniform(w.y) == fin && uniform(w.w) == fin) break;
          MSCCLX_POLL_PAUSE();
          if ((++spins & 0x3fu) == 0) {
            since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, step, watch.slice, (u64)pass, 1));
            if (since == ~0ull) { lost = true; break; }
          }
        }
        if (lost) break;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t i = i0 + 64u * (uint32_t)u;
        lo[u] = A::template ld<XP>(rin, (int)(i * 16));
        hi[u] = A::template ld<XP>(rin2, (int)(i * 16));
      }
      if ((++spins & 0x3fu) == 0) {
        since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, step, watch.slice, (u64)pass, 1));
        if (since == ~0ull) { lost = true; break; }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = u32x4{lo[u].x, lo[u].z, hi[u].x, hi[u].z};
  }
  MSCCLX_CHAIN_CLOCK(prof_got);
  MSCCLX_CHAIN_ADD(1, prof_ld, prof_got);
  if constexpr (has_b) {
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = R::combine(y[u], x[u]);
  }
  if (snd && gate) {  // the slot may still be being read
    unsigned spins = 0;
    u64 since = 0;
    while (uniform((uint64_t)gate_seen) < gate_target && !lost) {
      MSCCLX_POLL_PAUSE();
      gate_seen = load_counter(gate);
      if ((++spins & 0x3fu) == 0) {
        since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, step, watch.slice, (u64)pass, 2));
        if (since == ~0ull) lost = true;
      }
    }
  }
  if (lost) return false;  // (the same in all lanes: every wait above is uniform)
  if constexpr (snd) {  // the forwarded lines first: the next rank is waiting for them
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + 64u * (uint32_t)u;
      A::template st<XF>(rout, (int)(i * 16), u32x4{x[u].x, fout, x[u].y, fout});
      A::template st<XF>(rout2, (int)(i * 16), u32x4{x[u].z, fout, x[u].w, fout});
    }
  }
  if constexpr (to_local) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + 64u * (uint32_t)u;
      if (nt) A::template st<XN>(rdst, (int)(i * 16), x[u]);
      else A::template st<XS>(rdst, (int)(i * 16), x[u]);
    }
  }
#ifdef MSCCLX_PROFILE
  prof_mark = __builtin_amdgcn_s_memtime();
  prof_acc[2] += prof_mark - prof_got;
#endif
  return true;
}

// The step table seen through the constant address space: nothing on the device writes it, and a
// step's entry then arrives in scalar registers with three scalar loads (a vector load would bring it
// to every lane, to be carried back to scalar registers word by word).
typedef const __attribute__((address_space(4))) DevOp* ConstOps;
__device__ __forceinline__ DevOp fetch_step(ConstOps e) {  // (field by field: a struct cannot be copied out of another address space as a whole)
  DevOp r;
  r.word = e->word; r.dep_tb = e->dep_tb; r.dep_step = e->dep_step; r.dep_nops = e->dep_nops;
  r.extra = e->extra; r.steps = e->steps;
  r.src_addr = e->src_addr; r.dst_addr = e->dst_addr; r.in_addr = e->in_addr;
  return r;
}

// The rows of one step of type T (run_chain): packed in the slots, a chunk apart in the rank's buffers.
template <class R, int T>
__device__ __forceinline__ bool chain_rows(const unsigned char* in_row, unsigned char* out_row, u64 src_row, u64 dst_row, const u64 row_stride,
                                           const uint32_t cnt, const uint32_t n, const uint32_t row_line_bytes, const uint32_t local_bytes,
                                           const uint32_t lane, const bool nt, const uint32_t fin, const uint32_t fout, const u64* gate,
                                           const u64 gate_target, const ChainWatch& watch, const int step, const uint32_t pass,
                                           const __amdgpu_buffer_rsrc_t table, uint32_t ask_index, StepAhead& asked, u64* prof_acc, u64& prof_mark,
                                           const u64 prof_floor) {
  for (uint32_t row = 0; row < cnt; ++row) {
    // (a row of lines: the first halves of its n units, then the second halves; a descriptor for each)
    const uint32_t half = row_line_bytes >> 1;
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(in_row, half), rin2 = make_rsrc(in_row + half, half);
    const __amdgpu_buffer_rsrc_t rout = make_rsrc(out_row, half), rout2 = make_rsrc(out_row + half, half);
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc((const void*)src_row, local_bytes), rdst = make_rsrc((const void*)dst_row, local_bytes);
    if (n <= 64) {  // the shape of the smallest messages: one unit per lane, half the instructions
      if (!chain_round<R, 1, T>(rin, rin2, rout, rout2, rsrc, rdst, lane, n, nt, fin, fout, gate, gate_target, watch, step, pass, table, ask_index, asked,
                                prof_acc, prof_mark, prof_floor))
        return false;
      gate = nullptr;
      ask_index = ~0u;  // (the step's first round has asked)
    } else {
      for (uint32_t base = 0; base < n; base += 128) {
        if (!chain_round<R, 2, T>(rin, rin2, rout, rout2, rsrc, rdst, base + lane, n, nt, fin, fout, gate, gate_target, watch, step, pass, table, ask_index,
                                  asked, prof_acc, prof_mark, prof_floor))
          return false;
        gate = nullptr;
        ask_index = ~0u;
      }
    }
    in_row += row_line_bytes; out_row += row_line_bytes;
    src_row += row_stride; dst_row += row_stride;
  }
  return true;
}

// (prof_acc, profiling builds only: fine-clock ticks spent 0 waiting for a dependency, 1 from the first
// load of a message's lines until they are all there, 2 from there until the step's stores are issued,
// 3 from there to the next step's first load, 4 in all)
template <class R, bool RAGGED>
__device__ __forceinline__ void run_chain(const KernelParams& p, uint32_t epoch, int ctx, u64* prof_acc = nullptr) {
  const uint32_t lane = threadIdx.x;
  const bool writer = lane == 0;
  Hosted h;
  uint32_t left;  // units of the slice still to do (this pass included)
  u64 off;        // byte offset of this pass's piece inside every chunk
  {
    Context first;
    init_context<true, RAGGED>(h, first, p, epoch, ctx, writer);
    if (!first.active) return;
    left = uniform(first.left);
    off = uniform((uint64_t)first.off);
  }
  const ConstOps ops = (ConstOps)(p.ops + uniform(h.op_begin));
  const u64 row_stride = p.chunk_bytes;  // rows of a rank buffer are a chunk apart; rows of a slot are packed
  const uint32_t end_clip = RAGGED ? uniform(h.clip) : 0u;  // bytes that the last unit of the slice's last pass lacks (see move_units)
  unsigned char* const in_ring = p.fifo + (u64)uniform(h.in_slots) * 16;
  unsigned char* const out_ring = p.fifo + (u64)uniform(h.out_slots) * 16;
  const u64* const flags = p.sync_cur + uniform(h.flags);
  const u64* const out_tail = p.sync_cur + uniform(h.tail_in);  // what the receiver of the outgoing connection has consumed
  u64* const in_tail = p.sync_cur + uniform(h.tail_out);        // what this context has consumed of the incoming connection
  u64* const my_flag = p.sync_cur + uniform(h.my_flag);
  const uint32_t piece = p.piece_units, depth = (uint32_t)p.depth, nops = (uint32_t)uniform(h.nops), npasses = uniform(h.npasses);
  const uint32_t in_slot_bytes = uniform(h.in_slot_bytes), in_wrap = uniform(h.in_wrap), out_slot_bytes = uniform(h.out_slot_bytes), out_wrap = uniform(h.out_wrap);
  const ChainWatch watch{p.sync_cur, p.host_status, p.timeout_ticks, uniform(h.tb), uniform(h.slice)};
  uint32_t step = 0, pass = 0, rseq = 0, sseq = 0, rslot = 0, sslot = 0, count = 0;
  DevOp op = fetch_step(ops);
  const __amdgpu_buffer_rsrc_t table = make_rsrc(p.ops + uniform(h.op_begin), nops * (uint32_t)sizeof(DevOp));
  MSCCLX_CHAIN_CLOCK(prof_begin);
  u64 prof_mark = 0;  // profiling builds: when the previous step's stores were issued
#ifdef MSCCLX_PROFILE
  prof_mark = prof_begin;
#endif
  for (;;) {
    const StepAhead after = ask_step(table, step + 1 == nops ? 0 : step + 1);  // (it arrives while the wave waits)
    StepAhead not_asked;  // (only run_chain_flat asks from inside a round: measured, each loop as it runs fastest)
    MSCCLX_CHAIN_CLOCK(prof_dep0);
    const int t = (int)(op.word & 15u);
    const uint32_t cnt = op.word >> kOpCntShift;
    const uint32_t n = left < piece ? left : piece;
    if (op.dep_tb >= 0) {  // a step of another threadblock of this rank must have finished
      const u64* const flag = flags + (uint32_t)op.dep_tb * kSyncStrideWords;
      const u64 want = (u64)pass * (uint32_t)op.dep_nops + (uint32_t)op.dep_step + 1;
      unsigned spins = 0;
      u64 since = 0;
      while (uniform((uint64_t)load_counter(flag)) < want) {
        MSCCLX_POLL_PAUSE();
        if ((++spins & 0x3fu) == 0) {
          since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, (int)step, watch.slice, (u64)pass, 0));
          if (since == ~0ull) return;
        }
      }
    }
    if (__builtin_expect((count & 0x3fu) == 0x3fu, 0) && uniform((uint64_t)load_counter(watch.abort_word)) != 0) {  // a host's abort request, a lost launch
      note_abort(watch.abort_word, watch.host_status);
      return;
    }
    u64 prof_floor = 0;
#ifdef MSCCLX_PROFILE
    prof_floor = __builtin_amdgcn_s_memtime();
    prof_acc[0] += prof_floor - prof_dep0;
#endif
    const bool snd = ((0x5au >> t) & 1u) != 0;
    const bool nt = (op.word & kOpNtStore) != 0;
    const uint32_t fin = ll_flag(epoch, rseq), fout = ll_flag(epoch, sseq);
    const u64* gate = (snd && sseq >= depth) ? out_tail : nullptr;  // looked at in the step's first round only
    const u64 gate_target = (u64)sseq + 1 - depth;
    const uint32_t row_line_bytes = n * kLLUnitBytes;
    const uint32_t local_bytes = n * 16 - (left <= piece ? end_clip : 0u);  // rank-buffer rows may end inside their last unit; lines are whole
    bool ok = true;
#define MSCCLX_CHAIN_CASE(T)                                                                                                                                     \
  case T:                                                                                                                                                        \
    ok = chain_rows<R, T>(in_ring + rslot, out_ring + sslot, op.src_addr + off, op.dst_addr + off, row_stride, cnt, n, row_line_bytes, local_bytes, lane, nt, fin, \
                          fout, gate, gate_target, watch, (int)step, pass, table, ~0u, not_asked, prof_acc, prof_mark, prof_floor);                             \
    break
    switch (t) {  // (one copy of the step's instructions per type, with nothing left to decide inside)
      MSCCLX_CHAIN_CASE(MSCCLX_OP_SEND);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_RECV);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_RCS);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_RRS);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_RRC);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_RRCS);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_COPY);
      MSCCLX_CHAIN_CASE(MSCCLX_OP_REDUCE);
      default: break;  // nop
    }
#undef MSCCLX_CHAIN_CASE
    if (!ok) return;
    const bool rcv = ((0x7cu >> t) & 1u) != 0;
    // (in integers, not under `if (rcv)`: the compiler turns such an `if` into a per-lane select and
    // the running values would move to vector registers, and every address made from them with them)
    const uint32_t rcv_bit = (0x7cu >> t) & 1u, snd_bit = (0x5au >> t) & 1u;  // r rcs rrs rrc rrcs / s rcs rrs rrcs
    static_assert(MSCCLX_OP_SEND == 1 && MSCCLX_OP_RECV == 2 && MSCCLX_OP_RCS == 3 && MSCCLX_OP_RRS == 4 && MSCCLX_OP_RRC == 5 && MSCCLX_OP_RRCS == 6,
                  "the two masks above list the receiving and the sending step types by their codes");
    rseq += rcv_bit;
    rslot += in_slot_bytes & (0u - rcv_bit);
    rslot = rslot == in_wrap ? 0u : rslot;
    sseq += snd_bit;
    sslot += out_slot_bytes & (0u - snd_bit);
    sslot = sslot == out_wrap ? 0u : sslot;
    ++count;  // = pass * steps of the IR + IR step + 1 (nothing is folded under LL)
    if (op.word & kOpHasdep) {
      __builtin_amdgcn_s_waitcnt(0);
      if (writer) publish(my_flag, (u64)count);
    }
    if (++step == nops) {
      step = 0;
      left -= n;
      off += (u64)piece * 16;
      if (++pass >= npasses) {
        if (rcv && writer) publish(in_tail, (u64)rseq);
        break;
      }
    }
    if (rcv && writer) publish(in_tail, (u64)rseq);
    op = take_step(after);
  }
#ifdef MSCCLX_PROFILE
  prof_acc[4] = __builtin_amdgcn_s_memtime() - prof_begin;
#endif
}

// run_chain for a launch whose step table holds FlatOp records (plan.h): one pass, one row of at most 64 U units per step,
// no waits between the threadblocks of a rank, and every step's slots, flags and counter values worked out when the
// buffers were bound.  What is left per step is its one round and the request for the step after.
template <class R, int U>
__device__ __forceinline__ void run_chain_flat(const KernelParams& p, uint32_t epoch, int ctx) {
  const uint32_t lane = threadIdx.x;
  const bool writer = lane == 0;
  const DevCtx rec = p.ctxs[ctx];
  const Hosted h = rec.h;
  if (writer) {  // (as init_context: this context's counters in the area of the launch after this one)
    p.sync_nxt[h.my_flag] = 0;
    if (h.head_out) p.sync_nxt[h.head_out] = 0;
    if (h.tail_out) p.sync_nxt[h.tail_out] = 0;
  }
  const uint32_t nops = (uint32_t)uniform(h.nops);
  if (nops == 0 || uniform(h.npasses) == 0) return;
  const uint32_t n = uniform(rec.left);  // the units of this context's one piece
  const u64 off = uniform((uint64_t)rec.off);
  const unsigned char* const in_ring = p.fifo + (u64)uniform(h.in_slots) * 16;
  unsigned char* const out_ring = p.fifo + (u64)uniform(h.out_slots) * 16;
  const u64* const out_tail = p.sync_cur + uniform(h.tail_in);
  u64* const in_tail = p.sync_cur + uniform(h.tail_out);
  const ChainWatch watch{p.sync_cur, p.host_status, p.timeout_ticks, uniform(h.tb), uniform(h.slice)};
  const uint32_t flag_high = (epoch & 0x3ffu) << 22, half = n * 16;
  const __amdgpu_buffer_rsrc_t table = make_rsrc(p.ops + uniform(h.op_begin), nops * (uint32_t)sizeof(DevOp));
  FlatOp op = take_flat_step(ask_step(table, 0));
  StepAhead after = ask_step(table, nops > 1 ? 1u : 0u);  // (the table is read two steps ahead, as in run_chain)
  u64 no_clock = 0;
  for (uint32_t step = 0;;) {
    uint32_t second = step + 2;
    second = second >= nops ? second - nops : second;
    second = second >= nops ? 0u : second;
    StepAhead after_that;
    after_that.a = after_that.b = after_that.c = u32x4{0, 0, 0, 0};
    if (__builtin_expect((step & 0x3fu) == 0x3fu, 0) && uniform((uint64_t)load_counter(watch.abort_word)) != 0) {  // a host's abort request, a lost launch
      note_abort(watch.abort_word, watch.host_status);
      return;
    }
    const uint32_t t = op.word & 15u;
    const bool nt = (op.word & kOpNtStore) != 0;
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(in_ring + op.in_off, half), rin2 = make_rsrc(in_ring + op.in_off + half, half);
    const __amdgpu_buffer_rsrc_t rout = make_rsrc(out_ring + op.out_off, half), rout2 = make_rsrc(out_ring + op.out_off + half, half);
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc((const void*)(op.src_addr + off), half), rdst = make_rsrc((const void*)(op.dst_addr + off), half);
    const u64* const gate = op.gate ? out_tail : nullptr;
    bool ok = true;
#define MSCCLX_FLAT_CASE(T)                                                                                                                                  \
  case T:                                                                                                                                                    \
    ok = chain_round<R, U, T>(rin, rin2, rout, rout2, rsrc, rdst, lane, n, nt, flag_high | op.fin, flag_high | op.fout, gate, (u64)op.gate, watch, (int)step, 0u, \
                              table, second, after_that, nullptr, no_clock, 0);                                                                              \
    break
    switch (t) {
      MSCCLX_FLAT_CASE(MSCCLX_OP_SEND);
      MSCCLX_FLAT_CASE(MSCCLX_OP_RECV);
      MSCCLX_FLAT_CASE(MSCCLX_OP_RCS);
      MSCCLX_FLAT_CASE(MSCCLX_OP_RRS);
      MSCCLX_FLAT_CASE(MSCCLX_OP_RRC);
      MSCCLX_FLAT_CASE(MSCCLX_OP_RRCS);
      MSCCLX_FLAT_CASE(MSCCLX_OP_COPY);
      MSCCLX_FLAT_CASE(MSCCLX_OP_REDUCE);
      default: break;
    }
#undef MSCCLX_FLAT_CASE
    if (!ok) return;
    if (op.tail && writer) publish(in_tail, op.tail);
    if (++step == nops) break;
    op = take_flat_step(after);
    after = after_that;
  }
}

// One round of a step of run_chain_counters: units i0, i0 + 64, ... (U per lane) of one row of n
// units; out-of-range lanes load zeros and store nothing (the descriptors bound every access).
template <class R, int U>
__device__ __forceinline__ void chain_copy_round(const __amdgpu_buffer_rsrc_t ra, const __amdgpu_buffer_rsrc_t rb, const __amdgpu_buffer_rsrc_t rlocal,
                                                 const __amdgpu_buffer_rsrc_t rslot, const uint32_t i0, const bool has_b, const bool to_local,
                                                 const bool to_slot, const bool nt) {
  typedef Access<16> A;
  constexpr int XL = MSCCLX_AUX_LD, XS = MSCCLX_AUX_ST, XN = MSCCLX_AUX_ST_FINAL;
  u32x4 x[U], y[U];
#pragma unroll
  for (int u = 0; u < U; ++u) x[u] = A::template ld<XL>(ra, (int)((i0 + 64u * (uint32_t)u) * 16));
  if (has_b) {
#pragma unroll
    for (int u = 0; u < U; ++u) y[u] = A::template ld<XL>(rb, (int)((i0 + 64u * (uint32_t)u) * 16));
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = R::combine(y[u], x[u]);
  }
  if (to_slot) {  // the forwarded copy first: the next rank is waiting for it
#pragma unroll
    for (int u = 0; u < U; ++u) A::template st<XS>(rslot, (int)((i0 + 64u * (uint32_t)u) * 16), x[u]);
  }
  if (to_local) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (nt) A::template st<XN>(rlocal, (int)((i0 + 64u * (uint32_t)u) * 16), x[u]);
      else A::template st<XS>(rlocal, (int)((i0 + 64u * (uint32_t)u) * 16), x[u]);
    }
  }
}

// The counter protocol, one context on a workgroup of one wave: the same lean loop as run_chain for
// programs whose messages are announced by counters and mostly read where the sender keeps them.  A
// step waits for its (up to three) counters with one round of loads, moves its rows, waits until its
// stores are acknowledged and announces them.  Steps, waits and counters are those of the hosted
// path, so a workgroup running this loop can talk to workgroups running that one.
template <class R, bool RAGGED>
__device__ __forceinline__ void run_chain_counters(const KernelParams& p, int ctx, u64* prof_acc = nullptr) {
  const uint32_t lane = threadIdx.x;
  const bool writer = lane == 0;
  Hosted h;
  uint32_t left;  // units of the slice still to do (this pass included)
  u64 off;        // byte offset of this pass's piece inside every chunk
  {
    Context first;
    init_context<false, RAGGED>(h, first, p, 0, ctx, writer);
    if (!first.active) return;
    left = uniform(first.left);
    off = uniform((uint64_t)first.off);
  }
  const ConstOps ops = (ConstOps)(p.ops + uniform(h.op_begin));
  const u64 row_stride = p.chunk_bytes;  // rows of a rank buffer are a chunk apart; rows of a slot are packed
  const uint32_t end_clip = RAGGED ? uniform(h.clip) : 0u;  // bytes that the last unit of the slice's last pass lacks (see move_units)
  unsigned char* const in_ring = p.fifo + (u64)uniform(h.in_slots) * 16;
  unsigned char* const out_ring = p.fifo + (u64)uniform(h.out_slots) * 16;
  const u64* const flags = p.sync_cur + uniform(h.flags);
  const u64* const in_head = p.sync_cur + uniform(h.head_in);   // messages the sender of the incoming connection has announced
  u64* const in_tail = p.sync_cur + uniform(h.tail_out);        // messages this context has consumed of them
  u64* const out_head = p.sync_cur + uniform(h.head_out);       // messages this context has announced on the outgoing connection
  const u64* const out_tail = p.sync_cur + uniform(h.tail_in);  // messages its receiver has consumed
  u64* const my_flag = p.sync_cur + uniform(h.my_flag);
  const uint32_t piece = p.piece_units, depth = (uint32_t)p.depth, nops = (uint32_t)uniform(h.nops), npasses = uniform(h.npasses);
  const uint32_t in_slot_bytes = uniform(h.in_slot_bytes), in_wrap = uniform(h.in_wrap), out_slot_bytes = uniform(h.out_slot_bytes), out_wrap = uniform(h.out_wrap);
  const ChainWatch watch{p.sync_cur, p.host_status, p.timeout_ticks, uniform(h.tb), uniform(h.slice)};
  uint32_t step = 0, pass = 0, rseq = 0, sseq = 0, rslot = 0, sslot = 0, count = 0;
  DevOp op = fetch_step(ops);
  const __amdgpu_buffer_rsrc_t table = make_rsrc(p.ops + uniform(h.op_begin), nops * (uint32_t)sizeof(DevOp));
  // (prof_acc, profiling builds only: fine-clock ticks spent 0 waiting for the step's counters, 1 moving its rows,
  // 2 waiting for the stores' acknowledgement, 3 on the bookkeeping between steps, 4 in all)
  MSCCLX_CHAIN_CLOCK(prof_begin);
  for (;;) {
    MSCCLX_CHAIN_CLOCK(prof_top);
    const StepAhead after = ask_step(table, step + 1 == nops ? 0 : step + 1);  // (it arrives while the wave waits)
    const uint32_t t = op.word & 15u;
    const uint32_t cnt = op.word >> kOpCntShift;
    const uint32_t n = left < piece ? left : piece;
    const uint32_t rcv_bit = (0x7cu >> t) & 1u, snd_bit = (0x5au >> t) & 1u;  // r rcs rrs rrc rrcs / s rcs rrs rrcs
    static_assert(MSCCLX_OP_SEND == 1 && MSCCLX_OP_RECV == 2 && MSCCLX_OP_RCS == 3 && MSCCLX_OP_RRS == 4 && MSCCLX_OP_RRC == 5 && MSCCLX_OP_RRCS == 6,
                  "the two masks above list the receiving and the sending step types by their codes");
    {  // what the step waits for: a step of another threadblock, the incoming message, a free outgoing slot -- one round of loads for all
      const u64* const w0 = op.dep_tb >= 0 ? flags + (uint32_t)op.dep_tb * kSyncStrideWords : nullptr;
      const u64 t0 = (u64)pass * (uint32_t)op.dep_nops + (uint32_t)op.dep_step + 1;
      const u64* const w1 = (rcv_bit && !(op.steps & kStepsNoAnnouncement)) ? in_head : nullptr;  // (the bit is only set on payloads read in place)
      const u64 t1 = (u64)rseq + 1;
      const u64* const w2 = (snd_bit && sseq >= depth) ? out_tail : nullptr;
      const u64 t2 = (u64)sseq + 1 - depth;
      unsigned spins = 0;
      u64 since = 0;
      for (;;) {
        const u64 v0 = w0 ? load_counter(w0) : 0, v1 = w1 ? load_counter(w1) : 0, v2 = w2 ? load_counter(w2) : 0;
        const bool ok0 = !w0 || uniform((uint64_t)v0) >= t0, ok1 = !w1 || uniform((uint64_t)v1) >= t1, ok2 = !w2 || uniform((uint64_t)v2) >= t2;
        if (ok0 && ok1 && ok2) break;
        MSCCLX_POLL_PAUSE();
        if ((++spins & 0x3fu) == 0) {
          since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, (int)step, watch.slice, (u64)pass,
                                                     !ok0 ? 0 : !ok1 ? 1 : 2));
          if (since == ~0ull) return;
        }
      }
    }
    if (__builtin_expect((count & 0x3fu) == 0x3fu, 0) && uniform((uint64_t)load_counter(watch.abort_word)) != 0) {  // a host's abort request, a lost launch
      note_abort(watch.abort_word, watch.host_status);
      return;
    }
    MSCCLX_CHAIN_CLOCK(prof_ready);
    MSCCLX_CHAIN_ADD(0, prof_top, prof_ready);
    const bool rcv = rcv_bit != 0;
    const bool has_b = t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRS || t == MSCCLX_OP_RRCS || t == MSCCLX_OP_REDUCE;
    const bool to_local = t == MSCCLX_OP_RECV || t == MSCCLX_OP_RCS || t == MSCCLX_OP_RRC || t == MSCCLX_OP_RRCS || t == MSCCLX_OP_COPY || t == MSCCLX_OP_REDUCE;
    const bool to_slot = snd_bit && (op.word & kOpOutStaged);  // else the receiver reads the payload where this rank keeps it
    const bool nt = (op.word & kOpNtStore) != 0;
    if (to_local || to_slot) {
      // the step's rows: packed in the slots, a chunk apart in rank buffers (the sender's too, when the payload is read in place)
      const bool in_place = rcv && (op.word & kOpInPlace);
      u64 a_row = rcv ? (in_place ? op.in_addr + off : (u64)(in_ring + rslot)) : op.src_addr + off;
      const u64 a_stride = (rcv && !in_place) ? (u64)n * 16 : row_stride;
      u64 local_row = op.dst_addr + off, slot_row = (u64)(out_ring + sslot);
      const uint32_t row_total = n * 16 - (left <= piece ? end_clip : 0u);  // (slot rows are n units apart, and end where their rank-buffer rows do)
      // whole dwords through the descriptors; RAGGED kernels of 8- and 16-bit elements: then 1 to 3 bytes, element by element (see move_units)
      constexpr bool kTails = RAGGED && R::kElemBytes < 4;
      const uint32_t row_bytes = kTails ? row_total & ~3u : row_total, odd = row_total - row_bytes;
      for (uint32_t row = 0; row < cnt; ++row) {
        const __amdgpu_buffer_rsrc_t ra = make_rsrc((const void*)a_row, row_bytes), rlocal = make_rsrc((const void*)local_row, row_bytes);
        const __amdgpu_buffer_rsrc_t rslot_out = make_rsrc((const void*)slot_row, row_bytes);
        typedef Access<(R::kElemBytes < 4 ? R::kElemBytes : 1)> AE;
        typename AE::word tail_x{}, tail_y{};
        if constexpr (kTails) {
          if (odd && lane * R::kElemBytes < odd) {
            tail_x = AE::template ld<MSCCLX_AUX_LD>(make_rsrc((const void*)(a_row + row_bytes), odd), (int)(lane * R::kElemBytes));
            if (has_b) tail_y = AE::template ld<MSCCLX_AUX_LD>(make_rsrc((const void*)(local_row + row_bytes), odd), (int)(lane * R::kElemBytes));
          }
        }
        if (n <= 64) chain_copy_round<R, 1>(ra, rlocal, rlocal, rslot_out, lane, has_b, to_local, to_slot, nt);
        else if (n <= 128) chain_copy_round<R, 2>(ra, rlocal, rlocal, rslot_out, lane, has_b, to_local, to_slot, nt);
        else if (n <= 256) chain_copy_round<R, 4>(ra, rlocal, rlocal, rslot_out, lane, has_b, to_local, to_slot, nt);
        else  // (eight loads in flight per lane and operand, as the workgroup-wide mover has)
          for (uint32_t base = 0; base < n; base += 512) chain_copy_round<R, 8>(ra, rlocal, rlocal, rslot_out, base + lane, has_b, to_local, to_slot, nt);
        if constexpr (kTails) {
          if (odd && lane * R::kElemBytes < odd) {
            if (has_b) tail_x = R::combine(tail_y, tail_x);
            if (to_local) AE::template st<MSCCLX_AUX_ST>(make_rsrc((const void*)(local_row + row_bytes), odd), (int)(lane * R::kElemBytes), tail_x);
            if (to_slot) AE::template st<MSCCLX_AUX_ST>(make_rsrc((const void*)(slot_row + row_bytes), odd), (int)(lane * R::kElemBytes), tail_x);
          }
        }
        a_row += a_stride; local_row += row_stride; slot_row += (u64)n * 16;
      }
      MSCCLX_CHAIN_CLOCK(prof_issued);
      MSCCLX_CHAIN_ADD(1, prof_ready, prof_issued);
      __builtin_amdgcn_s_waitcnt(0);  // the stores are acknowledged: the counters below may announce them
      MSCCLX_CHAIN_CLOCK(prof_acked);
      MSCCLX_CHAIN_ADD(2, prof_issued, prof_acked);
    }
    MSCCLX_CHAIN_CLOCK(prof_moved);
    if (snd_bit && writer) publish(out_head, (u64)sseq + 1);
    if (rcv_bit && writer) publish(in_tail, (u64)rseq + 1);
    rseq += rcv_bit;
    rslot += in_slot_bytes & (0u - rcv_bit);
    rslot = rslot == in_wrap ? 0u : rslot;
    sseq += snd_bit;
    sslot += out_slot_bytes & (0u - snd_bit);
    sslot = sslot == out_wrap ? 0u : sslot;
    ++count;  // = pass * steps of the IR + IR step + 1 (programs with folded steps do not come here)
    if ((op.word & kOpHasdep) && writer) publish(my_flag, (u64)count);
    if (++step == nops) {
      step = 0;
      left -= n;
      off += (u64)piece * 16;
      if (++pass >= npasses) break;
    }
    op = take_step(after);
#ifdef MSCCLX_PROFILE
    prof_acc[3] += __builtin_amdgcn_s_memtime() - prof_moved;
#endif
  }
#ifdef MSCCLX_PROFILE
  prof_acc[4] = __builtin_amdgcn_s_memtime() - prof_begin;
#endif
}

// The start of a launch.  The number of launches so far is kept on the device, so a launch carries no host-side state
// and the same launch can be replayed: the control block holds up to kFinishCounters counters of finished workgroups,
// workgroup w counting itself in counter w mod `finish_counters` when it ends.  Such a counter grows by a known number
// per launch (the workgroups of its class), and a workgroup that reads its own class's counter when it starts finds
// (launches so far) x (that number) + (workgroups of its class that have already ended in this launch) -- fewer than
// the class has, the reader being one of them -- so the quotient is the launch's number however late the workgroup
// starts, and however early others have ended.  (Stream order guarantees that every workgroup of the launches before has counted itself.)  The number's lowest
// bit picks which of the two counter areas this launch uses; its low 10 bits mark the LL lines.  Returns that number.
__device__ __forceinline__ u64 begin_launch(KernelParams& p) {
  const uint32_t k = blockIdx.x & (p.finish_counters - 1u);
  const u64 ended = load_counter(p.sync_base + 8 + (uint64_t)k * kFinishStrideWords);
  // ended / (workgroups of my class), as a multiplication by ceil(2^64 / divisor), worked out on the host: exact for
  // dividends below 2^57 and divisors up to 128 (0 stands for a divisor of 1)
  const u64 magic = k < p.finish_more ? p.finish_magic_more : p.finish_magic_each;
  const u64 launch_no = magic ? __umul64hi(ended, magic) : ended;  // (left in vector registers: the counter areas' addresses made from it cost scalar registers the step loops need)
  const u64 parity = launch_no & 1ull;
  p.sync_cur = p.sync_base + kControlWords + parity * p.sync_words;
  p.sync_nxt = p.sync_base + kControlWords + (parity ^ 1ull) * p.sync_words;
  return launch_no;
}

// The end of a workgroup: it counts itself, and does not wait for the answer -- the last workgroup to finish its work
// used to find out that it was the last with one or two atomics that return, a microsecond at the end of every launch.
__device__ __forceinline__ void end_launch(const KernelParams& p) {
  if (threadIdx.x == 0)
    (void)__hip_atomic_fetch_add(p.sync_base + 8 + (uint64_t)(blockIdx.x & (p.finish_counters - 1u)) * kFinishStrideWords, 1ull, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
}

// A workgroup hosts up to 64 contexts, one per lane of wave 0.  Wave 0 polls the counters every
// active context waits for (one round of loads covers all of them), finishes steps that move no data
// on the spot, and picks a ready context whose step does move data; the whole workgroup then copies /
// reduces that step's piece.  No context ever blocks the workgroup, so any number of threadblocks can
// share the resident workgroups without deadlock.
// FOLD: steps may carry the dependencies of nop steps folded into them (a kernel of its own, so that
// programs without such steps do not pay for the check in the poll loop).
template <class R, bool LL, int FOLD, bool RAGGED>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4))) exec_kernel(const KernelParams launch_params) {
  KernelParams p = launch_params;
  const u64 launch_no = begin_launch(p);
  const uint32_t epoch = (uint32_t)launch_no & 0x3ffu;
  __shared__ int sh_choice;
  __shared__ Move sh_move;
  __shared__ uint32_t sh_seq[2];   // LL: numbers of the incoming and the outgoing message
  __shared__ int sh_who[4];        // LL: threadblock, step, slice, pass of the chosen step, for the watchdog's report
  u64* const abort_word = p.sync_cur;
  const int lane = threadIdx.x;
  const bool poller = threadIdx.x < 64;
  const int ctx_begin = p.one_each ? (int)blockIdx.x : p.wg_begin[blockIdx.x], hosted = p.one_each ? 1 : p.wg_begin[blockIdx.x + 1] - ctx_begin;
  // LL, one hosted context: nothing else could run while it waits for a message, so the lane does not
  // watch for it; the moving threads go straight to the lines and retry them until they are there.
  const bool direct = LL && hosted == 1;

  __shared__ Hosted sh_hosted[kMaxHosted];
  Hosted& h = sh_hosted[lane & (kMaxHosted - 1)];  // this lane's entry; lanes of other waves never look at it
  Context c;
  c.active = false;
#ifdef MSCCLX_PROFILE
  u64 prof_wait = 0, prof_move = 0, prof_ack = 0, prof_fin = 0;
  unsigned prof_moves = 0;
  const u64 prof_start = wall_clock64();
#endif
  if (threadIdx.x == 0 && blockIdx.x == 0) p.sync_nxt[0] = 0;
  if (LL && hosted == 1 && blockDim.x == 64) {  // (LL is configured only for chunks of whole dwords)
#ifdef MSCCLX_PROFILE
    u64 chain_acc[5] = {0, 0, 0, 0, 0};
    if constexpr (LL) run_chain<R, RAGGED>(p, epoch, ctx_begin, chain_acc);
    prof_fin = chain_acc[0]; prof_wait = chain_acc[1]; prof_move = chain_acc[2]; prof_ack = chain_acc[3];
    if (threadIdx.x == 0 && p.prof) p.prof[(size_t)blockIdx.x * kProfWords + 8] = chain_acc[4];
#else
    if constexpr (LL) {
      if (!RAGGED && p.flat) {  // (a loop for each number of units per lane: in one loop the longer rows cost the short ones 40 %)
        if (p.piece_units <= 64) run_chain_flat<R, 1>(p, epoch, ctx_begin);
        else run_chain_flat<R, 2>(p, epoch, ctx_begin);  // (four units per lane lost to the general loop: 64-rank chain on 4 KiB pieces 128 -> 147 us)
      } else {
        run_chain<R, RAGGED>(p, epoch, ctx_begin);
      }
    }
#endif
  } else if (!LL && !FOLD && hosted == 1 && blockDim.x == 64) {
#ifdef MSCCLX_PROFILE
    u64 chain_acc[5] = {0, 0, 0, 0, 0};
    if constexpr (!LL && !FOLD) run_chain_counters<R, RAGGED>(p, ctx_begin, chain_acc);
    prof_wait = chain_acc[0]; prof_move = chain_acc[1]; prof_ack = chain_acc[2]; prof_fin = chain_acc[3];
    if (threadIdx.x == 0 && p.prof) p.prof[(size_t)blockIdx.x * kProfWords + 8] = chain_acc[4];
#else
    if constexpr (!LL && !FOLD) run_chain_counters<R, RAGGED>(p, ctx_begin);
#endif
  } else {
  if (poller && lane < hosted) init_context<LL, RAGGED>(h, c, p, epoch, ctx_begin + lane, true);
  if (FOLD && poller && lane < hosted && c.active) mark_many_sources(c, p.ops[h.op_begin]);
  int cursor = 0;
  unsigned busy_rounds = 0;

  // A workgroup of one wave needs neither LDS nor a barrier to hand the chosen step to its threads:
  // they are the lanes of the polling wave, and take the operands from the chosen lane's registers.
  const bool one_wave = blockDim.x == 64;
  for (;;) {
#ifdef MSCCLX_PROFILE
    const u64 prof_t0 = wall_clock64();
#endif
    int chosen = -2;
    if (poller) {
      int choice = -2;
      unsigned spins = 0;
      // The watchdog period starts when this workgroup last made progress.  The clock is only read
      // while nothing is ready, so a workgroup that keeps finding work never pays for it.
      u64 deadline = 0;
      bool armed = false;
      while (choice == -2) {
        bool ready = false;
        if (c.active) {
          // the (up to three) counters are loaded together: one round trip to memory, not one each
          const bool watch1 = c.w1 && !direct;
          const u64 v0 = c.w0 ? load_counter(c.w0) : 0;
          const u64 v1 = watch1 ? load_counter(c.w1) : 0;
          const u64 v2 = c.w2 ? load_counter(c.w2) : 0;
          ready = (!c.w0 || v0 >= c.t0) && (!c.w2 || v2 >= c.t2) &&
                  (!watch1 || (LL ? (uint32_t)(v1 >> 32) == (uint32_t)c.t1 : v1 >= c.t1));
          if (FOLD && ready && (c.extra & 255u) && (c.extra & 255u) <= (uint32_t)kLaneExtraDeps) ready = extras_ready(c, h, p);  // the nops folded into this step
        }
        if (FOLD == 2) {  // long runs of folded nops, context by context
          u64 long_runs = __ballot(ready && (c.extra & 255u) > (uint32_t)kLaneExtraDeps);
          while (long_runs) {
            const int owner = __ffsll((long long)long_runs) - 1;
            long_runs &= long_runs - 1;
            const bool all_there = extras_ready_together(c, h, p, owner, lane);
            if (lane == owner) ready = all_there;
          }
        }
        bool progressed = false;
        if (ready && !c.moves) {  // nothing to copy: the step is complete as soon as it may start
          const DevOp next = fetch_next_op(c, h, p);
          finish_step<LL, RAGGED>(c, h, p, epoch, next);
          if (FOLD && c.active) mark_many_sources(c, next);
          progressed = true;
          ready = false;  // the context now stands at another step, whose conditions are not yet known
        }
        const u64 movers = __ballot(ready && c.moves && c.active);
        if (movers) {
          const u64 from_cursor = movers & ~((cursor >= 64) ? ~0ull : ((1ull << cursor) - 1ull));
          choice = __ffsll((long long)(from_cursor ? from_cursor : movers)) - 1;
          // a workgroup that always finds work never reaches the idle branch below: it looks at the
          // abort word once in 64 moves, so that a host's abort request ends it too
          if (__builtin_expect((++busy_rounds & 0x3fu) == 0, 0)) {
            bool stop = false;
            if (lane == 0) stop = load_counter(abort_word) != 0;
            if (__any(stop)) { if (lane == 0) note_abort_here(abort_word, p.host_status); choice = -3; }
          }
        } else if (!__any(c.active)) {
          choice = -1;  // every hosted context has run to its end
        } else if (__any(progressed)) {
          armed = false;
        } else {
          __builtin_amdgcn_s_sleep(1);
          if ((++spins & 0x3fu) == 0) {
            const u64 now = wall_clock64();
            if (!armed) { deadline = now + p.timeout_ticks; armed = true; }
            bool stop = false;
            if (lane == 0) stop = load_counter(abort_word) != 0;
            if (__any(stop)) { if (lane == 0) note_abort_here(abort_word, p.host_status); choice = -3; }
            else if (now > deadline) {
              // report the first context that is still waiting
              const u64 stuck = __ballot(c.active);
              const int who = __ffsll((long long)stuck) - 1;
              if (lane == who && atomicCAS(abort_word, 0ull, kAbortByWatchdog) == 0ull) {
                int what = 3;
                if (c.w0 && load_counter(c.w0) < c.t0) what = 0;
                else if (c.w1 && (LL ? (uint32_t)(load_counter(c.w1) >> 32) != (uint32_t)c.t1 : load_counter(c.w1) < c.t1)) what = 1;
                else if (c.w2 && load_counter(c.w2) < c.t2) what = 2;
                else if (FOLD && (c.extra & 255u)) what = 0;  // the dependency of a nop folded into this step
                mscclx_status* hs = p.host_status;
                hs->tb = h.tb; hs->step = c.step; hs->slice = h.slice; hs->pass = (int64_t)c.pass; hs->waiting_on = what;
                __threadfence_system();
                __hip_atomic_store(&hs->code, (int)MSCCLX_ERR_TIMEOUT, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
              }
              choice = -3;
            }
          }
        }
      }
      if (!one_wave) {
        if (choice >= 0 && lane == choice) {
          sh_move = c.m;
          if (LL) { sh_seq[0] = c.rseq; sh_seq[1] = c.sseq; sh_who[0] = h.tb; sh_who[1] = c.step; sh_who[2] = h.slice; sh_who[3] = (int)c.pass; }
        }
        if (lane == 0) sh_choice = choice;
      }
      chosen = choice;
      cursor = choice >= 0 ? (choice + 1) & 63 : cursor;
    }
    int choice;
    Move m;
    uint32_t rseq = 0, sseq = 0;
    int who_tb = 0, who_step = 0, who_slice = 0;
    unsigned who_pass = 0;
    if (one_wave) {
      choice = __builtin_amdgcn_readfirstlane(chosen);
      if (choice < 0) break;  // done (-1) or giving up (-3)
      m.a = lane_value(c.m.a, choice); m.dst = lane_value(c.m.dst, choice); m.out = lane_value(c.m.out, choice);
      m.n = lane_value(c.m.n, choice); m.rows = (int)lane_value((uint32_t)c.m.rows, choice); m.kind = (int)lane_value((uint32_t)c.m.kind, choice);
      if (LL) {
        rseq = lane_value(c.rseq, choice); sseq = lane_value(c.sseq, choice);
        who_tb = (int)lane_value((uint32_t)h.tb, choice); who_step = (int)lane_value((uint32_t)c.step, choice);
        who_slice = (int)lane_value((uint32_t)h.slice, choice); who_pass = lane_value(c.pass, choice);
      }
    } else {
      __syncthreads();
      choice = sh_choice;
      if (choice < 0) break;  // done (-1) or giving up (-3); uniform for the workgroup
      m = sh_move;
      if (LL) { rseq = sh_seq[0]; sseq = sh_seq[1]; who_tb = sh_who[0]; who_step = sh_who[1]; who_slice = sh_who[2]; who_pass = (unsigned)sh_who[3]; }
    }
#ifdef MSCCLX_PROFILE
    const u64 prof_t1 = wall_clock64();
#endif

    // ---- the chosen context's step: move one piece ----
    do_move<R, LL, FOLD, RAGGED>(m, p, epoch, rseq, sseq, who_tb, who_step, who_slice, who_pass);
#ifdef MSCCLX_PROFILE
    const u64 prof_t2 = wall_clock64();
#endif
    // every wave waits until its own device-scope stores are acknowledged (the context's lane asks
    // for its next step's description meanwhile); after the barrier that lane may announce the whole
    // workgroup's data with plain counter stores
    const bool mine = poller && lane == choice;
    DevOp next;
    if (mine) next = fetch_next_op(c, h, p);
    __builtin_amdgcn_s_waitcnt(0);
    if (!one_wave) __syncthreads();
#ifdef MSCCLX_PROFILE
    const u64 prof_t3 = wall_clock64();
#endif
    if (mine) {
      finish_step<LL, RAGGED>(c, h, p, epoch, next);
      if (FOLD && c.active) mark_many_sources(c, next);
    }
#ifdef MSCCLX_PROFILE
    if (threadIdx.x == 0) {
      const u64 prof_t4 = wall_clock64();
      prof_wait += prof_t1 - prof_t0;
      prof_move += prof_t2 - prof_t1;
      prof_ack += prof_t3 - prof_t2;
      prof_fin += prof_t4 - prof_t3;
      // the first kProfTrace moves of the workgroup: start (10 ns ticks since the workgroup began), duration up to the barrier, lane
      if (p.prof && prof_moves < kProfTrace)
        p.prof[(size_t)blockIdx.x * kProfWords + 8 + prof_moves] = ((prof_t1 - prof_start) << 32) | (((prof_t3 - prof_t1) & 0xffffffull) << 8) | (u64)(choice & 0xff);
      ++prof_moves;
    }
#endif
  }
  }  // hosted contexts
  end_launch(p);
#ifdef MSCCLX_PROFILE
  if (threadIdx.x == 0 && p.prof) {
    p.prof[(size_t)blockIdx.x * kProfWords + 0] = prof_wait;
    p.prof[(size_t)blockIdx.x * kProfWords + 1] = prof_move;
    p.prof[(size_t)blockIdx.x * kProfWords + 2] = wall_clock64() - prof_start;
    p.prof[(size_t)blockIdx.x * kProfWords + 3] = prof_start;
    p.prof[(size_t)blockIdx.x * kProfWords + 4] = prof_ack;
    p.prof[(size_t)blockIdx.x * kProfWords + 5] = prof_fin;
    // where the workgroup ran: HW_ID (compute unit, shader engine) and XCC_ID hardware registers
    p.prof[(size_t)blockIdx.x * kProfWords + 6] = __builtin_amdgcn_s_getreg(4 | (31 << 11));
    p.prof[(size_t)blockIdx.x * kProfWords + 7] = __builtin_amdgcn_s_getreg(20 | (31 << 11));
  }
#endif
}

// Programs with folded nops on one-wave workgroups with one context each (the all-pairs family on small messages: the
// all-reduce, all-gather and all-to-all plans below a few MiB per rank): a kernel of its own, so that neither loop pays
// for the other's registers.  The step waits of such programs are many -- a step that stands for a run of nops waits for
// each nop's threadblock, a receive that has taken over its sender's waits for those too -- and all of one kind: a
// counter that must reach a value.  So every wait of a step sits in a lane of its own (the folded ones first, then the
// step's own dependency, the incoming message's announcement, the outgoing connection's free slot), and one vector load
// and one ballot check them all: one round trip per poll however many counters a step waits for, where the hosting loop
// makes three in a row (its counters, the table of folded dependencies, their counters).  The table entries of the next
// step are asked for while this step waits.  The moves are the hosting loop's own (do_move), with the wave as the workgroup.
template <class R, bool RAGGED>
__global__ void __launch_bounds__(64) exec_kernel_chain_fold(const KernelParams launch_params) {
  KernelParams p = launch_params;
  // (the context's record is asked for in front of the launch's number: two round trips of a workgroup's start side by side)
  const DevCtx record = launch_params.ctxs[blockIdx.x];
  (void)begin_launch(p);
  const uint32_t lane = threadIdx.x;
  const bool writer = lane == 0;
  if (writer && blockIdx.x == 0) p.sync_nxt[0] = 0;
  Hosted h;
  uint32_t left;  // units of the slice still to do (this pass included)
  u64 off;        // byte offset of this pass's piece inside every chunk
  bool active;
  {
    Context first;
    init_context<false, RAGGED>(h, first, p, 0, (int)blockIdx.x, writer, &record);  // (a workgroup hosts the context of its own number)
    active = first.active;
    left = uniform(first.left);
    off = uniform((uint64_t)first.off);
  }
  if (active) {
    const ConstOps ops = (ConstOps)(p.ops + uniform(h.op_begin));
    const uint2* const extras = (const uint2*)p.extra_deps;
    const uint32_t end_clip = RAGGED ? uniform(h.clip) : 0u;
    unsigned char* const in_ring = p.fifo + (u64)uniform(h.in_slots) * 16;
    unsigned char* const out_ring = p.fifo + (u64)uniform(h.out_slots) * 16;
    const u64* const flags = p.sync_cur + uniform(h.flags);
    const u64* const in_head = p.sync_cur + uniform(h.head_in);
    u64* const in_tail = p.sync_cur + uniform(h.tail_out);
    u64* const out_head = p.sync_cur + uniform(h.head_out);
    const u64* const out_tail = p.sync_cur + uniform(h.tail_in);
    u64* const my_flag = p.sync_cur + uniform(h.my_flag);
    const uint32_t piece = p.piece_units, depth = (uint32_t)p.depth, nops = (uint32_t)uniform(h.nops), npasses = uniform(h.npasses);
    const uint32_t in_slot_bytes = uniform(h.in_slot_bytes), in_wrap = uniform(h.in_wrap), out_slot_bytes = uniform(h.out_slot_bytes), out_wrap = uniform(h.out_wrap);
    const ChainWatch watch{p.sync_cur, p.host_status, p.timeout_ticks, uniform(h.tb), uniform(h.slice)};
    uint32_t step = 0, pass = 0, rseq = 0, sseq = 0, rslot = 0, sslot = 0, count = 0;
    DevOp op = fetch_step(ops);
    const __amdgpu_buffer_rsrc_t table = make_rsrc(p.ops + uniform(h.op_begin), nops * (uint32_t)sizeof(DevOp));
    uint2 entry = {0u, 0u};  // this lane's folded dependency of the step `op`, if it has one
    if (lane < (op.extra & 255u)) entry = extras[(op.extra >> 8) + lane];
    // The table is read two steps ahead: the entry of the step after this one is there when this step begins, so
    // that its lanes can ask for their folded dependencies, and the entry of the step after that is on its way.
    StepAhead after = ask_step(table, nops > 1 ? 1u : 0u);
    for (;;) {
      uint32_t second = step + 2;
      second = second >= nops ? second - nops : second;
      second = second >= nops ? 0u : second;  // (a table of one step)
      const StepAhead after_that = ask_step(table, second);
      uint2 next_entry = {0u, 0u};
      if (lane < (after.b.x & 255u)) next_entry = extras[(after.b.x >> 8) + lane];  // (b.x: DevOp::extra)
      const uint32_t t = op.word & 15u;
      const uint32_t cnt = op.word >> kOpCntShift;
      const uint32_t n = left < piece ? left : piece;
      const uint32_t rcv_bit = (0x7cu >> t) & 1u, snd_bit = (0x5au >> t) & 1u;  // r rcs rrs rrc rrcs / s rcs rrs rrcs
      static_assert(MSCCLX_OP_SEND == 1 && MSCCLX_OP_RECV == 2 && MSCCLX_OP_RCS == 3 && MSCCLX_OP_RRS == 4 && MSCCLX_OP_RRC == 5 && MSCCLX_OP_RRCS == 6,
                    "the two masks above list the receiving and the sending step types by their codes");
      {  // what this lane waits for: nothing, or one counter and the value it must reach
        const uint32_t folded = op.extra & 255u;
        const u64* mine = nullptr;
        uint32_t target = 0;
        if (lane < folded) {
          mine = flags + entry.x;
          target = pass * (entry.y >> 16) + (entry.y & 0xffffu);
        } else if (lane == folded) {
          if (op.dep_tb >= 0) { mine = flags + (uint32_t)op.dep_tb * kSyncStrideWords; target = pass * (uint32_t)op.dep_nops + (uint32_t)op.dep_step + 1; }
        } else if (lane == folded + 1) {
          if (rcv_bit && !(op.steps & kStepsNoAnnouncement)) { mine = in_head; target = rseq + 1; }
        } else if (lane == folded + 2) {
          if (snd_bit && sseq >= depth) { mine = out_tail; target = sseq + 1 - depth; }
        }
        unsigned spins = 0;
        u64 since = 0;
        for (;;) {
          u64 seen = ~0ull;
          if (mine) seen = load_counter(mine);
          const u64 behind = __builtin_amdgcn_ballot_w64(seen < (u64)target);
          if (!behind) break;
          MSCCLX_POLL_PAUSE();
          if ((++spins & 0x3fu) == 0) {
            const uint32_t who = (uint32_t)__ffsll((long long)behind) - 1u;  // the first lane still waiting names what the report says
            since = uniform((uint64_t)chain_slow_check(watch.abort_word, watch.host_status, watch.timeout_ticks, since, watch.tb, (int)step, watch.slice, (u64)pass,
                                                       who <= folded ? 0 : who == folded + 1 ? 1 : 2));
            if (since == ~0ull) break;
          }
        }
        if (since == ~0ull) break;  // the launch is lost
      }
      if (__builtin_expect((count & 0x3fu) == 0x3fu, 0) && uniform((uint64_t)load_counter(watch.abort_word)) != 0) {  // a host's abort request
        note_abort(watch.abort_word, watch.host_status);
        break;
      }
      const bool out_staged = (op.word & kOpOutStaged) != 0;
      if (!(t == MSCCLX_OP_NOP || (t == MSCCLX_OP_SEND && !out_staged))) {
        // the step's operands, as the hosting loop's describe_step works them out, in scalar registers
        Move m;
        const u64 out = (snd_bit && out_staged) ? (u64)(out_ring + sslot) : 0;
        u64 in = 0;
        int in_packed = kAPacked;
        if (rcv_bit) {
          if (op.word & kOpInPlace) { in = op.in_addr + off; in_packed = 0; }
          else in = (u64)(in_ring + rslot);
        }
        m.n = n; m.rows = (int)cnt;
        m.a = in; m.dst = op.dst_addr + off; m.out = out;
        const int nt = (op.word & kOpNtStore) ? kNt1 : 0;
        int kind = 0;
        switch (t) {
          case MSCCLX_OP_SEND: m.a = op.src_addr + off; kind = (int)kToSlot; break;
          case MSCCLX_OP_RECV: kind = in_packed | nt; break;
          case MSCCLX_OP_RCS: kind = in_packed | (out ? (int)kHasO2 : 0); break;
          case MSCCLX_OP_RRC: kind = in_packed | kHasB; break;
          case MSCCLX_OP_RRS: kind = in_packed | kHasB | kToSlot; break;
          case MSCCLX_OP_RRCS: kind = in_packed | kHasB | (out ? (int)kHasO2 : 0); break;
          case MSCCLX_OP_COPY: m.a = op.src_addr + off; kind = nt; break;
          case MSCCLX_OP_REDUCE:
            m.a = op.src_addr + off;
            kind = kHasB;
            if (op.in_addr) { m.out = op.in_addr; kind = kMany | nt; }  // several sources, in_addr bytes apart
            break;
          default: break;
        }
        if constexpr (RAGGED) kind |= left <= piece ? (int)end_clip << kClipShift : 0;
        m.kind = kind;
        do_move<R, false, 1, RAGGED, 8>(m, p, 0u, 0u, 0u, 0, 0, 0, 0u);  // (short rows of a multi-chunk step go eight at a time here)
        __builtin_amdgcn_s_waitcnt(0);  // the stores are acknowledged: the counters below may announce them
      }
      if (snd_bit && writer) publish(out_head, (u64)sseq + 1);
      if (rcv_bit && writer) publish(in_tail, (u64)rseq + 1);
      rseq += rcv_bit;
      rslot += in_slot_bytes & (0u - rcv_bit);
      rslot = rslot == in_wrap ? 0u : rslot;
      sseq += snd_bit;
      sslot += out_slot_bytes & (0u - snd_bit);
      sslot = sslot == out_wrap ? 0u : sslot;
      count += op.steps & ~kStepsNoAnnouncement;  // = pass * steps of the IR + IR step + 1: a step may stand for folded ones too
      if ((op.word & kOpHasdep) && writer) publish(my_flag, (u64)count);
      if (++step == nops) {
        step = 0;
        left -= n;
        off += (u64)piece * 16;
        if (++pass >= npasses) break;
      }
      op = take_step(after);
      after = after_that;
      entry = next_entry;
    }
  }
  end_launch(p);
}

// ------------------------------------------------------------------------------------------------
// kernel table of one element type
// ------------------------------------------------------------------------------------------------
typedef void (*kernel_fn)(const KernelParams);

// ragged: chunks that are no multiple of 16 bytes -- rows may end inside a unit; the other kernels carry none of that
// fold: 0 = no step stands for folded nops, 1 = some do, at most kLaneExtraDeps each, 2 = some for more (the check
// of those costs scalar registers the other programs' poll loop has no room for: a kernel of its own), 3 = the loop for
// such programs on one-wave workgroups with one context each (exec_kernel_chain_fold)
template <int DT, int OP, bool RAGGED> kernel_fn pick_variant(bool ll, int fold) {
  if (ll) return !fold ? (kernel_fn)exec_kernel<Reducer<DT, OP>, true, 0, RAGGED> : nullptr;
  if (fold == 3) return (kernel_fn)exec_kernel_chain_fold<Reducer<DT, OP>, RAGGED>;
  if (fold == 2) return (kernel_fn)exec_kernel<Reducer<DT, OP>, false, 2, RAGGED>;
  if (fold) return (kernel_fn)exec_kernel<Reducer<DT, OP>, false, 1, RAGGED>;
  return (kernel_fn)exec_kernel<Reducer<DT, OP>, false, 0, RAGGED>;
}
template <int DT> kernel_fn pick_op(int op, bool ll, int fold, bool ragged) {
  switch (op) {
    case MSCCLX_SUM: return (ragged ? pick_variant<DT, MSCCLX_SUM, true>(ll, fold) : pick_variant<DT, MSCCLX_SUM, false>(ll, fold));
    case MSCCLX_PROD: return (ragged ? pick_variant<DT, MSCCLX_PROD, true>(ll, fold) : pick_variant<DT, MSCCLX_PROD, false>(ll, fold));
    case MSCCLX_MAX: return (ragged ? pick_variant<DT, MSCCLX_MAX, true>(ll, fold) : pick_variant<DT, MSCCLX_MAX, false>(ll, fold));
    case MSCCLX_MIN: return (ragged ? pick_variant<DT, MSCCLX_MIN, true>(ll, fold) : pick_variant<DT, MSCCLX_MIN, false>(ll, fold));
    default: return nullptr;
  }
}

}  // namespace mscclx
