// pccl_kernels.h -- device code of libpccl_hip.so: the gfx950 kernels for
// PCCL's reduction and placement work.  Included by pccl_hip.hip only (and by
// the host-side indexing check in tests/, which runs the same code thread by
// thread on the CPU; the kernels use no LDS and no barriers, so that is exact).
#ifndef PCCL_KERNELS_H
#define PCCL_KERNELS_H

#include <cstddef>
#include <cstdint>

#include "pccl_hip.h"

namespace pccl_kernels {

constexpr int kThreads = 256;              // 4 waves of 64 lanes
constexpr size_t kTileBytes = kThreads * 16;   // what a workgroup moves per operand with one vector per thread
constexpr size_t kXcds = 8;                    // accelerator dies of an MI355X; workgroup i runs on XCD i % 8
constexpr int kMaxSeg = PCCL_HIP_MAX_RANKS;

// The work items [begin, end) one launch covers.  Long schedules go out as
// several launches of bounded size: within one launch the XCDs drift apart in
// the address range they stream from, and throughput falls with its length.
struct Span {
  uint32_t begin, end;
};
constexpr unsigned kMaxGrid = 0x7fffffffu;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
template <bool NT>
__device__ __forceinline__ u32x4 ld16(const u32x4* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}

template <bool NT>
__device__ __forceinline__ void st16(u32x4* p, u32x4 v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// The same 16 bytes at ANY address.  gfx950 takes vector accesses that are not
// 16-byte (or even 4-byte) aligned; one that straddles its natural boundary is
// split into more requests, which is still far ahead of an element-wise loop
// (measured on MI355X: a bf16 fold of 12 shards whose blocks start at odd
// multiples of 2 bytes 2.2 -> 5.5 TB/s, an accumulate whose source is one element
// off the destination's alignment 3.3 -> 6.4, a copy one byte off 1.9 -> 6.4).
// For an aligned address it is the very same instruction.
typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(1)));

template <bool NT>
__device__ __forceinline__ u32x4 ld16u(const void* p) {
  if constexpr (NT) return __builtin_nontemporal_load((const u32x4_any*)p);
  else return *(const u32x4_any*)p;
}

// Round an fp32 value (given as bits) to bfloat16, ties to even; the result
// stays in the upper 16 bits so that it is again a valid fp32 operand.
// NaN becomes the canonical quiet NaN 0x7FC0, as on the host.
__device__ __forceinline__ uint32_t bf16_round_hi(float s) {
  uint32_t w = __float_as_uint(s);
  uint32_t r = (w + 0x7fffu + ((w >> 16) & 1u)) & 0xffff0000u;
  return (s != s) ? 0x7fc00000u : r;
}

// Two fp32 values to packed bfloat16 (lo in bits 0-15) with the gfx950 packed
// conversion: round to nearest even, identical to bf16_round_hi for every
// non-NaN input; a NaN stays a (quiet) NaN but keeps its payload, so results
// that may be NaN are canonicalised with bf16_round_hi when they are stored.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}

// own + received in fp32, where `own` is the rank's own block and `received` what
// its neighbour or partner sent: vectorAdd(a, b) of pccl/src/common.cu:5-19.
// The sum is commutative except for WHICH payload survives when both operands
// are NaN: the hardware add keeps the one in its first source, and the
// reference's compiled kernel has `b` there.  The compiler orders the sources of
// a plain `own + received` as it likes (it did the opposite here), so the
// instruction is written out; the host build of this file, which only checks
// indexing, adds plainly.
__device__ __forceinline__ float add_own_received(float own, float received) {
#if defined(__HIP_DEVICE_COMPILE__)
  float r;
  asm("v_add_f32 %0, %1, %2" : "=v"(r) : "v"(received), "v"(own));
  return r;
#else
  return own + received;
#endif
}

struct OpF32 {
  typedef float elem;
  static constexpr int kPerVec = 4;
  static __device__ __forceinline__ u32x4 add(u32x4 a, u32x4 b) {
    u32x4 r;
    r.x = __float_as_uint(add_own_received(__uint_as_float(a.x), __uint_as_float(b.x)));
    r.y = __float_as_uint(add_own_received(__uint_as_float(a.y), __uint_as_float(b.y)));
    r.z = __float_as_uint(add_own_received(__uint_as_float(a.z), __uint_as_float(b.z)));
    r.w = __float_as_uint(add_own_received(__uint_as_float(a.w), __uint_as_float(b.w)));
    return r;
  }
  static __device__ __forceinline__ elem add1(elem a, elem b) { return add_own_received(a, b); }
};

// Two bf16 values per 32-bit word, element 2i in the low half.
struct OpBF16 {
  typedef uint16_t elem;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ uint32_t add_word(uint32_t a, uint32_t b) {
    float lo = __uint_as_float(a << 16) + __uint_as_float(b << 16);
    float hi = __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u);
    return (bf16_round_hi(lo) >> 16) | bf16_round_hi(hi);
  }
  static __device__ __forceinline__ u32x4 add(u32x4 a, u32x4 b) {
    u32x4 r;
    r.x = add_word(a.x, b.x);
    r.y = add_word(a.y, b.y);
    r.z = add_word(a.z, b.z);
    r.w = add_word(a.w, b.w);
    return r;
  }
  static __device__ __forceinline__ elem add1(elem a, elem b) {
    float s = __uint_as_float((uint32_t)a << 16) + __uint_as_float((uint32_t)b << 16);
    return (elem)(bf16_round_hi(s) >> 16);
  }
};

// binary16 <-> binary32.  Widening is exact; narrowing rounds to nearest even
// (v_cvt_f16_f32), and NaN becomes the canonical 0x7E00.  An fp16 hop is
// RNE_fp16(float(a) + float(b)), what torch.add does on float16 tensors on the
// host; since binary32 carries 24 >= 2 * 11 + 2 significand bits, rounding the
// fp32 sum once more gives the correctly rounded fp16 sum.
__device__ __forceinline__ float f16_widen(uint32_t u16) {
  const uint16_t u = (uint16_t)u16;
  _Float16 h;
  __builtin_memcpy(&h, &u, 2);
  return (float)h;
}

__device__ __forceinline__ uint32_t f16_narrow(float s) {
  const _Float16 h = (_Float16)s;
  uint16_t u;
  __builtin_memcpy(&u, &h, 2);
  return (s != s) ? 0x7e00u : (uint32_t)u;
}

// Two fp16 values per 32-bit word, element 2i in the low half.
struct OpF16 {
  typedef uint16_t elem;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ uint32_t add_word(uint32_t a, uint32_t b) {
    const float lo = f16_widen(a & 0xffffu) + f16_widen(b & 0xffffu);
    const float hi = f16_widen(a >> 16) + f16_widen(b >> 16);
    return f16_narrow(lo) | (f16_narrow(hi) << 16);
  }
  static __device__ __forceinline__ u32x4 add(u32x4 a, u32x4 b) {
    u32x4 r;
    r.x = add_word(a.x, b.x);
    r.y = add_word(a.y, b.y);
    r.z = add_word(a.z, b.z);
    r.w = add_word(a.w, b.w);
    return r;
  }
  static __device__ __forceinline__ elem add1(elem a, elem b) {
    return (elem)f16_narrow(f16_widen(a) + f16_widen(b));
  }
};

// Partial sums of the fused reduce.  An accumulator is held as fp32 lanes; for
// bf16 with per-hop rounding the fp32 value is re-rounded to bf16 precision
// after every add, which is bit-identical to storing and re-loading bf16.
struct AccF32 {
  typedef OpF32 op;
  static constexpr int kLanes = 4;   // fp32 lanes per 16-byte input vector
  static __device__ __forceinline__ void widen(u32x4 v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  static __device__ __forceinline__ float widen1(float e) { return e; }
  static __device__ __forceinline__ float narrow1(float f) { return f; }
  static __device__ __forceinline__ float hop(float a, float b) { return a + b; }
  // one hop of a ring: the running sum `acc` is what the rank received, x its own block
  template <int L>
  static __device__ __forceinline__ void hop_lanes(float* acc, const float* x) {
#pragma unroll
    for (int l = 0; l < L; ++l) acc[l] = add_own_received(x[l], acc[l]);
  }
  // one round of halving: lo is the rank's own partial sum, hi its partner's
  template <int L>
  static __device__ __forceinline__ void join_lanes(float* lo, const float* hi) {
#pragma unroll
    for (int l = 0; l < L; ++l) lo[l] = add_own_received(lo[l], hi[l]);
  }
  static __device__ __forceinline__ u32x4 narrow(const float* f) {
    u32x4 r;
    r.x = __float_as_uint(f[0]); r.y = __float_as_uint(f[1]);
    r.z = __float_as_uint(f[2]); r.w = __float_as_uint(f[3]);
    return r;
  }
  // one hop on whole input vectors: partial sums can stay in input format
  static constexpr bool kPacked = true;
  static constexpr bool kAsmAdd = true;   // the add is an asm statement (add_own_received): loads are not hoisted over it
  static __device__ __forceinline__ u32x4 add_vec(u32x4 a, u32x4 b) { return OpF32::add(a, b); }
  static __device__ __forceinline__ u32x4 settle(u32x4 v) { return v; }
};

template <bool PER_HOP>
struct AccBF16 {
  typedef OpBF16 op;
  static constexpr int kLanes = 8;
  static __device__ __forceinline__ void widen(u32x4 v, float* f) {
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
  }
  static __device__ __forceinline__ float widen1(uint16_t e) { return __uint_as_float((uint32_t)e << 16); }
  static __device__ __forceinline__ uint16_t narrow1(float f) { return (uint16_t)(bf16_round_hi(f) >> 16); }
  static __device__ __forceinline__ float hop(float a, float b) {
    float s = a + b;
    if constexpr (PER_HOP) return __uint_as_float(bf16_round_hi(s));
    else return s;
  }
  // acc[l] = hop(acc[l], x[l]) for L lanes; lanes are rounded two at a time
  // with the packed conversion (NaN payloads are settled in narrow()).
  template <int L>
  static __device__ __forceinline__ void hop_lanes(float* acc, const float* x) {
    if constexpr (PER_HOP && (L % 2 == 0)) {
#pragma unroll
      for (int l = 0; l < L; l += 2) {
        const uint32_t p = cvt_pk_bf16(acc[l] + x[l], acc[l + 1] + x[l + 1]);
        acc[l] = __uint_as_float(p << 16);
        acc[l + 1] = __uint_as_float(p & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int l = 0; l < L; ++l) acc[l] = hop(acc[l], x[l]);
    }
  }
  // NaNs are stored as the canonical pattern, so the two operands' roles do not matter here
  template <int L>
  static __device__ __forceinline__ void join_lanes(float* lo, const float* hi) { hop_lanes<L>(lo, hi); }
  static __device__ __forceinline__ u32x4 narrow(const float* f) {
    u32x4 r;
    r.x = (bf16_round_hi(f[0]) >> 16) | bf16_round_hi(f[1]);
    r.y = (bf16_round_hi(f[2]) >> 16) | bf16_round_hi(f[3]);
    r.z = (bf16_round_hi(f[4]) >> 16) | bf16_round_hi(f[5]);
    r.w = (bf16_round_hi(f[6]) >> 16) | bf16_round_hi(f[7]);
    return r;
  }
  // With a rounding per hop every partial sum is a bf16 value again, so partial
  // sums can stay packed two to a word (half the registers of fp32 lanes).
  static constexpr bool kPacked = PER_HOP;
  static constexpr bool kAsmAdd = false;
  static __device__ __forceinline__ uint32_t add_word(uint32_t a, uint32_t b) {
    return cvt_pk_bf16(__uint_as_float(a << 16) + __uint_as_float(b << 16),
                       __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u));
  }
  static __device__ __forceinline__ u32x4 add_vec(u32x4 a, u32x4 b) {
    u32x4 r;
    r.x = add_word(a.x, b.x); r.y = add_word(a.y, b.y);
    r.z = add_word(a.z, b.z); r.w = add_word(a.w, b.w);
    return r;
  }
  // the NaN patterns of the packed conversion become the canonical one
  static __device__ __forceinline__ u32x4 settle(u32x4 v) {
    float f[8];
    widen(v, f);
    return narrow(f);
  }
};

template <bool PER_HOP>
struct AccF16 {
  typedef OpF16 op;
  static constexpr int kLanes = 8;
  static __device__ __forceinline__ void widen(u32x4 v, float* f) {
    f[0] = f16_widen(v.x & 0xffffu); f[1] = f16_widen(v.x >> 16);
    f[2] = f16_widen(v.y & 0xffffu); f[3] = f16_widen(v.y >> 16);
    f[4] = f16_widen(v.z & 0xffffu); f[5] = f16_widen(v.z >> 16);
    f[6] = f16_widen(v.w & 0xffffu); f[7] = f16_widen(v.w >> 16);
  }
  static __device__ __forceinline__ float widen1(uint16_t e) { return f16_widen(e); }
  static __device__ __forceinline__ uint16_t narrow1(float f) { return (uint16_t)f16_narrow(f); }
  static __device__ __forceinline__ float hop(float a, float b) {
    const float s = a + b;
    if constexpr (PER_HOP) return f16_widen(f16_narrow(s));
    else return s;
  }
  template <int L>
  static __device__ __forceinline__ void hop_lanes(float* acc, const float* x) {
#pragma unroll
    for (int l = 0; l < L; ++l) acc[l] = hop(acc[l], x[l]);
  }
  // NaNs are stored as the canonical pattern, so the two operands' roles do not matter here
  template <int L>
  static __device__ __forceinline__ void join_lanes(float* lo, const float* hi) { hop_lanes<L>(lo, hi); }
  static __device__ __forceinline__ u32x4 narrow(const float* f) {
    u32x4 r;
    r.x = f16_narrow(f[0]) | (f16_narrow(f[1]) << 16);
    r.y = f16_narrow(f[2]) | (f16_narrow(f[3]) << 16);
    r.z = f16_narrow(f[4]) | (f16_narrow(f[5]) << 16);
    r.w = f16_narrow(f[6]) | (f16_narrow(f[7]) << 16);
    return r;
  }
  // with a rounding per hop every partial sum is an fp16 value again and can stay packed
  static constexpr bool kPacked = PER_HOP;
  static constexpr bool kAsmAdd = false;
  static __device__ __forceinline__ u32x4 add_vec(u32x4 a, u32x4 b) { return OpF16::add(a, b); }
  static __device__ __forceinline__ u32x4 settle(u32x4 v) { return v; }   // OpF16::add stores canonical NaNs already
};

// How a segment of `n` elements splits into a head (elements before the first
// 16-byte boundary of the DESTINATION), a body of whole 128-bit vectors and a
// tail.  Stores of the body are aligned; the sources are read at whatever
// alignment they have (ld16u).  A destination that is not even element-aligned,
// or a segment shorter than one vector, is done element by element (vec == 0).
struct Split {
  size_t head;   // elements
  size_t vec;    // 16-byte vectors
  size_t tail;   // elements
};

__device__ __forceinline__ Split split_segment(uintptr_t dst, size_t n, unsigned esize) {
  Split s;
  const unsigned mis = (unsigned)(dst & 15u);
  if ((mis % esize) != 0) {
    s.head = n; s.vec = 0; s.tail = 0;
    return s;
  }
  size_t head = ((16u - mis) & 15u) / esize;
  if (head > n) head = n;
  size_t per = 16u / esize;
  s.head = head;
  s.vec = (n - head) / per;
  s.tail = n - head - s.vec * per;
  if (s.vec == 0) { s.head = n; s.tail = 0; }
  return s;
}

// dst = a + b over one tile of a segment, by a workgroup of T threads.  Tile
// `tile` covers vectors [tile*T*U, (tile+1)*T*U); tile 0 also does head and tail.
// `aligned` (decided on the host for the whole launch): every operand starts on
// a 16-byte boundary and n is a whole number of vectors, so there is no head,
// no tail and nothing to decide per segment.
template <class Op, int U, bool NTL, bool NTS, int T = kThreads>
__device__ __forceinline__ void add_tile(void* dstp, const void* ap, const void* bp, size_t n,
                                         size_t tile, bool aligned) {
  typedef typename Op::elem elem;
  if (aligned) {
    u32x4* dv = (u32x4*)dstp;
    const u32x4* av = (const u32x4*)ap;
    const u32x4* bv = (const u32x4*)bp;
    const size_t nvec = n / Op::kPerVec;
    const size_t v0 = tile * (size_t)(T * U) + threadIdx.x;
    if (v0 + (size_t)(U - 1) * T < nvec) {
      u32x4 x[U], y[U];
#pragma unroll
      for (int j = 0; j < U; ++j) x[j] = ld16<NTL>(av + v0 + (size_t)j * T);
#pragma unroll
      for (int j = 0; j < U; ++j) y[j] = ld16<NTL>(bv + v0 + (size_t)j * T);
#pragma unroll
      for (int j = 0; j < U; ++j) st16<NTS>(dv + v0 + (size_t)j * T, Op::add(x[j], y[j]));
    } else {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = v0 + (size_t)j * T;
        if (v < nvec) st16<NTS>(dv + v, Op::add(ld16<NTL>(av + v), ld16<NTL>(bv + v)));
      }
    }
    return;
  }
  const Split sp = split_segment((uintptr_t)dstp, n, sizeof(elem));
  elem* de = (elem*)dstp;
  const elem* ae = (const elem*)ap;
  const elem* be = (const elem*)bp;
  const unsigned tid = threadIdx.x;

  if (sp.vec == 0) {
    // a segment shorter than one vector: scalar path, each tile takes the
    // element range its vectors would have covered
    const size_t per_tile = (size_t)T * U * Op::kPerVec;
    size_t lo = tile * per_tile;
    size_t hi = lo + per_tile < sp.head ? lo + per_tile : sp.head;
    for (size_t i = lo + tid; i < hi; i += T) de[i] = Op::add1(ae[i], be[i]);
    return;
  }

  u32x4* dv = (u32x4*)(de + sp.head);
  const uint8_t* av = (const uint8_t*)(ae + sp.head);   // the sources may sit at any element alignment
  const uint8_t* bv = (const uint8_t*)(be + sp.head);
  const size_t base = tile * (size_t)(T * U);

  if (base + (size_t)T * U <= sp.vec) {
    u32x4 x[U], y[U];
#pragma unroll
    for (int j = 0; j < U; ++j) x[j] = ld16u<NTL>(av + (base + (size_t)j * T + tid) * 16);
#pragma unroll
    for (int j = 0; j < U; ++j) y[j] = ld16u<NTL>(bv + (base + (size_t)j * T + tid) * 16);
#pragma unroll
    for (int j = 0; j < U; ++j) st16<NTS>(dv + base + (size_t)j * T + tid, Op::add(x[j], y[j]));
  } else {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      size_t v = base + (size_t)j * T + tid;
      if (v < sp.vec) st16<NTS>(dv + v, Op::add(ld16u<NTL>(av + v * 16), ld16u<NTL>(bv + v * 16)));
    }
  }

  if (tile == 0) {
    if (tid < sp.head) de[tid] = Op::add1(ae[tid], be[tid]);
    if (tid >= T / 2 && tid - T / 2 < sp.tail) {   // head and tail are below 16 elements each
      size_t i = sp.head + sp.vec * Op::kPerVec + (tid - T / 2);
      de[i] = Op::add1(ae[i], be[i]);
    }
  }
}

// Vector j of this thread in tile `tile` of a copy.  The U vectors of a thread
// come from 4 KiB chunks 8 apart (tiles are taken in groups of 8, one per XCD as
// workgroups are dealt round robin), so chunk c of a segment is always moved by
// the same XCD, as it is with one vector per thread.  With contiguous 8 KiB
// tiles a copy runs 7 % slower on MI355X than with 4 KiB tiles; with this
// mapping two vectors per thread run 3-4 % faster.  The host rounds the tiles of
// a segment up to a multiple of 8 (copy_tiles_for).
template <int U>
__device__ __forceinline__ size_t copy_vec(size_t tile, int j) {
  return ((tile / kXcds) * (size_t)(kXcds * U) + tile % kXcds + (size_t)j * kXcds) * kThreads + threadIdx.x;
}

// Byte copy of one tile of a segment (same splitting, element = byte).
template <int U, bool NTL, bool NTS>
__device__ __forceinline__ void copy_tile(void* dstp, const void* srcp, size_t nbytes, size_t tile,
                                          bool aligned = false) {
  if (aligned) {   // 16-byte aligned ends on both sides: vectors only
    u32x4* dv = (u32x4*)dstp;
    const u32x4* sv = (const u32x4*)srcp;
    const size_t nvec = nbytes / 16;
    if (copy_vec<U>(tile, U - 1) < nvec) {   // the last vector of the thread is the farthest
      u32x4 x[U];
#pragma unroll
      for (int j = 0; j < U; ++j) x[j] = ld16<NTL>(sv + copy_vec<U>(tile, j));
#pragma unroll
      for (int j = 0; j < U; ++j) st16<NTS>(dv + copy_vec<U>(tile, j), x[j]);
    } else {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = copy_vec<U>(tile, j);
        if (v < nvec) st16<NTS>(dv + v, ld16<NTL>(sv + v));
      }
    }
    return;
  }
  const Split sp = split_segment((uintptr_t)dstp, nbytes, 1);
  uint8_t* d8 = (uint8_t*)dstp;
  const uint8_t* s8 = (const uint8_t*)srcp;
  const unsigned tid = threadIdx.x;

  if (sp.vec == 0) {
    const size_t per_tile = (size_t)kThreads * U * 16;
    size_t lo = tile * per_tile;
    if (lo >= sp.head) return;
    size_t hi = lo + per_tile < sp.head ? lo + per_tile : sp.head;
    if ((((uintptr_t)dstp | (uintptr_t)srcp) & 3u) == 0) {
      // both 4-byte aligned: move words, then the last 0-3 bytes
      size_t wlo = lo / 4, whi = hi / 4;
      uint32_t* d32 = (uint32_t*)dstp;
      const uint32_t* s32 = (const uint32_t*)srcp;
      for (size_t i = wlo + tid; i < whi; i += kThreads) d32[i] = s32[i];
      if (hi == sp.head) {
        size_t i = whi * 4 + tid;
        if (i < hi) d8[i] = s8[i];
      }
    } else {
      for (size_t i = lo + tid; i < hi; i += kThreads) d8[i] = s8[i];
    }
    return;
  }

  u32x4* dv = (u32x4*)(d8 + sp.head);
  const uint8_t* sv = s8 + sp.head;                      // any alignment
  if (copy_vec<U>(tile, U - 1) < sp.vec) {
    u32x4 x[U];
#pragma unroll
    for (int j = 0; j < U; ++j) x[j] = ld16u<NTL>(sv + copy_vec<U>(tile, j) * 16);
#pragma unroll
    for (int j = 0; j < U; ++j) st16<NTS>(dv + copy_vec<U>(tile, j), x[j]);
  } else {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t v = copy_vec<U>(tile, j);
      if (v < sp.vec) st16<NTS>(dv + v, ld16u<NTL>(sv + v * 16));
    }
  }
  if (tile == 0) {
    if (tid < sp.head) d8[tid] = s8[tid];
    if (tid >= 64 && tid - 64 < sp.tail) {
      size_t i = sp.head + sp.vec * 16 + (tid - 64);
      d8[i] = s8[i];
    }
  }
}

// ---------------------------------------------------------------------------
// kernels
// ---------------------------------------------------------------------------
struct AddSegs {
  void* dst[kMaxSeg];
  const void* a[kMaxSeg];
  const void* b[kMaxSeg];
};

// A segment may consist of s1*s2 pieces of `len` elements (bytes for copies):
// piece (p1, p2) of operand X starts at X + p1*X1 + p2*X2.  This is how the
// [inter, intra, m] <-> [intra, inter, m] block permutation of the 2-D
// collectives is read or written in place instead of being materialised.
// s1 = s2 = 1 describes a plain contiguous segment.
struct Pieces {
  unsigned s1, s2;
  size_t len;
  size_t d1, d2;   // destination strides
  size_t a1, a2;   // first operand (or copy source) strides
  size_t b1, b2;   // second operand strides
};

// `count` segments: dst[s] = a[s] + b[s], piece by piece.
template <class Op, int U, bool NTL, bool NTS, int T>
__global__ __launch_bounds__(T) void k_add_segs(AddSegs t, int count, Pieces pc,
                                                       size_t tiles_per_piece, int aligned, Span span) {
  typedef typename Op::elem elem;
  // work items are counted in 32 bits (the host refuses launches beyond 2^32 - 1)
  const uint32_t tpp = (uint32_t)tiles_per_piece;
  const uint32_t per_seg = pc.s1 * pc.s2 * tpp;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t s = w / per_seg;
    const uint32_t rem = w - s * per_seg;
    const uint32_t piece = rem / tpp;
    const size_t tile = rem - piece * tpp;
    const size_t p1 = piece / pc.s2, p2 = piece - (uint32_t)p1 * pc.s2;
    add_tile<Op, U, NTL, NTS, T>((elem*)t.dst[s] + p1 * pc.d1 + p2 * pc.d2,
                              (const elem*)t.a[s] + p1 * pc.a1 + p2 * pc.a2,
                              (const elem*)t.b[s] + p1 * pc.b1 + p2 * pc.b2, pc.len, tile,
                              aligned != 0);
  }
}

// The same adds for the common case, stripped to the bone: contiguous segments
// of nvec whole vectors, every operand 16-byte aligned.  One wave per workgroup,
// one vector per thread and operand; blockIdx.y is the segment and blockIdx.x
// the 1 KiB tile inside it, so no work item is decoded by division and nothing
// but three pointers is fetched before the loads go out.  Measured on MI355X
// (dst = a + b, bf16, operands of 1 GiB): 6.73 TB/s, against 6.50 for
// k_add_segs with the same workgroup shape and 6.36 with 256 threads and four
// vectors per thread.  A one-wave workgroup frees its slot the moment its
// store is out, so the address window the chip has in flight stays short and
// dense, which is what the DRAM pages like.
constexpr int kRowThreads = 64;

template <class Op, bool NTL, bool NTS>
__global__ __launch_bounds__(kRowThreads) void k_add_rows(AddSegs t, int row0, size_t nvec, uint32_t tile0) {
  const int s = row0 + (int)blockIdx.y;
  const size_t v = ((size_t)tile0 + blockIdx.x) * kRowThreads + threadIdx.x;
  if (v >= nvec) return;
  const u32x4 x = ld16<NTL>((const u32x4*)t.a[s] + v);
  const u32x4 y = ld16<NTL>((const u32x4*)t.b[s] + v);
  st16<NTS>((u32x4*)t.dst[s] + v, Op::add(x, y));
}

struct RhArgs {
  void* bufs[kMaxSeg];
  const void* src[kMaxSeg];
  void* outs[kMaxSeg];
};

// One recursive-halving round for all P ranks: the strided-half pairwise add.
// Rank r and its partner own the same active region [start, start + 2*count);
// the lower rank of the pair sums the lower halves into its buffer, the upper
// rank the upper halves into its own.
template <class Op, int U, bool NTL, bool NTS, int T>
__global__ __launch_bounds__(T) void k_rh_round(RhArgs t, int P, size_t B, int round,
                                                       int from_src, int to_outs,
                                                       size_t tiles_per_seg, int aligned, Span span) {
  typedef typename Op::elem elem;
  const int group = P >> round;
  const int half = group >> 1;
  const size_t count = (size_t)half * B;
  const uint32_t tps = (uint32_t)tiles_per_seg;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const int r = (int)(w / tps);
    const size_t tile = w - (uint32_t)r * tps;
    const bool lower = (r % group) < half;
    const int partner = lower ? r + half : r - half;
    const size_t off = (size_t)(r / group) * group * B + (lower ? 0 : count);
    const elem* a = (const elem*)(from_src ? t.src[r] : t.bufs[r]) + off;
    const elem* b = (const elem*)(from_src ? t.src[partner] : t.bufs[partner]) + off;
    elem* d = to_outs ? (elem*)t.outs[r] : (elem*)t.bufs[r] + off;
    add_tile<Op, U, NTL, NTS, T>(d, a, b, count, tile, aligned != 0);
  }
}

// The strided-half pairwise add in the same lean shape (P a power of two, every
// buffer and B*sizeof(elem) 16-byte aligned): blockIdx.y is the rank, partner and
// half come from shifts and masks.  nvec = vectors of one half.
template <class Op, bool NTL, bool NTS>
__global__ __launch_bounds__(kRowThreads) void k_rh_rows(RhArgs t, int row0, int log2_group, size_t B,
                                                         int from_src, int to_outs, size_t nvec, uint32_t tile0) {
  typedef typename Op::elem elem;
  const int r = row0 + (int)blockIdx.y;
  const size_t v = ((size_t)tile0 + blockIdx.x) * kRowThreads + threadIdx.x;
  if (v >= nvec) return;
  const int group = 1 << log2_group, half = group >> 1;
  const bool lower = (r & (group - 1)) < half;
  const int partner = lower ? r + half : r - half;
  const size_t off = (size_t)(r & ~(group - 1)) * B + (lower ? 0 : (size_t)half * B);
  const u32x4* a = (const u32x4*)((const elem*)(from_src ? t.src[r] : t.bufs[r]) + off);
  const u32x4* b = (const u32x4*)((const elem*)(from_src ? t.src[partner] : t.bufs[partner]) + off);
  u32x4* d = to_outs ? (u32x4*)t.outs[r] : (u32x4*)((elem*)t.bufs[r] + off);
  const u32x4 x = ld16<NTL>(a + v);
  const u32x4 y = ld16<NTL>(b + v);
  st16<NTS>(d + v, Op::add(x, y));
}

struct CopySegs {
  void* dst[kMaxSeg];
  const void* src[kMaxSeg];
  size_t nbytes[kMaxSeg];
};

// `count` byte segments; tiles_per_seg is sized for the longest one.
template <int U, bool NTL, bool NTS>
__global__ __launch_bounds__(kThreads) void k_copy_segs(CopySegs t, int count,
                                                        size_t tiles_per_seg, int aligned, Span span) {
  const uint32_t tps = (uint32_t)tiles_per_seg;
  const size_t tile_bytes = (size_t)kThreads * U * 16;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const int s = (int)(w / tps);
    const size_t tile = w - (uint32_t)s * tps;
    const size_t nb = t.nbytes[s];
    // a group of tiles past the end of a short segment has nothing to do (16
    // spare bytes cover the head shift of the vector body); tiles share their
    // chunks in groups of kXcds, see copy_vec
    if (tile != 0 && (tile / kXcds) * kXcds * tile_bytes >= nb + 16) continue;
    copy_tile<U, NTL, NTS>(t.dst[s], t.src[s], nb, tile, aligned != 0);
  }
}

struct CopyPairs {
  void* dst[kMaxSeg];
  const void* src[kMaxSeg];
};

// `count` segments of s1*s2 pieces of pc.len BYTES each (strides in bytes).
template <int U, bool NTL, bool NTS>
__global__ __launch_bounds__(kThreads) void k_copy_pieces(CopyPairs t, int count, Pieces pc,
                                                          size_t tiles_per_piece, int aligned, Span span) {
  // work items are counted in 32 bits (the host refuses launches beyond 2^32 - 1)
  const uint32_t tpp = (uint32_t)tiles_per_piece;
  const uint32_t per_seg = pc.s1 * pc.s2 * tpp;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t s = w / per_seg;
    const uint32_t rem = w - s * per_seg;
    const uint32_t piece = rem / tpp;
    const size_t tile = rem - piece * tpp;
    const size_t p1 = piece / pc.s2, p2 = piece - (uint32_t)p1 * pc.s2;
    copy_tile<U, NTL, NTS>((uint8_t*)t.dst[s] + p1 * pc.d1 + p2 * pc.d2,
                           (const uint8_t*)t.src[s] + p1 * pc.a1 + p2 * pc.a2, pc.len, tile, aligned != 0);
  }
}

struct GatherArgs {
  void* outs[kMaxSeg];
  const void* ins[kMaxSeg];
  size_t nbytes[kMaxSeg];
  size_t dst_off[kMaxSeg];
};

// Direct all_gather placement for all P ranks: a workgroup reads one tile of
// shard k and stores it into the outputs of one of `split` groups of ranks at
// dst_off[k].  With split == 1 every shard byte is read once; with more groups
// the same tile is read by `split` workgroups launched side by side, each with
// nout / split write streams.
template <int U, bool NTL, bool NTS>
__global__ __launch_bounds__(kThreads) void k_gather_multicast(GatherArgs t, int P, int nout,
                                                              size_t tiles_per_seg, int split, Span span) {
  const uint32_t tps = (uint32_t)tiles_per_seg;
  const size_t tile_bytes = (size_t)kThreads * U * 16;
  const unsigned tid = threadIdx.x;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64 / (uint32_t)split;
    const int grp = (int)((uint32_t)w64 - w * (uint32_t)split);
    const int r0 = (int)((long)nout * grp / split), r1 = (int)((long)nout * (grp + 1) / split);
    const int k = (int)(w / tps);
    const size_t tile = w - (uint32_t)k * tps;
    const size_t nb = t.nbytes[k];
    if (tile != 0 && (tile / kXcds) * kXcds * tile_bytes >= nb + 16) continue;
    const uint8_t* src = (const uint8_t*)t.ins[k];
    const size_t off = t.dst_off[k];
    // vector path only if the source and EVERY destination share alignment
    bool aligned = ((uintptr_t)src & 15u) == 0 && (off & 15u) == 0;
    for (int r = r0; r < r1; ++r) aligned = aligned && (((uintptr_t)t.outs[r]) & 15u) == 0;
    const size_t nvec = nb / 16;
    if (aligned && copy_vec<U>(tile, U - 1) < nvec) {   // the same chunks as copy_tile would take
      const u32x4* sv = (const u32x4*)src;
      u32x4 x[U];
#pragma unroll
      for (int j = 0; j < U; ++j) x[j] = ld16<NTL>(sv + copy_vec<U>(tile, j));
      for (int r = r0; r < r1; ++r) {
        u32x4* dv = (u32x4*)((uint8_t*)t.outs[r] + off);
#pragma unroll
        for (int j = 0; j < U; ++j) st16<NTS>(dv + copy_vec<U>(tile, j), x[j]);
      }
      if (tile == 0 && tid < nb - nvec * 16) {   // the last nb % 16 bytes of the shard
        const size_t i = nvec * 16 + tid;
        for (int r = r0; r < r1; ++r) ((uint8_t*)t.outs[r])[off + i] = src[i];
      }
    } else {
      for (int r = r0; r < r1; ++r)
        copy_tile<U, NTL, NTS>((uint8_t*)t.outs[r] + off, src, nb, tile);
    }
  }
}

// The same placement, blocked in time: workgroup w runs on XCD w % 8 (workgroups
// are dealt to the dies round robin), and the workgroups of one XCD, taken in
// index order, walk a strip of `strip` of that XCD's 4 KiB tiles of shard k once
// per output: first the whole strip into output 0, then the same strip into
// output 1, ...  At any moment an XCD therefore feeds one write stream (two
// around a change of output) instead of nout, and every pass after the first
// finds the strip in that XCD's L2.  XCD x owns the tiles t = x (mod 8) of every
// shard, as in copy_vec.  n_local = tiles per shard and XCD, a multiple of strip.
template <int U, bool NTL, bool NTS>
__global__ __launch_bounds__(kThreads) void k_gather_strips(GatherArgs t, int P, int nout, uint32_t n_local,
                                                           uint32_t strip, Span span) {
  // a work item moves U of its XCD's tiles (8 tiles apart in the shard); n_local and strip count work items
  const unsigned tid = threadIdx.x;
  const uint32_t per_shard = n_local * (uint32_t)nout;
  const uint32_t per_strip = strip * (uint32_t)nout;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t x = w % (uint32_t)kXcds, seq = w / (uint32_t)kXcds;
    const uint32_t k = seq / per_shard;
    uint32_t rem = seq - k * per_shard;
    const uint32_t s = rem / per_strip;
    rem -= s * per_strip;
    const uint32_t r = rem / strip;
    const size_t tile0 = (size_t)(s * strip + (rem - r * strip)) * (kXcds * U) + x;   // then tile0 + 8, + 16, ...
    const size_t nb = t.nbytes[k];
    if (tile0 != 0 && tile0 * kTileBytes >= nb + 16) continue;
    const uint8_t* src = (const uint8_t*)t.ins[k];
    uint8_t* dst = (uint8_t*)t.outs[r] + t.dst_off[k];
    // head up to the destination's first 16-byte boundary, aligned vector stores behind
    // it, the source read at whatever alignment that leaves it (ld16u), then the tail
    size_t head = (16u - (unsigned)((uintptr_t)dst & 15u)) & 15u;
    if (head > nb) head = nb;
    const size_t nvec = (nb - head) / 16;
    u32x4* dv = (u32x4*)(dst + head);
    const uint8_t* sv = src + head;
    const size_t v0 = tile0 * kThreads + tid;
    if (v0 + (size_t)(U - 1) * kXcds * kThreads < nvec) {
      u32x4 xv[U];
#pragma unroll
      for (int j = 0; j < U; ++j) xv[j] = ld16u<NTL>(sv + (v0 + (size_t)j * kXcds * kThreads) * 16);
#pragma unroll
      for (int j = 0; j < U; ++j) st16<NTS>(dv + v0 + (size_t)j * kXcds * kThreads, xv[j]);
    } else {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = v0 + (size_t)j * kXcds * kThreads;
        if (v < nvec) st16<NTS>(dv + v, ld16u<NTL>(sv + v * 16));
      }
    }
    if (tile0 == 0) {   // at most 15 bytes on either side of the body
      if (tid < head) dst[tid] = src[tid];
      const size_t done = head + nvec * 16;
      if (tid >= 64 && done + (tid - 64) < nb) dst[done + (tid - 64)] = src[done + (tid - 64)];
    }
  }
}

// dst[c][r][0:m] = src[r][c][0:m] (bytes): the 2-D block transpose.
template <int U, bool NTL, bool NTS>
__global__ __launch_bounds__(kThreads) void k_block_transpose(uint8_t* dst, const uint8_t* src,
                                                              size_t rows, size_t cols, size_t m,
                                                              size_t tiles_per_seg, int aligned, Span span) {
  const uint32_t tps = (uint32_t)tiles_per_seg;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t blk32 = w / tps;                  // destination block index c*rows + r
    const size_t tile = w - blk32 * tps;
    const size_t blk = blk32;
    const size_t c = blk32 / (uint32_t)rows, r = blk - c * rows;
    copy_tile<U, NTL, NTS>(dst + blk * m, src + (r * cols + c) * m, m, tile, aligned != 0);
  }
}

// Streaming probes: what this device sustains for a pure read and a pure
// write stream with the same access shape as the kernels above.  The read
// probe folds its data with xor and stores only if the result hits a value
// that zero-filled or random buffers never produce, so the loads stay live.
template <int U, bool NTL, int T = kThreads>
__global__ __launch_bounds__(T) void k_probe_read(const u32x4* src, u32x4* sink, size_t nvec) {
  const size_t base = (size_t)blockIdx.x * (T * U) + threadIdx.x;
  u32x4 x[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const size_t v = base + (size_t)j * T;
    x[j] = v < nvec ? ld16<NTL>(src + v) : u32x4{0, 0, 0, 0};
  }
  u32x4 acc = x[0];
#pragma unroll
  for (int j = 1; j < U; ++j) acc ^= x[j];
  if (acc.x == 0x9e3779b9u && acc.y == 0x7f4a7c15u && acc.z == 0xf39cc060u && acc.w == 0x5cedc834u)
    sink[threadIdx.x] = acc;
}

template <int U, bool NTS, int T = kThreads>
__global__ __launch_bounds__(T) void k_probe_write(u32x4* dst, size_t nvec, uint32_t value) {
  const size_t base = (size_t)blockIdx.x * (T * U) + threadIdx.x;
  const u32x4 v4 = {value, value, value, value};
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const size_t v = base + (size_t)j * T;
    if (v < nvec) st16<NTS>(dst + v, v4);
  }
}

struct MixArgs {
  const void* rd[kMaxSeg];
  void* wr[kMaxSeg];
};

// nr read streams and nw write streams of nvec vectors each in one launch, with
// no data flowing from the loads to the stores: what the device sustains for a
// given read:write mix when nothing but the memory system is in the way.
//   shape 0: workgroup t loads tile t of every read stream and stores tile t of
//            every write stream (the access shape of the add and fold kernels);
//   shape 1: every workgroup serves ONE stream: workgroup w tile w / (nr + nw)
//            of stream w % (nr + nw);
//   shapes 2 and 3: the same two with one-wave workgroups (T = 64).
// Loads are folded with xor and stored only on a value random data never hits.
template <int U, bool NTL, bool NTS, int T = kThreads>
__global__ __launch_bounds__(T) void k_probe_mix(MixArgs t, int nr, int nw, size_t nvec, int shape,
                                                       uint32_t value) {
  const u32x4 v4 = {value, value, value, value};
  u32x4 acc = {0, 0, 0, 0};
  if ((shape & 1) == 0) {
    const size_t base = (size_t)blockIdx.x * (T * U) + threadIdx.x;
    for (int q = 0; q < nr; ++q) {
      u32x4 x[U];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = base + (size_t)j * T;
        x[j] = v < nvec ? ld16<NTL>((const u32x4*)t.rd[q] + v) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int j = 0; j < U; ++j) acc ^= x[j];
    }
    for (int q = 0; q < nw; ++q) {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = base + (size_t)j * T;
        if (v < nvec) st16<NTS>((u32x4*)t.wr[q] + v, v4);
      }
    }
  } else {
    const unsigned streams = (unsigned)(nr + nw);
    const unsigned sidx = blockIdx.x % streams;
    const size_t base = (size_t)(blockIdx.x / streams) * (T * U) + threadIdx.x;
    if (sidx < (unsigned)nr) {
      u32x4 x[U];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = base + (size_t)j * T;
        x[j] = v < nvec ? ld16<NTL>((const u32x4*)t.rd[sidx] + v) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int j = 0; j < U; ++j) acc ^= x[j];
    } else {
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const size_t v = base + (size_t)j * T;
        if (v < nvec) st16<NTS>((u32x4*)t.wr[sidx - nr] + v, v4);
      }
    }
  }
  if (nw > 0 && acc.x == 0x9e3779b9u && acc.y == 0x7f4a7c15u && acc.z == 0xf39cc060u && acc.w == 0x5cedc834u)
    ((u32x4*)t.wr[0])[threadIdx.x] = acc;
}

struct KwayArgs {
  const void* shard[kMaxSeg];
  void* out[kMaxSeg];
  size_t eoff[kMaxSeg];   // element offset into every shard, per output
};

// S(M, H) of the halving butterfly over K leaves v[m] = shard[first ^ m]:
// S(M, K) = v[M];  S(M, H) = S(M, 2H) + S(M + H, 2H);  the result is S(0, 1).
// Unfolding v[m] += v[m+h] for h = K/2 .. 1 gives exactly this tree.  Every
// index is a template constant, so partial sums live in registers.
template <class Acc, int K, int M, int H, int L, class Load>
__device__ __forceinline__ void tree_sum(Load& load, int first, float* out) {
  if constexpr (H == K) {
    load(first ^ M, out);
  } else {
    float lo[L], hi[L];
    tree_sum<Acc, K, M, 2 * H, L>(load, first, lo);
    tree_sum<Acc, K, M + H, 2 * H, L>(load, first, hi);
#if defined(__HIP_DEVICE_COMPILE__)
    // Eight and sixteen shards: the two leaves of a pair are loaded together, ahead of their
    // add, and the next pair is not loaded before this one is summed (the sum must
    // exist at the second fence: an empty asm takes it as operand): two loads in
    // flight per wave, as in the ring order.  Left alone, the scheduler issues 6 of
    // the 8 loads up front for the 16-bit types and sinks every fp32 load down to
    // its add (an asm statement); both measured 4-6 % slower on MI355X (sixteen
    // shards: 2 % slower as subtrees side by side, see tree_vec).  Four shards
    // measured the same or slower with the fences and stay without; 32 and 64
    // shards are faster as subtrees side by side.
    if constexpr (2 * H == K && (K == 8 || K == 16)) __builtin_amdgcn_sched_barrier(0);
#endif
    Acc::template join_lanes<L>(lo, hi);
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (2 * H == K && (K == 8 || K == 16)) {
#pragma unroll
      for (int l = 0; l < L; ++l) asm volatile("" : "+v"(lo[l]));
      __builtin_amdgcn_sched_barrier(0);
    }
#endif
#pragma unroll
    for (int l = 0; l < L; ++l) out[l] = lo[l];
  }
}

// The same butterfly on whole vectors, G subtrees side by side: vec[r] holds
// S(r, G), the sum over the leaves m = r (mod G), so a leaf of this tree is the
// group of G adjacent operands G*b .. G*b+G-1 and load(b, vec) fetches all G.
// Depth first, a single subtree reads its operands in bit-reversed order
// (0, K/2, K/4, 3K/4, ...): consecutive loads lie half the operand range apart,
// which costs 10-15 % of the bandwidth on MI355X (same k and data in natural
// order: 6.5 TB/s, bit-reversed: 5.6; groups of 4-8 adjacent operands in
// bit-reversed group order: 6.3-6.6).  The caller finishes with the last
// log2 G levels, vec[r] += vec[r + h] for h = G/2 .. 1.
template <class Acc, int KG, int M, int H, int G, class Load>
__device__ __forceinline__ void tree_vec(Load& load, u32x4* out) {
  if constexpr (H == KG) {
    load(M, out);
  } else {
    u32x4 lo[G], hi[G];
    tree_vec<Acc, KG, M, 2 * H, G>(load, lo);
    tree_vec<Acc, KG, M + H, 2 * H, G>(load, hi);
#if defined(__HIP_DEVICE_COMPILE__)
    // 64 fp32 shards: both leaf groups are loaded ahead of their adds.  The fp32
    // add is an asm statement, and the scheduler otherwise sinks each load down to
    // its add: one load in flight, 0.70 of the peak on MI355X against 0.80 with the
    // fence.  The 16-bit types do not need it, and 16 and 32 shards measured 4-6 %
    // slower with it, whatever the type.
    if constexpr (2 * H == KG && KG >= 8 && Acc::kAsmAdd) __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
    for (int r = 0; r < G; ++r) out[r] = Acc::add_vec(lo[r], hi[r]);
#if defined(__HIP_DEVICE_COMPILE__)
    // After every pair of leaf groups: the sums must exist here (an empty asm
    // takes them as operands) and nothing moves across.  Left alone, the
    // scheduler issues all K loads first and sinks the adds to the end: every
    // loaded vector stays live (up to 256 VGPRs, one wave per SIMD).  With the
    // fence 2*G loads are in flight.
    if constexpr (2 * H == KG) {
#pragma unroll
      for (int r = 0; r < G; ++r) asm volatile("" : "+v"(out[r]));
      __builtin_amdgcn_sched_barrier(0);
    }
#endif
  }
}

// Subtrees evaluated side by side for a butterfly over K >= 32 operands (measured:
// 8 for K = 64 and 32; K = 8 and 16 are faster depth first with their leaves in pairs).
template <int K>
constexpr int tree_group() { return 8; }

// Left fold over `count` operands in cyclic order first, first+1, ...
// load(q, f) fills the L fp32 lanes of operand q; acc receives the result.
// Folds over kFoldPairedFrom or more operands issue their loads two at a time
// ahead of the adds, shorter ones one at a time: with the workgroups a CU holds,
// that keeps about as many bytes in flight as the memory system needs, and
// deeper batches measured slower on MI355X (the streams of the k shards then
// interleave more finely at the DRAM).
constexpr int kFoldBatch = 2;
constexpr int kFoldPairedFrom = 16;

template <class Acc, int L, int PF = kFoldPairedFrom, class Load>
__device__ __forceinline__ void ring_fold(Load&& load, int count, int first, float* acc) {
  int q = first;
  load(q, acc);
  int done = 1;
  if (count >= PF) {
    for (; done + kFoldBatch <= count; done += kFoldBatch) {
      float f[kFoldBatch][L];
#pragma unroll
      for (int i = 0; i < kFoldBatch; ++i) {
        q = q + 1 == count ? 0 : q + 1;
        load(q, f[i]);
      }
#if defined(__HIP_DEVICE_COMPILE__)
      // the loads of a batch are issued together, ahead of its adds: the fp32 add is
      // an asm statement (add_own_received), and the scheduler otherwise sinks each
      // load down to its add, which leaves one load in flight instead of two (-14 %)
      __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
      for (int i = 0; i < kFoldBatch; ++i) Acc::template hop_lanes<L>(acc, f[i]);
    }
  }
  for (; done < count; ++done) {
    q = q + 1 == count ? 0 : q + 1;
    float f[L];
    load(q, f);
    Acc::template hop_lanes<L>(acc, f);
  }
}

// Fold the k shards at one position in the order of a schedule.
//   K == 0 : ring order, runtime k (one level if g >= k, else two levels)
//   K >= 2 : halving order for k == K: leaves v[m] = shard[first ^ m] summed by
//            the butterfly v[m] += v[m+h], h = K/2 .. 1, evaluated depth first
//            by tree_sum (the same tree with only log2 K live partial sums).
template <class Acc, int K, int L, int PF = kFoldPairedFrom, class Load>
__device__ __forceinline__ void fold_shards(Load&& load, int k, int g, int first, int first_outer,
                                            float* acc) {
  if constexpr (K == 0) {
    if (g >= k) {
      ring_fold<Acc, L, PF>(load, k, first, acc);
    } else {
      // two-level ring: shards form k/g groups of g; every group is folded in
      // ring order from `first`, and the group sums are folded in ring order
      // from group `first_outer` (inner, then outer reduce_scatter of the 2-D
      // collective)
      const int groups = k / g;
      int go = first_outer;
      for (int og = 0; og < groups; ++og) {
        float part[L];
        ring_fold<Acc, L, PF>([&](int q, float* f) { load(go * g + q, f); }, g, first, part);
        if (og == 0) {
#pragma unroll
          for (int l = 0; l < L; ++l) acc[l] = part[l];
        } else {
          Acc::template hop_lanes<L>(acc, part);
        }
        go = go + 1 == groups ? 0 : go + 1;
      }
    }
  } else {
    tree_sum<Acc, K, 0, 1, L>(load, first, acc);
  }
}

// One 128-bit vector of one output: the fold over the k shards at byte offset
// wg_byte (uniform over the workgroup) + lane_byte, stored to dst.
template <class Acc, int K, bool NTL, bool NTS, int PF>
__device__ __forceinline__ void fold_vector(const KwayArgs& t, int k, int g, int first, int first_outer,
                                            size_t wg_byte, uint32_t lane_byte, u32x4* dst) {
  constexpr int L = Acc::kLanes;
  if constexpr (K >= 32 && Acc::kPacked) {
    constexpr int G = tree_group<K>();
    u32x4 part[G];
    auto group_load = [&](int b, u32x4* x) {
#pragma unroll
      for (int r = 0; r < G; ++r) {
        int q = first ^ (G * b + r);
#if defined(__HIP_DEVICE_COMPILE__)
        // ties the fetch of the shard pointer to this place: left alone, all K
        // pointers are fetched up front and spill out of the scalar registers
        asm volatile("" : "+s"(q));
#endif
        x[r] = ld16u<NTL>((const uint8_t*)t.shard[q] + wg_byte + lane_byte);
      }
    };
    tree_vec<Acc, K / G, 0, 1, G>(group_load, part);
#pragma unroll
    for (int h = G / 2; h >= 1; h /= 2) {
#pragma unroll
      for (int r = 0; r < h; ++r) part[r] = Acc::add_vec(part[r], part[r + h]);
    }
    st16<NTS>(dst, Acc::settle(part[0]));
  } else {
    float acc[L];
    fold_shards<Acc, K, L, PF>(
        [&](int q, float* f) {
          Acc::widen(ld16u<NTL>((const uint8_t*)t.shard[q] + wg_byte + lane_byte), f);
        },
        k, g, first, first_outer, acc);
    st16<NTS>(dst, Acc::narrow(acc));
  }
}

// Fused k-way reduce, one pass: output j = fold over the k shards of
// shard[.][eoff[j] + i], i < n, starting the schedule at shard
// (first0 + j) mod k (or, for the two-level ring, at the inner and outer
// successors of j).  Output and shards may start at any element alignment;
// the few elements around the vector body go one by one through the same fold.
template <class Acc, int K, int U, bool NTL, bool NTS, int T = kThreads, int PF = kFoldPairedFrom>
__global__ __launch_bounds__(T) void k_reduce_kway(KwayArgs t, int k, int g, int nout,
                                                          size_t n, int first0,
                                                          size_t tiles_per_seg, Span span) {
  typedef typename Acc::op Op;
  typedef typename Op::elem elem;
  const uint32_t tps = (uint32_t)tiles_per_seg;
  const unsigned tid = threadIdx.x;
  for (uint64_t w64 = (uint64_t)span.begin + blockIdx.x; w64 < span.end; w64 += gridDim.x) {
    const uint32_t w = (uint32_t)w64;
    const int j = (int)(w / tps);
    const size_t tile = w - (uint32_t)j * tps;
    // flat: the schedule of output j starts at shard (first0 + j) mod k;
    // two-level ring (g < k): inner start (j mod g) + 1, outer start (j / g) + 1
    const int first = g >= k ? (first0 + j) % k : (j % g + 1) % g;
    const int first_outer = g >= k ? 0 : (j / g + 1) % (k / g);
    const size_t eoff = t.eoff[j];
    elem* out = (elem*)t.out[j];

    // The elements up to the output's first 16-byte boundary (head) and those behind
    // its last whole vector (tail) go one by one, the body as aligned vector stores;
    // the shards are read at whatever element alignment that leaves them (ld16u).
    const unsigned mis = (unsigned)((uintptr_t)out & 15u);
    size_t head = (mis % sizeof(elem)) == 0 ? ((16u - mis) & 15u) / sizeof(elem) : n;
    if (head > n) head = n;
    const size_t nvec = (n - head) / Op::kPerVec;
    const size_t base = tile * (size_t)(T * U);

#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t v = base + (size_t)u * T + tid;
      // an address is a workgroup-uniform 64-bit base plus a 32-bit lane offset:
      // the unrolled folds then need no vector registers for their k addresses
      const size_t wg_byte = (eoff + head) * sizeof(elem) + (base + (size_t)u * T) * 16;
      const uint32_t lane_byte = tid * 16u;
      if (v < nvec)
        fold_vector<Acc, K, NTL, NTS, PF>(t, k, g, first, first_outer, wg_byte, lane_byte, (u32x4*)(out + head) + v);
    }

    // head and tail, by the first tile of the output
    const size_t body_end = head + nvec * Op::kPerVec;
    const size_t loose = tile == 0 ? head + (n - body_end) : 0;
    for (size_t e = tid; e < loose; e += T) {
      const size_t i = e < head ? e : body_end + (e - head);
      float acc1[1];
      fold_shards<Acc, K, 1>(
          [&](int q, float* f) {
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (K > 0) asm volatile("" : "+s"(q));   // fetch the pointer here, see group_load
#endif
            elem e = ((const elem*)t.shard[q] + eoff)[i];
            f[0] = Acc::widen1(e);
          },
          k, g, first, first_outer, acc1);
      out[i] = Acc::narrow1(acc1[0]);
    }
  }
}

// The same fold for the usual case -- every output, every shard and every
// element offset 16-byte aligned, n a whole number of vectors: one-wave
// workgroups on a 2-D grid (y = output, x = 1 KiB tile), nothing decoded by
// division and nothing peeled.
template <class Acc, int K, bool NTL, bool NTS, int PF>
__global__ __launch_bounds__(kRowThreads) void k_fold_rows(KwayArgs t, int k, int g, int first0, size_t nvec) {
  typedef typename Acc::op::elem elem;
  const int j = (int)blockIdx.y;
  const size_t tile_vec = (size_t)blockIdx.x * kRowThreads;
  if (tile_vec + threadIdx.x >= nvec) return;
  const int first = g >= k ? (first0 + j) % k : (j % g + 1) % g;
  const int first_outer = g >= k ? 0 : (j / g + 1) % (k / g);
  const size_t wg_byte = t.eoff[j] * sizeof(elem) + tile_vec * 16;
  fold_vector<Acc, K, NTL, NTS, PF>(t, k, g, first, first_outer, wg_byte, threadIdx.x * 16u,
                                    (u32x4*)t.out[j] + tile_vec + threadIdx.x);
}

}  // namespace pccl_kernels

#endif  // PCCL_KERNELS_H
