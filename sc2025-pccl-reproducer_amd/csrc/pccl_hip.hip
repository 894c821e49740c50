// libpccl_hip.so -- reduction and placement kernels of PCCL's collectives for
// gfx950 (MI355X), behind the C ABI declared in include/pccl_hip.h.
//
// Everything here is HBM-bandwidth bound (one add per 6-12 bytes, or a pure
// copy), so the kernels are organised around memory traffic only:
//   * every global access is a 128-bit load/store, consecutive lanes touch
//     consecutive 16-byte vectors (one wave instruction = 1 KiB contiguous);
//   * each thread issues all loads of its tile before the first use, so a
//     workgroup of 256 threads keeps 2*U*4 KiB of reads in flight (U = vectors
//     per thread and operand);
//   * a whole step of a schedule (all virtual ranks) is ONE launch: the
//     per-segment pointers travel in the kernel arguments, so nothing is
//     allocated or copied to the device to describe the step;
//   * workgroups walk the segments tile by tile in address order.
// No MFMA: there is no contraction anywhere on this path.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <type_traits>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "pccl_hip.h"

namespace {

// ---------------------------------------------------------------------------
// errors and tuning
// ---------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

// The status of a launch is what the launch call itself returns: hipGetLastError()
// would hand out (and clear) whatever an earlier, unrelated call of this thread
// left behind, and a caller's own check could eat ours.  The first failure of a
// call's launches is kept per thread until launch_status() reports it.
thread_local hipError_t t_launch_error = hipSuccess;

inline void note_launch(hipError_t e) {
  if (e != hipSuccess && t_launch_error == hipSuccess) t_launch_error = e;
}

int launch_status(const char* what) {
  const hipError_t e = t_launch_error;
  t_launch_error = hipSuccess;
  if (e != hipSuccess)
    return fail(PCCL_HIP_ELAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return PCCL_HIP_OK;
}

#ifndef PCCL_LAUNCH   // a host stand-in for the HIP runtime brings its own
template <class T> struct same_as { typedef T type; };
template <class... P>
hipError_t launch_kernel(void (*kernel)(P...), dim3 grid, dim3 block, unsigned lds, hipStream_t stream,
                         typename same_as<P>::type... args) {
  void* ptrs[] = {(void*)&args...};
  return hipLaunchKernel((const void*)kernel, grid, block, ptrs, lds, stream);
}
#define PCCL_LAUNCH(kernel, grid, block, lds, stream, ...) \
  note_launch(launch_kernel(kernel, grid, block, lds, stream, __VA_ARGS__))
#endif

std::atomic<long> g_grid_cap{0};
std::atomic<long> g_unroll{4};        // vectors per thread and operand, general add kernels
// Aligned contiguous adds go to the lean one-wave kernels (k_add_rows, k_rh_rows); 0 = always the general kernels
std::atomic<long> g_add_rows{1};
std::atomic<long> g_unroll_copy{2};   // ... copy kernels (two 4 KiB chunks per workgroup, 8 chunks apart: see copy_vec)
// Unused dynamic LDS requested per workgroup, only to bound how many workgroups
// share a CU (160 KiB of LDS): the fewer are resident, the narrower the address
// window the chip streams from at any moment.  0 = as many as fit (8).
std::atomic<long> g_lds_pad_copy{-1};  // copy kernels; -1 = chosen per launch (see copy_lds_pad)
std::atomic<long> g_lds_pad_kway{-1};  // fused reduce; -1 = chosen per launch (see launch_kway)
std::atomic<long> g_fold_rows{1};      // aligned folds of streams from HBM go to the lean kernel (k_fold_rows); 0 = always the general kernel
std::atomic<long> g_wg_kway{-1};       // threads per workgroup of the fused reduce: 64, 256, or -1 = 64 for streams from HBM
std::atomic<long> g_lds_pad_gather{-1}; // all_gather placement kernels; -1 = chosen per launch
std::atomic<long> g_gather_split{0};   // groups of outputs per shard tile in the multicast gather; 0 = four outputs a group
std::atomic<long> g_gather_nt{-1};     // non-temporal stores in the all_gather placement kernels (-1: by footprint, like nt_store)
std::atomic<long> g_unroll_gather{0};  // vectors per thread in the all_gather placement kernels; 0 = chosen per launch
std::atomic<long> g_gather_strip{-1};  // work items per XCD and strip of the time-blocked gather; 0 = the multicast kernel, -1 = chosen per launch
std::atomic<long> g_gather_strip_from{-1};  // shortest longest-shard (bytes) the time-blocked gather is chosen for when gather_strip = -1
std::atomic<unsigned long long> g_launches{0};   // kernel launches issued so far
// Non-temporal loads / stores: 1 = always, 0 = never, -1 = by the footprint of
// the call.  Data that fits the 256 MB Infinity Cache and the L2s is better left
// cacheable (the next step or call finds it there: a P=8 ring reduce_scatter of
// 16 MiB per rank runs 18 % faster, an accumulate of 64 MiB operands 6 %);
// streams beyond that are 10-12 % faster with the non-temporal hint.
std::atomic<long> g_nt_load{-1};
std::atomic<long> g_nt_store{-1};
constexpr size_t kStreamFrom = (size_t)288 << 20;   // 256 MiB Infinity Cache + 8 x 4 MiB L2
constexpr long kStripItems = 160;                   // work items per XCD and strip of the time-blocked gather
constexpr long kStripFrom = 2 << 20;                // ... chosen for shards of at least this many bytes

// Footprint of the collective being launched (inputs, work buffers and outputs of
// all ranks), set by the collective entry points; 0 inside a plain kernel call,
// where the traffic of the launch itself decides.
thread_local size_t t_call_bytes = 0;
struct CallBytes {
  size_t saved;
  explicit CallBytes(size_t bytes) : saved(t_call_bytes) { if (bytes > t_call_bytes) t_call_bytes = bytes; }
  ~CallBytes() { t_call_bytes = saved; }
};
bool stream_hint(long setting, size_t launch_bytes) {
  if (setting >= 0) return setting != 0;
  return (launch_bytes > t_call_bytes ? launch_bytes : t_call_bytes) >= kStreamFrom;
}

}  // namespace

#include "pccl_kernels.h"

namespace {

using namespace pccl_kernels;

// ---------------------------------------------------------------------------
// host side: launch geometry and dispatch over the tuning parameters
// ---------------------------------------------------------------------------
// Kernels count their work items (tiles) in 32 bits.
constexpr size_t kMaxWorkItems = 0xffffffffull;
constexpr int kMaxVirtualRanks = PCCL_HIP_MAX_VIRTUAL_RANKS;

int check_work_items(size_t segments, size_t tiles, const char* what) {
  if (tiles != 0 && segments > kMaxWorkItems / tiles)
    return fail(PCCL_HIP_EINVAL, "%s: %zu segments of %zu tiles exceed the 2^32 - 1 tiles of one launch", what,
                segments, tiles);
  return PCCL_HIP_OK;
}

unsigned grid_for(size_t total_tiles) {
  long cap = g_grid_cap.load(std::memory_order_relaxed);
  size_t g = total_tiles;
  if (cap > 0 && g > (size_t)cap) g = (size_t)cap;
  if (g > kMaxGrid) g = kMaxGrid;
  if (g == 0) g = 1;
  return (unsigned)g;
}

// One launch over the `items` work items of a schedule step: launch(span, grid).
// (Steps of the 256-thread add kernels used to go out as several launches of
// bounded size; with the one-wave kernels serving the aligned case that measured
// inside the run-to-run spread on MI355X and was dropped.)
template <class F>
void for_spans(size_t items, F&& launch) {
  if (items == 0) return;
  launch(Span{0u, (uint32_t)items}, grid_for(items));
  g_launches.fetch_add(1, std::memory_order_relaxed);
}

size_t tiles_for(size_t nbytes, int unroll, int threads = kThreads) {
  // one extra vector covers the shift of the body behind an unaligned head
  size_t nvec = nbytes / 16 + 2;
  size_t per = (size_t)threads * (size_t)unroll;
  return (nvec + per - 1) / per;
}

// Tiles of a copy: whole groups of kXcds, which share their chunks (copy_vec).
size_t copy_tiles_for(size_t nbytes, int unroll) {
  const size_t t = tiles_for(nbytes, unroll);
  return unroll > 1 ? (t + kXcds - 1) / kXcds * kXcds : t;
}

struct Tune {
  int unroll;
  bool ntl, nts;
  int threads;   // workgroup size of the add kernels
};

bool is16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// launch_bytes: what the launch moves (decides the non-temporal hints when the
// setting leaves them open).
Tune current_tune(bool copy, size_t launch_bytes) {
  Tune t;
  t.unroll = (int)(copy ? g_unroll_copy : g_unroll).load(std::memory_order_relaxed);
  t.threads = kThreads;
  t.ntl = stream_hint(g_nt_load.load(std::memory_order_relaxed), launch_bytes);
  t.nts = stream_hint(g_nt_store.load(std::memory_order_relaxed), launch_bytes);
  return t;
}

// Calls f.template operator()<U, NTL, NTS>() for the current tuning.
template <class F>
void with_tuning(const Tune& t, F&& f) {
#define PCCL_CASE(UV)                                                 \
  case UV:                                                            \
    if (t.ntl) {                                                      \
      if (t.nts) f.template operator()<UV, true, true>();             \
      else f.template operator()<UV, true, false>();                  \
    } else {                                                          \
      if (t.nts) f.template operator()<UV, false, true>();            \
      else f.template operator()<UV, false, false>();                 \
    }                                                                 \
    break;
  switch (t.unroll) {
    PCCL_CASE(1)
    PCCL_CASE(2)
    PCCL_CASE(8)
    default:
    PCCL_CASE(4)
  }
#undef PCCL_CASE
}

size_t esize_of(int dtype) {
  return dtype == PCCL_HIP_F32 ? 4 : (dtype == PCCL_HIP_BF16 || dtype == PCCL_HIP_F16) ? 2 : 0;
}

Pieces contiguous(size_t n) {
  Pieces pc{};
  pc.s1 = pc.s2 = 1;
  pc.len = n;
  return pc;
}

struct AddLaunch {
  const AddSegs* segs;
  int count, dtype;
  Pieces pc;
  size_t tiles;
  int aligned, threads;
  hipStream_t stream;
  template <int U, bool NTL, bool NTS, int T>
  void run() const {
    const unsigned lds = 0;
    for_spans((size_t)count * pc.s1 * pc.s2 * tiles, [&](Span span, unsigned grid) {
      if (dtype == PCCL_HIP_F32)
        PCCL_LAUNCH((k_add_segs<OpF32, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *segs, count, pc, tiles, aligned, span);
      else if (dtype == PCCL_HIP_BF16)
        PCCL_LAUNCH((k_add_segs<OpBF16, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *segs, count, pc, tiles, aligned, span);
      else
        PCCL_LAUNCH((k_add_segs<OpF16, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *segs, count, pc, tiles, aligned, span);
    });
  }
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    run<U, NTL, NTS, kThreads>();
  }
};

// The lean add for `count` contiguous, aligned segments of n elements.
void launch_add_rows(const AddSegs& segs, int count, size_t n, int dtype, const Tune& t, hipStream_t stream) {
  const size_t nvec = n * esize_of(dtype) / 16;
  const size_t tiles = (nvec + kRowThreads - 1) / kRowThreads;
  {
    const int row0 = 0;
    const uint32_t tile0 = 0;
#define PCCL_ROWS(OP, L, S) PCCL_LAUNCH((k_add_rows<OP, L, S>), dim3((unsigned)tiles, (unsigned)count), dim3(kRowThreads), 0, stream, segs, row0, nvec, tile0)
    if (dtype == PCCL_HIP_F32) {
      if (t.ntl) { if (t.nts) PCCL_ROWS(OpF32, true, true); else PCCL_ROWS(OpF32, true, false); }
      else { if (t.nts) PCCL_ROWS(OpF32, false, true); else PCCL_ROWS(OpF32, false, false); }
    } else if (dtype == PCCL_HIP_BF16) {
      if (t.ntl) { if (t.nts) PCCL_ROWS(OpBF16, true, true); else PCCL_ROWS(OpBF16, true, false); }
      else { if (t.nts) PCCL_ROWS(OpBF16, false, true); else PCCL_ROWS(OpBF16, false, false); }
    } else {
      if (t.ntl) { if (t.nts) PCCL_ROWS(OpF16, true, true); else PCCL_ROWS(OpF16, true, false); }
      else { if (t.nts) PCCL_ROWS(OpF16, false, true); else PCCL_ROWS(OpF16, false, false); }
    }
#undef PCCL_ROWS
    g_launches.fetch_add(1, std::memory_order_relaxed);
  }
}

// True if every piece of every operand starts on a 16-byte boundary and is a
// whole number of vectors: the kernels then skip all head/tail handling.
bool pieces_aligned(const Pieces& pc, size_t unit) {
  const size_t m = 16 / unit - 1;   // strides and length are in units of `unit` bytes
  auto ok = [&](size_t v) { return (v & m) == 0; };
  return ok(pc.len) && (pc.s1 < 2 || (ok(pc.d1) && ok(pc.a1) && ok(pc.b1))) &&
         (pc.s2 < 2 || (ok(pc.d2) && ok(pc.a2) && ok(pc.b2)));
}

int launch_add_pieces(const AddSegs& segs, int count, const Pieces& pc, int dtype, hipStream_t stream,
                      const char* what) {
  if (pc.len == 0 || count == 0 || pc.s1 == 0 || pc.s2 == 0) return PCCL_HIP_OK;
  Tune t = current_tune(false, 3 * (size_t)count * pc.s1 * pc.s2 * pc.len * esize_of(dtype));
  bool aligned = pieces_aligned(pc, esize_of(dtype));
  for (int s = 0; s < count && aligned; ++s) aligned = is16(segs.dst[s]) && is16(segs.a[s]) && is16(segs.b[s]);
  if (aligned && pc.s1 == 1 && pc.s2 == 1 && g_add_rows.load(std::memory_order_relaxed) &&
      pc.len * esize_of(dtype) / 16 <= (size_t)kMaxGrid * kRowThreads) {
    launch_add_rows(segs, count, pc.len, dtype, t, stream);
    return launch_status(what);
  }
  AddLaunch l{&segs, count, dtype, pc, tiles_for(pc.len * esize_of(dtype), t.unroll, t.threads), aligned ? 1 : 0,
              t.threads, stream};
  if (int rc = check_work_items((size_t)count * pc.s1 * pc.s2, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

int launch_add(const AddSegs& segs, int count, size_t n, int dtype, hipStream_t stream,
               const char* what) {
  return launch_add_pieces(segs, count, contiguous(n), dtype, stream, what);
}

// Unused LDS per workgroup of the copy kernels: six resident workgroups per CU
// instead of eight for copies that stream from HBM (+1-1.5 % on MI355X from
// 256 MiB per launch up); cache-sized copies keep all eight.
unsigned copy_lds_pad(size_t traffic) {
  const long pad = g_lds_pad_copy.load(std::memory_order_relaxed);
  if (pad >= 0) return (unsigned)pad;
  return stream_hint(-1, traffic) ? 24576u : 0u;
}

struct CopyLaunch {
  const CopySegs* segs;
  int count;
  size_t tiles;
  int aligned;
  size_t traffic;
  hipStream_t stream;
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    const unsigned lds = copy_lds_pad(traffic);
    for_spans((size_t)count * tiles, [&](Span span, unsigned grid) {
      PCCL_LAUNCH((k_copy_segs<U, NTL, NTS>), dim3(grid), dim3(kThreads), lds, stream, *segs, count, tiles, aligned, span);
    });
  }
};

int launch_copy(const CopySegs& segs, int count, hipStream_t stream, const char* what) {
  size_t longest = 0, total = 0;
  for (int s = 0; s < count; ++s) {
    longest = segs.nbytes[s] > longest ? segs.nbytes[s] : longest;
    total += segs.nbytes[s];
  }
  if (longest == 0 || count == 0) return PCCL_HIP_OK;
  Tune t = current_tune(true, 2 * total);
  bool aligned = true;
  for (int s = 0; s < count && aligned; ++s)
    aligned = segs.nbytes[s] == 0 || (is16(segs.dst[s]) && is16(segs.src[s]) && (segs.nbytes[s] & 15u) == 0);
  CopyLaunch l{&segs, count, copy_tiles_for(longest, t.unroll), aligned ? 1 : 0, 2 * total, stream};
  if (int rc = check_work_items((size_t)count, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

struct CopyPiecesLaunch {
  const CopyPairs* segs;
  int count;
  Pieces pc;
  size_t tiles;
  int aligned;
  hipStream_t stream;
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    const unsigned lds = copy_lds_pad(2 * (size_t)count * pc.s1 * pc.s2 * pc.len);
    for_spans((size_t)count * pc.s1 * pc.s2 * tiles, [&](Span span, unsigned grid) {
      PCCL_LAUNCH((k_copy_pieces<U, NTL, NTS>), dim3(grid), dim3(kThreads), lds, stream, *segs, count, pc, tiles, aligned, span);
    });
  }
};

int launch_copy_pieces(const CopyPairs& segs, int count, const Pieces& pc, hipStream_t stream,
                       const char* what) {
  if (pc.len == 0 || count == 0 || pc.s1 == 0 || pc.s2 == 0) return PCCL_HIP_OK;
  Tune t = current_tune(true, 2 * (size_t)count * pc.s1 * pc.s2 * pc.len);
  Pieces chk = pc;
  chk.b1 = chk.b2 = 0;
  bool aligned = pieces_aligned(chk, 1);
  for (int s = 0; s < count && aligned; ++s) aligned = is16(segs.dst[s]) && is16(segs.src[s]);
  CopyPiecesLaunch l{&segs, count, pc, copy_tiles_for(pc.len, t.unroll), aligned ? 1 : 0, stream};
  if (int rc = check_work_items((size_t)count * pc.s1 * pc.s2, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

struct RhLaunch {
  const RhArgs* args;
  int P, round, dtype, from_src, to_outs;
  size_t B, tiles;
  int aligned, threads;
  hipStream_t stream;
  template <int U, bool NTL, bool NTS, int T>
  void run() const {
    const unsigned lds = 0;
    for_spans((size_t)P * tiles, [&](Span span, unsigned grid) {
      if (dtype == PCCL_HIP_F32)
        PCCL_LAUNCH((k_rh_round<OpF32, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *args, P, B, round, from_src, to_outs, tiles, aligned, span);
      else if (dtype == PCCL_HIP_BF16)
        PCCL_LAUNCH((k_rh_round<OpBF16, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *args, P, B, round, from_src, to_outs, tiles, aligned, span);
      else
        PCCL_LAUNCH((k_rh_round<OpF16, U, NTL, NTS, T>), dim3(grid), dim3(T), lds, stream, *args, P, B, round, from_src, to_outs, tiles, aligned, span);
    });
  }
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    run<U, NTL, NTS, kThreads>();
  }
};

struct GatherLaunch {
  const GatherArgs* args;
  int P, nout, split;
  size_t tiles;
  bool nt;
  unsigned lds_pad;
  hipStream_t stream;
  // Plain loads whatever the tuning says; the stores follow their own setting.
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    for_spans((size_t)P * tiles * (size_t)split, [&](Span span, unsigned grid) {
      if (nt)
        PCCL_LAUNCH((k_gather_multicast<U, false, true>), dim3(grid), dim3(kThreads), lds_pad, stream, *args, P, nout, tiles, split, span);
      else
        PCCL_LAUNCH((k_gather_multicast<U, false, false>), dim3(grid), dim3(kThreads), lds_pad, stream, *args, P, nout, tiles, split, span);
    });
  }
};

struct TransposeLaunch {
  uint8_t* dst;
  const uint8_t* src;
  size_t rows, cols, m, tiles;
  int aligned;
  hipStream_t stream;
  template <int U, bool NTL, bool NTS>
  void operator()() const {
    for_spans(rows * cols * tiles, [&](Span span, unsigned grid) {
      PCCL_LAUNCH((k_block_transpose<U, NTL, NTS>), dim3(grid), dim3(kThreads), 0, stream, dst, src, rows, cols, m, tiles, aligned, span);
    });
  }
};

// The fused reduce runs one vector per thread whatever the unroll setting:
// a thread already streams k shards, and measurements on MI355X show one
// vector per thread ahead of two by 5-10 % for k = 8 and k = 32.
struct KwayLaunch {
  const KwayArgs* args;
  int k, g, nout, dtype, order, first0, per_hop;
  size_t n, tiles;
  unsigned lds_pad;
  int threads;
  bool rows;
  hipStream_t stream;

  template <class Acc, int U, bool NTL, bool NTS, int T, int PF>
  void run_wg() const {
    static_assert(U == 1, "the fused reduce is launched with one vector per thread");
#define PCCL_KWAY(KV) \
  PCCL_LAUNCH((k_reduce_kway<Acc, KV, U, NTL, NTS, T, PF>), dim3(grid), dim3(T), lds_pad, stream, *args, k, g, nout, n, first0, tiles, span)
    for_spans((size_t)nout * tiles, [&](Span span, unsigned grid) {
      if (order == PCCL_HIP_ORDER_RING) { PCCL_KWAY(0); return; }
      switch (k) {
        case 2: PCCL_KWAY(2); break;
        case 4: PCCL_KWAY(4); break;
        case 8: PCCL_KWAY(8); break;
        case 16: PCCL_KWAY(16); break;
        case 32: PCCL_KWAY(32); break;
        default: PCCL_KWAY(64); break;
      }
    });
#undef PCCL_KWAY
  }

  // ring order; every output, shard and element offset 16-byte aligned, whole vectors: the lean kernel on a 2-D grid
  template <class Acc>
  void run_rows() const {
    const size_t nvec = n * sizeof(typename Acc::op::elem) / 16;
    const dim3 grid((unsigned)((nvec + kRowThreads - 1) / kRowThreads), (unsigned)nout);
    PCCL_LAUNCH((k_fold_rows<Acc, 0, true, true, 2>), grid, dim3(kRowThreads), lds_pad, stream, *args, k, g, first0, nvec);
    g_launches.fetch_add(1, std::memory_order_relaxed);
  }

  template <class Acc, int U, bool NTL, bool NTS>
  void run() const {
    if constexpr (NTL && NTS) {
      // streams from HBM: one-wave workgroups, ring-order loads in pairs whatever k, one launch
      if constexpr (!std::is_same<Acc, AccF16<true>>::value && !std::is_same<Acc, AccF16<false>>::value) {
        if (threads == kRowThreads && rows) { run_rows<Acc>(); return; }
      }
      if (threads == kRowThreads) { run_wg<Acc, U, NTL, NTS, kRowThreads, 2>(); return; }
    }
    run_wg<Acc, U, NTL, NTS, kThreads, kFoldPairedFrom>();
  }

  template <int U, bool NTL, bool NTS>
  void operator()() const {
    constexpr int UK = 1;
    if (dtype == PCCL_HIP_F32) run<AccF32, UK, NTL, NTS>();
    else if (dtype == PCCL_HIP_BF16 && per_hop) run<AccBF16<true>, UK, NTL, NTS>();
    else if (dtype == PCCL_HIP_BF16) run<AccBF16<false>, UK, NTL, NTS>();
    else if (per_hop) run<AccF16<true>, UK, NTL, NTS>();
    else run<AccF16<false>, UK, NTL, NTS>();
  }
};

// Unused LDS per workgroup of the fused reduce, chosen for a launch: it takes the
// room of further workgroups on a CU (160 KiB of LDS), and fewer resident waves
// narrow the window each of the k streams has in flight.  Only the one-wave
// workgroups that streams from HBM get are limited; operands that fit the caches
// (the footprint rule of the non-temporal hints) and 256-thread workgroups run
// at full occupancy.  6 KiB leave 26 waves on a CU, 7 KiB 22, 8 KiB 20, 9 KiB 17, 10 KiB 16,
// 11 KiB 14, 12 KiB 13; 32 without.  Measured on MI355X, ring order with loads in
// pairs, 512 MiB per rank, fraction of 8 TB/s at the best setting (and without a
// limit); up to 16 shards in the lean kernel, beyond in the general one:
//   bf16   2 shards 0.85 without (7 KiB: 0.79)    3: 0.85 at 7 KiB (0.80)
//          4: 0.87 at 7 KiB (0.80)                 5: 0.855 at 8 KiB (0.80)
//          6: 0.83 at 8 KiB (0.79)                 8: 0.835-0.85 at 8 KiB (0.78)
//         12: 0.82 at 8 KiB (0.76)                16: 0.82 at 9 KiB (0.76)
//         24: 0.80 at 9-10 KiB (0.75)             32: 0.80 at 9-10 KiB (0.76)
//         64: 0.785 at 8-9 KiB (0.76)
//   fp16   (general kernel) 4 shards 0.85 at 6 KiB, 8: 0.845 at 7 KiB (0.78), 16: 0.80 at 8 KiB
//   fp32   2 and 3 shards 0.83, 0.815 without (flat up to 10 KiB for 3)
//          4: 0.83 at 9-10 KiB (0.80)              5: 0.835 at 11 KiB (0.795)
//          6, 8: 0.845 at 11 KiB (0.785)          12, 16: 0.82 at 11 KiB (0.76)
//         24: 0.80 at 11 KiB (0.74)               32: 0.84 at 11-12 KiB (0.76)
//         64: 0.79 at 9-10 KiB (0.755)
// A setting one step off costs 1-4 %, two steps off 3-10 %.  The two-level ring
// order of the 2-D collectives issues its loads in chains of g shards (one inner
// group at a time), wants more waves for it, and follows g, fp32 like bf16: best
// settings 4x2 bf16 7 KiB (0.815; 0.77 at 8 KiB), 2x4 6 KiB (0.81; 0.69 at 8 KiB),
// 3x2 7 KiB, 4x4 7 KiB, 8x8 8 KiB, 16x4 9-10 KiB; fp32 2x4 6 KiB (0.83), 4x2 and
// 4x4 7 KiB (0.84, 0.81), 6x2 8 KiB, 8x8 8-10 KiB; fp16 4x2 and 4x4 6 KiB.  Halving
// order (butterfly in registers; 8 and 16 shards with their loads in pairs): 4 shards
// bf16 0.81 at 9-10 KiB, fp16 0.815 at 9 KiB, fp32 0.83 at 8 KiB (0.80 without);
// 8 shards bf16 0.84 and fp16 0.82 at 7 KiB, fp32 0.85 at 11 KiB (0.79); 16 fp32
// shards 0.84 at 11 KiB (0.77), 16 bf16 shards 0.81 at 9-11 KiB (0.76), 16 fp16 shards 0.80 at 8 KiB;
// 32 fp32 shards 0.83 at 11 KiB, 32 bf16 / fp16 shards 0.80 at 18 KiB (0.775 at 11 KiB);
// the kernels for 32 and 64 shards hold 105-182 registers per lane, which bounds a
// CU to 8-16 waves by itself (64 shards: the same at every setting).
long kway_lds_pad(int k, int g, int dtype, int order, size_t traffic, int threads) {
  if (threads != kRowThreads || !stream_hint(-1, traffic)) return 0;
  if (k <= 2) return 0;
  if (order != PCCL_HIP_ORDER_RING) {
    if (traffic < ((size_t)512 << 20)) return 0;   // not measured below
    if (k == 4) return dtype == PCCL_HIP_F32 ? 8192 : dtype == PCCL_HIP_F16 ? 9216 : 10240;
    if (k == 8) return dtype == PCCL_HIP_F32 ? 11264 : 7168;
    if (k == 16) return dtype == PCCL_HIP_F32 ? 11264 : dtype == PCCL_HIP_F16 ? 8192 : 9216;
    if (dtype != PCCL_HIP_F32 && k == 32) return 18432;
    return 11264;
  }
  const long by_type = dtype == PCCL_HIP_F16 ? -1024 : 0;
  if (g < k) {                           // two-level: 1 KiB per doubling of the inner group, rounded up
    int doublings = 0;
    while ((1 << doublings) < g) ++doublings;
    return 5120 + 1024 * (long)doublings + by_type;
  }
  if (dtype == PCCL_HIP_F32) {
    // the wide limits of fp32 cost 1-4 % on launches of 320 MiB over 4 or 8 shards and gain from 0.6 GiB on
    if (k <= 8 && traffic < ((size_t)512 << 20)) return 0;
    return k <= 3 ? 0 : k == 4 ? 9216 : k <= 32 ? 11264 : 10240;
  }
  return (k <= 4 ? 7168 : k < 16 ? 8192 : k < 32 ? 9216 : k == 32 ? 10240 : 9216) + by_type;
}

// g = size of the inner groups of a two-level ring order (g >= k: one level).
int launch_kway(const KwayArgs& args, int k, int g, int nout, size_t n, int dtype, int order,
                int first0, int per_hop, hipStream_t stream, const char* what) {
  if (n == 0 || nout == 0) return PCCL_HIP_OK;
  // an output at an address that is no multiple of its element size would leave the whole fold to the
  // element-wise path of one workgroup: refused instead
  for (int j = 0; j < nout; ++j)
    if ((uintptr_t)args.out[j] % esize_of(dtype))
      return fail(PCCL_HIP_EINVAL, "%s: output %d is not aligned to its element size (%zu bytes)", what, j, esize_of(dtype));
  const size_t traffic = ((size_t)k + 1) * n * esize_of(dtype) * (size_t)nout;
  const Tune tune = current_tune(false, traffic);
  long wg = g_wg_kway.load(std::memory_order_relaxed);
  if (wg < 0) wg = stream_hint(-1, traffic) ? kRowThreads : kThreads;
  if (!(tune.ntl && tune.nts)) wg = kThreads;   // the one-wave variant exists for non-temporal streams only
  long pad = g_lds_pad_kway.load(std::memory_order_relaxed);
  if (pad < 0) pad = kway_lds_pad(k, g, dtype, order, traffic, (int)wg);
  const size_t es = esize_of(dtype);
  // The lean kernel for what it measured faster for on MI355X: the flat ring order over up to 16 fp32 or bf16
  // shards (+2-3 % at 4-16 shards; 32 and 64 shards, the two-level ring and the butterfly -2...0 %, float16 -1 %).
  bool rows = wg == kRowThreads && g_fold_rows.load(std::memory_order_relaxed) && order == PCCL_HIP_ORDER_RING &&
              g >= k && k <= 16 && dtype != PCCL_HIP_F16 && (n * es) % 16 == 0 &&
              n * es / 16 <= (size_t)kMaxGrid * kRowThreads;
  for (int q = 0; rows && q < k; ++q) rows = (uintptr_t)args.shard[q] % 16 == 0;
  for (int j = 0; rows && j < nout; ++j) rows = (uintptr_t)args.out[j] % 16 == 0 && (args.eoff[j] * es) % 16 == 0;
  KwayLaunch l{&args, k, g, nout, dtype, order, first0, per_hop, n, tiles_for(n * esize_of(dtype), 1, (int)wg),
               (unsigned)pad, (int)wg, rows, stream};
  if (int rc = check_work_items((size_t)nout, l.tiles, what)) return rc;
  with_tuning(tune, l);
  return launch_status(what);
}

// A step over more segments than one launch's kernel arguments hold goes out
// as several launches; the segments of a step are hazard-free, so their order
// does not matter.
struct AddTriple { void* dst; const void* a; const void* b; };

// One entry per virtual rank: on the stack up to the ranks of one launch (so a
// collective over at most PCCL_HIP_MAX_RANKS ranks touches no heap either), on
// the host heap beyond.
template <class T>
class RankList {
 public:
  explicit RankList(size_t n) : n_(n), p_(small_) {
    if (n > (size_t)kMaxSeg) { big_.resize(n); p_ = big_.data(); }
  }
  RankList(const RankList&) = delete;
  RankList& operator=(const RankList&) = delete;
  T& operator[](size_t i) { return p_[i]; }
  const T& operator[](size_t i) const { return p_[i]; }
  size_t size() const { return n_; }
 private:
  size_t n_;
  T* p_;
  T small_[kMaxSeg];
  std::vector<T> big_;
};

int launch_add_list(const RankList<AddTriple>& list, size_t n, int dtype, hipStream_t stream,
                    const char* what) {
  for (size_t i0 = 0; i0 < list.size(); i0 += kMaxSeg) {
    const int cnt = (int)(list.size() - i0 < (size_t)kMaxSeg ? list.size() - i0 : (size_t)kMaxSeg);
    AddSegs segs;
    for (int s = 0; s < cnt; ++s) { segs.dst[s] = list[i0 + s].dst; segs.a[s] = list[i0 + s].a; segs.b[s] = list[i0 + s].b; }
    if (int rc = launch_add(segs, cnt, n, dtype, stream, what)) return rc;
  }
  return PCCL_HIP_OK;
}

struct CopyItem { void* dst; const void* src; size_t nbytes; };

int launch_copy_list(const RankList<CopyItem>& list, hipStream_t stream, const char* what) {
  for (size_t i0 = 0; i0 < list.size(); i0 += kMaxSeg) {
    const int cnt = (int)(list.size() - i0 < (size_t)kMaxSeg ? list.size() - i0 : (size_t)kMaxSeg);
    CopySegs segs;
    for (int s = 0; s < cnt; ++s) { segs.dst[s] = list[i0 + s].dst; segs.src[s] = list[i0 + s].src; segs.nbytes[s] = list[i0 + s].nbytes; }
    if (int rc = launch_copy(segs, cnt, stream, what)) return rc;
  }
  return PCCL_HIP_OK;
}

// ---------------------------------------------------------------------------
// overlap of the buffers of one call
// ---------------------------------------------------------------------------
// A collective reads some buffers (inputs) and writes others (outputs, work
// space).  Readers may share memory among themselves; a written buffer may
// share memory with nothing, with ONE exception per rank that the kernels
// handle element by element (every element is read by the thread that
// overwrites it, and by no other): the in-place use the reference allows
// because it copies first (pccl/src/reduce_scatter.cpp:119-123,
// pccl/src/all_gather.cpp:31-35) -- a reduce_scatter output that IS block r of
// rank r's input, an all_gather shard that IS block r of rank r's output.
struct Extent {
  uintptr_t lo, hi;   // [lo, hi)
  int rank;           // index within its table
  char kind;          // 'i' read only, 'o' output, 'w' work space
  bool in_place;      // this written buffer coincides with its rank's reader exactly where the kernels allow it
};

class ExtentList {
 public:
  void add(const void* p, size_t bytes, int rank, char kind, bool in_place = false) {
    if (!p || bytes == 0) return;
    Extent e{(uintptr_t)p, (uintptr_t)p + bytes, rank, kind, in_place};
    if (n_ < kSmall) small_[n_++] = e;
    else { if (big_.empty()) big_.assign(small_, small_ + n_); big_.push_back(e); ++n_; }
  }
  // 0 if the call's buffers overlap only where that is allowed, else EINVAL with a message naming two of them
  int check(const char* what) {
    Extent* v = big_.empty() ? small_ : big_.data();
    std::sort(v, v + n_, [](const Extent& a, const Extent& b) { return a.lo != b.lo ? a.lo < b.lo : a.kind < b.kind; });
    // sweep by start address; `topw` is the started writer that reaches farthest (writers
    // never overlap each other, so it is the only one that can still be open), `topr` and
    // `nextr` the two started readers that reach farthest: a writer may start inside ONE
    // reader, its partner, so no other reader may reach to where it starts
    const Extent* topw = nullptr;
    const Extent* topr = nullptr;
    const Extent* nextr = nullptr;
    for (size_t i = 0; i < n_; ++i) {
      const Extent& x = v[i];
      const bool xw = x.kind != 'i';
      if (topw && topw->hi > x.lo) {           // a writer is still open here
        const Extent& w = *topw;
        const bool ok = !xw && w.in_place && w.kind == 'o' && x.rank == w.rank && pairs(x, w);
        if (!ok) return clash(what, w, x);
      }
      if (xw && topr && topr->hi > x.lo) {     // a reader is still open where this writer starts
        const Extent& r = *topr;
        const bool ok = x.in_place && x.kind == 'o' && r.rank == x.rank && pairs(r, x);
        if (!ok) return clash(what, r, x);
        if (nextr && nextr->hi > x.lo) return clash(what, *nextr, x);
      }
      if (xw) {
        if (!topw || x.hi > topw->hi) topw = &x;
      } else if (!topr || x.hi > topr->hi) {
        nextr = topr; topr = &x;
      } else if (!nextr || x.hi > nextr->hi) {
        nextr = &x;
      }
    }
    return PCCL_HIP_OK;
  }

 private:
  // one of the two contains the other: the only shape an allowed pair has
  static bool pairs(const Extent& r, const Extent& w) {
    return (r.lo <= w.lo && w.hi <= r.hi) || (w.lo <= r.lo && r.hi <= w.hi);
  }
  static const char* name(char kind) { return kind == 'i' ? "inputs" : kind == 'o' ? "outputs" : "work"; }
  static int clash(const char* what, const Extent& a, const Extent& b) {
    return fail(PCCL_HIP_EINVAL,
                "%s: %s[%d] and %s[%d] overlap in memory (a written buffer may share memory with nothing, except "
                "outputs[r] being exactly block r of inputs[r] in a reduce_scatter, or inputs[r] being exactly block r "
                "of outputs[r] in an all_gather)",
                what, name(a.kind), a.rank, name(b.kind), b.rank);
  }
  static constexpr size_t kSmall = 3 * (size_t)PCCL_HIP_MAX_RANKS;
  Extent small_[kSmall];
  std::vector<Extent> big_;
  size_t n_ = 0;
};

// two buffers of `bytes` bytes that share memory without being the same buffer
bool partly_overlap(const void* p, const void* q, size_t bytes) {
  const uintptr_t a = (uintptr_t)p, b = (uintptr_t)q;
  return a != b && a < b + bytes && b < a + bytes;
}

bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

int check_table(const void* const* tab, int count, const char* what, const char* name) {
  if (!tab) return fail(PCCL_HIP_EINVAL, "%s: %s is NULL", what, name);
  for (int i = 0; i < count; ++i)
    if (!tab[i]) return fail(PCCL_HIP_EINVAL, "%s: %s[%d] is NULL", what, name, i);
  return PCCL_HIP_OK;
}

int check_dtype(int dtype, const char* what) {
  if (esize_of(dtype) == 0)
    return fail(PCCL_HIP_EINVAL, "%s: unknown dtype %d (0 = float32, 1 = bfloat16, 2 = float16)", what, dtype);
  return PCCL_HIP_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" {

int pccl_hip_version(void) { return PCCL_HIP_ABI_VERSION; }

const char* pccl_hip_last_error(void) { return g_err; }

size_t pccl_hip_dtype_size(int dtype) { return esize_of(dtype); }

int pccl_hip_set_tuning(const char* key, long value) {
  if (!key) return fail(PCCL_HIP_EINVAL, "set_tuning: key is NULL");
  if (!strcmp(key, "grid_cap")) {
    if (value < 0) return fail(PCCL_HIP_EINVAL, "set_tuning: grid_cap must be >= 0");
    g_grid_cap = value;
  } else if (!strcmp(key, "unroll")) {
    if (value != 1 && value != 2 && value != 4 && value != 8)
      return fail(PCCL_HIP_EINVAL, "set_tuning: unroll must be 1, 2, 4 or 8");
    g_unroll = value;
  } else if (!strcmp(key, "wg_kway")) {
    if (value != -1 && value != 64 && value != 256)
      return fail(PCCL_HIP_EINVAL, "set_tuning: wg_kway must be -1, 64 or 256");
    g_wg_kway = value;
  } else if (!strcmp(key, "add_rows")) {
    g_add_rows = value != 0;
  } else if (!strcmp(key, "fold_rows")) {
    g_fold_rows = value != 0;
  } else if (!strcmp(key, "unroll_copy")) {
    if (value != 1 && value != 2 && value != 4 && value != 8)
      return fail(PCCL_HIP_EINVAL, "set_tuning: unroll_copy must be 1, 2, 4 or 8");
    g_unroll_copy = value;
  } else if (!strcmp(key, "lds_pad_copy") || !strcmp(key, "lds_pad_kway")) {
    if (value < -1 || value > 65536)   // -1: the copies and the fused reduce pick per launch
      return fail(PCCL_HIP_EINVAL, "set_tuning: %s must be in [-1, 65536]", key);
    (!strcmp(key, "lds_pad_copy") ? g_lds_pad_copy : g_lds_pad_kway) = value;
  } else if (!strcmp(key, "lds_pad_gather")) {
    if (value < -1 || value > 65536) return fail(PCCL_HIP_EINVAL, "set_tuning: lds_pad_gather must be in [-1, 65536]");
    g_lds_pad_gather = value;
  } else if (!strcmp(key, "gather_split")) {
    if (value < 0 || value > kMaxSeg) return fail(PCCL_HIP_EINVAL, "set_tuning: gather_split must be in [0, %d]", kMaxSeg);
    g_gather_split = value;
  } else if (!strcmp(key, "gather_strip")) {
    if (value < -1 || value > 65536) return fail(PCCL_HIP_EINVAL, "set_tuning: gather_strip must be in [-1, 65536]");
    g_gather_strip = value;
  } else if (!strcmp(key, "gather_strip_from")) {
    g_gather_strip_from = value < 0 ? -1 : value;
  } else if (!strcmp(key, "unroll_gather")) {
    if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8)
      return fail(PCCL_HIP_EINVAL, "set_tuning: unroll_gather must be 0, 1, 2, 4 or 8");
    g_unroll_gather = value;
  } else if (!strcmp(key, "gather_nt") || !strcmp(key, "nt_load") || !strcmp(key, "nt_store")) {
    // -1: non-temporal for calls whose footprint exceeds the caches, 0: never, other: always
    const long v = value < 0 ? -1 : value != 0;
    (!strcmp(key, "gather_nt") ? g_gather_nt : !strcmp(key, "nt_load") ? g_nt_load : g_nt_store) = v;
  } else {
    return fail(PCCL_HIP_EINVAL, "set_tuning: unknown key '%s'", key);
  }
  return PCCL_HIP_OK;
}

unsigned long long pccl_hip_launch_count(void) { return g_launches.load(std::memory_order_relaxed); }

long pccl_hip_get_tuning(const char* key) {
  if (!key) return -1;
  if (!strcmp(key, "grid_cap")) return g_grid_cap;
  if (!strcmp(key, "unroll")) return g_unroll;
  if (!strcmp(key, "wg_kway")) return g_wg_kway;
  if (!strcmp(key, "add_rows")) return g_add_rows;
  if (!strcmp(key, "fold_rows")) return g_fold_rows;
  if (!strcmp(key, "unroll_copy")) return g_unroll_copy;
  if (!strcmp(key, "lds_pad_copy")) return g_lds_pad_copy;
  if (!strcmp(key, "lds_pad_kway")) return g_lds_pad_kway;
  if (!strcmp(key, "lds_pad_gather")) return g_lds_pad_gather;
  if (!strcmp(key, "gather_split")) return g_gather_split;
  if (!strcmp(key, "unroll_gather")) return g_unroll_gather;
  if (!strcmp(key, "gather_strip")) return g_gather_strip;
  if (!strcmp(key, "gather_strip_from")) return g_gather_strip_from;
  if (!strcmp(key, "gather_nt")) return g_gather_nt;
  if (!strcmp(key, "nt_load")) return g_nt_load;
  if (!strcmp(key, "nt_store")) return g_nt_store;
  return -1;
}

int pccl_hip_add(void* dst, const void* a, const void* b, size_t n, int dtype, void* stream) {
  const char* what = "pccl_hip_add";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (n == 0) return PCCL_HIP_OK;
  if (!dst || !a || !b) return fail(PCCL_HIP_EINVAL, "%s: NULL operand", what);
  if (partly_overlap(dst, a, n * esize_of(dtype)) || partly_overlap(dst, b, n * esize_of(dtype)))
    return fail(PCCL_HIP_EINVAL, "%s: dst may be a or b exactly, but overlaps one of them partly", what);
  AddSegs segs;
  segs.dst[0] = dst; segs.a[0] = a; segs.b[0] = b;
  return launch_add(segs, 1, n, dtype, (hipStream_t)stream, what);
}

int pccl_hip_accumulate(void* dst, const void* src, size_t n, int dtype, void* stream) {
  const char* what = "pccl_hip_accumulate";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (n == 0) return PCCL_HIP_OK;
  if (!dst || !src) return fail(PCCL_HIP_EINVAL, "%s: NULL operand", what);
  if (partly_overlap(dst, src, n * esize_of(dtype)))
    return fail(PCCL_HIP_EINVAL, "%s: src may be dst exactly, but overlaps it partly", what);
  AddSegs segs;
  segs.dst[0] = dst; segs.a[0] = dst; segs.b[0] = src;
  return launch_add(segs, 1, n, dtype, (hipStream_t)stream, what);
}

int pccl_hip_add_batched(void* const* dst, const void* const* a, const void* const* b, int count,
                         size_t n, int dtype, void* stream) {
  const char* what = "pccl_hip_add_batched";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (count < 0 || count > kMaxSeg)
    return fail(PCCL_HIP_EINVAL, "%s: count %d outside [0, %d]", what, count, kMaxSeg);
  if (count == 0 || n == 0) return PCCL_HIP_OK;
  if (int rc = check_table((const void* const*)dst, count, what, "dst")) return rc;
  if (int rc = check_table(a, count, what, "a")) return rc;
  if (int rc = check_table(b, count, what, "b")) return rc;
  AddSegs segs;
  for (int s = 0; s < count; ++s) { segs.dst[s] = dst[s]; segs.a[s] = a[s]; segs.b[s] = b[s]; }
  return launch_add(segs, count, n, dtype, (hipStream_t)stream, what);
}

int pccl_hip_rh_round(void* const* bufs, const void* const* src, void* const* outs, int P, size_t B,
                      int round, int dtype, void* stream) {
  const char* what = "pccl_hip_rh_round";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (P < 2 || P > kMaxSeg || !pow2(P))
    return fail(PCCL_HIP_EINVAL, "%s: P = %d must be a power of two in [2, %d]", what, P, kMaxSeg);
  int rounds = 0;
  while ((1 << rounds) < P) ++rounds;
  if (round < 0 || round >= rounds)
    return fail(PCCL_HIP_EINVAL, "%s: round %d outside [0, %d)", what, round, rounds);
  const bool last = round == rounds - 1;
  const bool to_outs = outs != nullptr && last;
  // the work buffers are needed unless this round reads the inputs and writes the outputs
  const bool need_bufs = !(src != nullptr && to_outs);
  if (need_bufs) if (int rc = check_table((const void* const*)bufs, P, what, "bufs")) return rc;
  if (src) if (int rc = check_table(src, P, what, "src")) return rc;
  if (to_outs) if (int rc = check_table((const void* const*)outs, P, what, "outs")) return rc;
  if (B == 0) return PCCL_HIP_OK;
  RhArgs args;
  for (int r = 0; r < P; ++r) {
    args.bufs[r] = need_bufs ? bufs[r] : nullptr;
    args.src[r] = src ? src[r] : nullptr;
    args.outs[r] = to_outs ? outs[r] : nullptr;
  }
  const size_t count = (size_t)((P >> round) / 2) * B;
  Tune t = current_tune(false, 3 * (size_t)P * count * esize_of(dtype));
  // block offsets are multiples of B elements, so B must be a whole number of vectors too
  bool aligned = (B * esize_of(dtype)) % 16 == 0;
  for (int r = 0; r < P && aligned; ++r)
    aligned = is16(args.bufs[r]) && is16(args.src[r]) && is16(args.outs[r]);
  if (aligned && g_add_rows.load(std::memory_order_relaxed) && count * esize_of(dtype) / 16 <= (size_t)kMaxGrid * kRowThreads) {
    const size_t nvec = count * esize_of(dtype) / 16;
    const size_t tiles = (nvec + kRowThreads - 1) / kRowThreads;
    int log2_group = 0;
    while ((1 << log2_group) < (P >> round)) ++log2_group;
    const int from_src = src ? 1 : 0, outs_i = to_outs ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    {
      const int row0 = 0;
      const uint32_t tile0 = 0;
#define PCCL_RH(OP, L, S) PCCL_LAUNCH((k_rh_rows<OP, L, S>), dim3((unsigned)tiles, (unsigned)P), dim3(kRowThreads), 0, st, args, row0, log2_group, B, from_src, outs_i, nvec, tile0)
      if (dtype == PCCL_HIP_F32) {
        if (t.ntl) { if (t.nts) PCCL_RH(OpF32, true, true); else PCCL_RH(OpF32, true, false); }
        else { if (t.nts) PCCL_RH(OpF32, false, true); else PCCL_RH(OpF32, false, false); }
      } else if (dtype == PCCL_HIP_BF16) {
        if (t.ntl) { if (t.nts) PCCL_RH(OpBF16, true, true); else PCCL_RH(OpBF16, true, false); }
        else { if (t.nts) PCCL_RH(OpBF16, false, true); else PCCL_RH(OpBF16, false, false); }
      } else {
        if (t.ntl) { if (t.nts) PCCL_RH(OpF16, true, true); else PCCL_RH(OpF16, true, false); }
        else { if (t.nts) PCCL_RH(OpF16, false, true); else PCCL_RH(OpF16, false, false); }
      }
#undef PCCL_RH
      g_launches.fetch_add(1, std::memory_order_relaxed);
    }
    return launch_status(what);
  }
  RhLaunch l{&args, P, round, dtype, src ? 1 : 0, to_outs ? 1 : 0, B,
             tiles_for(count * esize_of(dtype), t.unroll, t.threads), aligned ? 1 : 0, t.threads, (hipStream_t)stream};
  if (int rc = check_work_items((size_t)P, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

int pccl_hip_reduce_kway(void* out, const void* const* shards, int k, size_t n, int dtype,
                         int order, int first, int per_hop_round, void* stream) {
  const char* what = "pccl_hip_reduce_kway";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (k < 2 || k > kMaxSeg) return fail(PCCL_HIP_EINVAL, "%s: k = %d outside [2, %d]", what, k, kMaxSeg);
  if (order != PCCL_HIP_ORDER_RING && order != PCCL_HIP_ORDER_HALVING)
    return fail(PCCL_HIP_EINVAL, "%s: unknown order %d", what, order);
  if (order == PCCL_HIP_ORDER_HALVING && !pow2(k))
    return fail(PCCL_HIP_EINVAL, "%s: halving order needs k = %d to be a power of two", what, k);
  if (first < 0 || first >= k) return fail(PCCL_HIP_EINVAL, "%s: first = %d outside [0, %d)", what, first, k);
  if (n == 0) return PCCL_HIP_OK;
  if (!out) return fail(PCCL_HIP_EINVAL, "%s: out is NULL", what);
  if (int rc = check_table(shards, k, what, "shards")) return rc;
  {
    ExtentList ext;
    for (int q = 0; q < k; ++q) ext.add(shards[q], n * esize_of(dtype), q, 'i');
    ext.add(out, n * esize_of(dtype), 0, 'o');
    if (int rc = ext.check(what)) return rc;
  }
  KwayArgs args;
  for (int q = 0; q < k; ++q) args.shard[q] = shards[q];
  args.out[0] = out;
  args.eoff[0] = 0;
  return launch_kway(args, k, k, 1, n, dtype, order, first, per_hop_round, (hipStream_t)stream, what);
}

int pccl_hip_copy_batched(void* const* dst, const void* const* src, const size_t* nbytes, int count,
                          void* stream) {
  const char* what = "pccl_hip_copy_batched";
  if (count < 0 || count > kMaxSeg)
    return fail(PCCL_HIP_EINVAL, "%s: count %d outside [0, %d]", what, count, kMaxSeg);
  if (count == 0) return PCCL_HIP_OK;
  if (!nbytes) return fail(PCCL_HIP_EINVAL, "%s: nbytes is NULL", what);
  if (!dst || !src) return fail(PCCL_HIP_EINVAL, "%s: NULL pointer table", what);
  CopySegs segs;
  for (int s = 0; s < count; ++s) {
    if (nbytes[s] && (!dst[s] || !src[s]))
      return fail(PCCL_HIP_EINVAL, "%s: segment %d has a NULL pointer", what, s);
    segs.dst[s] = dst[s]; segs.src[s] = src[s]; segs.nbytes[s] = nbytes[s];
  }
  return launch_copy(segs, count, (hipStream_t)stream, what);
}

int pccl_hip_gather_place(void* out, const void* const* shards, const size_t* nbytes,
                          const size_t* dst_off, int P, void* stream) {
  const char* what = "pccl_hip_gather_place";
  if (P < 1 || P > kMaxSeg) return fail(PCCL_HIP_EINVAL, "%s: P = %d outside [1, %d]", what, P, kMaxSeg);
  if (!out || !shards || !nbytes || !dst_off) return fail(PCCL_HIP_EINVAL, "%s: NULL argument", what);
  CopySegs segs;
  for (int k = 0; k < P; ++k) {
    if (nbytes[k] && !shards[k]) return fail(PCCL_HIP_EINVAL, "%s: shards[%d] is NULL", what, k);
    segs.dst[k] = (uint8_t*)out + dst_off[k]; segs.src[k] = shards[k]; segs.nbytes[k] = nbytes[k];
  }
  return launch_copy(segs, P, (hipStream_t)stream, what);
}

int pccl_hip_block_transpose(void* dst, const void* src, size_t rows, size_t cols, size_t m_bytes,
                             void* stream) {
  const char* what = "pccl_hip_block_transpose";
  if (rows == 0 || cols == 0 || m_bytes == 0) return PCCL_HIP_OK;
  if (!dst || !src) return fail(PCCL_HIP_EINVAL, "%s: NULL operand", what);
  Tune t = current_tune(true, 2 * rows * cols * m_bytes);
  const bool aligned = is16(dst) && is16(src) && (m_bytes & 15u) == 0;
  TransposeLaunch l{(uint8_t*)dst, (const uint8_t*)src, rows, cols, m_bytes,
                    copy_tiles_for(m_bytes, t.unroll), aligned ? 1 : 0, (hipStream_t)stream};
  if (rows > kMaxWorkItems || cols > kMaxWorkItems / rows)
    return fail(PCCL_HIP_EINVAL, "%s: rows*cols too large", what);
  if (int rc = check_work_items(rows * cols, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

}  // extern "C"

namespace {

// Places `nshards` shards (shard k: nbytes[k] bytes at byte offset dst_off[k]) into
// each of `nout` outputs in one launch; both counts at most kMaxSeg.
int gather_place_all(void* const* outputs, int nout, const void* const* inputs, const size_t* nbytes,
                     const size_t* dst_off, int nshards, void* stream, const char* what) {
  const int P = nshards;
  GatherArgs args;
  size_t longest = 0, payload = 0;
  for (int r = 0; r < nout; ++r) args.outs[r] = outputs[r];
  for (int k = 0; k < P; ++k) {
    if (nbytes[k] && !inputs[k]) return fail(PCCL_HIP_EINVAL, "%s: inputs[%d] is NULL", what, k);
    args.ins[k] = inputs[k];
    args.nbytes[k] = nbytes[k]; args.dst_off[k] = dst_off[k];
    longest = nbytes[k] > longest ? nbytes[k] : longest;
    payload += nbytes[k];
  }
  if (longest == 0) return PCCL_HIP_OK;
  const size_t moved = ((size_t)nout + 1) * payload;   // every shard read, and written to nout outputs
  Tune t = current_tune(false, moved);
  // Two kernels.  Time-blocked strips (k_gather_strips): an XCD walks a strip of
  // its tiles once per output, so it feeds one write stream at a time and re-reads
  // the strip from its L2.  Measured on MI355X against the multicast kernel below
  // (shards of 8 ... 512 MiB, 4 ... 64 ranks): +9 ... +15 %; 16 shards of 128 MiB
  // 5.85 -> 6.75 TB/s.  Four tiles per workgroup (with one the kernel is bound by
  // the latency of its load, 5.4 TB/s); strips of 160 work items = 2.5 MiB per XCD
  // (beyond the 4 MiB of an L2 the re-reads miss: 3.7 TB/s); three workgroups per
  // CU (48 KiB of unused LDS each, +1 %).  A strip that divides the shard exactly
  // is 5-15 % slower than a longer one (the two outputs an XCD writes around a
  // change of output then lie a power of two apart); for shards shorter than a
  // strip, strips of twice their work items (every other slot an empty workgroup)
  // measured 2-5 % ahead of strips a quarter longer, three times are slower.
  long strip = g_gather_strip.load(std::memory_order_relaxed);
  if (strip < 0) {
    long from = g_gather_strip_from.load(std::memory_order_relaxed);
    if (from < 0) from = kStripFrom;
    strip = (nout >= 2 && longest >= (size_t)from) ? kStripItems : 0;
  }
  const long unroll_set = g_unroll_gather.load(std::memory_order_relaxed);
  const long pad_set = g_lds_pad_gather.load(std::memory_order_relaxed);
  t.unroll = unroll_set > 0 ? (int)unroll_set : strip > 0 ? 4 : 1;
  size_t n_local = 0;
  if (strip > 0) {
    // work items per shard and XCD, each t.unroll tiles; whole strips
    const size_t items = (tiles_for(longest, 1) + kXcds * t.unroll - 1) / (kXcds * t.unroll);
    const bool automatic = g_gather_strip.load(std::memory_order_relaxed) < 0;
    if (automatic && 2 * items + 1 < (size_t)strip) strip = (long)(2 * items + 1);
    n_local = (items + (size_t)strip - 1) / (size_t)strip * (size_t)strip;
    // one work item per (shard, output, XCD, item): beyond what a launch counts, the automatic choice
    // falls back to the multicast kernel, which needs 1/16 of the work items
    if (n_local > kMaxWorkItems / ((size_t)P * (size_t)nout * kXcds)) {
      if (!automatic) return check_work_items((size_t)P * (size_t)nout * kXcds, n_local, what);
      strip = 0;
      t.unroll = unroll_set > 0 ? (int)unroll_set : 1;
    }
  }
  const unsigned lds = (unsigned)(pad_set >= 0 ? pad_set : strip > 0 ? 49152 : 0);
  if (strip > 0) {
    const int U = t.unroll;
    const bool nts = stream_hint(g_gather_nt.load(), moved);
    hipStream_t st = (hipStream_t)stream;
#define PCCL_STRIPS(UV)                                                                                              \
  case UV:                                                                                                          \
    if (nts) PCCL_LAUNCH((k_gather_strips<UV, false, true>), dim3(grid), dim3(kThreads), lds, st, args, P, nout, (uint32_t)n_local, (uint32_t)strip, span); \
    else PCCL_LAUNCH((k_gather_strips<UV, false, false>), dim3(grid), dim3(kThreads), lds, st, args, P, nout, (uint32_t)n_local, (uint32_t)strip, span);    \
    break;
    for_spans((size_t)P * (size_t)nout * kXcds * n_local, [&](Span span, unsigned grid) {
      switch (U) {
        PCCL_STRIPS(1)
        PCCL_STRIPS(2)
        PCCL_STRIPS(8)
        default:
        PCCL_STRIPS(4)
      }
    });
#undef PCCL_STRIPS
    return launch_status(what);
  }
  // A workgroup holds one 4 KiB tile of a shard and stores it into four of the
  // P outputs; the P/4 workgroups of a tile are launched side by side, so all but
  // the first find the tile in cache.  Measured on MI355X against one workgroup
  // per tile storing to all P outputs: +9 % (P = 16, 128 MiB shards), +12 %
  // (P = 32), +15 % (P = 64); more than four streams per workgroup or more
  // workgroups per tile are both slower.
  int split = (int)g_gather_split.load(std::memory_order_relaxed);
  if (split <= 0) split = (nout + 3) / 4;
  if (split > nout) split = nout;
  GatherLaunch l{&args, P, nout, split, copy_tiles_for(longest, t.unroll), stream_hint(g_gather_nt.load(), moved),
                 lds, (hipStream_t)stream};
  if (int rc = check_work_items((size_t)P * (size_t)split, l.tiles, what)) return rc;
  with_tuning(t, l);
  return launch_status(what);
}

}  // namespace

extern "C" {

int pccl_hip_all_gather_uneven_virtual(void* const* outputs, const void* const* inputs,
                                       const size_t* nbytes, const size_t* dst_off, int P,
                                       void* stream) {
  const char* what = "pccl_hip_all_gather_uneven_virtual";
  if (P < 1 || P > kMaxVirtualRanks)
    return fail(PCCL_HIP_EINVAL, "%s: P = %d outside [1, %d]", what, P, kMaxVirtualRanks);
  if (!nbytes || !dst_off) return fail(PCCL_HIP_EINVAL, "%s: NULL size table", what);
  if (int rc = check_table((const void* const*)outputs, P, what, "outputs")) return rc;
  if (!inputs) return fail(PCCL_HIP_EINVAL, "%s: inputs is NULL", what);
  size_t total = 0, end = 0;
  for (int k = 0; k < P; ++k) {
    total += nbytes[k];
    if (nbytes[k] && dst_off[k] + nbytes[k] > end) end = dst_off[k] + nbytes[k];
  }
  {
    ExtentList ext;
    for (int k = 0; k < P; ++k) ext.add(inputs[k], nbytes[k], k, 'i');
    for (int k = 0; k < P; ++k)
      ext.add(outputs[k], end, k, 'o', nbytes[k] != 0 && inputs[k] == (const uint8_t*)outputs[k] + dst_off[k]);
    if (int rc = ext.check(what)) return rc;
  }
  CallBytes footprint(((size_t)P + 1) * total);   // P shards and P outputs holding all of them
  // one launch places up to kMaxSeg shards into up to kMaxSeg outputs
  for (int k0 = 0; k0 < P; k0 += kMaxSeg) {
    const int nk = P - k0 < kMaxSeg ? P - k0 : kMaxSeg;
    for (int r0 = 0; r0 < P; r0 += kMaxSeg) {
      const int nr = P - r0 < kMaxSeg ? P - r0 : kMaxSeg;
      if (int rc = gather_place_all(outputs + r0, nr, inputs + k0, nbytes + k0, dst_off + k0, nk, stream, what)) return rc;
    }
  }
  return PCCL_HIP_OK;
}

}  // extern "C"

namespace {

// The argument checks of a reduce_scatter over virtual ranks, before anything touches the device.
int check_reduce_scatter_args(void* const* outputs, const void* const* inputs, int P, int dtype,
                              const char* algorithm, int mode, const char* what) {
  if (int rc = check_dtype(dtype, what)) return rc;
  if (!algorithm) return fail(PCCL_HIP_EINVAL, "%s: algorithm is NULL", what);
  const bool ring = !strcmp(algorithm, "ring");
  const bool rec = !strcmp(algorithm, "recursive");
  if (!ring && !rec)
    return fail(PCCL_HIP_EINVAL, "Unknown algorithm specified for reduce_scatter_mpi: %s", algorithm);
  if (P < 1 || P > kMaxVirtualRanks)
    return fail(PCCL_HIP_EINVAL, "%s: P = %d outside [1, %d]", what, P, kMaxVirtualRanks);
  if (rec && !pow2(P))
    return fail(PCCL_HIP_EINVAL, "%s: recursive halving needs a power-of-two P, got %d", what, P);
  if (mode != PCCL_HIP_MODE_STEPS && mode != PCCL_HIP_MODE_FUSED && mode != PCCL_HIP_MODE_FAITHFUL)
    return fail(PCCL_HIP_EINVAL, "%s: unknown mode %d", what, mode);
  if (int rc = check_table((const void* const*)outputs, P, what, "outputs")) return rc;
  if (int rc = check_table(inputs, P, what, "inputs")) return rc;
  return PCCL_HIP_OK;
}

// reduce_scatter over P virtual ranks; `what` names the entry point in messages.
int reduce_scatter_ranks(void* const* outputs, const void* const* inputs, void* const* work, int P,
                         size_t B, int dtype, const char* algorithm, int mode, void* stream,
                         const char* what) {
  if (int rc = check_reduce_scatter_args(outputs, inputs, P, dtype, algorithm, mode, what)) return rc;
  const bool ring = !strcmp(algorithm, "ring");
  // beyond the shards of one launch the fused halving order runs its first rounds step by step (see below)
  const bool fused_rounds = mode == PCCL_HIP_MODE_FUSED && !ring && P > kMaxSeg;
  const bool need_work = (mode == PCCL_HIP_MODE_FAITHFUL && P > 1) || (mode == PCCL_HIP_MODE_STEPS && P > 2) ||
                         fused_rounds;
  if (need_work) if (int rc = check_table((const void* const*)work, P, what, "work")) return rc;
  if (B == 0) return PCCL_HIP_OK;
  hipStream_t st = (hipStream_t)stream;
  const size_t es = esize_of(dtype);
  {
    // In place (outputs[r] is block r of inputs[r]) every mode reads an element before the same thread
    // overwrites it, except the fused ring beyond the shards of one launch: its chain of launches keeps the
    // running sum in outputs[r] while block r of inputs[r] is still to come as the last operand.
    const bool chained = mode == PCCL_HIP_MODE_FUSED && ring && P > kMaxSeg;
    ExtentList ext;
    for (int r = 0; r < P; ++r) ext.add(inputs[r], (size_t)P * B * es, r, 'i');
    for (int r = 0; r < P; ++r)
      ext.add(outputs[r], B * es, r, 'o', !chained && outputs[r] == (const uint8_t*)inputs[r] + (size_t)r * B * es);
    if (need_work) for (int r = 0; r < P; ++r) ext.add(work[r], (size_t)P * B * es, r, 'w');
    if (int rc = ext.check(what)) return rc;
  }
  // inputs, the work buffers if the mode uses them, and the outputs
  CallBytes footprint(((need_work ? 2 : 1) * (size_t)P * P + P) * B * es);

  if (P == 1) {  // zero steps: the output is the input block
    CopySegs c;
    c.dst[0] = outputs[0]; c.src[0] = inputs[0]; c.nbytes[0] = B * es;
    return launch_copy(c, 1, st, what);
  }

  if (mode == PCCL_HIP_MODE_FUSED && P <= kMaxSeg) {
    KwayArgs args;
    for (int r = 0; r < P; ++r) { args.shard[r] = inputs[r]; args.out[r] = outputs[r]; args.eoff[r] = (size_t)r * B; }
    // ring: block j is folded from rank j+1 on; halving: the butterfly rooted at rank j
    return launch_kway(args, P, P, P, B, dtype, ring ? PCCL_HIP_ORDER_RING : PCCL_HIP_ORDER_HALVING,
                       ring ? 1 : 0, 1, st, what);
  }

  if (mode == PCCL_HIP_MODE_FUSED && ring) {
    // More ranks than one launch has shard pointers: the left fold of block j is cut
    // into launches of at most kMaxSeg operands, and every launch after the first
    // takes the running sum (already in output j) as its first operand.  A partial
    // sum is stored in the element type, which is what every hop rounds to anyway,
    // so the bits are those of the single fold.  One chain of launches per output.
    for (int j = 0; j < P; ++j) {
      int rank = (j + 1) % P;   // the fold of block j starts at rank j+1 and ends with rank j
      int left = P;
      bool running = false;
      while (left > 0) {
        KwayArgs args;
        int k = 0;
        if (running) args.shard[k++] = outputs[j];
        while (k < kMaxSeg && left > 0) {
          args.shard[k++] = (const uint8_t*)inputs[rank] + (size_t)j * B * es;
          rank = rank + 1 == P ? 0 : rank + 1;
          --left;
        }
        args.out[0] = outputs[j];
        args.eoff[0] = 0;
        if (int rc = launch_kway(args, k, k, 1, B, dtype, PCCL_HIP_ORDER_RING, 0, 1, st, what)) return rc;
        running = true;
      }
    }
    return PCCL_HIP_OK;
  }

  const bool faithful = mode == PCCL_HIP_MODE_FAITHFUL;
  RankList<CopyItem> copies((size_t)P);
  if (faithful) {  // buf <- input
    for (int r = 0; r < P; ++r) copies[r] = CopyItem{work[r], inputs[r], (size_t)P * B * es};
    if (int rc = launch_copy_list(copies, st, what)) return rc;
  }
  auto copy_out = [&]() {   // output <- buf[rank]
    for (int r = 0; r < P; ++r)
      copies[r] = CopyItem{outputs[r], (const uint8_t*)work[r] + (size_t)r * B * es, B * es};
    return launch_copy_list(copies, st, what);
  };
  RankList<AddTriple> adds((size_t)P);

  if (ring) {
    for (int step = 0; step < P - 1; ++step) {
      const bool first = step == 0, last = step == P - 2;
      for (int r = 0; r < P; ++r) {
        const int recv_idx = ((r - step - 2) % P + P) % P;
        const int source = (r - 1 + P) % P;
        const size_t off = (size_t)recv_idx * B * es;
        if (faithful) {
          adds[r].dst = (uint8_t*)work[r] + off;
          adds[r].a = adds[r].dst;
          adds[r].b = (const uint8_t*)work[source] + off;
        } else {
          // rank r's block recv_idx is still its input; the running sum of the
          // left neighbour is its input at step 0 and its work buffer after
          adds[r].a = (const uint8_t*)inputs[r] + off;
          adds[r].b = first ? (const uint8_t*)inputs[source] + off : (const uint8_t*)work[source] + off;
          adds[r].dst = last ? outputs[r] : (void*)((uint8_t*)work[r] + off);
        }
      }
      if (int rc = launch_add_list(adds, B, dtype, st, what)) return rc;
    }
    return faithful ? copy_out() : PCCL_HIP_OK;
  }

  // recursive halving
  int rounds = 0;
  while ((1 << rounds) < P) ++rounds;
  for (int round = 0; round < rounds; ++round) {
    if (fused_rounds && (P >> round) == kMaxSeg) {
      // The rest of the butterfly stays inside groups of kMaxSeg ranks whose partial
      // sums lie in the work buffers: one fused launch per group finishes it.
      for (int g0 = 0; g0 < P; g0 += kMaxSeg) {
        KwayArgs args;
        for (int q = 0; q < kMaxSeg; ++q) {
          args.shard[q] = work[g0 + q]; args.out[q] = outputs[g0 + q]; args.eoff[q] = (size_t)(g0 + q) * B;
        }
        if (int rc = launch_kway(args, kMaxSeg, kMaxSeg, kMaxSeg, B, dtype, PCCL_HIP_ORDER_HALVING, 0, 1, st, what))
          return rc;
      }
      return PCCL_HIP_OK;
    }
    const bool from_inputs = !faithful && round == 0;
    const bool to_outputs = !faithful && round == rounds - 1;
    if (P <= kMaxSeg) {   // the pairwise kernel finds partner and halves from (rank, round) itself
      if (int rc = pccl_hip_rh_round(work, from_inputs ? inputs : nullptr, to_outputs ? outputs : nullptr, P,
                                     B, round, dtype, stream))
        return rc;
      continue;
    }
    const int group = P >> round, half = group / 2;
    const size_t count = (size_t)half * B;
    for (int r = 0; r < P; ++r) {
      const bool lower = (r % group) < half;
      const int partner = lower ? r + half : r - half;
      const size_t off = ((size_t)(r / group) * group * B + (lower ? 0 : count)) * es;
      adds[r].a = from_inputs ? (const uint8_t*)inputs[r] + off : (const uint8_t*)work[r] + off;
      adds[r].b = from_inputs ? (const uint8_t*)inputs[partner] + off : (const uint8_t*)work[partner] + off;
      adds[r].dst = to_outputs ? outputs[r] : (void*)((uint8_t*)work[r] + off);
    }
    if (int rc = launch_add_list(adds, count, dtype, st, what)) return rc;
  }
  return faithful ? copy_out() : PCCL_HIP_OK;
}

// Work buffers of pccl_hip_reduce_scatter_virtual_noalloc: one array per GPU,
// part of the loaded code object, held until the process ends.  `scratch` is a
// host-side stand-in for the symbol; the address of a device's copy comes from
// hipGetSymbolAddress with that device current and is kept per device.
constexpr size_t kScratchBytes = PCCL_HIP_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int scratch_of_current_device(void** out, const char* what) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(PCCL_HIP_ENODEV, "%s: hipGetDevice failed: %s", what, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(PCCL_HIP_ENODEV, "%s: device index %d outside [0, %d)", what, dev, kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(PCCL_HIP_ENODEV, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", what, dev,
                  hipGetErrorString(e));
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // two threads racing here store the same address
  }
  *out = p;
  return PCCL_HIP_OK;
}

}  // namespace

extern "C" {

int pccl_hip_reduce_scatter_virtual(void* const* outputs, const void* const* inputs,
                                    void* const* work, int P, size_t B, int dtype,
                                    const char* algorithm, int mode, void* stream) {
  return reduce_scatter_ranks(outputs, inputs, work, P, B, dtype, algorithm, mode, stream,
                              "pccl_hip_reduce_scatter_virtual");
}

int pccl_hip_reduce_scatter_virtual_noalloc(void* const* outputs, const void* const* inputs, int P,
                                            size_t B, int dtype, const char* algorithm, void* stream) {
  const char* what = "pccl_hip_reduce_scatter_virtual_noalloc";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (P < 1 || P > kMaxSeg)
    return fail(PCCL_HIP_EINVAL, "%s: P = %d outside [1, %d]", what, P, kMaxSeg);
  // rank r works in scratch[r * slice, (r + 1) * slice), slice = P*B elements rounded up to 256 bytes
  const size_t es = esize_of(dtype);
  if (B > kScratchBytes / es / (size_t)P)
    return fail(PCCL_HIP_EINVAL, "%s: P = %d ranks of %zu elements need more than the %zu bytes of built-in scratch",
                what, P, B, kScratchBytes);
  const size_t slice = ((size_t)P * B * es + 255) / 256 * 256;
  if (slice * (size_t)P > kScratchBytes)
    return fail(PCCL_HIP_EINVAL,
                "%s: work buffers of %d ranks x %zu bytes exceed the %zu bytes of built-in scratch; "
                "use pccl_hip_reduce_scatter_virtual with caller-owned work buffers",
                what, P, slice, kScratchBytes);
  if (int rc = check_reduce_scatter_args(outputs, inputs, P, dtype, algorithm, PCCL_HIP_MODE_STEPS, what)) return rc;
  if (B == 0) return PCCL_HIP_OK;
  void* work[kMaxSeg];
  const bool need_work = P > 2;   // the per-step mode needs no work buffers for one or two ranks
  if (need_work) {
    void* base = nullptr;
    if (int rc = scratch_of_current_device(&base, what)) return rc;
    for (int r = 0; r < P; ++r) work[r] = (uint8_t*)base + (size_t)r * slice;
  }
  return reduce_scatter_ranks(outputs, inputs, need_work ? work : nullptr, P, B, dtype, algorithm,
                              PCCL_HIP_MODE_STEPS, stream, what);
}

int pccl_hip_all_gather_virtual(void* const* outputs, const void* const* inputs, int P,
                                size_t block_bytes, const char* algorithm, int mode, void* stream) {
  const char* what = "pccl_hip_all_gather_virtual";
  if (!algorithm) return fail(PCCL_HIP_EINVAL, "%s: algorithm is NULL", what);
  const bool ring = !strcmp(algorithm, "ring");
  const bool rec = !strcmp(algorithm, "recursive");
  if (!ring && !rec)
    return fail(PCCL_HIP_EINVAL, "Unknown algorithm specified for all_gather_mpi: %s", algorithm);
  if (P < 1 || P > kMaxVirtualRanks)
    return fail(PCCL_HIP_EINVAL, "%s: P = %d outside [1, %d]", what, P, kMaxVirtualRanks);
  if (rec && !pow2(P))
    return fail(PCCL_HIP_EINVAL, "%s: recursive doubling needs a power-of-two P, got %d", what, P);
  if (mode != PCCL_HIP_MODE_STEPS && mode != PCCL_HIP_MODE_FUSED && mode != PCCL_HIP_MODE_FAITHFUL)
    return fail(PCCL_HIP_EINVAL, "%s: unknown mode %d", what, mode);
  if (int rc = check_table((const void* const*)outputs, P, what, "outputs")) return rc;
  if (int rc = check_table(inputs, P, what, "inputs")) return rc;
  if (block_bytes == 0) return PCCL_HIP_OK;
  hipStream_t st = (hipStream_t)stream;
  {
    ExtentList ext;
    for (int r = 0; r < P; ++r) ext.add(inputs[r], block_bytes, r, 'i');
    for (int r = 0; r < P; ++r)
      ext.add(outputs[r], (size_t)P * block_bytes, r, 'o', inputs[r] == (const uint8_t*)outputs[r] + (size_t)r * block_bytes);
    if (int rc = ext.check(what)) return rc;
  }
  CallBytes footprint(((size_t)P * P + P) * block_bytes);   // P shards and P outputs of P blocks

  if (mode == PCCL_HIP_MODE_FUSED) {
    // one launch places up to kMaxSeg shards into up to kMaxSeg outputs
    size_t nbytes[kMaxSeg], off[kMaxSeg];
    for (int k0 = 0; k0 < P; k0 += kMaxSeg) {
      const int nk = P - k0 < kMaxSeg ? P - k0 : kMaxSeg;
      for (int k = 0; k < nk; ++k) { nbytes[k] = block_bytes; off[k] = (size_t)(k0 + k) * block_bytes; }
      for (int r0 = 0; r0 < P; r0 += kMaxSeg) {
        const int nr = P - r0 < kMaxSeg ? P - r0 : kMaxSeg;
        if (int rc = gather_place_all(outputs + r0, nr, inputs + k0, nbytes, off, nk, stream, what)) return rc;
      }
    }
    return PCCL_HIP_OK;
  }

  // out[r][r] <- in[r]   (pccl/src/all_gather.cpp:31-35)
  RankList<CopyItem> c((size_t)P);
  for (int r = 0; r < P; ++r)
    c[r] = CopyItem{(uint8_t*)outputs[r] + (size_t)r * block_bytes, inputs[r], block_bytes};
  if (int rc = launch_copy_list(c, st, what)) return rc;

  if (rec) {
    for (int seg = 1; seg < P; seg *= 2) {
      for (int r = 0; r < P; ++r) {
        const int partner = r ^ seg;
        const int group_start = (r / (2 * seg)) * (2 * seg);
        const size_t recv_off = (size_t)(r < partner ? group_start + seg : group_start) * block_bytes;
        // the partner's send offset equals this rank's receive offset
        c[r] = CopyItem{(uint8_t*)outputs[r] + recv_off, (const uint8_t*)outputs[partner] + recv_off,
                        (size_t)seg * block_bytes};
      }
      if (int rc = launch_copy_list(c, st, what)) return rc;
    }
    return PCCL_HIP_OK;
  }

  for (int step = 0; step < P - 1; ++step) {
    for (int r = 0; r < P; ++r) {
      const int j = ((r - step - 1) % P + P) % P;
      const int source = (r - 1 + P) % P;
      c[r] = CopyItem{(uint8_t*)outputs[r] + (size_t)j * block_bytes,
                      (const uint8_t*)outputs[source] + (size_t)j * block_bytes, block_bytes};
    }
    if (int rc = launch_copy_list(c, st, what)) return rc;
  }
  return PCCL_HIP_OK;
}

int pccl_hip_reduce_scatter_2d_virtual(void* const* outputs, const void* const* inputs,
                                       void* const* work, void* const* mid, int intra, int inter,
                                       size_t m, int dtype, const char* algorithm, int mode,
                                       void* stream) {
  const char* what = "pccl_hip_reduce_scatter_2d_virtual";
  if (int rc = check_dtype(dtype, what)) return rc;
  if (!algorithm) return fail(PCCL_HIP_EINVAL, "%s: algorithm is NULL", what);
  const bool ring = !strcmp(algorithm, "ring");
  const bool rec = !strcmp(algorithm, "recursive");
  if (!ring && !rec)
    return fail(PCCL_HIP_EINVAL, "Unknown algorithm specified for reduce_scatter_mpi: %s", algorithm);
  if (intra < 1 || inter < 1 || (long)intra * inter > kMaxVirtualRanks)
    return fail(PCCL_HIP_EINVAL, "%s: intra = %d, inter = %d: need intra, inter >= 1 and intra*inter <= %d",
                what, intra, inter, kMaxVirtualRanks);
  if (rec && (!pow2(intra) || !pow2(inter)))
    return fail(PCCL_HIP_EINVAL, "%s: recursive halving needs power-of-two group sizes, got %d x %d", what,
                intra, inter);
  if (mode != PCCL_HIP_MODE_STEPS && mode != PCCL_HIP_MODE_FUSED)
    return fail(PCCL_HIP_EINVAL, "%s: mode %d not offered here (steps or fused)", what, mode);
  const int W = intra * inter;
  // a grid beyond the shards of one launch is fused level by level: one fold per node, then one per local rank
  const bool fused = mode == PCCL_HIP_MODE_FUSED;
  const bool two_folds = fused && W > kMaxSeg;
  if (two_folds && (intra > kMaxSeg || inter > kMaxSeg))
    return fail(PCCL_HIP_EINVAL, "%s: the fused mode takes groups of at most %d ranks per level, got %d x %d (use the per-step mode)",
                what, kMaxSeg, intra, inter);
  if (int rc = check_table((const void* const*)outputs, W, what, "outputs")) return rc;
  if (int rc = check_table(inputs, W, what, "inputs")) return rc;
  const bool need_mid = (!fused || two_folds) && intra > 1 && inter > 1;
  const bool need_work = !fused && (intra > 2 || inter > 2);
  if (need_mid) if (int rc = check_table((const void* const*)mid, W, what, "mid")) return rc;
  if (need_work) if (int rc = check_table((const void* const*)work, W, what, "work")) return rc;
  if (m == 0) return PCCL_HIP_OK;
  hipStream_t st = (hipStream_t)stream;
  const size_t es = esize_of(dtype);
  {
    ExtentList ext;
    for (int w = 0; w < W; ++w) ext.add(inputs[w], (size_t)W * m * es, w, 'i');
    for (int w = 0; w < W; ++w)
      ext.add(outputs[w], m * es, w, 'o', outputs[w] == (const uint8_t*)inputs[w] + (size_t)w * m * es);
    if (need_work) for (int w = 0; w < W; ++w) ext.add(work[w], (size_t)W * m * es, w, 'w');
    if (need_mid) for (int w = 0; w < W; ++w) ext.add(mid[w], (size_t)inter * m * es, w, 'w');
    if (int rc = ext.check(what)) return rc;
  }
  // inputs of W*m elements per rank, as much work space in the per-step mode, the outputs
  CallBytes footprint(((fused ? 1 : 2) * (size_t)W * W + W) * m * es);
  auto at = [es](const void* p, size_t elems) { return (const void*)((const uint8_t*)p + elems * es); };
  auto atw = [es](void* p, size_t elems) { return (void*)((uint8_t*)p + elems * es); };

  if (W == 1) {
    CopySegs c;
    c.dst[0] = outputs[0]; c.src[0] = inputs[0]; c.nbytes[0] = m * es;
    return launch_copy(c, 1, st, what);
  }

  if (fused && !two_folds) {
    KwayArgs args;
    if (ring) {
      // world order; block w of every input; inner ring inside each node, then the ring across nodes
      for (int w = 0; w < W; ++w) { args.shard[w] = inputs[w]; args.out[w] = outputs[w]; args.eoff[w] = (size_t)w * m; }
      // (one rank per node, or one node: the flat ring, whose loads go out in pairs)
      return launch_kway(args, W, (inter == 1 || intra == 1) ? W : intra, W, m, dtype, PCCL_HIP_ORDER_RING, 1, 1, st, what);
    }
    // halving inside the node, then across nodes = ONE butterfly over the index
    // q = i*inter + j (inner bits above outer bits), rooted at the output's own q
    for (int j = 0; j < inter; ++j)
      for (int i = 0; i < intra; ++i) {
        const int w = j * intra + i, q = i * inter + j;
        args.shard[q] = inputs[w]; args.out[q] = outputs[w]; args.eoff[q] = (size_t)w * m;
      }
    return launch_kway(args, W, W, W, m, dtype, PCCL_HIP_ORDER_HALVING, 0, 1, st, what);
  }

  // result of the inner stage: [inter, m] per rank
  RankList<const void*> midr((size_t)W);
  RankList<void*> midw((size_t)W);
  for (int w = 0; w < W; ++w) {
    if (intra == 1) { midr[w] = inputs[w]; midw[w] = nullptr; }
    else if (inter == 1) { midr[w] = outputs[w]; midw[w] = outputs[w]; }
    else { midr[w] = mid[w]; midw[w] = mid[w]; }
  }
  const size_t B1 = (size_t)inter * m;   // inner block: one piece of m per node
  const int order = ring ? PCCL_HIP_ORDER_RING : PCCL_HIP_ORDER_HALVING;

  if (two_folds) {
    // Inner level, node by node: element (jj, i) of rank (j, i)'s intermediate is the fold, in the inner
    // schedule's order for local rank i, of block jj*intra + i of the node's `intra` inputs.  The outputs of
    // a launch are taken in the order o = jj*intra + i, whole rows of `intra` at a time, so that output o of
    // a launch starts its schedule at shard (first0 + o) mod intra as the flat collective does.
    if (intra > 1) {
      const int rows_per = kMaxSeg / intra;   // rows jj of one launch
      for (int j = 0; j < inter; ++j)
        for (int jj0 = 0; jj0 < inter; jj0 += rows_per) {
          const int rows = inter - jj0 < rows_per ? inter - jj0 : rows_per;
          KwayArgs args;
          for (int i = 0; i < intra; ++i) args.shard[i] = inputs[j * intra + i];
          for (int r = 0; r < rows; ++r)
            for (int i = 0; i < intra; ++i) {
              const int o = r * intra + i, jj = jj0 + r;
              args.out[o] = atw(midw[j * intra + i], (size_t)jj * m);
              args.eoff[o] = (size_t)(jj * intra + i) * m;
            }
          if (int rc = launch_kway(args, intra, intra, rows * intra, m, dtype, order, ring ? 1 : 0, 1, st, what)) return rc;
        }
    }
    // Outer level, local rank by local rank: a flat fused reduce_scatter over the `inter` intermediates.
    if (inter > 1) {
      for (int i = 0; i < intra; ++i) {
        KwayArgs args;
        for (int j = 0; j < inter; ++j) {
          args.shard[j] = midr[j * intra + i]; args.out[j] = outputs[j * intra + i]; args.eoff[j] = (size_t)j * m;
        }
        if (int rc = launch_kway(args, inter, inter, inter, m, dtype, order, ring ? 1 : 0, 1, st, what)) return rc;
      }
    }
    return PCCL_HIP_OK;
  }

  // per-step mode: one step of a level for ALL its groups is one launch per kMaxSeg ranks
  RankList<AddTriple> adds((size_t)W);
  auto launch_step = [&](const Pieces& pc) {
    for (int w0 = 0; w0 < W; w0 += kMaxSeg) {
      const int cnt = W - w0 < kMaxSeg ? W - w0 : kMaxSeg;
      AddSegs segs;
      for (int q = 0; q < cnt; ++q) { segs.dst[q] = adds[w0 + q].dst; segs.a[q] = adds[w0 + q].a; segs.b[q] = adds[w0 + q].b; }
      if (int rc = launch_add_pieces(segs, cnt, pc, dtype, st, what)) return rc;
    }
    return (int)PCCL_HIP_OK;
  };

  // ---- inner stage: groups of `intra` ranks, inputs read through the permutation ----
  if (intra > 1 && ring) {
    for (int s = 0; s < intra - 1; ++s) {
      const bool first = s == 0, last = s == intra - 2;
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i;
          const int b = ((i - s - 2) % intra + intra) % intra;
          const int src = j * intra + (i - 1 + intra) % intra;
          adds[w].a = at(inputs[w], (size_t)b * m);
          adds[w].b = first ? at(inputs[src], (size_t)b * m) : at(work[src], (size_t)b * B1);
          adds[w].dst = last ? midw[w] : atw(work[w], (size_t)b * B1);
        }
      Pieces pc{};
      pc.s1 = (unsigned)inter; pc.s2 = 1; pc.len = m;
      pc.a1 = (size_t)intra * m; pc.b1 = first ? (size_t)intra * m : m; pc.d1 = m;
      if (int rc = launch_step(pc)) return rc;
    }
  } else if (intra > 1) {
    int rounds = 0;
    while ((1 << rounds) < intra) ++rounds;
    for (int t = 0; t < rounds; ++t) {
      const int g = intra >> t, half = g / 2;
      const bool first = t == 0, last = t == rounds - 1;
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i;
          const bool lower = (i % g) < half;
          const int p = j * intra + (lower ? i + half : i - half);
          const size_t b0 = (size_t)(i / g) * g + (lower ? 0 : half);   // first block this rank keeps
          if (first) {
            adds[w].a = at(inputs[w], b0 * m);
            adds[w].b = at(inputs[p], b0 * m);
          } else {
            adds[w].a = at(work[w], b0 * B1);
            adds[w].b = at(work[p], b0 * B1);
          }
          adds[w].dst = last ? midw[w] : atw(work[w], b0 * B1);
        }
      Pieces pc{};
      if (first) {   // piece (node jj, block bb): strided in the input, contiguous rows in the work layout
        pc.s1 = (unsigned)inter; pc.s2 = (unsigned)half; pc.len = m;
        pc.a1 = pc.b1 = (size_t)intra * m; pc.a2 = pc.b2 = m;
        pc.d1 = m; pc.d2 = B1;
      } else {
        pc = contiguous((size_t)half * B1);
      }
      if (int rc = launch_step(pc)) return rc;
    }
  }

  // ---- outer stage: groups of `inter` ranks on the [inter, m] intermediates ----
  if (inter > 1 && ring) {
    for (int s = 0; s < inter - 1; ++s) {
      const bool first = s == 0, last = s == inter - 2;
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i;
          const int b = ((j - s - 2) % inter + inter) % inter;
          const int src = ((j - 1 + inter) % inter) * intra + i;
          adds[w].a = at(midr[w], (size_t)b * m);
          adds[w].b = first ? at(midr[src], (size_t)b * m) : at(work[src], (size_t)b * m);
          adds[w].dst = last ? outputs[w] : atw(work[w], (size_t)b * m);
        }
      if (int rc = launch_step(contiguous(m))) return rc;
    }
  } else if (inter > 1) {
    int rounds = 0;
    while ((1 << rounds) < inter) ++rounds;
    for (int t = 0; t < rounds; ++t) {
      const int g = inter >> t, half = g / 2;
      const bool first = t == 0, last = t == rounds - 1;
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i;
          const bool lower = (j % g) < half;
          const int p = (lower ? j + half : j - half) * intra + i;
          const size_t b0 = (size_t)(j / g) * g + (lower ? 0 : half);
          adds[w].a = first ? at(midr[w], b0 * m) : at(work[w], b0 * m);
          adds[w].b = first ? at(midr[p], b0 * m) : at(work[p], b0 * m);
          adds[w].dst = last ? outputs[w] : atw(work[w], b0 * m);
        }
      if (int rc = launch_step(contiguous((size_t)half * m))) return rc;
    }
  }
  return PCCL_HIP_OK;
}

int pccl_hip_all_gather_2d_virtual(void* const* outputs, const void* const* inputs, void* const* mid,
                                   int intra, int inter, size_t block_bytes, const char* algorithm,
                                   int mode, void* stream) {
  const char* what = "pccl_hip_all_gather_2d_virtual";
  if (!algorithm) return fail(PCCL_HIP_EINVAL, "%s: algorithm is NULL", what);
  const bool ring = !strcmp(algorithm, "ring");
  const bool rec = !strcmp(algorithm, "recursive");
  if (!ring && !rec)
    return fail(PCCL_HIP_EINVAL, "Unknown algorithm specified for all_gather_mpi: %s", algorithm);
  if (intra < 1 || inter < 1 || (long)intra * inter > kMaxVirtualRanks)
    return fail(PCCL_HIP_EINVAL, "%s: intra = %d, inter = %d: need intra, inter >= 1 and intra*inter <= %d",
                what, intra, inter, kMaxVirtualRanks);
  if (rec && (!pow2(intra) || !pow2(inter)))
    return fail(PCCL_HIP_EINVAL, "%s: recursive doubling needs power-of-two group sizes, got %d x %d", what,
                intra, inter);
  if (mode != PCCL_HIP_MODE_STEPS && mode != PCCL_HIP_MODE_FUSED)
    return fail(PCCL_HIP_EINVAL, "%s: mode %d not offered here (steps or fused)", what, mode);
  const int W = intra * inter;
  if (int rc = check_table((const void* const*)outputs, W, what, "outputs")) return rc;
  if (int rc = check_table(inputs, W, what, "inputs")) return rc;
  const size_t n = block_bytes;
  if (n == 0) return PCCL_HIP_OK;
  hipStream_t st = (hipStream_t)stream;
  {
    ExtentList ext;
    for (int w = 0; w < W; ++w) ext.add(inputs[w], n, w, 'i');
    for (int w = 0; w < W; ++w) ext.add(outputs[w], (size_t)W * n, w, 'o', inputs[w] == (const uint8_t*)outputs[w] + (size_t)w * n);
    if (mode == PCCL_HIP_MODE_STEPS && intra > 1 && inter > 1 && mid)
      for (int w = 0; w < W; ++w) ext.add(mid[w], (size_t)inter * n, w, 'w');
    if (int rc = ext.check(what)) return rc;
  }
  CallBytes footprint(((size_t)W * W + W) * n);   // W shards and W outputs of W blocks

  if (W == 1) {
    CopySegs one;
    one.dst[0] = outputs[0]; one.src[0] = inputs[0]; one.nbytes[0] = n;
    return launch_copy(one, 1, st, what);
  }

  if (mode == PCCL_HIP_MODE_FUSED) {   // the 2-D result is the concatenation in world order
    RankList<size_t> nbytes((size_t)W), off((size_t)W);
    for (int w = 0; w < W; ++w) { nbytes[w] = n; off[w] = (size_t)w * n; }
    return pccl_hip_all_gather_uneven_virtual(outputs, inputs, &nbytes[0], &off[0], W, stream);
  }

  const bool need_mid = intra > 1 && inter > 1;
  if (need_mid) if (int rc = check_table((const void* const*)mid, W, what, "mid")) return rc;
  // outer result per rank, [inter, n]; with one rank per node it IS the output
  RankList<uint8_t*> M((size_t)W);
  for (int w = 0; w < W; ++w)
    M[w] = inter == 1 ? (uint8_t*)inputs[w] : intra == 1 ? (uint8_t*)outputs[w] : (uint8_t*)mid[w];
  // one step of a level for ALL its groups: one launch per kMaxSeg ranks
  struct Pair { void* dst; const void* src; };
  RankList<Pair> c((size_t)W);
  auto launch_step = [&](const Pieces& pieces) {
    for (int w0 = 0; w0 < W; w0 += kMaxSeg) {
      const int cnt = W - w0 < kMaxSeg ? W - w0 : kMaxSeg;
      CopyPairs cp;
      for (int q = 0; q < cnt; ++q) { cp.dst[q] = c[w0 + q].dst; cp.src[q] = c[w0 + q].src; }
      if (int rc = launch_copy_pieces(cp, cnt, pieces, st, what)) return rc;
    }
    return (int)PCCL_HIP_OK;
  };

  // ---- outer stage: gather across nodes into M ----
  if (inter > 1) {
    for (int j = 0; j < inter; ++j)
      for (int i = 0; i < intra; ++i) { const int w = j * intra + i; c[w].dst = M[w] + (size_t)j * n; c[w].src = inputs[w]; }
    if (int rc = launch_step(contiguous(n))) return rc;
    if (rec) {
      for (int seg = 1; seg < inter; seg *= 2) {
        for (int j = 0; j < inter; ++j)
          for (int i = 0; i < intra; ++i) {
            const int w = j * intra + i, pj = j ^ seg, p = pj * intra + i;
            const int gs = (j / (2 * seg)) * (2 * seg);
            const size_t off = (size_t)(j < pj ? gs + seg : gs) * n;
            c[w].dst = M[w] + off; c[w].src = M[p] + off;
          }
        if (int rc = launch_step(contiguous((size_t)seg * n))) return rc;
      }
    } else {
      for (int s = 0; s < inter - 1; ++s) {
        for (int j = 0; j < inter; ++j)
          for (int i = 0; i < intra; ++i) {
            const int w = j * intra + i, src = ((j - 1 + inter) % inter) * intra + i;
            const size_t off = (size_t)(((j - s - 1) % inter + inter) % inter) * n;
            c[w].dst = M[w] + off; c[w].src = M[src] + off;
          }
        if (int rc = launch_step(contiguous(n))) return rc;
      }
    }
  }
  if (intra == 1) return PCCL_HIP_OK;

  // ---- inner stage: gather inside the node, written through the un-permutation:
  // inner block ii of the [intra, inter, n] layout is the pieces (jj*intra + ii)*n of the output ----
  Pieces pc{};
  pc.s1 = (unsigned)inter; pc.s2 = 1; pc.len = n; pc.d1 = (size_t)intra * n; pc.a1 = n;
  for (int j = 0; j < inter; ++j)
    for (int i = 0; i < intra; ++i) { const int w = j * intra + i; c[w].dst = (uint8_t*)outputs[w] + (size_t)i * n; c[w].src = M[w]; }
  if (int rc = launch_step(pc)) return rc;
  pc.a1 = (size_t)intra * n;   // from here on both sides are output layouts
  if (rec) {
    for (int seg = 1; seg < intra; seg *= 2) {
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i, pi = i ^ seg, p = j * intra + pi;
          const int gs = (i / (2 * seg)) * (2 * seg);
          const size_t off = (size_t)(i < pi ? gs + seg : gs) * n;
          c[w].dst = (uint8_t*)outputs[w] + off; c[w].src = (const uint8_t*)outputs[p] + off;
        }
      pc.len = (size_t)seg * n;
      if (int rc = launch_step(pc)) return rc;
    }
  } else {
    for (int s = 0; s < intra - 1; ++s) {
      for (int j = 0; j < inter; ++j)
        for (int i = 0; i < intra; ++i) {
          const int w = j * intra + i, src = j * intra + (i - 1 + intra) % intra;
          const size_t off = (size_t)(((i - s - 1) % intra + intra) % intra) * n;
          c[w].dst = (uint8_t*)outputs[w] + off; c[w].src = (const uint8_t*)outputs[src] + off;
        }
      pc.len = n;
      if (int rc = launch_step(pc)) return rc;
    }
  }
  return PCCL_HIP_OK;
}

int pccl_hip_probe_stream(int kind, void* buf, size_t nbytes, void* stream) {
  const char* what = "pccl_hip_probe_stream";
  if (kind != 0 && kind != 1) return fail(PCCL_HIP_EINVAL, "%s: kind must be 0 (read) or 1 (write)", what);
  if (nbytes < 16384) return fail(PCCL_HIP_EINVAL, "%s: buffer must hold at least 16384 bytes", what);
  if (!buf || ((uintptr_t)buf & 15u)) return fail(PCCL_HIP_EINVAL, "%s: buffer must be 16-byte aligned", what);
  const size_t nvec = nbytes / 16;
  // the shapes that sustain the most on MI355X: reads, workgroups of 1024 threads with one vector each
  // (7.5 TB/s over 2 GiB against 7.0 with 256 threads); writes, 256 threads with one vector each
  // (6.8 TB/s with 4 KiB per workgroup against 6.2 with 16 KiB)
  const size_t per_tile = kind == 0 ? 1024 : (size_t)kThreads;
  const size_t tiles = (nvec + per_tile - 1) / per_tile;
  if (tiles > kMaxGrid) return fail(PCCL_HIP_EINVAL, "%s: buffer too large", what);
  hipStream_t st = (hipStream_t)stream;
  if (kind == 0)
    PCCL_LAUNCH((k_probe_read<1, true, 1024>), dim3((unsigned)tiles), dim3(1024), 0, st,
                (const u32x4*)buf, (u32x4*)buf, nvec);
  else
    PCCL_LAUNCH((k_probe_write<1, false, kThreads>), dim3((unsigned)tiles), dim3(kThreads), 0, st, (u32x4*)buf, nvec,
                0x3f803f80u);
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return launch_status(what);
}

int pccl_hip_probe_mix(const void* const* reads, int nr, void* const* writes, int nw, size_t nbytes,
                       int shape, int vectors, void* stream) {
  const char* what = "pccl_hip_probe_mix";
  if (nr < 0 || nw < 0 || nr > kMaxSeg || nw > kMaxSeg || nr + nw < 1)
    return fail(PCCL_HIP_EINVAL, "%s: need 0 <= nr, nw <= %d and nr + nw >= 1", what, kMaxSeg);
  if (shape < 0 || shape > 3)
    return fail(PCCL_HIP_EINVAL, "%s: shape must be 0 (a workgroup serves all streams), 1 (one stream per workgroup), or 2 / 3 (the same with one-wave workgroups)", what);
  if (vectors != 1 && vectors != 2 && vectors != 4) return fail(PCCL_HIP_EINVAL, "%s: vectors per thread must be 1, 2 or 4", what);
  if (nbytes < 4096 || (nbytes & 15u)) return fail(PCCL_HIP_EINVAL, "%s: streams must hold a multiple of 16 and at least 4096 bytes", what);
  if (nr) if (int rc = check_table(reads, nr, what, "reads")) return rc;
  if (nw) if (int rc = check_table((const void* const*)writes, nw, what, "writes")) return rc;
  MixArgs args;
  for (int q = 0; q < nr; ++q) { if (!is16(reads[q])) return fail(PCCL_HIP_EINVAL, "%s: reads[%d] is not 16-byte aligned", what, q); args.rd[q] = reads[q]; }
  for (int q = 0; q < nw; ++q) { if (!is16(writes[q])) return fail(PCCL_HIP_EINVAL, "%s: writes[%d] is not 16-byte aligned", what, q); args.wr[q] = writes[q]; }
  const size_t nvec = nbytes / 16;
  const int threads = shape >= 2 ? kRowThreads : kThreads;
  const size_t per_tile = (size_t)threads * (size_t)vectors;
  size_t tiles = (nvec + per_tile - 1) / per_tile;
  if (shape & 1) tiles *= (size_t)(nr + nw);
  if (tiles > kMaxGrid) return fail(PCCL_HIP_EINVAL, "%s: streams too long for one launch", what);
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)tiles;
#define PCCL_MIX(UV, TV) PCCL_LAUNCH((k_probe_mix<UV, true, true, TV>), dim3(grid), dim3(TV), 0, st, args, nr, nw, nvec, shape, 0x3f803f80u)
  if (threads == kRowThreads) {
    switch (vectors) {
      case 1: PCCL_MIX(1, kRowThreads); break;
      case 2: PCCL_MIX(2, kRowThreads); break;
      default: PCCL_MIX(4, kRowThreads); break;
    }
  } else {
    switch (vectors) {
      case 1: PCCL_MIX(1, kThreads); break;
      case 2: PCCL_MIX(2, kThreads); break;
      default: PCCL_MIX(4, kThreads); break;
    }
  }
#undef PCCL_MIX
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return launch_status(what);
}

}  // extern "C"
