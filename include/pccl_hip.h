/*
 * pccl_hip.h -- C ABI of libpccl_hip.so: the per-GPU reduction and placement
 * compute of PCCL's reduce_scatter / all_gather, written for gfx950 (MI355X).
 *
 * The library replaces the torch/pybind11 extension module that the reference
 * builds at run time (pccl/build_kernels.py:102-105 compiles pccl/src/pccl.cpp,
 * all_gather.cpp, reduce_scatter.cpp and common.cu into a module named "pccl").
 * It is torch-free: every argument is a plain pointer, size or enum, so it can
 * be bound from ctypes, cffi, pybind11 or C.
 *
 * Model. P "virtual ranks" live on ONE GPU: rank r's send and receive buffers
 * are ordinary device allocations in that GPU's HBM, and the MPI_Sendrecv the
 * reference issues between two device kernels (pccl/src/reduce_scatter.cpp:67-69,
 * :140-142; pccl/src/all_gather.cpp:61-63) becomes a direct read of the
 * partner's buffer by the kernel of the next step.  No inter-GPU collective is
 * ever issued.
 *
 * Conventions
 *  - Every entry point returns 0 on success and a negative PCCL_HIP_E* code on
 *    failure; pccl_hip_last_error() then holds a message for the calling
 *    thread.  Nothing here prints or terminates the process (the reference's
 *    CUDA_CHECK calls exit(1): pccl/include/common.h:8-15).
 *  - Pointer tables (void* const*) are HOST arrays of DEVICE pointers; they are
 *    consumed before the call returns (copied into kernel arguments).
 *  - The library never allocates, frees or retains device memory: the caller
 *    passes inputs, outputs and workspaces (the reference shim allocates them
 *    as torch tensors for the same reason: pccl/src/pccl.cpp:54-59,71-73).
 *  - Work is only enqueued on `stream` (a hipStream_t; NULL = the default
 *    stream).  No call synchronises the host.
 *  - Sizes are size_t elements unless a name says bytes.  The reference uses
 *    `int` for both (pccl/include/reduce_scatter.h:8,15, all_gather.h:8), so it
 *    cannot address a 2 GiB buffer; this ABI can.
 *  - Buffers passed to one call must not overlap except where a function
 *    documents in-place use.
 */
#ifndef PCCL_HIP_H
#define PCCL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCCL_HIP_ABI_VERSION 1

/* Largest number of segments / shards one LAUNCH takes (their pointers travel
 * in the kernel arguments): the limit of the batched kernels and of the 2-D
 * entry points. */
#define PCCL_HIP_MAX_RANKS 64

/* Largest number of virtual ranks of pccl_hip_reduce_scatter_virtual /
 * pccl_hip_all_gather_virtual: a step (or a fused collective) over more than
 * PCCL_HIP_MAX_RANKS ranks goes out as several launches. */
#define PCCL_HIP_MAX_VIRTUAL_RANKS 4096

/* Element types.  bf16 and fp16 sums are computed as RNE(float(a) + float(b))
 * at every hop, which is what torch.add does on bfloat16 and float16 tensors
 * in the reference's Python algorithms (pccl/reduce_scatter.py:24,83,95,106,158;
 * float16 is what ZeRO hands them through pccl/patch_deepspeed.py:42-59).  The
 * reference's compiled extension takes float32 only (pccl/src/pccl.cpp:42-45).
 * NaN results are stored as the canonical quiet NaN of the type (0x7FC0,
 * 0x7E00), as the host conversions of c10 do for bfloat16. */
enum pccl_hip_dtype {
  PCCL_HIP_F32 = 0,
  PCCL_HIP_BF16 = 1,
  PCCL_HIP_F16 = 2
};

/* Summation orders for the fused reduce (bit-exact replay of a schedule). */
enum pccl_hip_order {
  /* Left fold over ranks first, first+1, ... (mod k), i.e. the order in which
   * the ring of pccl/src/reduce_scatter.cpp:127-146 accumulates block j when
   * first = (j + 1) mod P. */
  PCCL_HIP_ORDER_RING = 0,
  /* XOR butterfly of recursive halving (pccl/src/reduce_scatter.cpp:50-89):
   * v[m] = shard[first ^ m]; for h = k/2 .. 1: v[m] += v[m + h], m < h. */
  PCCL_HIP_ORDER_HALVING = 1
};

/* How a whole collective is executed on the virtual ranks. */
enum pccl_hip_mode {
  /* One batched launch per step of the reference schedule; the input->work
   * copy and the final copy-out are folded into the first and last step. */
  PCCL_HIP_MODE_STEPS = 0,
  /* One launch for the whole collective (k-way reduce / direct placement),
   * reproducing the same summation order. */
  PCCL_HIP_MODE_FUSED = 1,
  /* The reference's memory operations one for one: copy input to the work
   * buffer, add in place per step, copy the result block out
   * (pccl/src/reduce_scatter.cpp:32-36,92-96,119-123,148-152). */
  PCCL_HIP_MODE_FAITHFUL = 2
};

enum pccl_hip_status {
  PCCL_HIP_OK = 0,
  PCCL_HIP_EINVAL = -1,   /* bad argument (message says which) */
  PCCL_HIP_ELAUNCH = -2,  /* the HIP runtime refused a launch */
  PCCL_HIP_ENODEV = -3    /* no usable gfx950 device */
};

/* ABI version of the loaded library (== PCCL_HIP_ABI_VERSION). */
int pccl_hip_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char* pccl_hip_last_error(void);

/* Size in bytes of one element of `dtype`, 0 if unknown. */
size_t pccl_hip_dtype_size(int dtype);

/* ---- a1: the accumulate kernel ------------------------------------------
 * dst[i] = dst[i] + src[i], i < n.  Replaces vectorAdd / vectorAddKernel
 * (pccl/src/common.cu:5-19; float only there).  Same result bits as the
 * reference for fp32 (one IEEE add per element). */
int pccl_hip_accumulate(void* dst, const void* src, size_t n, int dtype,
                        void* stream);

/* dst[i] = a[i] + b[i].  dst may alias a or b exactly (in-place), but must
 * not partially overlap either.  This three-address form is what lets a
 * schedule skip the reference's input->work copy. */
int pccl_hip_add(void* dst, const void* a, const void* b, size_t n, int dtype,
                 void* stream);

/* `count` independent adds of n elements each in ONE launch:
 * dst[s][i] = a[s][i] + b[s][i].  One ring step or halving round over all
 * virtual ranks is one such call.  Segments must be pairwise hazard-free
 * (no segment writes what another reads or writes). count <= PCCL_HIP_MAX_RANKS. */
int pccl_hip_add_batched(void* const* dst, const void* const* a,
                         const void* const* b, int count, size_t n, int dtype,
                         void* stream);

/* ---- a3: strided-half pairwise kernel (one recursive-halving round) -------
 * bufs[r] is rank r's work buffer of P*B elements.  Round `round`
 * (0 <= round < log2 P), group = P >> round, half = group/2 blocks,
 * count = half*B, start(r) = (r / group) * group * B:
 *   lower rank k (k % group <  half), partner p = k + half:
 *       bufs[k][start : start+count]          += bufs[p][start : start+count]
 *   upper rank p:
 *       bufs[p][start+count : start+2*count]  += bufs[k][start+count : start+2*count]
 * exactly the two branches of pccl/src/reduce_scatter.cpp:58-88 with the
 * received half read from the partner's buffer.  All P ranks in one launch.
 * If `src` is non-NULL the operands are read from src[] instead of bufs[]
 * (first round straight from the inputs); if `outs` is non-NULL the sums of
 * the LAST round (count == B) are written to outs[r][0:B] instead. */
int pccl_hip_rh_round(void* const* bufs, const void* const* src,
                      void* const* outs, int P, size_t B, int round, int dtype,
                      void* stream);

/* ---- fused one-pass k-way reduce -----------------------------------------
 * out[i] = sum over the k shards of shard[.][i], i < n, added in `order`
 * starting from shard `first`.  With per_hop_round != 0 a bf16 partial sum is
 * rounded to bf16 after every add (bit-exact to k-1 calls of
 * pccl_hip_accumulate); with 0 the partial sum stays in fp32 and is rounded
 * once.  For PCCL_HIP_F32 the flag has no effect.  2 <= k <= PCCL_HIP_MAX_RANKS;
 * PCCL_HIP_ORDER_HALVING needs k to be a power of two.  out must not overlap
 * any shard. */
int pccl_hip_reduce_kway(void* out, const void* const* shards, int k, size_t n,
                         int dtype, int order, int first, int per_hop_round,
                         void* stream);

/* ---- placement copies ---------------------------------------------------
 * `count` independent byte copies in one launch: dst[s][0:nbytes[s]] =
 * src[s][0:nbytes[s]].  Any alignment and any size (0 allowed); 16-byte
 * aligned segments take the 128-bit path.  count <= PCCL_HIP_MAX_RANKS.
 * Replaces the cudaMemcpyAsync placement copies of pccl/src/all_gather.cpp:31-35
 * and pccl/src/reduce_scatter.cpp:32-36,92-96,119-123,148-152. */
int pccl_hip_copy_batched(void* const* dst, const void* const* src,
                          const size_t* nbytes, int count, void* stream);

/* out[dst_off[k] : dst_off[k] + nbytes[k]] = shard[k][0 : nbytes[k]] for
 * k < P: materialise one rank's all_gather output from the P shards in one
 * launch.  Uneven shards are expressed by nbytes[]/dst_off[] (bytes); gaps
 * between shards (padding) are left untouched. */
int pccl_hip_gather_place(void* out, const void* const* shards,
                          const size_t* nbytes, const size_t* dst_off, int P,
                          void* stream);

/* dst viewed as [cols][rows][m] = src viewed as [rows][cols][m], m in bytes:
 * the block transpose that reduce_scatter_2D applies before the inner
 * collective (pccl/reduce_scatter.py:226, rows = inter, cols = intra) and
 * all_gather_2D applies after it (pccl/all_gather.py:158-159, rows = intra,
 * cols = inter).  dst must not overlap src. */
int pccl_hip_block_transpose(void* dst, const void* src, size_t rows,
                             size_t cols, size_t m_bytes, void* stream);

/* ---- whole collectives on virtual ranks -----------------------------------
 * reduce_scatter over P virtual ranks.  Replaces reduce_scatter_mpi
 * (pccl/src/pccl.cpp:11-85) and the two algorithms it dispatches to
 * (pccl/src/reduce_scatter.cpp:16-99 "recursive", :101-155 "ring").
 *   inputs[r]  : rank r's input, P*B elements (read only)
 *   outputs[r] : rank r's output, B elements = sum_k inputs[k][r*B:(r+1)*B]
 *   work[r]    : rank r's workspace, P*B elements; may be NULL as a whole
 *                for P <= 2 and for PCCL_HIP_MODE_FUSED (except "recursive"
 *                with P > PCCL_HIP_MAX_RANKS, see below)
 *   algorithm  : "ring" or "recursive" (recursive needs P a power of two);
 *                any other string is an error, as at pccl.cpp:83.
 * The summation order of each output block is that of the named algorithm in
 * every mode.  1 <= P <= PCCL_HIP_MAX_VIRTUAL_RANKS.  PCCL_HIP_MODE_FUSED is
 * one launch up to PCCL_HIP_MAX_RANKS ranks.  Beyond, "ring" folds every
 * output block in ceil((P-1)/63) launches of at most 64 operands, the running
 * sum (kept in the output) being the first operand of the next launch, and
 * "recursive" runs halving rounds step by step until groups of 64 ranks
 * remain (this needs work[]) and finishes each group with one launch. */
int pccl_hip_reduce_scatter_virtual(void* const* outputs,
                                    const void* const* inputs,
                                    void* const* work, int P, size_t B,
                                    int dtype, const char* algorithm, int mode,
                                    void* stream);

/* The per-step reduce_scatter (PCCL_HIP_MODE_STEPS of the call above, same
 * schedules, same bits) for callers that cannot allocate device memory and have
 * no workspace to pass: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference (its shim
 * allocates the work buffers as torch tensors on every call,
 * pccl/src/pccl.cpp:58-59,71-73).  The work buffers live in an array that is
 * part of the library's code object: PCCL_HIP_NOALLOC_SCRATCH_BYTES of device
 * memory on every GPU the library is used on, held until the process ends.
 * The call allocates and frees nothing, on the device or on the host.
 *   limit : P <= PCCL_HIP_MAX_RANKS, and P slices of P*B elements, each rounded
 *           up to 256 bytes, must fit PCCL_HIP_NOALLOC_SCRATCH_BYTES; larger
 *           shapes are refused with PCCL_HIP_EINVAL (use the call above with
 *           caller-owned work buffers).
 *   set-up: the first call on a device looks the array's address up
 *           (hipGetSymbolAddress) with that device current; make it outside
 *           graph capture.  Later calls only enqueue.
 *   sharing: every call on a GPU uses that GPU's one array, so calls that can
 *           overlap on one GPU (different streams, different threads) race;
 *           calls on one stream are ordered and safe.  Nothing has to be
 *           cleared between calls: every scratch element a call reads has been
 *           written earlier in the same call. */
#define PCCL_HIP_NOALLOC_SCRATCH_BYTES (32u * 1024u * 1024u)
int pccl_hip_reduce_scatter_virtual_noalloc(void* const* outputs,
                                            const void* const* inputs, int P,
                                            size_t B, int dtype,
                                            const char* algorithm, void* stream);

/* all_gather over P virtual ranks, in bytes.  Replaces all_gather_mpi
 * (pccl/src/pccl.cpp:87-142) and recursiveDoublingAllGatherGPU
 * (pccl/src/all_gather.cpp:15-69).
 *   inputs[r]  : rank r's shard, block_bytes bytes
 *   outputs[r] : rank r's output, P*block_bytes bytes = concatenation of the
 *                shards in rank order
 *   algorithm  : "recursive" (doubling, P a power of two) or "ring"
 *                (the ring schedule the reference leaves to MPI_Allgather,
 *                pccl/all_gather.py:124-128).
 * PCCL_HIP_MODE_STEPS replays one batched copy per step;
 * PCCL_HIP_MODE_FUSED places every shard directly (one launch per 64 shards
 * and 64 outputs); FAITHFUL == STEPS.  1 <= P <= PCCL_HIP_MAX_VIRTUAL_RANKS. */
int pccl_hip_all_gather_virtual(void* const* outputs, const void* const* inputs,
                                int P, size_t block_bytes,
                                const char* algorithm, int mode, void* stream);

/* Uneven all_gather: shard k has nbytes[k] bytes and lands at byte offset
 * dst_off[k] of every output (the caller chooses offsets, e.g. each shard
 * padded to a multiple of 256 bytes).  One launch places all P*P segments
 * (one per 64 shards and 64 outputs beyond PCCL_HIP_MAX_RANKS ranks).
 * 1 <= P <= PCCL_HIP_MAX_VIRTUAL_RANKS.  Not a reference feature (it requires
 * equal shards, pccl/src/pccl.cpp:111-116). */
int pccl_hip_all_gather_uneven_virtual(void* const* outputs,
                                       const void* const* inputs,
                                       const size_t* nbytes,
                                       const size_t* dst_off, int P,
                                       void* stream);

/* ---- 2-D (hierarchical) collectives on virtual ranks ------------------------
 * World of intra*inter ranks, rank w = j*intra + i (node j, local rank i):
 * the inner group of w is its node {j*intra + i'}, the outer group the ranks
 * {j'*intra + i} (pccl/process_groups.py:97-98).  Replaces reduce_scatter_2D
 * (pccl/reduce_scatter.py:205-235): input viewed [inter, intra, m] is permuted
 * to [intra, inter, m], reduce-scattered inside the node, then across nodes.
 * The permutation is never materialised: the first inner step reads the inputs
 * through it (strided pieces).  One launch per step serves ALL groups of a
 * level, i.e. (intra-1)+(inter-1) launches for "ring" (one launch per
 * PCCL_HIP_MAX_RANKS ranks of the grid and step).
 *   inputs[w]  : intra*inter*m elements;  outputs[w] : m elements
 *   work[w]    : intra*inter*m elements (needed if intra > 2 or inter > 2)
 *   mid[w]     : inter*m elements (needed if intra > 1 and inter > 1)
 *   mode       : PCCL_HIP_MODE_STEPS, or PCCL_HIP_MODE_FUSED = ONE launch that
 *                folds all intra*inter inputs in the two-level order
 *                (work and mid may then be NULL).  A grid of more than
 *                PCCL_HIP_MAX_RANKS ranks is fused level by level instead: one
 *                fold per node over its `intra` inputs into mid[] (which is
 *                then needed; work is not), then one fold per local rank over
 *                the `inter` intermediates; intra, inter <= PCCL_HIP_MAX_RANKS.
 * Both levels use `algorithm`; intra*inter <= PCCL_HIP_MAX_VIRTUAL_RANKS. */
int pccl_hip_reduce_scatter_2d_virtual(void* const* outputs,
                                       const void* const* inputs,
                                       void* const* work, void* const* mid,
                                       int intra, int inter, size_t m, int dtype,
                                       const char* algorithm, int mode,
                                       void* stream);

/* all_gather_2D (pccl/all_gather.py:136-159): gather across nodes, gather
 * inside the node, un-permute [intra, inter, n] -> [inter, intra, n]; the inner
 * stage writes through the un-permutation, so no extra pass is made.
 *   inputs[w]  : block_bytes bytes;  outputs[w] : intra*inter*block_bytes
 *   mid[w]     : inter*block_bytes bytes (needed if intra > 1 and inter > 1)
 * PCCL_HIP_MODE_FUSED places every shard directly (one launch per 64 shards
 * and 64 outputs).  intra*inter <= PCCL_HIP_MAX_VIRTUAL_RANKS. */
int pccl_hip_all_gather_2d_virtual(void* const* outputs,
                                   const void* const* inputs, void* const* mid,
                                   int intra, int inter, size_t block_bytes,
                                   const char* algorithm, int mode, void* stream);

/* ---- bandwidth probe (for measurement) --------------------------------------
 * One pure streaming pass over buf[0:nbytes]: kind 0 reads every byte (nothing
 * is written; workgroups of 1024 threads, the fastest shape measured for
 * reads), kind 1 overwrites every byte with the bf16 pattern of 1.0
 * (workgroups of 256 threads, the fastest for writes).  Timing it gives the
 * read and write bandwidth this device sustains, reference points beside the
 * 2-reads-1-write kernels.  No counterpart in the reference.  buf must be
 * 16-byte aligned, nbytes >= 16384. */
int pccl_hip_probe_stream(int kind, void* buf, size_t nbytes, void* stream);

/* A read:write MIX in one launch: nr read streams and nw write streams of
 * nbytes bytes each, with no data flowing from the loads to the stores (the
 * loads are folded and dropped, the stores write a constant).  Timing it gives
 * what the device sustains for the 2:1 mix of the add kernels, the k:1 mix of
 * the fused reduce or the 1:P mix of the all_gather placement when nothing but
 * the memory system is in the way.  shape 0: workgroup t serves tile t of every
 * stream; shape 1: every workgroup serves one stream; shapes 2 and 3: the same
 * two with one-wave workgroups (64 threads, the shape of the lean add kernels
 * and of the fused reduce on streams from HBM).  vectors = 128-bit vectors per
 * thread and stream (1, 2 or 4).  The best of these shapes is a reference
 * point, not an upper bound: a library kernel that orders its work in time
 * (the time-blocked all_gather) runs ahead of all of them.  No counterpart in
 * the reference.
 * Streams must be 16-byte aligned, nbytes a multiple of 16, nr, nw <= 64. */
int pccl_hip_probe_mix(const void* const* reads, int nr, void* const* writes,
                       int nw, size_t nbytes, int shape, int vectors,
                       void* stream);

/* ---- launch tuning (for measurement) ------------------------------------
 * key: "grid_cap" (max workgroups per launch of the 256-thread kernels,
 *                  0 = one tile per workgroup),
 *      "add_rows" (1, the default: adds over contiguous 16-byte aligned
 *                  segments run in the lean one-wave kernels, one 128-bit
 *                  vector per thread; 0: everything in the general kernels),
 *      "fold_rows" (1, the default: a ring-order fused reduce over at most 16
 *                  fp32 or bfloat16 shards that streams from HBM, with every
 *                  operand 16-byte aligned, runs in the lean kernel on a 2-D
 *                  grid; 0: always the general kernel),
 *      "unroll"   (128-bit vectors per thread per operand of the general add
 *                  kernels: 1, 2, 4 or 8), "unroll_copy" (the same for the copy
 *                  kernels),
 *      "nt_load" / "nt_store" (non-temporal global loads / stores: 1 always,
 *                  0 never, -1, the default: for calls whose footprint exceeds
 *                  the Infinity Cache and the L2s, 288 MiB),
 *      "wg_kway"  (threads per workgroup of the fused reduce: 64, 256, or -1,
 *                  the default: 64 with loads in pairs for streams from HBM,
 *                  256 for operands that fit the caches),
 *      "lds_pad_copy" / "lds_pad_kway" / "lds_pad_gather" (bytes of unused LDS
 *                  per workgroup, 0..65536: bounds the workgroups resident per
 *                  CU; -1, the default, lets the launch choose),
 *      "unroll_gather" (vectors per thread of the all_gather placement kernels:
 *                  1, 2, 4, 8; 0, the default: one in the multicast kernel,
 *                  four in the time-blocked one),
 *      "gather_strip"  (fused all_gather: work items per XCD and strip of the
 *                  time-blocked kernel, in which an XCD walks a strip of its
 *                  tiles once per output; 0 = the multicast kernel, in which a
 *                  workgroup stores its tile to several outputs at once; -1, the
 *                  default: time-blocked, 160, for shards of at least
 *                  "gather_strip_from" bytes, default 2 MiB),
 *      "gather_split"  (multicast kernel: workgroups sharing one shard tile,
 *                  each storing to 1/gather_split of the outputs;
 *                  0, the default = four outputs per workgroup),
 *      "gather_nt" (non-temporal stores in both kernels: 1, 0 or -1 as above).
 * Every default that is not the plain setting is backed by an A/B measurement
 * over fresh processes on MI355X; a setting whose gain was inside the
 * run-to-run spread has been removed.
 * Returns 0, or PCCL_HIP_EINVAL for an unknown key or value.
 * The settings are process-wide: besides the per-thread error message, they,
 * the launch counter below and the per-device address of the built-in scratch
 * array are the only state the library keeps.  Every value is one atomic word
 * that a launch reads once, so changing a setting while another thread
 * launches is safe, but that launch may see either value.  They exist for
 * measurement; the defaults are what the kernels were tuned to. */
int pccl_hip_set_tuning(const char* key, long value);
long pccl_hip_get_tuning(const char* key);

/* Kernel launches this process has issued through the library so far (a step
 * of a schedule is one launch up to 64 ranks and one per 64 ranks beyond; a
 * fused collective is one or a few, see the entry points).  For measurement: the
 * difference around a timed region is the number of launches in it.  No
 * counterpart in the reference. */
unsigned long long pccl_hip_launch_count(void);

#ifdef __cplusplus
}
#endif
#endif /* PCCL_HIP_H */
