#!/usr/bin/env python3
"""Benchmark of the per-GPU reduce/copy kernels of PCCL's collectives on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--mode M]

Prints ONE JSON line.  A "step" is one whole collective over the virtual ranks
of the workload with all inputs already resident in HBM; `value` is the
algorithmic bytes of that collective divided by its time (GB/s, 1 GB = 1e9 B).
Timing follows benchmark_raw_collectives/utils.py:16-33 of the reference:
warm-up calls, then the mean over the timed calls between two device events
recorded on the stream the library launches on.

With no --workload the headline is `cfg2` in the per-step mode (the
configuration the metric is quoted on: the per-hop accumulate kernel), and
`config.workloads` carries one row for every other configuration and mode, each
timed the same way, each with its roofline fraction and a `verified` flag that
comes from a closed form recomputed with torch (never from a second run of the
library); `config.latency_us`, `config.ceilings` and `config.drop_in` follow.

Workloads:
  cfg1  ring reduce_scatter, P=4, fp32, 16 Mi elements per rank
  cfg2  ring reduce_scatter, P=8, bf16, 256 Mi elements per rank, per-hop
        accumulate with bf16 rounding at every hop
  cfg2h the cfg2 shape in float16 (the third element type; not one of the published configurations)
  cfg2d reduce_scatter_2D of the cfg2 data on a grid of 2 nodes x 4 local ranks, ring on
        both levels, as one fused launch (what the reference's harness runs with
        --library pccl; not one of the published configurations)
  cfg2dh the same with recursive halving on both levels (one 8-way butterfly; what the
        reference's DeepSpeed patch calls for reduce_scatter_tensor)
  cfg2ar all_reduce of the cfg2 data: ring reduce_scatter + all_gather, one fused launch each
  cfg3  recursive-halving round at its largest shape: a pair of ranks adding
        512 MiB strided halves (bf16), i.e. round 0 of P=64 with 1 GiB per rank
  cfg3full  the whole recursive-halving reduce_scatter over P=64 resident ranks,
        bf16, 1 GiB per rank (64 GiB of inputs + 64 GiB of work buffers in HBM)
  cfg4  all_gather placement, P=16, bf16 shards of 128 MiB into 2 GiB outputs
  cfg4u the same with uneven shards padded to 256 bytes
  cfg5  fused one-pass reduce of 32 fp32 shards of 32 Mi elements
  ceilings  what the device sustains for plain streams of 1 GiB (read-only,
        write-only, copy, add) and for read:write mixes with no data flowing
        from the loads to the stores (1:1, 2:1, 8:1, 32:1, 1:16)
  sweep  GB/s against message size, 64 MiB .. 2 GiB per operand
  latency  small messages, 4 KiB .. 1 MiB in bf16: microseconds per call
  placement  the cfg2 shape on six separately allocated groups of buffers in one
        process: the spread that comes from where the buffers lie physically
  all   (default) cfg2/steps as the headline plus every row above

The CPU baseline (the reference's per-rank algorithm on host cores, one process
per rank over MPI_Sendrecv, or fork+shared memory where no MPI launcher
exists) is timed on a bounded sample and reported beside the GPU number; it is
a baseline, not a target.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import shutil
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "sc2025-pccl-reproducer_amd"))

METRIC = "reduce/copy kernel HBM GB/s and % of MI355X peak at 64MB-2GB messages"
HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published peak
MiB = 1 << 20
WARM_MS = 60.0               # least duration of the untimed warm-up before a timed region, see time_steps

WORKLOADS = ["cfg1", "cfg2", "cfg2h", "cfg2d", "cfg2dh", "cfg2ar", "cfg3", "cfg3full", "cfg4", "cfg4u", "cfg5"]
# every (workload, mode) row of the default run besides the headline cfg2/steps
ALL_ROWS = [("cfg1", "steps"), ("cfg1", "fused"), ("cfg2", "fused"), ("cfg2h", "steps"), ("cfg2h", "fused"), ("cfg2d", "fused"),
            ("cfg2dh", "fused"), ("cfg2ar", "fused"), ("cfg3", "steps"),
            ("cfg3full", "steps"), ("cfg3full", "fused"), ("cfg4", "steps"), ("cfg4", "fused"),
            ("cfg4u", "fused"), ("cfg5", "fused"), ("cfg5", "steps")]


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all"] + WORKLOADS + ["latency", "ceilings", "sweep", "placement"])
    ap.add_argument("--mode", default=None, choices=["steps", "fused", "faithful"],
                    help="execution mode of the collective (default: per-step replay for the reductions, "
                         "one fused launch for cfg4, cfg4u and cfg5)")
    ap.add_argument("--scale", type=float, default=1.0,
                    help="shrink the per-rank message by this factor (1.0 = full size)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--layout", choices=["auto", "slab", "separate"], default="auto",
                    help="rank buffers carved from one allocation with a per-rank skew, one allocation each, "
                         "or (auto) the former from 32 ranks on")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed region launch one plain 1 GiB device copy (k_copy_segs): its "
                         "FETCH_SIZE / WRITE_SIZE readings scale the hardware counters of a rocprofv3 --pmc run")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch tuning of the library: any key of pccl_hip_set_tuning (grid_cap, unroll, unroll_copy, "
                         "nt_load, nt_store, add_rows, fold_rows, wg_kway, lds_pad_*, gather_strip, gather_split, unroll_gather, gather_nt)")
    return ap.parse_args()


# ---------------------------------------------------------------------------
# workloads: each builder returns {mode: (run_step, info)} on shared inputs
# resident on the GPU
# ---------------------------------------------------------------------------

def _randn_bf16(n, std, seed, device, out=None, dtype=None):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if out is None:
        out = torch.empty(n, dtype=dtype or torch.bfloat16, device=device)
    chunk = 1 << 26
    for i in range(0, n, chunk):      # bounded fp32 temporaries
        m = min(chunk, n - i)
        out[i:i + m] = (torch.randn(m, generator=g, device=device) * std).to(out.dtype)
    return out


def _rand_f32(n, seed, device, uniform=True, out=None):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if out is None:
        out = torch.empty(n, dtype=torch.float32, device=device)
    chunk = 1 << 26
    for i in range(0, n, chunk):
        m = min(chunk, n - i)
        if uniform:
            out[i:i + m] = torch.rand(m, generator=g, device=device) * 2 - 1
        else:
            out[i:i + m] = torch.randn(m, generator=g, device=device)
    return out


LAYOUT = "auto"


def _slab(P, numel, dtype, device):
    """The buffers of P virtual ranks.  'separate': one allocation per rank, what a
    caller with torch tensors has.  'slab': carved from one allocation with a
    per-rank skew (pccl.kernels.rank_slab).  'auto': the slab from 32 ranks on,
    where it measures faster (64 x 1 GiB inputs, fused halving: +8 %), separate
    allocations below (P = 8: the slab is 2 % slower)."""
    import torch
    from pccl import kernels
    use_slab = LAYOUT == "slab" or (LAYOUT == "auto" and P >= 32)
    if not use_slab:
        lens = [numel] * P if isinstance(numel, int) else list(numel)
        return [torch.empty(n, dtype=dtype, device=device) for n in lens]
    return kernels.rank_slab(P, numel, dtype, device)


def _mode_name(m):
    return {0: "steps", 1: "fused", 2: "faithful"}[m]


def _windows(n, width=1 << 20):
    """Element windows of a block that a closed form is recomputed on: its first
    and its last `width` elements (the whole block if it is shorter)."""
    if n <= 2 * width:
        return [(0, n)]
    return [(0, width), (n - width, n)]


def _hop(acc, x):
    """One hop of the reference's accumulate on torch tensors: an IEEE fp32 add,
    rounded to bfloat16 (nearest even) when the data is bfloat16."""
    import torch
    if acc.dtype in (torch.bfloat16, torch.float16):
        return (acc.float() + x.float()).to(acc.dtype)
    return acc + x


def _same_bits(a, b):
    import torch
    it = torch.int32 if a.dtype == torch.float32 else torch.int16
    return torch.equal(a.view(it), b.view(it))


def make_ring_rs(P, elems_per_rank, dtype, modes, device, seed=1234, std=1.0):
    import torch
    from pccl import kernels
    B = elems_per_rank // P
    total = B * P
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype]
    ins = _slab(P, total, tdt, device)
    for r in range(P):
        if dtype in ("bf16", "f16"):
            _randn_bf16(total, std, seed + r, device, out=ins[r])
        else:
            _rand_f32(total, seed + r, device, out=ins[r])
    es = 4 if dtype == "f32" else 2
    outs = _slab(P, B, tdt, device)
    shared = {}

    def verify():
        # closed form of the ring: block j is the left fold over ranks j+1, j+2, ..., j
        # (pccl/src/reduce_scatter.cpp:127-146), one rounding per hop
        torch.cuda.synchronize()
        for j in sorted({0, P // 2, P - 1}):
            for lo, hi in _windows(B):
                acc = ins[(j + 1) % P][j * B + lo:j * B + hi]
                for t in range(2, P + 1):
                    acc = _hop(acc, ins[(j + t) % P][j * B + lo:j * B + hi])
                if not _same_bits(outs[j][lo:hi], acc):
                    return False
        return True

    out = {}
    for mode in modes:
        m = kernels.mode_code(mode)
        if m != kernels.MODE_FUSED and P > 2 and "work" not in shared:
            shared["work"] = _slab(P, total, tdt, device)
        work = shared.get("work") if m != kernels.MODE_FUSED else None

        def step(m=m, work=work):
            kernels.reduce_scatter_ranks(outs, ins, "ring", m, work)

        launches = {kernels.MODE_STEPS: P - 1, kernels.MODE_FUSED: 1, kernels.MODE_FAITHFUL: P + 1}[m]
        if m == kernels.MODE_FUSED:
            kernel_bytes = (P * P + P) * B * es             # reads every input once, writes every output
            alg_bytes = kernel_bytes
            # aligned ring folds over at most 16 fp32 / bf16 shards run in the lean kernel
            kernel = "k_fold_rows" if P <= 16 and dtype in ("bf16", "f32") else "k_reduce_kway"
        else:
            kernel_bytes = 3 * P * B * es                   # one batched step: 2 reads + 1 write per rank
            alg_bytes = (P - 1) * kernel_bytes
            kernel = "k_add_rows"
        out[mode] = (step, dict(
            alg_bytes=alg_bytes, kernel=kernel, kernel_bytes=kernel_bytes,
            kernel_launches=(P - 1 if m != kernels.MODE_FUSED else 1), launches=launches,
            desc=f"ring reduce_scatter, P={P} virtual ranks, {dtype}, {total} elements per rank "
                 f"({total * es / MiB:.0f} MiB), block {B} elements, mode={_mode_name(m)}",
            dtype=dtype, P=P, B=B, verify=verify,
            verify_how="left fold from rank j+1 recomputed with torch on windows of blocks 0, P/2, P-1"))
    return out


def make_all_reduce(P, elems_per_rank, dtype, modes, device, seed=2468, std=1e-2):
    """all_reduce = reduce_scatter + all_gather with the ring schedules (pccl/all_reduce.py:21-55,
    pccl/src/yacl.cpp:146-177), each as one fused launch; the gathered sums land in separate
    buffers so that every timed call reduces the same inputs."""
    import torch
    from pccl import kernels
    B = elems_per_rank // P
    total = B * P
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype]
    es = 4 if dtype == "f32" else 2
    ins = _slab(P, total, tdt, device)
    for r in range(P):
        if dtype == "f32":
            _rand_f32(total, seed + r, device, out=ins[r])
        else:
            _randn_bf16(total, std, seed + r, device, out=ins[r])
    blocks = _slab(P, B, tdt, device)
    sums = _slab(P, total, tdt, device)

    def verify():
        torch.cuda.synchronize()
        for j in sorted({0, P // 2, P - 1}):
            for lo, hi in _windows(B):
                acc = ins[(j + 1) % P][j * B + lo:j * B + hi]
                for t in range(2, P + 1):
                    acc = _hop(acc, ins[(j + t) % P][j * B + lo:j * B + hi])
                for r in (0, P - 1):
                    if not _same_bits(sums[r][j * B + lo:j * B + hi], acc):
                        return False
        return True

    out = {}
    for mode in modes:
        if kernels.mode_code(mode) != kernels.MODE_FUSED:
            raise ValueError("the all_reduce workload is measured in the fused mode")

        def step():
            kernels.reduce_scatter_ranks(blocks, ins, "ring", "fused")
            kernels.all_gather_ranks(sums, blocks, "ring", "fused")

        nbytes = 2 * (P * P + P) * B * es     # the fold reads P*P*B and writes P*B; the placement reads P*B and writes P*P*B
        out[mode] = (step, dict(
            alg_bytes=nbytes, kernel="k_fold_rows + k_gather_strips", kernel_bytes=nbytes // 2, kernel_launches=2,
            launches=2,
            desc=f"all_reduce = ring reduce_scatter + all_gather, P={P} virtual ranks, {dtype}, {total} elements per rank "
                 f"({total * es / MiB:.0f} MiB), one fused launch each",
            dtype=dtype, P=P, B=B, verify=verify,
            verify_how="every block of the gathered sums of ranks 0 and P-1 against the left fold from rank j+1, "
                       "recomputed with torch on windows of blocks 0, P/2, P-1"))
    return out


def make_grid_rs(intra, inter, elems_per_rank, dtype, modes, device, seed=4321, std=1e-2, algorithm="ring"):
    """reduce_scatter_2D (pccl/reduce_scatter.py:205-235) over a grid of inter nodes x intra
    local ranks, ring order (or recursive halving, use_rh=True) on both levels, as ONE fused
    launch: what the reference's benchmark harness runs with --library pccl, and with
    halving what its DeepSpeed patch calls (pccl/patch_deepspeed.py:42-59)."""
    import torch
    from pccl import kernels
    W = intra * inter
    m = elems_per_rank // W
    total = m * W
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype]
    es = 4 if dtype == "f32" else 2
    ins = _slab(W, total, tdt, device)
    for r in range(W):
        if dtype == "f32":
            _rand_f32(total, seed + r, device, out=ins[r])
        else:
            _randn_bf16(total, std, seed + r, device, out=ins[r])
    outs = _slab(W, m, tdt, device)

    def ring_fold(parts, j):
        if algorithm != "ring":
            # the XOR butterfly rooted at j: v[m] = parts[j ^ m]; v[m] += v[m + h] for h = K/2 .. 1
            v = [parts[j ^ q] for q in range(len(parts))]
            h = len(parts) // 2
            while h >= 1:
                for q in range(h):
                    v[q] = _hop(v[q], v[q + h])
                h //= 2
            return v[0]
        acc = parts[(j + 1) % len(parts)]
        for t in range(2, len(parts) + 1):
            acc = _hop(acc, parts[(j + t) % len(parts)])
        return acc

    def verify():
        # rank w = node * intra + local ends with block w: first the ring order of block `local` over the
        # locals of every node, then the ring order of block `node` over the nodes, one rounding per hop
        torch.cuda.synchronize()
        for w in sorted({0, W // 2, W - 1}):
            node, local = divmod(w, intra)
            for lo, hi in _windows(m):
                per_node = [ring_fold([ins[n * intra + l][w * m + lo:w * m + hi] for l in range(intra)], local)
                            for n in range(inter)]
                if not _same_bits(outs[w][lo:hi], ring_fold(per_node, node)):
                    return False
        return True

    out = {}
    for mode in modes:
        if kernels.mode_code(mode) != kernels.MODE_FUSED:
            raise ValueError("the 2-D workload is measured in the fused mode")

        def step():
            kernels.reduce_scatter_2d_ranks(outs, ins, intra, inter, algorithm, "fused")

        nbytes = (W * W + W) * m * es
        out[mode] = (step, dict(
            alg_bytes=nbytes, kernel="k_reduce_kway", kernel_bytes=nbytes, kernel_launches=1, launches=1,
            desc=f"reduce_scatter_2D, {inter} nodes x {intra} local ranks (virtual), "
                 f"{'ring' if algorithm == 'ring' else 'recursive halving'} on both levels, {dtype}, "
                 f"{total} elements per rank ({total * es / MiB:.0f} MiB), block {m} elements, mode=fused",
            dtype=dtype, P=W, B=m, verify=verify,
            verify_how=("two-level left fold (locals from local+1, then nodes from node+1)" if algorithm == "ring" else
                        "XOR butterfly over the locals rooted at local, then over the nodes rooted at node")
            + " recomputed with torch on windows of blocks 0, W/2, W-1"))
    return out


def make_rh_pair(count_elems, device, seed=7):
    """Round 0 of recursive halving at P=64 with 1 GiB per rank, seen by one
    pair of ranks: P=2 here with B = count, so each rank adds one half."""
    import torch
    from pccl import _native, kernels
    B = count_elems
    ins = _slab(2, 2 * B, torch.bfloat16, device)
    work = _slab(2, 2 * B, torch.bfloat16, device)
    for r in range(2):
        _randn_bf16(2 * B, 1.0, seed + r, device, out=ins[r])
        work[r].copy_(ins[r])
    lib = _native.load()

    def step():
        lib.rh_round([w.data_ptr() for w in work], None, None, 2, B, 0, _native.BF16, kernels.stream_handle())

    def verify():
        # in place on the work buffers: redo once from the inputs and compare with torch
        for w, i in zip(work, ins):
            w.copy_(i)
        step()
        torch.cuda.synchronize()
        for lo, hi in _windows(B, 1 << 23):
            low = _hop(ins[0][lo:hi], ins[1][lo:hi])
            high = _hop(ins[1][B + lo:B + hi], ins[0][B + lo:B + hi])
            if not (_same_bits(work[0][lo:hi], low) and _same_bits(work[1][B + lo:B + hi], high)):
                return False
        return True

    kb = 2 * 3 * B * 2
    info = dict(alg_bytes=kb, kernel="k_rh_rows", kernel_bytes=kb, kernel_launches=1, launches=1,
                desc=f"recursive-halving round, one pair of ranks, bf16, halves of {B * 2 / MiB:.0f} MiB "
                     f"(round 0 of P=64 with {4 * B / MiB:.0f} MiB per rank)",
                dtype="bf16", P=2, B=B, verify=verify,
                verify_how="lower and upper half sums recomputed with torch on windows")
    return {"steps": (step, info)}


def make_rh_full(P, elems_per_rank, modes, device, seed=21):
    """Recursive-halving reduce_scatter with all P ranks resident."""
    import torch
    from pccl import kernels
    B = elems_per_rank // P
    total = B * P
    ins = _slab(P, total, torch.bfloat16, device)
    for r in range(P):
        _randn_bf16(total, 1.0, seed + r, device, out=ins[r])
    outs = _slab(P, B, torch.bfloat16, device)
    shared = {}

    def verify():
        # the halving order of block 0 and block P-1 recomputed with torch on windows
        torch.cuda.synchronize()
        for j in (0, P - 1):
            for lo, hi in _windows(B, 1 << 19):
                v = [ins[j ^ q][j * B + lo:j * B + hi] for q in range(P)]
                h = P // 2
                while h >= 1:
                    for q in range(h):
                        v[q] = _hop(v[q], v[q + h])
                    h //= 2
                if not _same_bits(outs[j][lo:hi], v[0]):
                    return False
        return True

    rounds = P.bit_length() - 1
    out = {}
    for mode in modes:
        m = kernels.mode_code(mode)
        if m != kernels.MODE_FUSED and "work" not in shared:
            shared["work"] = _slab(P, total, torch.bfloat16, device)
        work = shared.get("work") if m != kernels.MODE_FUSED else None

        def step(m=m, work=work):
            kernels.reduce_scatter_ranks(outs, ins, "recursive", m, work)

        if m == kernels.MODE_FUSED:
            kb = (P * P + P) * B * 2
            alg, kernel, kl, launches = kb, "k_reduce_kway", 1, 1
        else:
            # round r adds (P / 2^(r+1)) blocks per rank: 2 reads + 1 write per element
            alg = sum(3 * P * (P >> (r + 1)) * B * 2 for r in range(rounds))
            kb, kernel, kl, launches = alg, "k_rh_rows", 1, rounds
        out[mode] = (step, dict(
            alg_bytes=alg, kernel=kernel, kernel_bytes=kb, kernel_launches=kl, launches=launches,
            desc=f"recursive-halving reduce_scatter, P={P} resident virtual ranks, bf16, {total} elements per "
                 f"rank ({total * 2 / MiB:.0f} MiB), {rounds} rounds, mode={_mode_name(m)}",
            dtype="bf16", P=P, B=B, verify=verify,
            verify_how="XOR butterfly of blocks 0 and P-1 recomputed with torch on windows"))
    return out


def make_all_gather(P, shard_bytes, modes, device, uneven=False, seed=3):
    import torch
    from pccl import _native, kernels
    if isinstance(modes, str) or modes is None:      # a single mode: return its (step, info)
        return make_all_gather(P, shard_bytes, [modes or "fused"], device, uneven, seed)[modes or "fused"]
    n = shard_bytes // 2
    if uneven:
        g = torch.Generator().manual_seed(seed)
        lens = [int(n - int(torch.randint(0, n // 8, (1,), generator=g))) for _ in range(P)]
    else:
        lens = [n] * P
    ins = _slab(P, lens, torch.bfloat16, device)
    for r, l in enumerate(lens):
        _randn_bf16(l, 1.0, seed + r, device, out=ins[r])
    nbytes = [2 * l for l in lens]
    off = kernels.padded_offsets(nbytes, 256) if uneven else [r * shard_bytes for r in range(P)]
    total = off[-1] + (nbytes[-1] + 255) // 256 * 256 if uneven else P * shard_bytes
    outs = _slab(P, total // 2, torch.bfloat16, device)

    def verify():
        torch.cuda.synchronize()
        cat = torch.cat([t.view(torch.uint8) for t in ins]) if not uneven else None
        for o in (outs[0], outs[P // 2], outs[P - 1]):
            ob = o.view(torch.uint8)
            if uneven:
                for k in range(P):
                    if not torch.equal(ob[off[k]:off[k] + nbytes[k]], ins[k].view(torch.uint8)):
                        return False
            elif not torch.equal(ob, cat):
                return False
        return True

    payload = sum(nbytes)
    out = {}
    for mode in modes:
        m = kernels.mode_code(mode if mode else "fused")
        # the fused placement is the time-blocked kernel from 2 MiB shards on, the multicast kernel below
        strips = _native.load().get_tuning("gather_strip") != 0 and max(nbytes) >= (
            max(_native.load().get_tuning("gather_strip_from"), 0) or 2 * MiB)
        gather_kernel = "k_gather_strips" if strips else "k_gather_multicast"
        if uneven:
            def step():
                kernels.all_gather_uneven_ranks(outs, ins, off)
            launches, kernel = 1, gather_kernel
        else:
            def step(m=m):
                kernels.all_gather_ranks(outs, ins, "ring", m)
            launches = 1 if m == kernels.MODE_FUSED else P
            kernel = gather_kernel if m == kernels.MODE_FUSED else "k_copy_segs"
        if kernel == gather_kernel:
            # every shard is read once and written into each of the P outputs
            alg = (1 + P) * payload
            kb, kl = alg, 1
        else:
            alg = 2 * payload * P                   # 2 * bytes per materialised output, P outputs
            kb, kl = 2 * P * shard_bytes, P         # one batched step moves one shard per rank
        out[mode] = (step, dict(
            alg_bytes=alg, kernel=kernel, kernel_bytes=kb, kernel_launches=kl, launches=launches,
            desc=f"all_gather placement, P={P} virtual ranks, bf16 shards of ~{shard_bytes / MiB:.0f} MiB"
                 f"{' (uneven, padded to 256 B)' if uneven else ''} into {total / MiB:.0f} MiB outputs, "
                 f"all {P} outputs materialised, mode={_mode_name(m) if not uneven else 'fused'}",
            dtype="bf16", P=P, B=n, verify=verify,
            verify_how="outputs 0, P/2, P-1 byte-equal to the concatenation of the shards (torch.cat)"))
    return out


def make_kway(k, n, modes, device, seed=11):
    """k shards folded in ring order from shard 1: in one pass (fused), or as
    the k-1 per-hop accumulate launches the pass replaces (steps)."""
    import torch
    from pccl import kernels
    # 128 MiB shards: one allocation each measures 2 % faster than the skewed slab
    # (the slab pays off for buffers of 512 MiB and more)
    shards = _slab(k, n, torch.float32, device) if LAYOUT == "slab" else \
        [torch.empty(n, dtype=torch.float32, device=device) for _ in range(k)]
    for r in range(k):
        _rand_f32(n, seed + r, device, uniform=False, out=shards[r])
    out_t = torch.empty(n, device=device)

    def fused():
        kernels.reduce_kway(out_t, shards, "ring", 1 % k)

    def hops():
        kernels.add(out_t, shards[1 % k], shards[2 % k])
        for t in range(2, k):
            kernels.accumulate(out_t, shards[(1 + t) % k])

    def verify():
        torch.cuda.synchronize()
        for lo, hi in _windows(n, 1 << 21):
            acc = shards[1 % k][lo:hi].clone()
            for t in range(1, k):
                acc += shards[(1 + t) % k][lo:hi]
            if not _same_bits(out_t[lo:hi], acc):
                return False
        return True

    out = {}
    for mode in modes:
        per_hop = kernels.mode_code(mode if mode else "fused") != kernels.MODE_FUSED
        if per_hop:
            kb = 3 * n * 4                                       # one hop: 2 reads + 1 write
            info = dict(alg_bytes=(k - 1) * kb, kernel="k_add_rows", kernel_bytes=kb, kernel_launches=k - 1,
                        launches=k - 1,
                        desc=f"reduce of {k} fp32 shards of {n} elements ({n * 4 / MiB:.0f} MiB each) as {k - 1} "
                             f"per-hop accumulate launches, ring order", dtype="f32", P=k, B=n, verify=verify)
        else:
            kb = (k + 1) * n * 4
            info = dict(alg_bytes=kb, kernel="k_reduce_kway", kernel_bytes=kb, kernel_launches=1, launches=1,
                        desc=f"fused one-pass reduce of {k} fp32 shards of {n} elements ({n * 4 / MiB:.0f} MiB each), "
                             f"ring order", dtype="f32", P=k, B=n, verify=verify)
        info["verify_how"] = "left fold from shard 1 recomputed with torch fp32 adds on windows"
        out[mode] = (hops if per_hop else fused, info)
    return out


def default_mode(name):
    return "fused" if name in ("cfg2d", "cfg2dh", "cfg2ar", "cfg4", "cfg4u", "cfg5") else "steps"


def build_workloads(name, modes, scale, device):
    """{mode: (step, info)} of one configuration, on shared inputs."""
    def sc(x, q=1024):
        return max(q, int(x * scale) // q * q)
    modes = [m or default_mode(name) for m in modes]
    if name == "cfg1":
        return make_ring_rs(4, sc(16 * MiB), "f32", modes, device)
    if name == "cfg2":
        return make_ring_rs(8, sc(256 * MiB), "bf16", modes, device, std=1e-2)
    if name == "cfg2h":
        return make_ring_rs(8, sc(256 * MiB), "f16", modes, device, std=1e-2)
    if name == "cfg2d":
        return make_grid_rs(4, 2, sc(256 * MiB), "bf16", modes, device)
    if name == "cfg2ar":
        return make_all_reduce(8, sc(256 * MiB), "bf16", modes, device)
    if name == "cfg2dh":
        return make_grid_rs(4, 2, sc(256 * MiB), "bf16", modes, device, algorithm="recursive")
    if name == "cfg3":
        pair = make_rh_pair(sc(256 * MiB), device)
        return {m: pair["steps"] for m in modes}
    if name == "cfg3full":
        return make_rh_full(64, sc(512 * MiB, 1 << 16), modes, device)
    if name == "cfg4":
        return make_all_gather(16, sc(128 * MiB), modes, device)
    if name == "cfg4u":
        return make_all_gather(16, sc(128 * MiB), modes, device, uneven=True)
    if name == "cfg5":
        return make_kway(32, sc(32 * MiB), modes, device)
    raise ValueError(name)


def build_workload(name, mode, scale, device):
    mode = mode or default_mode(name)
    return build_workloads(name, [mode], scale, device)[mode]


# ---------------------------------------------------------------------------
# timing
# ---------------------------------------------------------------------------

def time_steps(step, steps, warmup, lib):
    """Warm-up calls, then `steps` timed calls between two events on the stream
    the library launches on.  Returns device ms, wall ms and launches per step."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # The device needs about 20 ms of continuous streaming before its rate settles (per-call times of a 0.75 ms
    # fold from a cold start: 0.82, 0.79, ... 0.73 of peak after 5 ms, 0.80 after 12 ms, 0.82-0.83 from 20 ms
    # on), so the untimed warm-up is at least `warmup` steps AND at least WARM_MS of device work.
    t_warm = time.perf_counter()
    while (time.perf_counter() - t_warm) * 1e3 < WARM_MS:
        for _ in range(max(1, warmup)):
            step()
        torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    launches0 = lib.launch_count()
    start.record(stream)
    for _ in range(steps):
        step()
    end.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(end), wall_ms, (lib.launch_count() - launches0) / steps


def roofline_of(info, dev_ms, steps, launched):
    """Roofline of the dominant kernel from the live timing: the timed region
    holds nothing but that kernel's launches (plus, in faithful mode, copies),
    so its mean launch time is region / launches and the bytes of a mean launch
    are the step's kernel bytes / launches."""
    if not (info["launches"] == info["kernel_launches"] or info["kernel_bytes"] == info["alg_bytes"]):
        return None
    step_kernel_bytes = (info["kernel_bytes"] * info["kernel_launches"]
                         if info["launches"] == info["kernel_launches"] else info["kernel_bytes"])
    kernel_ms = dev_ms / (steps * launched)
    launch_bytes = step_kernel_bytes / launched
    achieved = launch_bytes / (kernel_ms * 1e-3) / 1e9
    return {"bound": "hbm", "kernel": info["kernel"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
            "bytes_per_launch": int(round(launch_bytes)), "avg_launch_ms": round(kernel_ms, 5)}


def source_hash():
    """Digest of the kernel sources: a counter reading taken from another
    version of the kernels says nothing about this one."""
    h = hashlib.sha256()
    for f in ("pccl_kernels.h", "pccl_hip.hip"):
        with open(os.path.join(ROOT, "sc2025-pccl-reproducer_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def profiled_traffic(workload, mode, kernel, lib, scale):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 counter runs
    (profiles/traffic.json), or None with the reason: the entry must have been
    taken with these kernel sources, the default tuning and the full size."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as fh:
            table = json.load(fh)
    except Exception:                                         # noqa: BLE001
        return None, "no profiles/traffic.json"
    entry = table.get("entries", {}).get(f"{workload}:{mode}:{kernel}")
    if entry is None:
        return None, "no counter run recorded for this workload and mode"
    if table.get("source_sha256_16") != source_hash():
        return None, "recorded with other kernel sources than the ones loaded"
    if scale != 1.0 or any(lib.get_tuning(k) != v for k, v in table.get("tuning", {}).items()):
        return None, "recorded at the default tuning and full size, not this run's"
    return entry, None


def run_row(name, mode, step, info, steps, warmup, lib, verify=True):
    dev_ms, wall_ms, launched = time_steps(step, steps, warmup, lib)
    ms = dev_ms / steps
    gbps = info["alg_bytes"] / (ms * 1e-3) / 1e9
    roof = roofline_of(info, dev_ms, steps, launched)
    ok = bool(info["verify"]()) if verify else None
    row = {"workload": name, "mode": mode, "kernel": info["kernel"], "ms": round(ms, 4), "GBps": round(gbps, 1),
           "frac": round(gbps / HBM_PEAK_GBPS, 4), "launches": launched,
           "bytes_per_launch": roof["bytes_per_launch"] if roof else None,
           "avg_launch_ms": roof["avg_launch_ms"] if roof else None,
           "algorithmic_bytes": info["alg_bytes"], "steps": steps, "warmup": warmup,
           "verified": ok, "verified_by": info.get("verify_how") if verify else None}
    return row, roof, dev_ms, wall_ms, launched


def _stream_gbps(fn, nbytes, steps, warmup):
    """GB/s of `fn` moving nbytes per call: `warmup` untimed calls and at least WARM_MS of
    them (see time_steps), then `steps` calls between two events."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    while (time.perf_counter() - t_warm) * 1e3 < WARM_MS:
        for _ in range(max(1, warmup)):
            fn()
        torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(steps):
        fn()
    e.record()
    torch.cuda.synchronize()
    return round(nbytes / (s.elapsed_time(e) / steps * 1e-3) / 1e9, 1)


def ceilings(steps, warmup, device):
    """GB/s of pure read, pure write, copy and add streams over 1 GiB buffers, and
    of read:write mixes with no data flowing from the loads to the stores."""
    import torch
    from pccl import _native, kernels
    lib = _native.load()
    n = 1 << 30
    a = torch.zeros(n, dtype=torch.uint8, device=device)
    b = torch.zeros(n, dtype=torch.uint8, device=device)
    c = torch.zeros(n, dtype=torch.uint8, device=device)
    fa, fb, fc = (t.view(torch.float32) for t in (a, b, c))

    def gbps(fn, nbytes):
        return _stream_gbps(fn, nbytes, steps, warmup)

    st = kernels.stream_handle()
    res = {
        "read_only": gbps(lambda: lib.probe_stream(0, a.data_ptr(), n, st), n),
        "write_only": gbps(lambda: lib.probe_stream(1, c.data_ptr(), n, st), n),
        "copy": gbps(lambda: kernels.copy(c, a), 2 * n),
        "add_2r1w_f32": gbps(lambda: kernels.add(fc, fa, fb), 3 * n),
        "torch_copy_": gbps(lambda: c.copy_(a), 2 * n),
        "torch_add_f32": gbps(lambda: torch.add(fa, fb, out=fc), 3 * n),
    }
    del a, b, c, fa, fb, fc
    # read:write mixes, the best of the probe's shapes (all streams per workgroup or
    # one stream per workgroup; 256 threads or one wave per workgroup; 1, 2 or 4 vectors
    # per thread), beside the library kernel of the same mix on the same buffers.  The
    # probes are reference points, not bounds: a ratio above 1 says that the library
    # kernel orders its work better than any of the probe's plain shapes.
    mixes = {}
    for nr, nw, mib in ((1, 1, 1024), (2, 1, 1024), (8, 1, 256), (32, 1, 128), (1, 16, 128)):
        nb = mib * MiB
        rd = [torch.empty(nb // 4, device=device).normal_() for _ in range(nr)]
        wr = [torch.empty(nb // 4, device=device) for _ in range(nw)]
        rp, wp = [t.data_ptr() for t in rd], [t.data_ptr() for t in wr]
        best, shape = 0.0, None
        for sh in (0, 1, 2, 3):
            for u in (1, 2, 4):
                v = gbps(lambda: lib.probe_mix(rp, wp, nb, sh, u, st), (nr + nw) * nb)
                if v > best:
                    best, shape = v, f"shape {sh}, {u} vectors per thread"
        if nw == 1 and nr == 1:
            mine, kname = gbps(lambda: kernels.copy(wr[0], rd[0]), 2 * nb), "k_copy_segs"
        elif nw == 1 and nr == 2:
            mine, kname = gbps(lambda: kernels.add(wr[0], rd[0], rd[1]), 3 * nb), "k_add_rows"
        elif nw == 1:
            mine, kname = gbps(lambda: kernels.reduce_kway(wr[0], rd, "ring", 1), (nr + 1) * nb), \
                "k_fold_rows" if nr <= 16 else "k_reduce_kway"
        else:
            # nw shards of nb / nw bytes into nw outputs of nb bytes: nb read, nw * nb written
            g_out = [w.view(torch.uint8) for w in wr]
            g_in = [rd[0].view(torch.uint8)[q * (nb // nw):(q + 1) * (nb // nw)] for q in range(nw)]
            mine, kname = gbps(lambda: kernels.all_gather_ranks(g_out, g_in, "ring", "fused"), (1 + nw) * nb), \
                "k_gather_strips"
            del g_out, g_in
        mixes[f"{nr}r{nw}w_{mib}MiB"] = {"probe": best, "probe_shape": shape, "library_kernel": kname,
                                         "library": mine, "library_over_probe": round(mine / best, 3)}
        del rd, wr
    res["reference_mixes"] = mixes
    res["reference_mixes_note"] = ("dependence-free probes of the same read:write mix: reference points, not bounds "
                                   "(a ratio above 1 = the library kernel orders its work better than the probe's plain shapes)")
    return res


def size_sweep(steps, warmup, device):
    """Achieved GB/s of the per-hop, copy and fused kernels against message size."""
    import torch
    from pccl import _native, kernels

    def gbps(fn, nbytes):
        return _stream_gbps(fn, nbytes, steps, warmup)

    rows = []
    for mib in (64, 128, 256, 512, 1024, 2048):
        nb = mib * MiB
        a16, b16 = _randn_bf16(nb // 2, 1e-2, 1, device), _randn_bf16(nb // 2, 1e-2, 2, device)
        a32, b32 = a16.view(torch.float32), b16.view(torch.float32)
        c = torch.empty_like(a16)
        k = 8
        shards = [_randn_bf16(nb // 2 // k, 1e-2, 10 + i, device) for i in range(k)]
        out = torch.empty_like(shards[0])
        # the fold goes straight to the C entry point with its pointer list built once: at 64 MiB its kernel
        # (12 us) is shorter than the argument checks of the Python wrapper
        lib, st = _native.load(), kernels.stream_handle()
        shard_ptrs, out_ptr, n_el = [t.data_ptr() for t in shards], out.data_ptr(), out.numel()
        rows.append({
            "MiB": mib,
            "accumulate_bf16": gbps(lambda: kernels.accumulate(a16, b16), 3 * nb),
            "accumulate_f32": gbps(lambda: kernels.accumulate(a32, b32), 3 * nb),
            "copy": gbps(lambda: kernels.copy(c, a16), 2 * nb),
            "reduce_8way_bf16_total_input": gbps(lambda: lib.reduce_kway(out_ptr, shard_ptrs, n_el, _native.BF16, _native.ORDER_RING,
                                                                        1, True, st), (k + 1) * nb // k),
        })
        del a16, b16, a32, b32, c, shards, out
    return rows


def placement_spread(sets, steps, warmup, device):
    """The cfg2 shape on `sets` separately allocated groups of rank buffers, all of
    them alive at once: every group lies on other physical pages, and the same code
    on the same virtual layout runs at a rate that depends on the group.  Returns,
    per group, the GB/s of the per-step mode and of the fused mode."""
    import torch
    from pccl import _native
    lib = _native.load()
    groups, rows = [], []
    for g in range(sets):
        groups.append(make_ring_rs(8, 256 * MiB, "bf16", ["steps", "fused"], device, seed=1234 + 100 * g, std=1e-2))
    for g, built in enumerate(groups):
        row = {"group": g}
        for mode in ("steps", "fused"):
            step, info = built[mode]
            dev_ms, _, launched = time_steps(step, steps, warmup, lib)
            ms = dev_ms / steps
            row[mode + "_GBps"] = round(info["alg_bytes"] / (ms * 1e-3) / 1e9, 1)
            row[mode + "_frac"] = round(row[mode + "_GBps"] / HBM_PEAK_GBPS, 4)
        rows.append(row)
    return rows


def latency_sweep(steps, warmup, device):
    """Microseconds per call for launch-bound message sizes (bf16), through the
    ordinary Python API unless a column says otherwise."""
    import torch
    from pccl import kernels

    def us(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / steps

    rows = []
    P = 8
    for nbytes in [4096 << i for i in range(9)]:            # 4 KiB .. 1 MiB
        n = nbytes // 2
        x, y = _randn_bf16(n, 1.0, 1, device), _randn_bf16(n, 1.0, 2, device)
        z = torch.empty_like(x)
        B = max(8, n // P)
        ins = [_randn_bf16(P * B, 1.0, 10 + r, device) for r in range(P)]
        outs = [torch.empty(B, dtype=torch.bfloat16, device=device) for _ in range(P)]
        gouts = [torch.empty(P * B, dtype=torch.bfloat16, device=device) for _ in range(P)]
        work = [torch.empty_like(t) for t in ins]
        graph = torch.cuda.CUDAGraph()             # the 7 step launches captured once
        kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)
        plan_fused = kernels.plan_reduce_scatter(outs, ins, "ring", "fused")
        rows.append({
            "bytes": nbytes,
            "accumulate_us": round(us(lambda: kernels.accumulate(x, y)), 2),
            "copy_us": round(us(lambda: kernels.copy(z, x)), 2),
            "ring_rs_p8_fused_us": round(us(lambda: kernels.reduce_scatter_ranks(outs, ins, "ring", "fused")), 2),
            "ring_rs_p8_fused_plan_us": round(us(plan_fused), 2),
            "ring_rs_p8_steps_us": round(us(lambda: kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)), 2),
            "ring_rs_p8_steps_graph_us": round(us(graph.replay), 2),
            "all_gather_p8_fused_us": round(us(lambda: kernels.all_gather_ranks(gouts, outs, "ring", "fused")), 2),
        })
    return rows


def latency_from_c():
    """The same small-message table measured from plain C (csrc/examples/latency_from_c.c, built by
    `make -C sc2025-pccl-reproducer_amd/csrc example`): what the C ABI itself costs per call."""
    exe = os.path.join(ROOT, "sc2025-pccl-reproducer_amd", "csrc", "build", "latency_from_c")
    if not os.path.exists(exe):
        return {"error": "csrc/build/latency_from_c is not built"}
    try:
        p = subprocess.run([exe], capture_output=True, text=True, timeout=120)
        line = [l for l in p.stdout.splitlines() if l.startswith("[")]
        if p.returncode == 0 and line:
            return json.loads(line[-1])
        return {"error": f"exit code {p.returncode}: {p.stderr[-200:]}"}
    except Exception as e:                                    # noqa: BLE001
        return {"error": str(e)}


def drop_in(device, steps=5, warmup=2):
    """Wall time of the reference-shaped per-rank calls at the cfg2 size: 8
    virtual ranks (one Python thread each, as `mpirun -np 8` would start them)
    call pccl._reduce_scatter / pccl.reduce_scatter_2D / pccl.all_gather_2D with
    use_pccl_cpp_backend=True (pccl/reduce_scatter.py:164-235, pccl/all_gather.py:136-159)."""
    import torch
    import pccl
    P, total = 8, 256 * MiB
    B = total // P
    ins = [_randn_bf16(total, 1e-2, 50 + r, device) for r in range(P)]
    outs = [torch.empty(B, dtype=torch.bfloat16, device=device) for _ in range(P)]
    gouts = [torch.empty(total, dtype=torch.bfloat16, device=device) for _ in range(P)]
    world = pccl.VirtualWorld(P, device)
    res = {}

    def timed(name, call, setup=None):
        def rank_main(comm):
            r = comm.Get_rank()
            ctx = setup(comm) if setup else None
            t0 = None
            for it in range(warmup + steps):
                if it == warmup:
                    comm.Barrier()
                    if r == 0:
                        torch.cuda.synchronize()
                    comm.Barrier()
                    t0 = time.perf_counter()
                call(comm, r, ctx)
            comm.Barrier()
            if r == 0:
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) * 1e3 / steps
            return None
        res[name] = round(world.run(rank_main)[0], 4)

    def grid(comm):
        return pccl.ProcessGroups(4, 2, inner_group_backend="mpi", outer_group_backend="mpi", comm=comm)

    timed("_reduce_scatter_ring_ms",
          lambda comm, r, _: pccl._reduce_scatter(outs[r], ins[r], group=comm, use_pccl_cpp_backend=True))
    timed("reduce_scatter_2D_4x2_ring_ms",
          lambda comm, r, pg: pccl.reduce_scatter_2D(outs[r], ins[r], group=pg, use_pccl_cpp_backend=True), grid)
    timed("reduce_scatter_2D_4x2_halving_ms",
          lambda comm, r, pg: pccl.reduce_scatter_2D(outs[r], ins[r], group=pg, use_rh=True,
                                                     use_pccl_cpp_backend=True), grid)
    timed("all_gather_2D_4x2_doubling_ms",
          lambda comm, r, pg: pccl.all_gather_2D(gouts[r], outs[r], group=pg, use_rd=True,
                                                 use_pccl_cpp_backend=True), grid)
    # the same collective through the single-thread driver call, for scale
    from pccl import kernels
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        kernels.reduce_scatter_ranks(outs, ins, "ring")
    torch.cuda.synchronize()
    res["driver_reduce_scatter_ranks_ring_ms"] = round((time.perf_counter() - t0) * 1e3 / steps, 4)
    res["what"] = (f"wall ms per call, {P} virtual ranks = {P} Python threads meeting per call, bf16, "
                   f"{total * 2 // MiB} MiB per rank, default execution mode ({kernels.DEFAULT_MODE}), "
                   f"{warmup} warm-up + {steps} timed calls")
    return res


# ---------------------------------------------------------------------------
# CPU baseline (oracle/cpu_baseline.c), bounded sample
# ---------------------------------------------------------------------------

def _run_reaped(cmd, timeout):
    """Run a launcher in a process group of its own and leave nothing of it behind:
    an MPI launcher returns before its proxies have gone, so the group is waited
    for (two seconds at most) and then ended."""
    import signal
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, start_new_session=True)
    try:
        out, _ = proc.communicate(timeout=timeout)
        rc = proc.returncode
    except subprocess.TimeoutExpired:
        out, rc = "", -1
    pgid = proc.pid                      # the session leader's pid is the group's id
    deadline = time.time() + 2.0
    while True:
        try:
            os.killpg(pgid, 0)
        except (ProcessLookupError, PermissionError):
            break                        # nobody left in the group
        if time.time() > deadline:
            try:
                os.killpg(pgid, signal.SIGKILL)
            except (ProcessLookupError, PermissionError):
                pass
            break
        time.sleep(0.02)
    if proc.poll() is None:
        proc.wait()
    return rc, out


def _cpu_leg(ranks, dtype, block, iters, algs, scale):
    """One shape of the per-rank CPU program for the algorithms in `algs`
    ('ring': the reference's ring over MPI_Sendrecv, pccl/src/reduce_scatter.cpp:101-155;
    'mpi_block': MPI_Reduce_scatter_block, what pccl/reduce_scatter.py:197 calls).
    Returns {alg: result of the program}, the transport used and the wall seconds."""
    build = os.path.join(ROOT, "oracle", "build")
    mpi_bin = os.path.join(build, "cpu_baseline_mpi")
    shm_bin = os.path.join(build, "cpu_baseline_shm")
    launcher = None
    for cand in ("/opt/conda/bin/mpiexec.hydra", shutil.which("mpiexec.hydra"), shutil.which("mpiexec")):
        if cand and os.path.exists(cand):
            launcher = cand
            break
    res, transport, t0 = {}, None, time.time()
    for alg in algs:
        args = ["--alg", alg, "--dtype", dtype, "--block", str(block), "--warmup", "1", "--iters", str(iters),
                "--scale", scale]
        attempts = []
        if launcher and os.path.exists(mpi_bin):
            attempts.append(([launcher, "-np", str(ranks), mpi_bin] + args, "MPI_Sendrecv (MPICH)"))
        if alg == "ring":                # the vendor collective exists over MPI only
            attempts.append(([shm_bin, "--ranks", str(ranks)] + args, "fork+shared memory"))
        for cmd, how in attempts:
            try:
                rc, out = _run_reaped(cmd, 400)
            except Exception:                                 # noqa: BLE001
                continue
            line = [l for l in out.splitlines() if l.startswith("{")]
            if rc == 0 and line:
                res[alg] = json.loads(line[-1])
                transport = transport or how
                break
    return res, transport, time.time() - t0


def cpu_baseline(info):
    """The reference's per-rank algorithms on the host cores (oracle/cpu_baseline.c),
    timed on bounded samples: the headline's own shape (ring reduce_scatter over
    MPI_Sendrecv), and the reference's CPU-runnable configuration -- ring
    reduce_scatter, P = 4, fp32, 16 Mi elements per rank -- both as the
    hand-written ring and as the vendor's MPI_Reduce_scatter_block."""
    build = os.path.join(ROOT, "oracle", "build")
    if not os.path.exists(os.path.join(build, "cpu_baseline_shm")):
        try:
            subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
        except Exception as e:                               # noqa: BLE001
            return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": f"not built: {e}"}
    P = info["P"] if info["kernel"] in ("k_add_rows", "k_add_segs", "k_reduce_kway", "k_fold_rows") and info["P"] <= 8 else 8
    dtype = "bf16" if info["dtype"] == "bf16" else "f32"
    host_cores = os.cpu_count() or 1
    ranks = min(P, max(1, host_cores))
    if ranks & (ranks - 1):
        ranks = 1 << (ranks.bit_length() - 1)
    if info["kernel"] in ("k_add_rows", "k_add_segs") and ranks == info["P"]:
        block, sample = info["B"], "the workload itself (same P, dtype and block size)"
    else:
        block = (1 << 22) if dtype == "bf16" else (1 << 21)                 # 8 MiB blocks
        sample = "a ring reduce_scatter of the same dtype with 8 MiB blocks"
    # about ten seconds of timed calls, assuming ~15 GB/s of algorithmic bytes on the host
    job_bytes = 3 * (ranks - 1) * block * (2 if dtype == "bf16" else 4) * ranks
    iters = max(5, min(500, int(10.0 / max(job_bytes / 15e9, 1e-3))))
    head, transport, wall = _cpu_leg(ranks, dtype, block, iters, ["ring"], "0.01" if dtype == "bf16" else "1.0")
    # configuration 1 of the published list, the one the reference can run on CPUs: P = 4, fp32, blocks of 4 Mi elements
    c1_ranks = min(4, ranks if ranks >= 2 else 1)
    c1, c1_transport, c1_wall = _cpu_leg(c1_ranks, "f32", 1 << 22, 20, ["ring", "mpi_block"], "1.0")
    cfg1 = {
        "ring_GBps": round(c1["ring"]["GBps"], 3) if "ring" in c1 else None,
        "ring_ms_per_call": round(c1["ring"]["ms_per_call"], 3) if "ring" in c1 else None,
        "mpi_reduce_scatter_block_GBps": round(c1["mpi_block"]["GBps"], 3) if "mpi_block" in c1 else None,
        "mpi_reduce_scatter_block_ms_per_call": round(c1["mpi_block"]["ms_per_call"], 3) if "mpi_block" in c1 else None,
        "cores": c1_ranks,
        "sample": f"ring reduce_scatter, P = {c1_ranks}, fp32, {c1_ranks << 22} elements per rank: the reference's ring "
                  f"(pccl/src/reduce_scatter.cpp:101-155) and MPI_Reduce_scatter_block (pccl/reduce_scatter.py:197) on host "
                  f"buffers, {c1_ranks} processes over {c1_transport}, 1 warm-up + 20 timed calls each, {c1_wall:.1f} s wall",
    }
    if "ring" not in head:
        return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "baseline program failed", "cfg1": cfg1}
    r = head["ring"]
    return {"value": round(r["GBps"], 3), "unit": "GB/s", "cores": ranks, "kind": "port",
            "ms_per_call": round(r["ms_per_call"], 3), "host_cores": host_cores,
            "sample": f"{sample}: ring reduce_scatter of the reference "
                      f"(pccl/src/reduce_scatter.cpp:101-155) on host buffers, {ranks} ranks = {ranks} "
                      f"processes over {transport}, {dtype}, {block} elements per block "
                      f"({ranks * block} per rank), 1 warm-up + {iters} timed calls, {wall:.1f} s wall",
            "cfg1": cfg1}


# ---------------------------------------------------------------------------

TUNING_KEYS = ("grid_cap", "unroll", "add_rows", "fold_rows", "wg_kway", "unroll_copy", "nt_load", "nt_store", "gather_strip",
               "gather_split", "unroll_gather", "gather_nt", "lds_pad_copy", "lds_pad_kway",
               "lds_pad_gather")


def main():
    global LAYOUT
    args = parse_args()
    LAYOUT = args.layout
    if args.gpus != 1:
        print(f"bench.py: this build runs all virtual ranks on ONE GPU and issues no inter-GPU collective; "
              f"--gpus {args.gpus} is not supported (use --gpus 1).", file=sys.stderr)
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback.", file=sys.stderr)
        return 3
    from pccl import _native
    from pccl.build_kernels import build
    lib = build()
    for kv in args.tune:
        k, v = kv.split("=")
        lib.set_tuning(k, int(v))
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.workload == "ceilings":
        res = ceilings(args.steps, args.warmup, device)
        print(json.dumps({
            "metric": METRIC, "value": res["add_2r1w_f32"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(3 * (1 << 30) / res["add_2r1w_f32"] / 1e6, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "ceilings: plain streams over 1 GiB buffers and read:write mixes; "
                                   "value = the library's add kernel", "GBps": res},
            "roofline": None, "cpu_baseline": None}), flush=True)
        return 0

    if args.workload == "sweep":
        rows = size_sweep(args.steps, args.warmup, device)
        big = [r for r in rows if r["MiB"] >= 256]
        val = round(sum(r["accumulate_bf16"] for r in big) / len(big), 1)
        print(json.dumps({
            "metric": METRIC, "value": val, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
            "data": "synthetic",
            "config": {"workload": "sweep: GB/s against message size (MiB per operand); value = mean accumulate "
                                   "bf16 at >= 256 MiB", "GBps": rows,
                       "pct_of_hbm_peak": round(100 * val / HBM_PEAK_GBPS, 2)},
            "roofline": None, "cpu_baseline": None}), flush=True)
        return 0

    if args.workload == "placement":
        rows = placement_spread(6, min(args.steps, 10), min(args.warmup, 3), device)
        vals = [r["steps_GBps"] for r in rows]
        val = round(sum(vals) / len(vals), 1)
        print(json.dumps({
            "metric": METRIC, "value": val, "unit": "GB/s", "n_gpus": 1, "steps": min(args.steps, 10),
            "warmup": min(args.warmup, 3), "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "placement: cfg2 (ring reduce_scatter, P=8, bf16, 512 MiB per rank) on six separately "
                                   "allocated groups of buffers; value = mean of the per-step mode", "groups": rows,
                       "steps_min_max": [min(vals), max(vals)],
                       "fused_min_max": [min(r["fused_GBps"] for r in rows), max(r["fused_GBps"] for r in rows)]},
            "roofline": None, "cpu_baseline": None}), flush=True)
        return 0

    if args.workload == "latency":
        rows = latency_sweep(max(args.steps, 50), max(args.warmup, 10), device)
        last = rows[-1]
        print(json.dumps({
            "metric": METRIC, "value": round(3 * last["bytes"] / last["accumulate_us"] / 1e3, 1), "unit": "GB/s",
            "n_gpus": 1, "steps": max(args.steps, 50), "warmup": max(args.warmup, 10),
            "ms_per_step": round(last["accumulate_us"] / 1e3, 5), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "latency: bf16 messages of 4 KiB .. 1 MiB; value = accumulate at 1 MiB; "
                                   "microseconds per call include the Python/ctypes launch path",
                       "latency_us": rows, "latency_c_us": latency_from_c()},
            "roofline": None, "cpu_baseline": None}), flush=True)
        return 0

    everything = args.workload == "all"
    head_name = "cfg2" if everything else args.workload
    head_mode = (args.mode or default_mode(head_name)) if not everything else "steps"
    want_modes = [head_mode]
    rows, all_ok = [], True
    sub_steps, sub_warm = min(args.steps, 10), min(args.warmup, 3)

    def add_row(name, mode, step_fn, info_):
        nonlocal all_ok
        r, _, _, _, _ = run_row(name, mode, step_fn, info_, sub_steps, sub_warm, lib, verify=not args.no_verify)
        rows.append(r)
        all_ok = all_ok and r["verified"] in (None, True)

    # Where a workload's buffers lie decides 1-3 % of a fused fold: memory that has been returned to the driver
    # (empty_cache) and is allocated again runs them slower than memory allocated for the first time (cfg5:
    # 0.812 of the peak against 0.838 in a fresh process), and buffers carved out of the cached blocks of an
    # earlier, larger workload lie a power of two apart (cfg1: 0.763 against 0.787).  So that every row is what
    # a fresh process measures, the workloads that fit side by side keep their buffers until all of them have
    # run (each then allocates for the first time); only the three that need tens of GiB run after a release.
    held = []

    def run_group(name, hold):
        group = build_workloads(name, [m for n, m in ALL_ROWS if n == name], args.scale, device)
        for m in group:
            add_row(name, m, *group[m])
        if hold:
            held.append(group)
        else:
            del group
            torch.cuda.empty_cache()

    if everything:
        want_modes += [m for n, m in ALL_ROWS if n == head_name and m != head_mode]
    built = build_workloads(head_name, want_modes, args.scale, device)
    step, info = built[head_mode]
    torch.cuda.synchronize()

    row, roof, dev_ms, wall_ms, launched = run_row(head_name, head_mode, step, info, args.steps, args.warmup, lib,
                                                   verify=False)
    ms_per_step = dev_ms / args.steps
    value = info["alg_bytes"] / (ms_per_step * 1e-3) / 1e9

    if args.calibrate_copy:
        from pccl import kernels
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device).fill_(7)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        kernels.copy(dst, src)            # exactly 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst

    ok = None
    if not args.no_verify:
        step()                            # the outputs of this mode, not of a later one
        ok = bool(info["verify"]())
    if roof:
        roof["traffic"], roof["traffic_note"] = profiled_traffic(head_name, head_mode, info["kernel"], lib, args.scale)
        if roof["traffic"] is not None:
            roof["traffic_note"] = ("HBM bytes per launch from the rocprofv3 FETCH_SIZE/WRITE_SIZE runs summarised in "
                                    "profiles/ (same kernel sources, default tuning, full size); not measured in this run")

    all_ok = all_ok and ok in (None, True)
    extra = {}
    if everything:
        for m in want_modes[1:]:
            add_row(head_name, m, *built[m])
        held.append(built)
        del built, step
        info = {k: v for k, v in info.items() if k != "verify"}
        names = [n for n in dict.fromkeys(n for n, _ in ALL_ROWS) if n != head_name]
        large = [n for n in names if n in ("cfg3full", "cfg4", "cfg4u")]
        for name in names:
            if name not in large:
                run_group(name, hold=True)
        held.clear()
        torch.cuda.empty_cache()
        for name in large:
            run_group(name, hold=False)
        rows.sort(key=lambda r: ALL_ROWS.index((r["workload"], r["mode"])))
        extra["latency_us"] = latency_sweep(50, 10, device)
        extra["latency_c_us"] = latency_from_c()
        extra["ceilings"] = ceilings(10, 3, device)
        extra["drop_in"] = drop_in(device)

    cpu = None if args.no_cpu_baseline else cpu_baseline(info)

    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": info["dtype"], "data": "synthetic",
        "config": {"workload": f"{head_name}: {info['desc']}", "algorithmic_bytes_per_step": info["alg_bytes"],
                   "launches_per_step": launched, "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
                   "wall_ms_per_step": round(wall_ms / args.steps, 4), "verified": ok,
                   "verified_by": info.get("verify_how"), "layout": LAYOUT,
                   "tuning": {k: lib.get_tuning(k) for k in TUNING_KEYS}},
        "roofline": roof, "cpu_baseline": cpu,
    }
    if everything:
        out["config"]["workloads"] = rows
        out["config"].update(extra)
    print(json.dumps(out), flush=True)
    return 0 if all_ok else 1


if __name__ == "__main__":
    sys.exit(main())
