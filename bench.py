#!/usr/bin/env python3
"""Benchmark of the per-GPU reduce/copy kernels of PCCL's collectives on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--mode M]

Prints ONE JSON line.  A "step" is one whole collective over the virtual ranks
of the workload with all inputs already resident in HBM; `value` is the
algorithmic bytes of that collective divided by its time (GB/s, 1 GB = 1e9 B).
Timing follows benchmark_raw_collectives/utils.py:16-33 of the reference:
warm-up calls, then the mean over the timed calls between two device events.

Workloads (`cfg2` is the one the headline metric is quoted on):
  cfg1  ring reduce_scatter, P=4, fp32, 16 Mi elements per rank
  cfg2  ring reduce_scatter, P=8, bf16, 256 Mi elements per rank, per-hop
        accumulate with bf16 rounding at every hop              (default)
  cfg3  recursive-halving round at its largest shape: a pair of ranks adding
        512 MiB strided halves (bf16), i.e. round 0 of P=64 with 1 GiB per rank
  cfg3full  the whole recursive-halving reduce_scatter over P=64 resident ranks,
        bf16, 1 GiB per rank (64 GiB of inputs + 64 GiB of work buffers in HBM)
  cfg4  all_gather placement, P=16, bf16 shards of 128 MiB into 2 GiB outputs
  cfg4u the same with uneven shards padded to 256 bytes
  cfg5  fused one-pass reduce of 32 fp32 shards of 32 Mi elements
  ceilings  what the device sustains for plain streams of 1 GiB: read-only,
        write-only, copy and 2-reads-1-write add (the practical roofline)
  sweep  GB/s against message size, 64 MiB .. 2 GiB per operand: accumulate
        (bf16 and fp32), copy, and the fused 8-way reduce
  latency  small messages, 4 KiB .. 1 MiB in bf16: microseconds per accumulate,
        per copy and per whole P=8 ring reduce_scatter (per-step and fused)

The CPU baseline (the reference's per-rank algorithm on host cores, one process
per rank over MPI_Sendrecv, or fork+shared memory where no MPI launcher
exists) is timed on a bounded sample and reported beside the GPU number; it is
a baseline, not a target.
"""
from __future__ import annotations

import argparse
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


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2",
                    choices=["cfg1", "cfg2", "cfg3", "cfg3full", "cfg4", "cfg4u", "cfg5", "latency", "ceilings", "sweep"])
    ap.add_argument("--mode", default=None, choices=["steps", "fused", "faithful"],
                    help="execution mode of the collective (default: per-step replay)")
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
                         "nt_load, nt_store, lds_pad*, launch_mib, gather_split, unroll_gather, gather_nt)")
    return ap.parse_args()


# ---------------------------------------------------------------------------
# workloads: each returns (run_step, info) with inputs resident on the GPU
# ---------------------------------------------------------------------------

def _randn_bf16(n, std, seed, device, out=None):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if out is None:
        out = torch.empty(n, dtype=torch.bfloat16, device=device)
    chunk = 1 << 26
    for i in range(0, n, chunk):      # bounded fp32 temporaries
        m = min(chunk, n - i)
        out[i:i + m] = (torch.randn(m, generator=g, device=device) * std).to(torch.bfloat16)
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


def make_ring_rs(P, elems_per_rank, dtype, mode, device, seed=1234, std=1.0):
    import torch
    from pccl import kernels
    B = elems_per_rank // P
    total = B * P
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    ins = _slab(P, total, tdt, device)
    for r in range(P):
        if dtype == "bf16":
            _randn_bf16(total, std, seed + r, device, out=ins[r])
        else:
            _rand_f32(total, seed + r, device, out=ins[r])
    es = 2 if dtype == "bf16" else 4
    outs = _slab(P, B, tdt, device)
    m = kernels.mode_code(mode)
    work = _slab(P, total, tdt, device) if m != kernels.MODE_FUSED and P > 2 else None

    def step():
        kernels.reduce_scatter_ranks(outs, ins, "ring", m, work)

    def verify():
        # the three execution modes must agree bit for bit
        ref = [torch.empty_like(o) for o in outs]
        other = kernels.MODE_FUSED if m != kernels.MODE_FUSED else kernels.MODE_STEPS
        w2 = work if work is not None else _slab(P, total, tdt, device)
        kernels.reduce_scatter_ranks(ref, ins, "ring", other, w2)
        torch.cuda.synchronize()
        return all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(outs, ref))

    launches = {kernels.MODE_STEPS: P - 1, kernels.MODE_FUSED: 1, kernels.MODE_FAITHFUL: P + 1}[m]
    if m == kernels.MODE_FUSED:
        kernel_bytes = (P * P + P) * B * es             # reads every input once, writes every output
        alg_bytes = kernel_bytes
        kernel = "k_reduce_kway"
    else:
        kernel_bytes = 3 * P * B * es                   # one batched step: 2 reads + 1 write per rank
        alg_bytes = (P - 1) * kernel_bytes
        kernel = "k_add_segs"
    info = dict(alg_bytes=alg_bytes, kernel=kernel, kernel_bytes=kernel_bytes,
                kernel_launches=(P - 1 if m != kernels.MODE_FUSED else 1), launches=launches,
                desc=f"ring reduce_scatter, P={P} virtual ranks, {dtype}, {total} elements per rank "
                     f"({total * es / MiB:.0f} MiB), block {B} elements, mode={_mode_name(m)}",
                dtype=dtype, P=P, B=B, verify=verify)
    return step, info


def _mode_name(m):
    return {0: "steps", 1: "fused", 2: "faithful"}[m]


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
        n = min(B, 1 << 24)
        lo = (ins[0][:n].float() + ins[1][:n].float()).bfloat16()
        hi = (ins[1][B:B + n].float() + ins[0][B:B + n].float()).bfloat16()
        return torch.equal(work[0][:n], lo) and torch.equal(work[1][B:B + n], hi)

    kb = 2 * 3 * B * 2
    info = dict(alg_bytes=kb, kernel="k_rh_round", kernel_bytes=kb, kernel_launches=1, launches=1,
                desc=f"recursive-halving round, one pair of ranks, bf16, halves of {B * 2 / MiB:.0f} MiB "
                     f"(round 0 of P=64 with {4 * B / MiB:.0f} MiB per rank)",
                dtype="bf16", P=2, B=B, verify=verify)
    return step, info


def make_rh_full(P, elems_per_rank, mode, device, seed=21):
    """Recursive-halving reduce_scatter with all P ranks resident."""
    import torch
    from pccl import kernels
    B = elems_per_rank // P
    total = B * P
    ins = _slab(P, total, torch.bfloat16, device)
    for r in range(P):
        _randn_bf16(total, 1.0, seed + r, device, out=ins[r])
    outs = _slab(P, B, torch.bfloat16, device)
    m = kernels.mode_code(mode)
    work = _slab(P, total, torch.bfloat16, device) if m != kernels.MODE_FUSED else None

    def step():
        kernels.reduce_scatter_ranks(outs, ins, "recursive", m, work)

    def verify():
        # the halving order of block 0 and block P-1 recomputed with torch on a window
        n = min(B, 1 << 20)
        for j in (0, P - 1):
            v = [ins[j ^ q][j * B:j * B + n].float() for q in range(P)]
            h = P // 2
            while h >= 1:
                for q in range(h):
                    v[q] = (v[q] + v[q + h]).bfloat16().float()
                h //= 2
            if not torch.equal(outs[j][:n].float(), v[0]):
                return False
        return True

    rounds = P.bit_length() - 1
    if m == kernels.MODE_FUSED:
        kb = (P * P + P) * B * 2
        alg, kernel, kl, launches = kb, "k_reduce_kway", 1, 1
    else:
        # round r adds (P / 2^(r+1)) blocks per rank: 2 reads + 1 write per element
        alg = sum(3 * P * (P >> (r + 1)) * B * 2 for r in range(rounds))
        kb, kernel, kl, launches = alg, "k_rh_round", 1, rounds
    info = dict(alg_bytes=alg, kernel=kernel, kernel_bytes=kb, kernel_launches=kl, launches=launches,
                desc=f"recursive-halving reduce_scatter, P={P} resident virtual ranks, bf16, {total} elements per "
                     f"rank ({total * 2 / MiB:.0f} MiB), {rounds} rounds, mode={_mode_name(m)}",
                dtype="bf16", P=P, B=B, verify=verify)
    return step, info


def make_all_gather(P, shard_bytes, mode, device, uneven=False, seed=3):
    import torch
    from pccl import kernels
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
    m = kernels.mode_code(mode if mode else "fused")

    if uneven:
        def step():
            kernels.all_gather_uneven_ranks(outs, ins, off)
        launches, kernel = 1, "k_gather_multicast"
    else:
        def step():
            kernels.all_gather_ranks(outs, ins, "ring", m)
        launches = 1 if m == kernels.MODE_FUSED else P
        kernel = "k_gather_multicast" if m == kernels.MODE_FUSED else "k_copy_segs"

    def verify():
        cat = torch.cat([t.view(torch.uint8) for t in ins]) if not uneven else None
        for o in (outs[0], outs[P - 1]):
            ob = o.view(torch.uint8)
            if uneven:
                for k in range(P):
                    if not torch.equal(ob[off[k]:off[k] + nbytes[k]], ins[k].view(torch.uint8)):
                        return False
            elif not torch.equal(ob, cat):
                return False
        return True

    payload = sum(nbytes)
    if kernel == "k_gather_multicast":
        # every shard is read once and written into each of the P outputs
        alg = (1 + P) * payload
        kb, kl = alg, 1
    else:
        alg = 2 * payload * P                   # 2 * bytes per materialised output, P outputs
        kb, kl = 2 * P * shard_bytes, P         # one batched step moves one shard per rank
    info = dict(alg_bytes=alg, kernel=kernel, kernel_bytes=kb, kernel_launches=kl, launches=launches,
                desc=f"all_gather placement, P={P} virtual ranks, bf16 shards of ~{shard_bytes / MiB:.0f} MiB"
                     f"{' (uneven, padded to 256 B)' if uneven else ''} into {total / MiB:.0f} MiB outputs, "
                     f"all {P} outputs materialised, mode={_mode_name(m) if not uneven else 'fused'}",
                dtype="bf16", P=P, B=n, verify=verify)
    return step, info


def make_kway(k, n, mode, device, seed=11):
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
    out = torch.empty(n, device=device)
    per_hop = kernels.mode_code(mode if mode else "fused") != kernels.MODE_FUSED

    def fused():
        kernels.reduce_kway(out, shards, "ring", 1 % k)

    def hops():
        kernels.add(out, shards[1 % k], shards[2 % k])
        for t in range(2, k):
            kernels.accumulate(out, shards[(1 + t) % k])

    step = hops if per_hop else fused

    def verify():
        got = out.clone()
        (fused if per_hop else hops)()          # the other way must give the same bits
        torch.cuda.synchronize()
        if not torch.equal(got.view(torch.int32), out.view(torch.int32)):
            return False
        m = min(n, 1 << 22)
        acc = shards[1 % k][:m].clone()
        for t in range(1, k):
            acc += shards[(1 + t) % k][:m]
        return torch.equal(got[:m], acc)

    if per_hop:
        kb = 3 * n * 4                                       # one hop: 2 reads + 1 write
        info = dict(alg_bytes=(k - 1) * kb, kernel="k_add_segs", kernel_bytes=kb, kernel_launches=k - 1,
                    launches=k - 1,
                    desc=f"reduce of {k} fp32 shards of {n} elements ({n * 4 / MiB:.0f} MiB each) as {k - 1} "
                         f"per-hop accumulate launches, ring order", dtype="f32", P=k, B=n, verify=verify)
    else:
        kb = (k + 1) * n * 4
        info = dict(alg_bytes=kb, kernel="k_reduce_kway", kernel_bytes=kb, kernel_launches=1, launches=1,
                    desc=f"fused one-pass reduce of {k} fp32 shards of {n} elements ({n * 4 / MiB:.0f} MiB each), "
                         f"ring order", dtype="f32", P=k, B=n, verify=verify)
    return step, info


def build_workload(name, mode, scale, device):
    def sc(x, q=1024):
        return max(q, int(x * scale) // q * q)
    if name == "cfg1":
        return make_ring_rs(4, sc(16 * MiB), "f32", mode, device)
    if name == "cfg2":
        return make_ring_rs(8, sc(256 * MiB), "bf16", mode, device, std=1e-2)
    if name == "cfg3":
        return make_rh_pair(sc(256 * MiB), device)
    if name == "cfg3full":
        return make_rh_full(64, sc(512 * MiB, 1 << 16), mode, device)
    if name == "cfg4":
        return make_all_gather(16, sc(128 * MiB), mode, device)
    if name == "cfg4u":
        return make_all_gather(16, sc(128 * MiB), mode, device, uneven=True)
    if name == "cfg5":
        return make_kway(32, sc(32 * MiB), mode, device)
    raise ValueError(name)


def ceilings(steps, warmup, device):
    """GB/s of pure read, pure write, copy and add streams over 1 GiB buffers."""
    import torch
    from pccl import _native, kernels
    lib = _native.load()
    n = 1 << 30
    a = torch.zeros(n, dtype=torch.uint8, device=device)
    b = torch.zeros(n, dtype=torch.uint8, device=device)
    c = torch.zeros(n, dtype=torch.uint8, device=device)
    fa, fb, fc = (t.view(torch.float32) for t in (a, b, c))

    def gbps(fn, nbytes):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return round(nbytes / (s.elapsed_time(e) / steps * 1e-3) / 1e9, 1)

    st = kernels.stream_handle()
    return {
        "read_only": gbps(lambda: lib.probe_stream(0, a.data_ptr(), n, st), n),
        "write_only": gbps(lambda: lib.probe_stream(1, c.data_ptr(), n, st), n),
        "copy": gbps(lambda: kernels.copy(c, a), 2 * n),
        "add_2r1w_f32": gbps(lambda: kernels.add(fc, fa, fb), 3 * n),
        "torch_copy_": gbps(lambda: c.copy_(a), 2 * n),
        "torch_add_f32": gbps(lambda: torch.add(fa, fb, out=fc), 3 * n),
    }


def size_sweep(steps, warmup, device):
    """Achieved GB/s of the per-hop, copy and fused kernels against message size."""
    import torch
    from pccl import kernels

    def gbps(fn, nbytes):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return round(nbytes / (s.elapsed_time(e) / steps * 1e-3) / 1e9, 1)

    rows = []
    for mib in (64, 128, 256, 512, 1024, 2048):
        nb = mib * MiB
        a16, b16 = _randn_bf16(nb // 2, 1e-2, 1, device), _randn_bf16(nb // 2, 1e-2, 2, device)
        a32, b32 = a16.view(torch.float32), b16.view(torch.float32)
        c = torch.empty_like(a16)
        k = 8
        shards = [_randn_bf16(nb // 2 // k, 1e-2, 10 + i, device) for i in range(k)]
        out = torch.empty_like(shards[0])
        rows.append({
            "MiB": mib,
            "accumulate_bf16": gbps(lambda: kernels.accumulate(a16, b16), 3 * nb),
            "accumulate_f32": gbps(lambda: kernels.accumulate(a32, b32), 3 * nb),
            "copy": gbps(lambda: kernels.copy(c, a16), 2 * nb),
            "reduce_8way_bf16_total_input": gbps(lambda: kernels.reduce_kway(out, shards, "ring", 1), (k + 1) * nb // k),
        })
        del a16, b16, a32, b32, c, shards, out
    return rows


def latency_sweep(steps, warmup, device):
    """Microseconds per call for launch-bound message sizes (bf16)."""
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
        work = [torch.empty_like(t) for t in ins]
        graph = torch.cuda.CUDAGraph()             # the 7 step launches captured once
        kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)
        plan_fused = kernels.plan_reduce_scatter(outs, ins, "ring", "fused")
        plan_steps = kernels.plan_reduce_scatter(outs, ins, "ring", "steps", work)
        rows.append({
            "bytes": nbytes,
            "accumulate_us": round(us(lambda: kernels.accumulate(x, y)), 2),
            "copy_us": round(us(lambda: kernels.copy(z, x)), 2),
            "ring_rs_p8_steps_us": round(us(lambda: kernels.reduce_scatter_ranks(outs, ins, "ring", "steps", work)), 2),
            "ring_rs_p8_steps_graph_us": round(us(graph.replay), 2),
            "ring_rs_p8_steps_plan_us": round(us(plan_steps), 2),
            "ring_rs_p8_fused_plan_us": round(us(plan_fused), 2),
            "ring_rs_p8_fused_us": round(us(lambda: kernels.reduce_scatter_ranks(outs, ins, "ring", "fused")), 2),
        })
    return rows


# ---------------------------------------------------------------------------
# CPU baseline (oracle/cpu_baseline.c), bounded sample
# ---------------------------------------------------------------------------

def cpu_baseline(info):
    """Time the reference's per-rank ring reduce_scatter on host cores for a
    bounded sample of the workload (same P and dtype, shorter blocks)."""
    build = os.path.join(ROOT, "oracle", "build")
    mpi_bin = os.path.join(build, "cpu_baseline_mpi")
    shm_bin = os.path.join(build, "cpu_baseline_shm")
    if not os.path.exists(shm_bin):
        try:
            subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
        except Exception as e:                               # noqa: BLE001
            return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": f"not built: {e}"}
    P = info["P"] if info["kernel"] in ("k_add_segs", "k_reduce_kway") and info["P"] <= 8 else 8
    dtype = "bf16" if info["dtype"] == "bf16" else "f32"
    host_cores = os.cpu_count() or 1
    ranks = min(P, max(1, host_cores))
    if ranks & (ranks - 1):
        ranks = 1 << (ranks.bit_length() - 1)
    if info["kernel"] == "k_add_segs" and ranks == info["P"]:
        block, sample = info["B"], "the workload itself (same P, dtype and block size)"
    else:
        block = (1 << 22) if dtype == "bf16" else (1 << 21)                 # 8 MiB blocks
        sample = "a ring reduce_scatter of the same dtype with 8 MiB blocks"
    # about ten seconds of timed calls, assuming ~15 GB/s of algorithmic bytes on the host
    job_bytes = 3 * (ranks - 1) * block * (2 if dtype == "bf16" else 4) * ranks
    iters = max(5, min(500, int(10.0 / max(job_bytes / 15e9, 1e-3))))
    args = ["--alg", "ring", "--dtype", dtype, "--block", str(block), "--warmup", "1", "--iters", str(iters),
            "--scale", "0.01" if dtype == "bf16" else "1.0"]
    launcher = None
    for cand in ("/opt/conda/bin/mpiexec.hydra", shutil.which("mpiexec.hydra"), shutil.which("mpiexec")):
        if cand and os.path.exists(cand):
            launcher = cand
            break
    attempts = []
    if launcher and os.path.exists(mpi_bin):
        attempts.append(([launcher, "-np", str(ranks), mpi_bin] + args, "MPI_Sendrecv (MPICH)"))
    attempts.append(([shm_bin, "--ranks", str(ranks)] + args, "fork+shared memory"))
    for cmd, transport in attempts:
        try:
            t0 = time.time()
            p = subprocess.run(cmd, capture_output=True, text=True, timeout=400)
            line = [l for l in p.stdout.splitlines() if l.startswith("{")]
            if p.returncode == 0 and line:
                r = json.loads(line[-1])
                vendor = None
                if dtype == "f32" and cmd[0] == launcher:
                    # the vendor collective the reference reaches with --library mpi
                    # --pccl-disable-cpp-backend (pccl/reduce_scatter.py:197), same shape
                    vcmd = [a if a != "ring" else "mpi_block" for a in cmd]
                    try:
                        pv = subprocess.run(vcmd, capture_output=True, text=True, timeout=400)
                        vl = [l for l in pv.stdout.splitlines() if l.startswith("{")]
                        if pv.returncode == 0 and vl:
                            vendor = round(json.loads(vl[-1])["GBps"], 3)
                    except Exception:                         # noqa: BLE001
                        vendor = None
                return {"value": round(r["GBps"], 3), "unit": "GB/s", "cores": ranks, "kind": "port",
                        "mpi_reduce_scatter_block_GBps": vendor,
                        "ms_per_call": round(r["ms_per_call"], 3), "host_cores": host_cores,
                        "sample": f"{sample}: ring reduce_scatter of the reference "
                                  f"(pccl/src/reduce_scatter.cpp:101-155) on host buffers, {ranks} ranks = {ranks} "
                                  f"processes over {transport}, {dtype}, {block} elements per block "
                                  f"({ranks * block} per rank), 1 warm-up + {iters} timed calls, "
                                  f"{time.time() - t0:.1f} s wall"}
        except Exception:                                     # noqa: BLE001
            continue
    return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "baseline program failed"}


# ---------------------------------------------------------------------------

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
            "config": {"workload": "ceilings: plain streams over 1 GiB buffers; value = the library's add kernel",
                       "GBps": res}, "roofline": None, "cpu_baseline": None}), flush=True)
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
                       "latency_us": rows}, "roofline": None, "cpu_baseline": None}), flush=True)
        return 0

    step, info = build_workload(args.workload, args.mode, args.scale, device)
    torch.cuda.synchronize()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()           # the stream the library launches on
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    launches0 = lib.launch_count()
    start.record(stream)
    for _ in range(args.steps):
        step()
    end.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    dev_ms = start.elapsed_time(end)
    # a step of a schedule goes out as several launches of bounded size (launch_mib)
    launched = (lib.launch_count() - launches0) / args.steps
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
        ok = bool(info["verify"]())

    # the timed region holds nothing but the dominant kernel's launches (plus, in
    # faithful mode, the copies), so its mean launch time is region / launches and
    # the bytes of a mean launch are the step's kernel bytes / launches
    if info["launches"] == info["kernel_launches"] or info["kernel_bytes"] == info["alg_bytes"]:
        step_kernel_bytes = (info["kernel_bytes"] * info["kernel_launches"]
                             if info["launches"] == info["kernel_launches"] else info["kernel_bytes"])
        kernel_ms = dev_ms / (args.steps * launched)
        launch_bytes = step_kernel_bytes / launched
    else:
        kernel_ms = None
    roof = None
    if kernel_ms:
        achieved = launch_bytes / (kernel_ms * 1e-3) / 1e9
        traffic = None
        tfile = os.path.join(ROOT, "profiles", "traffic.json")
        if os.path.exists(tfile):
            try:
                traffic = json.load(open(tfile)).get(f"{args.workload}:{info['kernel']}")
            except Exception:                                 # noqa: BLE001
                traffic = None
        roof = {"bound": "hbm", "kernel": info["kernel"], "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": traffic, "bytes_per_launch": int(round(launch_bytes)),
                "avg_launch_ms": round(kernel_ms, 5)}

    cpu = None if args.no_cpu_baseline else cpu_baseline(info)

    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": info["dtype"], "data": "synthetic",
        "config": {"workload": f"{args.workload}: {info['desc']}", "algorithmic_bytes_per_step": info["alg_bytes"],
                   "launches_per_step": launched, "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
                   "wall_ms_per_step": round(wall_ms / args.steps, 4), "verified": ok, "layout": LAYOUT,
                   "tuning": {k: lib.get_tuning(k) for k in ("grid_cap", "unroll", "unroll_copy", "nt_load", "nt_store", "launch_mib")}},
        "roofline": roof, "cpu_baseline": cpu,
    }
    print(json.dumps(out), flush=True)
    return 0 if ok in (None, True) else 1


if __name__ == "__main__":
    sys.exit(main())
