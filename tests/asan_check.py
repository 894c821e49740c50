"""Run by tests/test_sanitizer.py in a child process with the AddressSanitizer
runtime preloaded: drives the ASan-instrumented CPU build of the library over
numpy buffers whose sizes leave no slack, so any out-of-bounds access of a
kernel aborts the process.  Shapes: ragged, empty, misaligned, every mode."""
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
spec = importlib.util.spec_from_file_location(
    "pccl_native", os.path.join(ROOT, "sc2025-pccl-reproducer_amd", "pccl", "_native.py"))
nat = importlib.util.module_from_spec(spec)
spec.loader.exec_module(nat)
from oracle import pccl_oracle as O  # noqa: E402

lib = nat.NativeLib(sys.argv[1])
rng = np.random.default_rng(0)


def arr(n, dtype):
    x = rng.standard_normal(n).astype(np.float32)
    return x if dtype == O.F32 else O.f32_to_bf16(x)


def ptr(a, shift=0):
    return a.ctypes.data + shift * a.itemsize


checked = 0
# the fused reduce with one-wave workgroups and loads in pairs (what streams from HBM get), and the general add
# kernels on aligned data (add_rows = 0): forced here, on exact-size buffers
lib.set_tuning("wg_kway", 64); lib.set_tuning("nt_load", 1); lib.set_tuning("nt_store", 1); lib.set_tuning("add_rows", 0)
for dtype, code in ((O.F32, 0), (O.BF16, 1)):
    for P in (2, 3, 4, 8, 16):
        for B in (1, 7, 64, 1024, 4099):
            for alg in ("ring", "recursive"):
                if alg == "recursive" and P & (P - 1):
                    continue
                ins = [arr(P * B, dtype) for _ in range(P)]
                want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
                for mode in (0, 1):
                    outs = [np.zeros(B, ins[0].dtype) for _ in range(P)]
                    work = [np.zeros(P * B, ins[0].dtype) for _ in range(P)]
                    lib.reduce_scatter_virtual([ptr(o) for o in outs], [ptr(i) for i in ins],
                                               [ptr(w) for w in work], B, code, alg, mode)
                    for r in range(P):
                        assert np.array_equal(outs[r].view(np.uint8), want[r].view(np.uint8)), (dtype, P, B, alg, mode)
                    checked += 1
lib.set_tuning("wg_kway", -1); lib.set_tuning("nt_load", -1); lib.set_tuning("nt_store", -1); lib.set_tuning("add_rows", 1)
for unroll in (1, 4, 8):
    lib.set_tuning("unroll", unroll)
    for dtype, code in ((O.F32, 0), (O.BF16, 1)):
        for P in (1, 2, 3, 4, 8):
            for B in (1, 7, 1024, 4099):
                for alg in ("ring", "recursive"):
                    if alg == "recursive" and P & (P - 1):
                        continue
                    ins = [arr(P * B, dtype) for _ in range(P)]
                    want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
                    for mode in (0, 1, 2):
                        outs = [np.zeros(B, ins[0].dtype) for _ in range(P)]
                        work = [np.zeros(P * B, ins[0].dtype) for _ in range(P)]
                        lib.reduce_scatter_virtual([ptr(o) for o in outs], [ptr(i) for i in ins],
                                                   [ptr(w) for w in work], B, code, alg, mode)
                        for r in range(P):
                            assert np.array_equal(outs[r].view(np.uint8), want[r].view(np.uint8)), (dtype, P, B, alg, mode)
                        checked += 1
        # misaligned single adds: exact-size views into exact-size arrays
        for n in (1, 5, 33, 5000):
            for sd, sa, sb in ((0, 0, 0), (1, 1, 1), (1, 2, 3), (3, 0, 1)):
                a, b = arr(n + sa, dtype), arr(n + sb, dtype)
                d = np.zeros(n + sd, a.dtype)
                lib.add(ptr(d, sd), ptr(a, sa), ptr(b, sb), n, code)
                assert np.array_equal(d[sd:].view(np.uint8), O.vector_add(a[sa:], b[sb:], dtype).view(np.uint8))
                checked += 1
    for P in (1, 2, 4, 8, 3, 5):
        for blk in (1, 3, 17, 4096 + 7, 70001):
            for alg in ("ring", "recursive"):
                if alg == "recursive" and P & (P - 1):
                    continue
                ins = [rng.integers(0, 256, blk, dtype=np.uint8) for _ in range(P)]
                cat = np.concatenate(ins)
                for mode in (0, 1):
                    outs = [np.zeros(P * blk, np.uint8) for _ in range(P)]
                    lib.all_gather_virtual([ptr(o) for o in outs], [ptr(i) for i in ins], blk, alg, mode)
                    for o in outs:
                        assert np.array_equal(o, cat)
                    checked += 1
    # 2-D with folded permutations, and uneven gather
    for intra, inter in ((1, 1), (2, 2), (4, 2), (2, 3), (3, 1), (1, 4)):
        W = intra * inter
        for m in (1, 9, 1030):
            for alg in ("ring", "recursive"):
                if alg == "recursive" and ((intra & (intra - 1)) or (inter & (inter - 1))):
                    continue
                ins = [arr(W * m, O.BF16) for _ in range(W)]
                want = O.reduce_scatter_2d(ins, intra, inter, O.BF16, alg)
                for mode in (0, 1):
                    outs = [np.zeros(m, np.uint16) for _ in range(W)]
                    work = [np.zeros(W * m, np.uint16) for _ in range(W)]
                    mid = [np.zeros(inter * m, np.uint16) for _ in range(W)]
                    lib.reduce_scatter_2d_virtual([ptr(o) for o in outs], [ptr(i) for i in ins], [ptr(w) for w in work],
                                                  [ptr(x) for x in mid], intra, inter, m, 1, alg, mode)
                    for w in range(W):
                        assert np.array_equal(outs[w], want[w]), (intra, inter, m, alg, mode)
                    gouts = [np.zeros(W * m, np.uint16) for _ in range(W)]
                    lib.all_gather_2d_virtual([ptr(g) for g in gouts], [ptr(o) for o in outs], [ptr(x) for x in mid],
                                              intra, inter, 2 * m, alg, mode)
                    for g in gouts:
                        assert np.array_equal(g, np.concatenate(want))
                    checked += 1
    lens = [5, 0, 4097, 33, 70000]
    shards = [rng.integers(0, 256, n, dtype=np.uint8) for n in lens]
    off, o = [], 0
    for n in lens:
        off.append(o)
        o += (n + 255) // 256 * 256
    outs = [np.zeros(off[-1] + lens[-1], np.uint8) for _ in lens]       # no slack behind the last shard
    lib.all_gather_uneven_virtual([ptr(x) for x in outs], [ptr(s) if s.size else 0 for s in shards], lens, off)
    for x in outs:
        for k, n in enumerate(lens):
            assert np.array_equal(x[off[k]:off[k] + n], shards[k])
    checked += 1
# the time-blocked placement kernel (chosen for long shards by default: forced here), every tile count per workgroup
lib.set_tuning("gather_strip_from", 0)
cases = [(ug, strip, P, blk) for ug in (0, 1, 8) for strip in (-1, 3) for P in (2, 5) for blk in (17, 4096 + 7, 70001)]
cases += [(0, -1, 16, 4096 + 7), (2, 1, 3, 1), (0, 160, 2, 70001)]
for ug, strip, P, blk in cases:
    lib.set_tuning("unroll_gather", ug)
    lib.set_tuning("gather_strip", strip)
    ins = [rng.integers(0, 256, blk, dtype=np.uint8) for _ in range(P)]
    outs = [np.zeros(P * blk, np.uint8) for _ in range(P)]
    lib.all_gather_virtual([ptr(o) for o in outs], [ptr(i) for i in ins], blk, "ring", 1)
    for o in outs:
        assert np.array_equal(o, np.concatenate(ins))
    checked += 1
for ug, strip in ((0, -1), (1, 3), (8, 2)):
    lib.set_tuning("unroll_gather", ug)
    lib.set_tuning("gather_strip", strip)
    outs = [np.zeros(off[-1] + lens[-1], np.uint8) for _ in lens]
    lib.all_gather_uneven_virtual([ptr(x) for x in outs], [ptr(s) if s.size else 0 for s in shards], lens, off)
    for x in outs:
        for k, n in enumerate(lens):
            assert np.array_equal(x[off[k]:off[k] + n], shards[k])
    checked += 1
lib.set_tuning("gather_strip", -1); lib.set_tuning("gather_strip_from", -1); lib.set_tuning("unroll_gather", 0)

# fused modes beyond the ranks of one launch, and the entry point with built-in work buffers
for alg, P, B in (("ring", 65, 5), ("recursive", 128, 3)):
    ins = [arr(P * B, O.BF16) for _ in range(P)]
    want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, O.BF16)
    outs = [np.zeros(B, np.uint16) for _ in range(P)]
    work = [np.zeros(P * B, np.uint16) for _ in range(P)]
    lib.reduce_scatter_virtual([ptr(o) for o in outs], [ptr(i) for i in ins], [ptr(w) for w in work], B, 1, alg, 1)
    for r in range(P):
        assert np.array_equal(outs[r], want[r]), (alg, P, r)
    gouts = [np.zeros(P * B, np.uint16) for _ in range(P)]
    lib.all_gather_virtual([ptr(g) for g in gouts], [ptr(o) for o in outs], 2 * B, alg, 1)
    for g in gouts:
        assert np.array_equal(g, np.concatenate(want))
    checked += 1
for alg, P, B in (("ring", 8, 4099), ("recursive", 4, 515), ("ring", 3, 1)):
    for dtype, code in ((O.F32, 0), (O.BF16, 1)):
        ins = [arr(P * B, dtype) for _ in range(P)]
        want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
        outs = [np.zeros(B, ins[0].dtype) for _ in range(P)]
        lib.reduce_scatter_virtual_noalloc([ptr(o) for o in outs], [ptr(i) for i in ins], B, code, alg)
        for r in range(P):
            assert np.array_equal(outs[r].view(np.uint8), want[r].view(np.uint8)), (alg, P, dtype, r)
        checked += 1

# the measurement probes on exact-size buffers
for nb in (4096, 4096 * 5 + 16, 70000 // 16 * 16):
    bufs = [np.zeros(nb, np.uint8) for _ in range(4)]
    if nb >= 16384:
        lib.probe_stream(0, ptr(bufs[0]), nb)
        lib.probe_stream(1, ptr(bufs[1]), nb)
    for shape in (0, 1, 2, 3):
        for vec in (1, 2, 4):
            lib.probe_mix([ptr(bufs[0]), ptr(bufs[1])], [ptr(bufs[2]), ptr(bufs[3])], nb, shape, vec)
            lib.probe_mix([ptr(bufs[0])], [], nb, shape, vec)
            lib.probe_mix([], [ptr(bufs[3])], nb, shape, vec)
            checked += 1
print(f"ASAN CHECK OK ({checked} cases)")
