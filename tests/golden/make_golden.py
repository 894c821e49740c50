#!/usr/bin/env python3
"""Writes the golden vectors in this folder from the CPU oracle.

The reference ships no fixtures (its only check is an allclose against NCCL on
unseeded inputs, benchmark_raw_collectives/utils.py:35-42), so these vectors
come from this repository's oracle (oracle/pccl_oracle.py), whose schedules
are pinned independently by the closed forms in tests/test_oracle.py.  Each
.npz holds the inputs of every rank and the expected output of every rank:
    in_<r>   rank r's input   (float32, or uint16 bfloat16 / binary16 bit patterns)
    out_<r>  rank r's output
    meta     JSON: collective, algorithm, dtype, P, block elements; for the 2-D
             collectives also the grid (intra, inter), for the uneven all_gather
             the shard lengths and byte offsets
Run:  python tests/golden/make_golden.py         (writes the files that are missing)
      python tests/golden/make_golden.py --all   (rewrites every file)
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import pccl_oracle as O  # noqa: E402


def inputs(P, n, dtype, seed, kind):
    xs = []
    for r in range(P):
        rng = np.random.default_rng(seed + r)
        if kind == "uniform":                      # the P=4 fp32 workload: uniform[-1, 1], seed + rank
            x = (rng.random(n, dtype=np.float32) * 2 - 1)
        elif kind == "grad":                       # the P=8 bf16 workload: normal(0, 1e-2)
            x = rng.standard_normal(n, dtype=np.float32) * np.float32(1e-2)
        else:                                      # normal(0, 1)
            x = rng.standard_normal(n, dtype=np.float32)
        xs.append(x if dtype == O.F32 else O.f32_to_bf16(x) if dtype == O.BF16 else O.f32_to_f16(x))
    return xs


CASES = [
    # name, collective, algorithm, dtype, P, B, input kind
    ("rs_ring_p4_f32_uniform", "reduce_scatter", "ring", O.F32, 4, 48, "uniform"),
    ("rs_ring_p8_bf16_grad", "reduce_scatter", "ring", O.BF16, 8, 40, "grad"),
    ("rs_ring_p3_bf16", "reduce_scatter", "ring", O.BF16, 3, 19, "normal"),
    ("rs_halving_p8_bf16", "reduce_scatter", "recursive", O.BF16, 8, 24, "normal"),
    ("rs_halving_p4_f32", "reduce_scatter", "recursive", O.F32, 4, 33, "normal"),
    ("rs_halving_p2_f32", "reduce_scatter", "recursive", O.F32, 2, 64, "uniform"),
    ("ag_doubling_p8_bf16", "all_gather", "recursive", O.BF16, 8, 21, "normal"),
    ("ag_ring_p5_f32", "all_gather", "ring", O.F32, 5, 7, "normal"),
    ("ar_halving_p4_f32", "all_reduce", "recursive", O.F32, 4, 13, "normal"),
    ("ar_ring_p3_bf16", "all_reduce", "ring", O.BF16, 3, 11, "grad"),
    ("rs_ring_p4_f16", "reduce_scatter", "ring", O.F16, 4, 35, "normal"),
    ("rs_halving_p8_f16_grad", "reduce_scatter", "recursive", O.F16, 8, 18, "grad"),
    ("ar_ring_p3_f16", "all_reduce", "ring", O.F16, 3, 14, "normal"),
]

GRID_CASES = [
    # name, collective, algorithm, dtype, intra, inter, elements per output block, input kind
    ("rs2d_halving_2x2_bf16", "reduce_scatter_2d", "recursive", O.BF16, 2, 2, 17, "normal"),
    ("rs2d_ring_3x2_f32", "reduce_scatter_2d", "ring", O.F32, 3, 2, 9, "uniform"),
    ("rs2d_halving_4x2_f32", "reduce_scatter_2d", "recursive", O.F32, 4, 2, 5, "grad"),
    ("ag2d_doubling_2x4_bf16", "all_gather_2d", "recursive", O.BF16, 2, 4, 6, "normal"),
    ("ag2d_ring_3x2_f32", "all_gather_2d", "ring", O.F32, 3, 2, 10, "normal"),
    ("rs2d_ring_2x3_f16", "reduce_scatter_2d", "ring", O.F16, 2, 3, 11, "normal"),
]

UNEVEN_CASES = [
    # name, shard lengths in bytes, gap between shards in bytes
    ("ag_uneven_p5", [37, 0, 4096, 1, 513], 3),
    ("ag_uneven_p3_packed", [100, 7, 64], 0),
]


def wanted(name):
    return "--all" in sys.argv or not os.path.exists(os.path.join(HERE, name + ".npz"))


def save(name, arrays, meta):
    arrays["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    np.savez(os.path.join(HERE, name + ".npz"), **arrays)
    print("wrote", name)


def main():
    for name, coll, alg, dtype, P, B, kind in CASES:
        if not wanted(name):
            continue
        if coll == "reduce_scatter":
            xs = inputs(P, P * B, dtype, 1234, kind)
            fn = O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter
            outs = fn(xs, dtype)
        elif coll == "all_reduce":
            xs = inputs(P, P * B, dtype, 1234, kind)
            outs = O.all_reduce(xs, dtype, alg)
        else:
            xs = inputs(P, B, dtype, 1234, kind)
            fn = O.ring_all_gather if alg == "ring" else O.recursive_doubling_all_gather
            outs = [o.view(xs[0].dtype) for o in fn(xs)]
        arrays = {f"in_{r}": xs[r] for r in range(P)}
        arrays.update({f"out_{r}": outs[r] for r in range(P)})
        meta = dict(collective=coll, algorithm=alg, dtype=dtype, P=P, B=B, inputs=kind)
        save(name, arrays, meta)
    for name, coll, alg, dtype, intra, inter, m, kind in GRID_CASES:
        if not wanted(name):
            continue
        W = intra * inter
        if coll == "reduce_scatter_2d":
            xs = inputs(W, W * m, dtype, 4321, kind)
            outs = O.reduce_scatter_2d(xs, intra, inter, dtype, alg)
        else:
            xs = inputs(W, m, dtype, 4321, kind)
            outs = [o.view(xs[0].dtype) for o in O.all_gather_2d(xs, intra, inter, alg)]
        arrays = {f"in_{r}": xs[r] for r in range(W)}
        arrays.update({f"out_{r}": outs[r] for r in range(W)})
        save(name, arrays, dict(collective=coll, algorithm=alg, dtype=dtype, P=W, B=m, intra=intra, inter=inter,
                                inputs=kind))
    for name, nbytes, gap in UNEVEN_CASES:
        if not wanted(name):
            continue
        P = len(nbytes)
        xs = [np.random.default_rng(99 + r).integers(0, 256, n, dtype=np.uint8) for r, n in enumerate(nbytes)]
        off = [int(v) for v in np.cumsum([0] + [n + gap for n in nbytes[:-1]])]
        total = off[-1] + nbytes[-1] + gap
        outs = O.uneven_all_gather(xs, off, total)       # bytes outside the shards hold 0xA5
        arrays = {f"in_{r}": xs[r] for r in range(P)}
        arrays.update({f"out_{r}": outs[r] for r in range(P)})
        save(name, arrays, dict(collective="all_gather_uneven", algorithm="ring", dtype="u8", P=P, nbytes=nbytes,
                                dst_off=off, total=total, fill=0xA5))


if __name__ == "__main__":
    main()
