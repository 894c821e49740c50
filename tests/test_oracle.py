"""Pins the CPU oracle without the reference's code.

The reference holds no golden vectors or unit tests, so every part of the
oracle is checked against something a plausible mistake would break:
library arithmetic (numpy / torch CPU), closed-form summation orders written
independently of the simulation, exact integer sums, schedule invariants,
special cases, a second restatement in C, and the committed fixtures."""
import glob
import json
import os
import subprocess

import numpy as np
import pytest

from helpers import assert_bits_equal, grid_closed_form, halving_closed_form, make_inputs, ring_closed_form
from oracle import pccl_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [O.F32, O.BF16]


# ---- element arithmetic ------------------------------------------------------

def test_bf16_rounding_matches_torch_for_every_upper_half_and_tie_pattern():
    import torch
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1).astype(np.uint32)
    x = bits.view(np.float32)
    want = torch.from_numpy(x.copy()).bfloat16().view(torch.int16).numpy().view(np.uint16)
    got = O.f32_to_bf16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN stays NaN in both; the oracle uses the canonical pattern
    assert (got[nan] == 0x7FC0).all()
    assert np.isnan(O.bf16_to_f32(want[nan])).all()


def test_bf16_rounding_against_exact_arithmetic():
    """RNE by definition: the nearer of the two neighbouring bf16 values, ties
    to the one with an even mantissa; done in float64 on finite normal values."""
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-20, 20, 20000))).astype(np.float32)
    got = O.bf16_to_f32(O.f32_to_bf16(x)).astype(np.float64)
    down = (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32).astype(np.float64)
    up_bits = (x.view(np.uint32) & np.uint32(0xFFFF0000)) + np.uint32(0x10000)
    up = up_bits.view(np.float32).astype(np.float64)
    xd = x.astype(np.float64)
    d_down, d_up = np.abs(xd - down), np.abs(up - xd)
    even_down = ((x.view(np.uint32) >> 16) & 1) == 0
    want = np.where(d_down < d_up, down, np.where(d_up < d_down, up, np.where(even_down, down, up)))
    assert np.array_equal(got, want)


def test_bf16_add_is_torch_add():
    """The hop arithmetic of the Python algorithms: torch.add on bfloat16."""
    import torch
    a = np.arange(65536, dtype=np.uint16)
    partners = np.concatenate([np.arange(0, 65536, 1024, dtype=np.uint16) | np.uint16(0x35),
                               np.array([0x0000, 0x8000, 0x7F80, 0xFF80, 0x0001, 0x7F7F], np.uint16)])
    A = np.tile(a, partners.size)
    B = np.repeat(partners, a.size)
    ta = torch.from_numpy(A.view(np.int16).copy()).view(torch.bfloat16)
    tb = torch.from_numpy(B.view(np.int16).copy()).view(torch.bfloat16)
    want = torch.add(ta, tb).view(torch.int16).numpy().view(np.uint16)
    got = O.vector_add(A, B, O.BF16)
    nan = np.isnan(O.bf16_to_f32(want))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(O.bf16_to_f32(got[nan])).all()


def test_f32_add_is_ieee_binary32():
    import torch
    rng = np.random.default_rng(1)
    a = (rng.standard_normal(100000) * np.exp(rng.uniform(-30, 30, 100000))).astype(np.float32)
    b = (rng.standard_normal(100000) * np.exp(rng.uniform(-30, 30, 100000))).astype(np.float32)
    want = (torch.from_numpy(a) + torch.from_numpy(b)).numpy()
    assert_bits_equal(O.vector_add(a, b, O.F32), want)
    # and it is NOT the float64 sum rounded late (double rounding would differ somewhere)
    assert_bits_equal(O.vector_add(a, b, O.F32), (a.astype(np.float64) + b.astype(np.float64)).astype(np.float32))


# ---- ring reduce_scatter -------------------------------------------------------

@pytest.mark.parametrize("P", range(1, 17))
def test_ring_schedule_invariants(P):
    """Index algebra of pccl/src/reduce_scatter.cpp:127-146."""
    for step in range(P - 1):
        for r in range(P):
            send_idx = (r - step - 1) % P
            recv_idx_right = ((r + 1) - step - 2) % P
            assert send_idx == recv_idx_right          # what r sends is what r+1 reduces into
    for r in range(P):
        touched = [(r - step - 2) % P for step in range(P - 1)]
        assert len(set(touched)) == P - 1              # every block but one reduced exactly once
        if P > 1:
            assert touched[-1] == r                    # the last one is the rank's own block
            assert (r - 1) % P not in touched          # block r-1 is only ever sent


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P", [1, 2, 3, 4, 5, 7, 8, 12, 16])
def test_ring_equals_left_fold_from_rank_j_plus_1(dtype, P):
    ins = make_inputs(P, P * 37, dtype, seed=2)
    got = O.ring_reduce_scatter(ins, dtype)
    want = ring_closed_form(ins, dtype)
    for r in range(P):
        assert_bits_equal(got[r], want[r], f"block {r}")


def test_ring_order_matters_so_the_closed_form_has_teeth():
    """A fold that starts at rank j (a plausible off-by-one) gives other bits."""
    P, B = 8, 4096
    ins = make_inputs(P, P * B, O.F32, seed=4)
    right = ring_closed_form(ins, O.F32)
    diff = 0
    for j in range(P):
        acc = ins[j][j * B:(j + 1) * B]
        for t in range(1, P):
            acc = O.vector_add(acc, ins[(j + t) % P][j * B:(j + 1) * B], O.F32)
        diff += int((acc.view(np.uint32) != right[j].view(np.uint32)).sum())
    assert diff > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_p2_is_one_add(dtype):
    a, b = make_inputs(2, 2 * 100, dtype, seed=6)
    for fn in (O.ring_reduce_scatter, O.recursive_halving_reduce_scatter):
        out = fn([a, b], dtype)
        assert_bits_equal(out[0], O.vector_add(a[:100], b[:100], dtype))
        assert_bits_equal(out[1], O.vector_add(a[100:], b[100:], dtype))


# ---- recursive halving --------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P", [1, 2, 4, 8, 16, 32, 64])
def test_halving_equals_xor_butterfly(dtype, P):
    ins = make_inputs(P, P * 11, dtype, seed=8)
    got = O.recursive_halving_reduce_scatter(ins, dtype)
    want = halving_closed_form(ins, dtype)
    for r in range(P):
        assert_bits_equal(got[r], want[r], f"block {r}")


def test_halving_differs_from_ring_in_rounding_only():
    P, B = 8, 2048
    ins = make_inputs(P, P * B, O.F32, seed=9)
    ring = O.ring_reduce_scatter(ins, O.F32)
    halv = O.recursive_halving_reduce_scatter(ins, O.F32)
    exact = np.sum(np.stack(ins).astype(np.float64), axis=0)
    ndiff = 0
    for r in range(P):
        ndiff += int((ring[r].view(np.uint32) != halv[r].view(np.uint32)).sum())
        for got in (ring[r], halv[r]):
            assert np.allclose(got, exact[r * B:(r + 1) * B], rtol=1e-5, atol=1e-6)
    assert ndiff > 0        # different association -> different bits somewhere


@pytest.mark.parametrize("fn", [O.ring_reduce_scatter, O.recursive_halving_reduce_scatter])
@pytest.mark.parametrize("dtype", DTYPES)
def test_integer_inputs_sum_exactly(fn, dtype):
    P, B = 8, 50
    ins = make_inputs(P, P * B, dtype, seed=10, dist="int")
    as_f = [x if dtype == O.F32 else O.bf16_to_f32(x) for x in ins]
    total = np.sum(np.stack(as_f).astype(np.float64), axis=0)
    outs = fn(ins, dtype)
    for r in range(P):
        got = outs[r] if dtype == O.F32 else O.bf16_to_f32(outs[r])
        assert np.array_equal(got.astype(np.float64), total[r * B:(r + 1) * B])


def test_reduce_scatter_rejects_bad_shapes():
    with pytest.raises(ValueError, match="divisible"):
        O.ring_reduce_scatter([np.zeros(10, np.float32)] * 3, O.F32)
    with pytest.raises(ValueError, match="power-of-two"):
        O.recursive_halving_reduce_scatter([np.zeros(9, np.float32)] * 3, O.F32)


# ---- all_gather -------------------------------------------------------------

@pytest.mark.parametrize("P", [1, 2, 4, 8, 16, 32])
@pytest.mark.parametrize("blk", [1, 7, 64])
def test_doubling_all_gather_is_concatenation(P, blk):
    rng = np.random.default_rng(P * 100 + blk)
    ins = [rng.integers(0, 256, blk, dtype=np.uint8) for _ in range(P)]
    outs = O.recursive_doubling_all_gather(ins, fill=0xEE)
    cat = np.concatenate(ins)
    for o in outs:
        assert np.array_equal(o, cat)


@pytest.mark.parametrize("P", range(1, 12))
def test_ring_all_gather_is_concatenation_and_keeps_its_invariant(P):
    rng = np.random.default_rng(P)
    ins = [rng.integers(0, 256, 5, dtype=np.uint8) for _ in range(P)]
    outs = O.ring_all_gather(ins, fill=0xEE)
    cat = np.concatenate(ins)
    for o in outs:
        assert np.array_equal(o, cat)
    # what r sends at step s is what r+1 receives; after step s rank r holds blocks r-s-1 .. r
    for s in range(P - 1):
        for r in range(P):
            assert (r - s) % P == ((r + 1) - s - 1) % P


def test_doubling_segments_partner_symmetry():
    """Receiver's recv offset equals the sender's send offset at every step
    (pccl/src/all_gather.cpp:42-52)."""
    for P in (2, 4, 8, 16, 64):
        seg = 1
        while seg < P:
            for r in range(P):
                p = r ^ seg
                gs_r = (r // (2 * seg)) * 2 * seg
                gs_p = (p // (2 * seg)) * 2 * seg
                recv_r = gs_r + seg if r < p else gs_r
                send_p = gs_p if p < r else gs_p + seg
                assert recv_r == send_p
            seg *= 2


def test_uneven_all_gather_leaves_padding():
    ins = [np.full(n, k + 1, np.uint8) for k, n in enumerate([3, 0, 5])]
    off = [0, 256, 256]
    outs = O.uneven_all_gather(ins, off, 512, fill=0xAA)
    for o in outs:
        assert (o[:3] == 1).all() and (o[3:256] == 0xAA).all() and (o[256:261] == 3).all() and (o[261:] == 0xAA).all()


# ---- 2-D -------------------------------------------------------------------

@pytest.mark.parametrize("intra,inter,grids", [(2, 2, 1), (4, 2, 1), (2, 4, 1), (2, 2, 2), (8, 1, 1), (1, 4, 2)])
def test_grid_groups_are_rows_and_columns(intra, inter, grids):
    world = intra * inter * grids
    inner, outer = O.grid_groups(world, intra, inter)
    grid = np.arange(world).reshape(grids, inter, intra)
    for g in range(grids):
        for j in range(inter):
            for i in range(intra):
                r = int(grid[g, j, i])
                assert inner[r] == [int(x) for x in grid[g, j, :]]
                assert outer[r] == [int(x) for x in grid[g, :, i]]


@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("intra,inter", [(2, 2), (4, 2), (2, 4)])
def test_reduce_scatter_2d_gives_block_r_of_the_total(alg, intra, inter):
    """With integer inputs every order is exact, so rank r must end with block r
    of the world-wide sum: pins the permutation and both group levels."""
    world = intra * inter
    m = 9
    ins = make_inputs(world, world * m, O.F32, seed=12, dist="int")
    total = np.sum(np.stack(ins), axis=0)
    outs = O.reduce_scatter_2d(ins, intra, inter, O.F32, alg)
    for r in range(world):
        assert np.array_equal(outs[r], total[r * m:(r + 1) * m]), r


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("alg,intra,inter", [("ring", 2, 2), ("ring", 3, 2), ("ring", 4, 3), ("ring", 1, 5), ("ring", 5, 1),
                                             ("recursive", 2, 2), ("recursive", 4, 2), ("recursive", 2, 8),
                                             ("recursive", 8, 4)])
def test_reduce_scatter_2d_rounds_in_the_order_of_both_levels(dtype, alg, intra, inter):
    """Floating-point inputs: the bits fix the order of summation, first inside
    every node, then across the nodes, each in its schedule's order."""
    world = intra * inter
    ins = make_inputs(world, world * 13, dtype, seed=14)
    got = O.reduce_scatter_2d(ins, intra, inter, dtype, alg)
    want = grid_closed_form(ins, intra, inter, dtype, alg)
    for r in range(world):
        assert_bits_equal(got[r], want[r], f"rank {r}")


def test_2d_order_differs_from_the_flat_order_so_the_closed_form_has_teeth():
    world, m = 8, 4096
    ins = make_inputs(world, world * m, O.F32, seed=15)
    grid = grid_closed_form(ins, 4, 2, O.F32, "ring")
    flat = ring_closed_form(ins, O.F32)
    swapped = grid_closed_form(ins, 2, 4, O.F32, "ring")
    assert sum(int((a.view(np.uint32) != b.view(np.uint32)).sum()) for a, b in zip(grid, flat)) > 0
    assert sum(int((a.view(np.uint32) != b.view(np.uint32)).sum()) for a, b in zip(grid, swapped)) > 0


@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("intra,inter", [(2, 2), (4, 2), (2, 4)])
def test_all_gather_2d_is_concatenation_in_world_order(alg, intra, inter):
    world = intra * inter
    ins = [np.full(6, r, np.uint8) for r in range(world)]
    outs = O.all_gather_2d(ins, intra, inter, alg)
    cat = np.concatenate(ins)
    for o in outs:
        assert np.array_equal(o, cat)


def test_all_reduce_is_the_sum_everywhere():
    ins = make_inputs(4, 4 * 10, O.F32, seed=13, dist="int")
    total = np.sum(np.stack(ins), axis=0)
    for alg in ("ring", "recursive"):
        for o in O.all_reduce(ins, O.F32, alg):
            assert np.array_equal(o, total)


# ---- the C restatement agrees with the numpy one -----------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P", [1, 2, 3, 4, 8, 16])
def test_c_oracle_matches_numpy_oracle(liboracle, dtype, P):
    B = 29
    code = 0 if dtype == O.F32 else 1
    ins = make_inputs(P, P * B, dtype, seed=14)
    flat = np.concatenate(ins)
    out = np.zeros(P * B, flat.dtype)
    assert liboracle.oracle_ring_reduce_scatter(out.ctypes.data, flat.ctypes.data, P, B, code) == 0
    want = O.ring_reduce_scatter(ins, dtype)
    assert_bits_equal(out, np.concatenate(want), "ring")
    if P & (P - 1) == 0:
        out[:] = 0
        assert liboracle.oracle_rh_reduce_scatter(out.ctypes.data, flat.ctypes.data, P, B, code) == 0
        assert_bits_equal(out, np.concatenate(O.recursive_halving_reduce_scatter(ins, dtype)), "halving")
        shards = np.concatenate([x[:B] for x in ins]).view(np.uint8)
        blk = shards.size // P
        ag = np.zeros(P * P * blk, np.uint8)
        assert liboracle.oracle_rd_all_gather(ag.ctypes.data, shards.ctypes.data, P, blk) == 0
        assert np.array_equal(ag, np.tile(shards, P))
    shards = np.concatenate([x[:B] for x in ins]).view(np.uint8)
    blk = shards.size // P
    ag = np.zeros(P * P * blk, np.uint8)
    assert liboracle.oracle_ring_all_gather(ag.ctypes.data, shards.ctypes.data, P, blk) == 0
    assert np.array_equal(ag, np.tile(shards, P))


def test_c_bf16_rounding_matches_numpy(liboracle):
    rng = np.random.default_rng(15)
    x = rng.standard_normal(2000).astype(np.float32)
    x[:6] = [np.inf, -np.inf, np.nan, 0.0, -0.0, 1e-40]
    want = O.f32_to_bf16(x)
    got = np.array([liboracle.oracle_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- per-rank CPU baseline programs reproduce the oracle ---------------------

def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15))
    x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def _baseline_input(n, dtype, seed, rank, scale):
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(rank))
        u = (_splitmix64(base + np.arange(n, dtype=np.uint64)) >> np.uint64(40)).astype(np.uint32)
    x = ((u.astype(np.float32) / np.float32(8388608.0)) - np.float32(1.0)) * np.float32(scale)
    return x if dtype == O.F32 else O.f32_to_bf16(x)


@pytest.mark.parametrize("transport", ["shm", "mpi"])
@pytest.mark.parametrize("alg,P", [("ring", 4), ("ring", 3), ("recursive", 4)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_cpu_baseline_programs_match_oracle(tmp_path, transport, alg, P, dtype):
    build = os.path.join(ROOT, "oracle", "build")
    if not os.path.exists(os.path.join(build, "cpu_baseline_shm")):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    B, seed, scale = 1000, 77, 0.5
    dump = str(tmp_path / "out.bin")
    common = ["--alg", alg, "--dtype", dtype, "--block", str(B), "--warmup", "0", "--iters", "1",
              "--seed", str(seed), "--scale", str(scale), "--dump", dump]
    if transport == "shm":
        cmd = [os.path.join(build, "cpu_baseline_shm"), "--ranks", str(P)] + common
    else:
        launcher = "/opt/conda/bin/mpiexec.hydra"
        binary = os.path.join(build, "cpu_baseline_mpi")
        if not (os.path.exists(launcher) and os.path.exists(binary)):
            pytest.skip("no MPI launcher in this environment")
        cmd = [launcher, "-np", str(P), binary] + common
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    info = json.loads([l for l in p.stdout.splitlines() if l.startswith("{")][-1])
    assert info["ranks"] == P and info["algorithm"] == alg
    ins = [_baseline_input(P * B, dtype, seed, r, scale) for r in range(P)]
    want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
    got = np.fromfile(dump, dtype=np.float32 if dtype == O.F32 else np.uint16)
    assert_bits_equal(got, np.concatenate(want), f"{transport} {alg}")


# ---- committed fixtures ----------------------------------------------------------

def golden_cases():
    return sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "*.npz")))


@pytest.mark.parametrize("path", golden_cases(), ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_golden_vectors(path):
    z = np.load(path)
    meta = json.loads(bytes(z["meta"]).decode())
    P, dtype = meta["P"], meta["dtype"]
    ins = [z[f"in_{r}"] for r in range(P)]
    kind = meta["collective"]
    if kind in ("reduce_scatter_2d", "all_gather_2d", "all_reduce", "all_gather_uneven"):
        # what the mathematics fixes first, then the oracle against the fixture
        alg = meta["algorithm"]
        if kind == "reduce_scatter_2d":
            closed = grid_closed_form(ins, meta["intra"], meta["inter"], dtype, alg)
            outs = O.reduce_scatter_2d(ins, meta["intra"], meta["inter"], dtype, alg)
        elif kind == "all_gather_2d":
            closed = [np.concatenate(ins)] * P
            outs = [o.view(ins[0].dtype) for o in O.all_gather_2d(ins, meta["intra"], meta["inter"], alg)]
        elif kind == "all_reduce":
            blocks = (ring_closed_form if alg == "ring" else halving_closed_form)(ins, dtype)
            closed = [np.concatenate(blocks)] * P
            outs = O.all_reduce(ins, dtype, alg)
        else:
            one = np.full(meta["total"], meta["fill"], np.uint8)
            for k in range(P):
                one[meta["dst_off"][k]:meta["dst_off"][k] + meta["nbytes"][k]] = ins[k]
            closed = [one] * P
            outs = O.uneven_all_gather(ins, meta["dst_off"], meta["total"], meta["fill"])
        for r in range(P):
            assert_bits_equal(z[f"out_{r}"], closed[r], f"fixture vs closed form, rank {r}")
            assert_bits_equal(outs[r], z[f"out_{r}"], f"oracle vs fixture, rank {r}")
        return
    if meta["collective"] == "reduce_scatter":
        fn = O.ring_reduce_scatter if meta["algorithm"] == "ring" else O.recursive_halving_reduce_scatter
        outs = fn(ins, dtype)
        closed = (ring_closed_form if meta["algorithm"] == "ring" else halving_closed_form)(ins, dtype)
        for r in range(P):
            assert_bits_equal(z[f"out_{r}"], closed[r], "fixture vs closed form")
    else:
        fn = O.ring_all_gather if meta["algorithm"] == "ring" else O.recursive_doubling_all_gather
        outs = fn(ins)
        for r in range(P):
            assert_bits_equal(z[f"out_{r}"], np.concatenate(ins), "fixture vs concatenation")
    for r in range(P):
        assert_bits_equal(outs[r], z[f"out_{r}"], f"rank {r}")


# ---- binary16 ---------------------------------------------------------------------

def _f16_partners():
    return np.concatenate([np.arange(0, 65536, 1024, dtype=np.uint16) | np.uint16(0x135),
                           np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF,
                                     0x3C00, 0x3C01, 0x7E00, 0x7D01], np.uint16)])


def test_f16_add_is_torch_add():
    """The hop arithmetic of the reference's Python algorithms on float16 tensors
    (pccl/reduce_scatter.py:24,83,95,158): torch.add, all 65 536 patterns against
    78 partners (every exponent, zeros, infinities, subnormals, the largest finite
    values, NaNs)."""
    import torch
    a = np.arange(65536, dtype=np.uint16)
    partners = _f16_partners()
    A, B = np.tile(a, partners.size), np.repeat(partners, a.size)
    ta = torch.from_numpy(A.view(np.int16).copy()).view(torch.float16)
    tb = torch.from_numpy(B.view(np.int16).copy()).view(torch.float16)
    want = torch.add(ta, tb).view(torch.int16).numpy().view(np.uint16)
    got = O.vector_add(A, B, O.F16)
    nan = np.isnan(want.view(np.float16))
    assert nan.any() and (~nan).sum() > 4_000_000
    assert np.array_equal(got[~nan], want[~nan])
    assert (got[nan] == 0x7E00).all()                 # the oracle stores the canonical quiet NaN


def test_f16_add_is_the_correctly_rounded_sum():
    """float64 holds the sum of two binary16 values exactly; rounding it ONCE to
    binary16 (nearest even) must give the oracle's result, which rounds twice
    (to binary32, then to binary16): 24 >= 2 * 11 + 2 bits make that harmless.
    Rounding toward zero instead gives other bits (the check has teeth)."""
    a = np.arange(65536, dtype=np.uint16)
    partners = _f16_partners()
    A, B = np.tile(a, partners.size), np.repeat(partners, a.size)
    with np.errstate(over="ignore", invalid="ignore"):
        exact = A.view(np.float16).astype(np.float64) + B.view(np.float16).astype(np.float64)
        want = exact.astype(np.float16).view(np.uint16)
    got = O.vector_add(A, B, O.F16)
    ok = ~np.isnan(exact)
    assert np.array_equal(got[ok], want[ok])
    with np.errstate(over="ignore", invalid="ignore"):
        toward_zero = np.where(np.abs(want.view(np.float16).astype(np.float64)) > np.abs(exact),
                               want - np.uint16(1), want)
    assert (toward_zero[ok] != got[ok]).sum() > 100_000


def test_f16_conversions_round_trip_and_saturate_to_infinity():
    u = np.arange(65536, dtype=np.uint16)
    f = O.f16_to_f32(u)
    back = O.f32_to_f16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], u[~nan]) and (back[nan] == 0x7E00).all()
    assert O.f32_to_f16(np.array([65504.0, 65519.9, 65520.0, -65520.0, 1e-8, 5.96e-8], np.float32)).tolist() == \
        [0x7BFF, 0x7BFF, 0x7C00, 0xFC00, 0x0000, 0x0001]


@pytest.mark.parametrize("alg", ["ring", "recursive"])
def test_f16_schedules_follow_the_closed_forms(alg):
    P, B = 8, 257
    ins = make_inputs(P, P * B, O.F16, seed=40)
    if alg == "ring":
        got, want = O.ring_reduce_scatter(ins, O.F16), ring_closed_form(ins, O.F16)
    else:
        got, want = O.recursive_halving_reduce_scatter(ins, O.F16), halving_closed_form(ins, O.F16)
    for r in range(P):
        assert_bits_equal(got[r], want[r], f"rank {r}")
