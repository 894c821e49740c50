"""GPU parity of whole collectives on virtual ranks against the CPU oracle:
driver API (all ranks' tensors in one call), every execution mode, and the
per-rank API run SPMD (one thread per virtual rank) with both backends."""
import numpy as np
import pytest

from helpers import assert_bits_equal, make_inputs, ring_closed_form, to_numpy, to_torch
from oracle import pccl_oracle as O

DTYPES = [O.F32, O.BF16]
MODES = ["steps", "fused", "faithful"]


def _tdtype(dtype):
    import torch
    return {O.F32: torch.float32, O.BF16: torch.bfloat16, O.F16: torch.float16}[dtype]


def _rs_oracle(alg):
    return O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg,P", [("ring", 1), ("ring", 2), ("ring", 3), ("ring", 4), ("ring", 8), ("ring", 13),
                                   ("recursive", 1), ("recursive", 2), ("recursive", 4), ("recursive", 8),
                                   ("recursive", 16), ("recursive", 64)])
def test_reduce_scatter_driver(target, dtype, mode, alg, P):
    import torch
    from pccl import kernels
    B = 1031 if P <= 16 else 130          # ragged: not a multiple of the vector width
    print(f"reduce_scatter alg={alg} P={P} B={B} dtype={dtype} mode={mode}", flush=True)
    ins = make_inputs(P, P * B, dtype, seed=21)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(B, dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
    kernels.reduce_scatter_ranks(t_out, t_in, algorithm=alg, mode=mode)
    target.sync()
    want = _rs_oracle(alg)(ins, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"rank {r}")
        assert_bits_equal(to_numpy(t_in[r], dtype), ins[r], f"input of rank {r} modified")


@pytest.mark.parametrize("alg,P", [("ring", 65), ("ring", 100), ("ring", 128), ("recursive", 128), ("recursive", 256)])
@pytest.mark.parametrize("mode", ["steps", "faithful", "fused"])
def test_more_ranks_than_one_launch_holds(target, alg, P, mode):
    """Beyond 64 ranks a step goes out as several launches; the fused ring
    order chains folds of at most 64 operands with the running sum as the first
    operand, the fused halving order runs rounds until groups of 64 remain and
    finishes each group with one butterfly launch."""
    import torch
    from pccl import kernels
    B, dtype = 21, O.BF16
    ins = make_inputs(P, P * B, dtype, seed=77)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(B, dtype=torch.bfloat16, device=target.device) for _ in range(P)]
    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
    target.sync()
    want = _rs_oracle(alg)(ins, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"rank {r}")
    g_out = [torch.zeros(P * B, dtype=torch.bfloat16, device=target.device) for _ in range(P)]
    kernels.all_gather_ranks(g_out, t_out, alg, "fused" if mode == "fused" else "steps")
    target.sync()
    for r in (0, 63, 64, P // 2, P - 1):
        assert_bits_equal(to_numpy(g_out[r], dtype), np.concatenate(want), f"gather rank {r}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_config1_shape_small_ring_p4_uniform(target, dtype):
    """The P=4 fp32 workload at reduced length: uniform[-1,1], seed + rank;
    all three modes agree with the oracle and with the closed-form left fold."""
    import torch
    from pccl import kernels
    P, B = 4, 1 << 16
    ins = make_inputs(P, P * B, dtype, seed=1234, dist="uniform")
    want = O.ring_reduce_scatter(ins, dtype)
    closed = ring_closed_form(ins, dtype)
    for r in range(P):
        assert_bits_equal(want[r], closed[r], "oracle vs closed form")
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    for mode in MODES:
        t_out = [torch.zeros(B, dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode)
        target.sync()
        for r in range(P):
            assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"{mode} rank {r}")


@pytest.mark.parametrize("alg", ["ring", "recursive"])
def test_integer_inputs_give_exact_sums(target, alg):
    """Small integers make every order exact: isolates placement from rounding."""
    import torch
    from pccl import kernels
    P, B = 8, 999
    for dtype in DTYPES:
        ins = make_inputs(P, P * B, dtype, seed=3, dist="int")
        as_f = [x if dtype == O.F32 else O.bf16_to_f32(x) for x in ins]
        total = np.sum(np.stack(as_f).astype(np.float64), axis=0)
        t_in = [to_torch(x, dtype, target.device) for x in ins]
        for mode in MODES:
            t_out = [torch.zeros(B, dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
            kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
            target.sync()
            for r in range(P):
                got = t_out[r].float().cpu().numpy().astype(np.float64)
                assert np.array_equal(got, total[r * B:(r + 1) * B]), (alg, dtype, mode, r)


@pytest.mark.parametrize("mode", ["steps", "fused"])
@pytest.mark.parametrize("alg,P", [("recursive", 1), ("recursive", 2), ("recursive", 4), ("recursive", 16),
                                   ("ring", 1), ("ring", 2), ("ring", 3), ("ring", 7), ("ring", 16)])
@pytest.mark.parametrize("blk", [1, 6, 256, 4096 + 2, 100_000])
def test_all_gather_driver(target, mode, alg, P, blk):
    import torch
    from pccl import kernels
    print(f"all_gather alg={alg} P={P} blk={blk} mode={mode}", flush=True)
    rng = np.random.default_rng(5)
    ins = [rng.integers(0, 256, blk, dtype=np.uint8) for _ in range(P)]
    t_in = [torch.from_numpy(x).to(target.device) for x in ins]
    t_out = [torch.full((P * blk,), 0xA5, dtype=torch.uint8, device=target.device) for _ in range(P)]
    kernels.all_gather_ranks(t_out, t_in, algorithm=alg, mode=mode)
    target.sync()
    want = (O.ring_all_gather if alg == "ring" else O.recursive_doubling_all_gather)(ins)
    cat = torch.cat(t_in)
    for r in range(P):
        assert np.array_equal(t_out[r].cpu().numpy(), want[r]), f"rank {r}"
        assert torch.equal(t_out[r], cat)


def test_all_gather_bf16_and_f32_typed(target):
    import torch
    from pccl import kernels
    for td in (torch.bfloat16, torch.float32):
        P, n = 4, 3001
        t_in = [torch.randn(n, device=target.device).to(td) for _ in range(P)]
        t_out = [torch.zeros(P * n, dtype=td, device=target.device) for _ in range(P)]
        kernels.all_gather_ranks(t_out, t_in, "recursive", "steps")
        target.sync()
        for r in range(P):
            assert torch.equal(t_out[r].view(torch.uint8), torch.cat(t_in).view(torch.uint8))


def test_all_gather_uneven_padded_to_256(target):
    """Uneven ZeRO-style shards, each padded to 256 bytes: equals torch.cat of
    the unpadded shards at the padded offsets; padding bytes stay untouched."""
    import torch
    from pccl import kernels
    rng = np.random.default_rng(8)
    P = 16
    lens = [int(x) for x in rng.integers(1, 40_000, P)]
    lens[3] = 0
    lens[5] = 2 * 17          # not a multiple of 4 bytes
    t_in = [torch.from_numpy(rng.integers(0, 2 ** 15, n, dtype=np.int16)).to(target.device).view(torch.bfloat16)
            if n else torch.empty(0, dtype=torch.bfloat16, device=target.device) for n in lens]

    def as_bytes(t):
        return t.view(torch.uint8) if t.numel() else torch.empty(0, dtype=torch.uint8, device=t.device)
    nbytes = [2 * n for n in lens]
    off = kernels.padded_offsets(nbytes, 256)
    total = off[-1] + (nbytes[-1] + 255) // 256 * 256
    t_out = [torch.full((total,), 0xA5, dtype=torch.uint8, device=target.device) for _ in range(P)]
    used = kernels.all_gather_uneven_ranks(t_out, t_in, align=256)
    target.sync()
    assert used == off and all(o % 256 == 0 for o in off)
    want = O.uneven_all_gather([as_bytes(t).cpu().numpy() for t in t_in], off, total)
    for r in range(P):
        assert np.array_equal(t_out[r].cpu().numpy(), want[r]), f"rank {r}"
    # closed form: the shards, unpadded, in rank order
    got = torch.cat([t_out[0][o:o + nb] for o, nb in zip(off, nbytes)])
    assert torch.equal(got, torch.cat([as_bytes(t) for t in t_in]))


def test_all_gather_uneven_more_ranks_than_one_launch_holds(target):
    import torch
    from pccl import kernels
    P = 70
    rng = np.random.default_rng(70)
    nbytes = [int(x) for x in rng.integers(0, 3000, P)]
    t_in = [torch.from_numpy(rng.integers(0, 256, n, dtype=np.uint8)).to(target.device) for n in nbytes]
    off = kernels.padded_offsets(nbytes, 256)
    total = off[-1] + nbytes[-1]
    t_out = [torch.full((total,), 0x5A, dtype=torch.uint8, device=target.device) for _ in range(P)]
    kernels.all_gather_uneven_ranks(t_out, t_in, off)
    target.sync()
    want = O.uneven_all_gather([t.cpu().numpy() for t in t_in], off, total, fill=0x5A)
    for r in (0, 63, 64, 69):
        assert np.array_equal(t_out[r].cpu().numpy(), want[r]), f"rank {r}"


@pytest.mark.parametrize("P", [1, 3, 5, 16])
@pytest.mark.parametrize("split,strip", [(0, 0), (1, 0), (2, 0), (3, 0), (64, 0), (0, 1), (0, 2), (0, 256), (0, -1)])
@pytest.mark.parametrize("unroll,nt", [(1, 1), (4, 0)])
def test_multicast_gather_tunings_give_the_same_bytes(target, P, split, strip, unroll, nt):
    """However the outputs of a shard tile are shared among workgroups
    (gather_split), or walked strip by strip and output by output
    (gather_strip), the gathered bytes are the same; ragged lengths and odd
    rank counts included."""
    import torch
    from pccl import kernels
    lib = target.native
    keys = ("gather_split", "unroll_gather", "gather_nt", "gather_strip", "gather_strip_from")
    saved = {k: lib.get_tuning(k) for k in keys}
    rng = np.random.default_rng(100 + P)
    nbytes = [int(x) for x in rng.integers(0, 30_000, P)]
    nbytes[0] = 4096 * 3 + 5
    t_in = [torch.from_numpy(rng.integers(0, 256, n, dtype=np.uint8)).to(target.device) for n in nbytes]
    off = kernels.padded_offsets(nbytes, 16)
    total = off[-1] + nbytes[-1] + 7
    try:
        lib.set_tuning("gather_split", split)
        lib.set_tuning("gather_strip", strip)
        lib.set_tuning("gather_strip_from", 0)      # strip = -1: the automatic choice, also for these short shards
        lib.set_tuning("unroll_gather", unroll)
        lib.set_tuning("gather_nt", nt)
        t_out = [torch.full((total,), 0x5A, dtype=torch.uint8, device=target.device) for _ in range(P)]
        lib.all_gather_uneven_virtual([t.data_ptr() for t in t_out], [t.data_ptr() for t in t_in], nbytes, off,
                                      target.stream())
        target.sync()
    finally:
        for k, v in saved.items():
            lib.set_tuning(k, v)
    want = O.uneven_all_gather([t.cpu().numpy() for t in t_in], off, total, fill=0x5A)
    for r in range(P):
        assert np.array_equal(t_out[r].cpu().numpy(), want[r]), f"rank {r}"


def _golden_cases():
    import glob
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    return sorted(glob.glob(os.path.join(here, "golden", "*.npz")))


@pytest.mark.parametrize("path", _golden_cases(), ids=lambda p: p.split("/")[-1][:-4])
@pytest.mark.parametrize("mode", MODES)
def test_golden_vectors(target, path, mode, monkeypatch):
    """The committed fixtures (tests/golden/make_golden.py) through the library."""
    import json
    import torch
    from pccl import kernels
    z = np.load(path)
    meta = json.loads(bytes(z["meta"]).decode())
    P, dtype, kind = meta["P"], meta["dtype"], meta["collective"]
    if kind == "all_gather_uneven":
        t_in = [torch.from_numpy(z[f"in_{r}"].copy()).to(target.device) for r in range(P)]
        t_out = [torch.full((meta["total"],), meta["fill"], dtype=torch.uint8, device=target.device) for _ in range(P)]
        kernels.all_gather_uneven_ranks(t_out, t_in, meta["dst_off"])
        target.sync()
        for r in range(P):
            assert np.array_equal(t_out[r].cpu().numpy(), z[f"out_{r}"]), f"rank {r}"
        return
    t_in = [to_torch(z[f"in_{r}"], dtype, target.device) for r in range(P)]
    if kind == "all_reduce":
        import pccl
        world = pccl.VirtualWorld(P, target.device)
        monkeypatch.setenv("PCCL_VIRTUAL_MODE", mode)
        world.run(lambda comm: pccl._all_reduce(t_in[comm.Get_rank()], group=comm,
                                                use_rh_and_rd=meta["algorithm"] == "recursive"))
        t_out = t_in                                       # in place, like the reference
    elif kind == "reduce_scatter":
        t_out = [torch.zeros(meta["B"], dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
        kernels.reduce_scatter_ranks(t_out, t_in, meta["algorithm"], mode)
    elif kind == "reduce_scatter_2d":
        t_out = [torch.zeros(meta["B"], dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
        kernels.reduce_scatter_2d_ranks(t_out, t_in, meta["intra"], meta["inter"], meta["algorithm"], mode)
    elif kind == "all_gather_2d":
        t_out = [torch.zeros(P * meta["B"], dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
        kernels.all_gather_2d_ranks(t_out, t_in, meta["intra"], meta["inter"], meta["algorithm"], mode)
    else:
        t_out = [torch.zeros(P * meta["B"], dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
        kernels.all_gather_ranks(t_out, t_in, meta["algorithm"], mode)
    target.sync()
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), z[f"out_{r}"], f"rank {r}")


# ---------------------------------------------------------------------------
# per-rank API, SPMD
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_rh,P", [(False, 4), (False, 5), (True, 4), (True, 8)])
@pytest.mark.parametrize("cpp", [True, False])
def test_reduce_scatter_per_rank_api(target, dtype, use_rh, P, cpp):
    """_reduce_scatter(out, in, group=comm, ...) called by every virtual rank;
    the native backend and the Python algorithms give the oracle's bits."""
    import torch
    import pccl
    B = 777
    print(f"_reduce_scatter P={P} rh={use_rh} cpp={cpp} dtype={dtype}", flush=True)
    ins = make_inputs(P, P * B, dtype, seed=31)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(B, dtype=_tdtype(dtype), device=target.device) for _ in range(P)]
    world = pccl.VirtualWorld(P, target.device)

    def rank_main(comm):
        r = comm.Get_rank()
        return pccl._reduce_scatter(t_out[r], t_in[r], group=comm, use_rh=use_rh, use_pccl_cpp_backend=cpp)

    assert world.run(rank_main) == [None] * P
    target.sync()
    want = _rs_oracle("recursive" if use_rh else "ring")(ins, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"rank {r}")


@pytest.mark.parametrize("cpp", [True, False])
@pytest.mark.parametrize("use_rd", [True, False])
def test_all_gather_per_rank_api(target, cpp, use_rd):
    import torch
    import pccl
    P, n = 8, 1234
    t_in = [torch.randn(n, device=target.device).bfloat16() for _ in range(P)]
    t_out = [torch.zeros(P * n, dtype=torch.bfloat16, device=target.device) for _ in range(P)]
    world = pccl.VirtualWorld(P, target.device)
    world.run(lambda comm: pccl._all_gather(t_out[comm.Get_rank()], t_in[comm.Get_rank()], group=comm,
                                            use_rd=use_rd, use_pccl_cpp_backend=cpp))
    target.sync()
    for r in range(P):
        assert torch.equal(t_out[r].view(torch.int16), torch.cat(t_in).view(torch.int16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("intra,inter", [(2, 2), (4, 2), (2, 4)])
@pytest.mark.parametrize("use_rh", [True, False])
@pytest.mark.parametrize("cpp", [True, False])
def test_reduce_scatter_2D(target, dtype, intra, inter, use_rh, cpp):
    import torch
    import pccl
    world_size = intra * inter
    m = 333
    print(f"reduce_scatter_2D {intra}x{inter} rh={use_rh} cpp={cpp} dtype={dtype}", flush=True)
    ins = make_inputs(world_size, world_size * m, dtype, seed=41)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(m, dtype=_tdtype(dtype), device=target.device) for _ in range(world_size)]
    world = pccl.VirtualWorld(world_size, target.device)

    def rank_main(comm):
        r = comm.Get_rank()
        pg = pccl.ProcessGroups(intra, inter, inner_group_backend="mpi", outer_group_backend="mpi", comm=comm)
        assert pg.get_world_size() == [intra, inter]
        pccl.reduce_scatter_2D(t_out[r], t_in[r], group=pg, use_rh=use_rh, use_pccl_cpp_backend=cpp)

    world.run(rank_main)
    target.sync()
    want = O.reduce_scatter_2d(ins, intra, inter, dtype, "recursive" if use_rh else "ring")
    for r in range(world_size):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"rank {r}")


@pytest.mark.parametrize("intra,inter", [(2, 2), (4, 2), (2, 4)])
@pytest.mark.parametrize("use_rd", [True, False])
@pytest.mark.parametrize("cpp", [True, False])
def test_all_gather_2D(target, intra, inter, use_rd, cpp):
    import torch
    import pccl
    world_size = intra * inter
    n = 501
    t_in = [torch.randn(n, device=target.device) for _ in range(world_size)]
    t_out = [torch.zeros(world_size * n, device=target.device) for _ in range(world_size)]
    world = pccl.VirtualWorld(world_size, target.device)

    def rank_main(comm):
        r = comm.Get_rank()
        pg = pccl.ProcessGroups(intra, inter, comm=comm)
        pccl.all_gather_2D(t_out[r], t_in[r], group=pg, use_rd=use_rd, use_pccl_cpp_backend=cpp)

    world.run(rank_main)
    target.sync()
    want = O.all_gather_2d([t.cpu().numpy() for t in t_in], intra, inter, "recursive" if use_rd else "ring")
    cat = torch.cat(t_in)
    for r in range(world_size):
        assert np.array_equal(t_out[r].view(torch.uint8).cpu().numpy(), want[r]), f"rank {r}"
        assert torch.equal(t_out[r], cat)      # the 2-D all_gather is a plain concatenation


# the last row: more ranks than one launch has pointers for (steps: launches of 64 ranks; fused: level by level)
GRIDS = [(1, 1), (2, 1), (1, 2), (2, 2), (4, 2), (2, 4), (3, 2), (2, 3), (1, 8), (8, 1), (4, 4), (8, 8), (16, 4),
         (8, 16), (16, 16), (5, 13), (43, 3), (1, 128), (128, 1)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("intra,inter", GRIDS)
@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("mode", ["steps", "fused"])
def test_reduce_scatter_2d_driver(target, dtype, intra, inter, alg, mode):
    """The whole 2-D collective in one call: permutation read in place, all
    groups of a level in one launch, or everything in one fused launch."""
    import torch
    from pccl import kernels
    if alg == "recursive" and ((intra & (intra - 1)) or (inter & (inter - 1))):
        pytest.skip("halving needs power-of-two groups")
    W = intra * inter
    m = 261 if W <= 16 else 37 if W <= 64 else 13
    print(f"reduce_scatter_2d {intra}x{inter} alg={alg} mode={mode} dtype={dtype}", flush=True)
    ins = make_inputs(W, W * m, dtype, seed=61)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(m, dtype=_tdtype(dtype), device=target.device) for _ in range(W)]
    kernels.reduce_scatter_2d_ranks(t_out, t_in, intra, inter, alg, mode)
    target.sync()
    want = O.reduce_scatter_2d(ins, intra, inter, dtype, alg)
    for w in range(W):
        assert_bits_equal(to_numpy(t_out[w], dtype), want[w], f"rank {w}")
        assert_bits_equal(to_numpy(t_in[w], dtype), ins[w], f"input of rank {w} modified")


@pytest.mark.parametrize("intra,inter", GRIDS)
@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("mode", ["steps", "fused"])
def test_all_gather_2d_driver(target, intra, inter, alg, mode):
    import torch
    from pccl import kernels
    if alg == "recursive" and ((intra & (intra - 1)) or (inter & (inter - 1))):
        pytest.skip("doubling needs power-of-two groups")
    W = intra * inter
    n = 1030 if W <= 16 else 70 if W <= 64 else 22
    rng = np.random.default_rng(71)
    ins = [rng.integers(0, 256, n, dtype=np.uint8) for _ in range(W)]
    t_in = [torch.from_numpy(x).to(target.device) for x in ins]
    t_out = [torch.full((W * n,), 0xA5, dtype=torch.uint8, device=target.device) for _ in range(W)]
    kernels.all_gather_2d_ranks(t_out, t_in, intra, inter, alg, mode)
    target.sync()
    want = O.all_gather_2d(ins, intra, inter, alg)
    for w in range(W):
        assert np.array_equal(t_out[w].cpu().numpy(), want[w]), f"rank {w}"


@pytest.mark.parametrize("mode", ["steps", "fused"])
def test_2d_per_rank_api_with_two_grids(target, mode, monkeypatch):
    """world = 2 grids of 2x2: every grid is an independent 2-D collective."""
    import torch
    import pccl
    monkeypatch.setenv("PCCL_VIRTUAL_MODE", mode)
    intra, inter, grids = 2, 2, 2
    world_size = intra * inter * grids
    m = 129
    ins = make_inputs(world_size, intra * inter * m, O.BF16, seed=81)
    t_in = [to_torch(x, O.BF16, target.device) for x in ins]
    t_out = [torch.zeros(m, dtype=torch.bfloat16, device=target.device) for _ in range(world_size)]
    g_out = [torch.zeros(intra * inter * m, dtype=torch.bfloat16, device=target.device) for _ in range(world_size)]
    world = pccl.VirtualWorld(world_size, target.device)

    def rank_main(comm):
        r = comm.Get_rank()
        pg = pccl.ProcessGroups(intra, inter, inner_group_backend="mpi", outer_group_backend="mpi", comm=comm)
        pccl.reduce_scatter_2D(t_out[r], t_in[r], group=pg, use_rh=True, use_pccl_cpp_backend=True)
        pccl.all_gather_2D(g_out[r], t_out[r], group=pg, use_rd=True, use_pccl_cpp_backend=True)

    world.run(rank_main)
    target.sync()
    per = intra * inter
    for g in range(grids):
        want = O.reduce_scatter_2d(ins[g * per:(g + 1) * per], intra, inter, O.BF16, "recursive")
        for k in range(per):
            assert_bits_equal(to_numpy(t_out[g * per + k], O.BF16), want[k], f"grid {g} rank {k}")
            assert_bits_equal(to_numpy(g_out[g * per + k], O.BF16), np.concatenate(want), f"gather grid {g} rank {k}")


@pytest.mark.parametrize("mode", MODES)
def test_plans_replay_on_fresh_data(target, mode):
    """A validated plan replays the collective with no per-call checks."""
    import torch
    from pccl import kernels
    P, B, dtype = 4, 515, O.F32
    ins = make_inputs(P, P * B, dtype, seed=91)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(B, device=target.device) for _ in range(P)]
    plan = kernels.plan_reduce_scatter(t_out, t_in, "ring", mode)
    g_out = [torch.zeros(P * B, device=target.device) for _ in range(P)]
    gplan = kernels.plan_all_gather(g_out, t_out, "ring", mode)
    fresh = make_inputs(P, P * B, dtype, seed=92)
    for t, x in zip(t_in, fresh):
        t.copy_(to_torch(x, dtype, target.device))
    plan()
    gplan()
    target.sync()
    want = O.ring_reduce_scatter(fresh, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"rank {r}")
        assert_bits_equal(to_numpy(g_out[r], dtype), np.concatenate(want), f"gather rank {r}")


@pytest.mark.parametrize("mode", ["fused", "steps"])
def test_repeated_calls_replay_the_checked_arguments(target, mode):
    """The ordinary API keeps the checked argument pack of a call and replays it
    when called again on the same tensor objects; fresh data, a storage swapped
    under one of the tensors and the death of a tensor are all handled."""
    import gc
    import torch
    from pccl import kernels
    P, B, dtype = 4, 515, O.F32
    t_in = [torch.zeros(P * B, device=target.device) for _ in range(P)]
    t_out = [torch.zeros(B, device=target.device) for _ in range(P)]
    g_out = [torch.zeros(P * B, device=target.device) for _ in range(P)]
    work = [torch.empty(P * B, device=target.device) for _ in range(P)]
    gc.collect()
    before = set(kernels._PLANS)                      # entries of tensors other tests still hold
    for seed in (91, 92, 93):
        ins = make_inputs(P, P * B, dtype, seed=seed)
        for t, x in zip(t_in, ins):
            t.copy_(to_torch(x, dtype, target.device))
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)
        kernels.all_gather_ranks(g_out, t_out, "ring", mode)
        target.sync()
        want = O.ring_reduce_scatter(ins, dtype)
        for r in range(P):
            assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"seed {seed} rank {r}")
            assert_bits_equal(to_numpy(g_out[r], dtype), np.concatenate(want), f"seed {seed} gather rank {r}")
    mine = set(kernels._PLANS) - before
    assert len(mine) == 2                             # one entry per collective, however often it ran
    # the same tensor object on another storage: the recorded address no longer matches
    moved = to_torch(make_inputs(1, P * B, dtype, seed=94)[0], dtype, target.device)
    t_in[2].set_(moved.untyped_storage(), 0, moved.shape)
    kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)
    target.sync()
    ins[2] = to_numpy(moved, dtype)
    want = O.ring_reduce_scatter(ins, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"after set_ rank {r}")
    # a work buffer moved to another storage: the call must use the new one (the old one may be freed memory)
    if mode != "fused":
        stale = work[1]
        stale_bits = stale.clone()
        work[1] = stale                      # same object ...
        work[1].set_(torch.full((P * B,), 7.0, device=target.device).untyped_storage(), 0, (P * B,))
        kept = torch.full((P * B,), 3.0, device=target.device)
        old_storage_view = kept                # stands in for whatever now owns the old address
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)
        target.sync()
        for r in range(P):
            assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"after work set_ rank {r}")
        assert not torch.equal(work[1], torch.full((P * B,), 7.0, device=target.device))   # the new storage was used
        assert torch.equal(old_storage_view, torch.full((P * B,), 3.0, device=target.device))
    # a wrong size is still refused although an entry for these objects exists: on the first output ...
    t_out[1].set_(torch.zeros(B + 1, device=target.device).untyped_storage(), 0, (B + 1,))
    with pytest.raises(RuntimeError, match="block_size"):
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)
    t_out[1].set_(torch.zeros(B, device=target.device).untyped_storage(), 0, (B,))
    kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)       # an entry for the repaired objects again
    # ... and on a later one, shrunk in place (same address, fewer elements)
    t_out[3].resize_(B - 1)
    with pytest.raises(RuntimeError, match="block_size"):
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", mode, work)
    del t_in, t_out, g_out, work, moved
    gc.collect()
    assert not (set(kernels._PLANS) & mine)           # entries die with their tensors


def test_repeated_folds_replay_the_checked_arguments(target):
    """kernels.reduce_kway on the same tensor objects: fresh data, another order,
    a storage swapped under a shard, a shard of another size."""
    import gc
    import torch
    from pccl import kernels
    k, n, dtype = 5, 1031, O.BF16
    shards = [torch.zeros(n, dtype=torch.bfloat16, device=target.device) for _ in range(k)]
    out = torch.zeros(n, dtype=torch.bfloat16, device=target.device)
    gc.collect()
    before = set(kernels._PLANS)

    def want(xs, first):
        acc = xs[first]
        for t in range(1, k):
            acc = O.vector_add(acc, xs[(first + t) % k], dtype)
        return acc

    for seed, first in ((61, 0), (62, 0), (63, 3), (64, 3)):
        xs = make_inputs(k, n, dtype, seed=seed)
        for t, x in zip(shards, xs):
            t.copy_(to_torch(x, dtype, target.device))
        kernels.reduce_kway(out, shards, "ring", first)
        target.sync()
        assert_bits_equal(to_numpy(out, dtype), want(xs, first), f"seed {seed}")
    mine = set(kernels._PLANS) - before
    assert len(mine) == 2                              # one entry per (tensors, order, first)
    moved = to_torch(make_inputs(1, n, dtype, seed=65)[0], dtype, target.device)
    shards[1].set_(moved.untyped_storage(), 0, moved.shape)
    kernels.reduce_kway(out, shards, "ring", 3)
    target.sync()
    xs[1] = to_numpy(moved, dtype)
    assert_bits_equal(to_numpy(out, dtype), want(xs, 3), "after set_")
    shards[0].set_(torch.zeros(n + 1, dtype=torch.bfloat16, device=target.device).untyped_storage(), 0, (n + 1,))
    with pytest.raises(RuntimeError, match="shards must match"):
        kernels.reduce_kway(out, shards, "ring", 3)
    del shards, out, moved
    gc.collect()
    assert not (set(kernels._PLANS) & mine)


@pytest.mark.parametrize("rec,kwargs", [(True, {}), (False, {}), (True, {"use_yacl": True}),
                                        (False, {"use_yacl": True, "use_pccl_cpp_backend": False}),
                                        (False, {"directly_call_mpi": True})])
def test_all_reduce(target, rec, kwargs):
    """The reference's keywords (pccl/all_reduce.py:21-28) are accepted; the
    direct-MPI route sums in ring order."""
    import torch
    import pccl
    P, n = 4, 4 * 257
    dtype = O.F32
    ins = make_inputs(P, n, dtype, seed=51)
    t = [to_torch(x, dtype, target.device) for x in ins]
    world = pccl.VirtualWorld(P, target.device)
    world.run(lambda comm: pccl._all_reduce(t[comm.Get_rank()], group=comm, use_rh_and_rd=rec, **kwargs))
    target.sync()
    want = O.all_reduce(ins, dtype, "recursive" if rec else "ring")
    for r in range(P):
        assert_bits_equal(to_numpy(t[r], dtype), want[r], f"rank {r}")


def test_request_wait_runs_epilogue(target):
    import torch
    import pccl
    if target.device == "cpu":
        pytest.skip("a StreamRequest records a HIP event")
    P, n = 2, 64
    t_in = [torch.randn(n, device=target.device) for _ in range(P)]
    t_out = [torch.zeros(P * n, device=target.device) for _ in range(P)]
    world = pccl.VirtualWorld(P, target.device)
    called = []

    def rank_main(comm):
        r = comm.Get_rank()
        req = pccl._all_gather(t_out[r], t_in[r], group=comm, async_op=True)
        assert isinstance(req, pccl.Request)
        req.wait(lambda: called.append(r))

    world.run(rank_main)
    assert sorted(called) == [0, 1]
    assert torch.equal(t_out[0], torch.cat(t_in))


def test_patch_deepspeed_routes_world_collectives(target, monkeypatch):
    """pccl/patch_deepspeed.py:95-126 against a stand-in for deepspeed's
    TorchBackend (deepspeed itself is not installed): world-group SUM
    collectives go through the 2-D PCCL path, the rest falls through."""
    import enum
    import sys
    import types
    import torch
    import pccl
    from pccl import build_kernels, patch_deepspeed as pd

    class ReduceOp(enum.Enum):
        SUM = 0
        MAX = 1

    fell_through = []

    class TorchBackend:
        def all_gather_into_tensor(self, o, i, group=None, async_op=False): fell_through.append("ag")
        def reduce_scatter_tensor(self, o, i, op=None, group=None, async_op=False): fell_through.append("rs")
        def all_reduce(self, t, op=None, group=None, async_op=False): fell_through.append("ar")
        def broadcast(self, t, src, group=None, async_op=False): fell_through.append("bc")
        def barrier(self, group=None, async_op=False, device_ids=None): fell_through.append("barrier")

    ds = types.ModuleType("deepspeed"); comm_m = types.ModuleType("deepspeed.comm")
    torch_m = types.ModuleType("deepspeed.comm.torch"); op_m = types.ModuleType("deepspeed.comm.reduce_op")
    torch_m.TorchBackend = TorchBackend; op_m.ReduceOp = ReduceOp
    for name, mod in (("deepspeed", ds), ("deepspeed.comm", comm_m), ("deepspeed.comm.torch", torch_m),
                      ("deepspeed.comm.reduce_op", op_m)):
        monkeypatch.setitem(sys.modules, name, mod)
    monkeypatch.setattr(build_kernels, "build", lambda *a, **k: None)
    monkeypatch.setattr(pd, "build", lambda *a, **k: None)

    W, intra, m, dtype = 8, 4, 97, O.BF16
    ins = make_inputs(W, W * m, dtype, seed=123)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [torch.zeros(m, dtype=torch.bfloat16, device=target.device) for _ in range(W)]
    g_out = [torch.zeros(W * m, dtype=torch.bfloat16, device=target.device) for _ in range(W)]
    ar = [to_torch(x, dtype, target.device) for x in make_inputs(W, 64, dtype, seed=5)]
    ar_in = make_inputs(W, 64, dtype, seed=5)
    bc = [torch.full((33,), float(r), device=target.device) for r in range(W)]
    world = pccl.VirtualWorld(W, target.device)

    def rank_main(comm):
        r = comm.Get_rank()
        pd.patch_deepspeed(intra, comm=comm)
        be = TorchBackend()
        assert be.reduce_scatter_tensor(t_out[r], t_in[r], op=ReduceOp.SUM, async_op=True).wait() is None
        be.all_gather_into_tensor(g_out[r], t_out[r])
        be.all_reduce(ar[r], op=ReduceOp.SUM)
        be.broadcast(bc[r], 3)
        be.barrier()
        if r == 0:      # not the world group / not a sum: the original methods run
            be.reduce_scatter_tensor(t_out[r], t_in[r], op=ReduceOp.MAX)
            be.all_gather_into_tensor(g_out[r], t_out[r], group=comm.world.subcomm([0, 1], 0))

    world.run(rank_main)
    target.sync()
    assert fell_through == ["rs", "ag"]
    want = O.reduce_scatter_2d(ins, intra, W // intra, dtype, "recursive")
    want_ar = O.all_reduce(ar_in, dtype, "recursive")
    for r in range(W):
        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"reduce_scatter rank {r}")
        assert_bits_equal(to_numpy(g_out[r], dtype), np.concatenate(want), f"all_gather rank {r}")
        assert_bits_equal(to_numpy(ar[r], dtype), want_ar[r], f"all_reduce rank {r}")
        assert bool((bc[r] == 3.0).all())


def test_patch_deepspeed_without_a_virtual_communicator_is_refused_at_patch_time():
    from pccl import patch_deepspeed as pd
    with pytest.raises(RuntimeError, match="virtual ranks only"):
        pd.patch_deepspeed(2)
    with pytest.raises(TypeError, match="must be a pccl.VirtualComm"):
        pd.patch_deepspeed(2, comm=object())


def test_patch_deepspeed_without_deepspeed_raises(target):
    import pccl
    from pccl import patch_deepspeed as pd
    with pytest.raises(RuntimeError, match="needs the deepspeed package"):
        pd.patch_deepspeed(2, comm=pccl.VirtualWorld(2, target.device).comm(0))


# ---------------------------------------------------------------------------
# buffers that share memory
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("alg,P", [("ring", 5), ("ring", 8), ("recursive", 8), ("recursive", 2)])
@pytest.mark.parametrize("mode", ["steps", "fused", "faithful"])
def test_reduce_scatter_in_place(target, dtype, alg, P, mode):
    """outputs[r] may BE block r of inputs[r] (the reference tolerates it because it
    copies the input first, pccl/src/reduce_scatter.cpp:119-123): every mode reads
    an element before the same thread overwrites it."""
    from pccl import kernels
    B = 1027
    ins = make_inputs(P, P * B, dtype, seed=70 + P)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [t_in[r][r * B:(r + 1) * B] for r in range(P)]
    want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
    target.sync()
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r].clone(), dtype), want[r], f"{alg}/{mode} rank {r}")
        # the other blocks of the input are untouched
        other = np.delete(to_numpy(t_in[r].clone(), dtype).reshape(P, B), r, axis=0)
        assert_bits_equal(other.reshape(-1), np.delete(ins[r].reshape(P, B), r, axis=0).reshape(-1), f"rank {r} input")


@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("mode", ["steps", "fused"])
def test_all_gather_in_place(target, alg, mode):
    """inputs[r] may BE block r of outputs[r] (pccl/src/all_gather.cpp:31-35 copies it there first)."""
    import torch
    from pccl import kernels
    P, n, dtype = 8, 1031, O.F32
    shards = make_inputs(P, n, dtype, seed=77)
    t_out = [torch.zeros(P * n, device=target.device) for _ in range(P)]
    t_in = []
    for r in range(P):
        t_out[r][r * n:(r + 1) * n] = to_torch(shards[r], dtype, target.device)
        t_in.append(t_out[r][r * n:(r + 1) * n])
    kernels.all_gather_ranks(t_out, t_in, alg, mode)
    target.sync()
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], dtype), np.concatenate(shards), f"rank {r}")


def test_overlapping_buffers_are_refused(target):
    """Any other sharing of memory between a written buffer and another buffer of
    the call is an argument error, reported before anything is launched."""
    import torch
    from pccl import kernels
    P, B = 4, 64
    dev = target.device
    t_in = [torch.zeros(P * B, device=dev) for _ in range(P)]
    t_out = [torch.zeros(B, device=dev) for _ in range(P)]
    work = [torch.zeros(P * B, device=dev) for _ in range(P)]

    def refused(outs, ins, mode="steps", wk=None, alg="ring"):
        with pytest.raises(RuntimeError, match="overlap in memory"):
            kernels.reduce_scatter_ranks(outs, ins, alg, mode, wk)

    # the wrong block of the own input, and another rank's input
    refused([t_in[0][B:2 * B]] + t_out[1:], t_in, "fused")
    refused([t_in[1][0:B]] + t_out[1:], t_in, "fused")
    # the right block, shifted by one element
    refused([t_in[0][1:B + 1]] + t_out[1:], t_in, "steps", work)
    # two outputs on the same memory; work space on an input; work space on an output
    refused([t_out[0], t_out[0]] + t_out[2:], t_in, "fused")
    refused(t_out, t_in, "steps", [t_in[2]] + work[1:])
    big = torch.zeros(P * B + B, device=dev)
    refused([big[P * B - 8:][:B]] + t_out[1:], t_in, "faithful", [big[:P * B]] + work[1:])
    # inputs may share memory among themselves
    kernels.reduce_scatter_ranks(t_out, [t_in[0]] * P, "ring", "fused")
    # ... but an output that is in place in its own input must not lie in a second input as well,
    # whichever of the two aliased inputs comes first in the table
    refused([t_in[0][0:B]] + t_out[1:], [t_in[0], t_in[0]] + t_in[2:], "fused")
    refused([t_out[0], t_in[1][B:2 * B]] + t_out[2:], [t_in[1]] + t_in[1:], "steps", work)
    refused(t_out[:3] + [t_in[3][3 * B:]], t_in[:2] + [t_in[3], t_in[3]], "fused")
    # all_gather: a shard inside another rank's output, outputs on top of each other
    g_out = [torch.zeros(P * B, device=dev) for _ in range(P)]
    g_in = [torch.zeros(B, device=dev) for _ in range(P)]
    with pytest.raises(RuntimeError, match="overlap in memory"):
        kernels.all_gather_ranks(g_out, [g_out[1][0:B]] + g_in[1:], "ring", "fused")
    with pytest.raises(RuntimeError, match="overlap in memory"):
        kernels.all_gather_ranks([g_out[0], g_out[0]] + g_out[2:], g_in, "recursive", "steps")
    # the fold: the output on one of its shards; add: a partial overlap
    sh = [torch.zeros(B, device=dev) for _ in range(3)]
    with pytest.raises(RuntimeError, match="overlap in memory"):
        target.native.reduce_kway(sh[1].data_ptr(), [t.data_ptr() for t in sh], B, 0, 0, 0, True, target.stream())
    with pytest.raises(RuntimeError, match="partly"):
        target.native.add(big[4:].data_ptr(), big.data_ptr(), sh[0].data_ptr(), B, 0, target.stream())
    target.sync()


def test_fused_ring_beyond_one_launch_refuses_in_place(target):
    """More ranks than one launch has shard pointers: the chain of launches keeps
    the running sum in outputs[r] while block r of inputs[r] is still to be added,
    so in-place use is refused there (the per-step modes take it)."""
    import torch
    from pccl import kernels
    P, B, dtype = 65, 16, O.F32
    ins = make_inputs(P, P * B, dtype, seed=5)
    t_in = [to_torch(x, dtype, target.device) for x in ins]
    t_out = [t_in[r][r * B:(r + 1) * B] for r in range(P)]
    with pytest.raises(RuntimeError, match="overlap in memory"):
        kernels.reduce_scatter_ranks(t_out, t_in, "ring", "fused")
    want = O.ring_reduce_scatter(ins, dtype)
    kernels.reduce_scatter_ranks(t_out, t_in, "ring", "steps")
    target.sync()
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r].clone(), dtype), want[r], f"rank {r}")
