"""GPU parity of the individual HIP kernels against the CPU oracle, through the
C ABI (ctypes -> libpccl_hip.so).  Bit-exact: these are IEEE adds in a fixed
order and byte copies."""
import numpy as np
import pytest

from helpers import assert_bits_equal, make_inputs, to_numpy, to_torch
from oracle import pccl_oracle as O

DTYPES = [O.F32, O.BF16]
CODE = {O.F32: 0, O.BF16: 1}


# sizes: empty, sub-vector, one vector, ragged, exactly one tile (256*4 vectors), several tiles + tail
SIZES = [0, 1, 3, 4, 8, 9, 255, 1024, 4096, 4097, 8192 + 5, 300_001]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", SIZES)
def test_accumulate_matches_oracle(target, dtype, n):
    import torch
    print(f"accumulate dtype={dtype} n={n}", flush=True)
    a, b = make_inputs(2, n, dtype, seed=11)
    ta, tb = to_torch(a, dtype, target.device), to_torch(b, dtype, target.device)
    target.native.accumulate(ta.data_ptr(), tb.data_ptr(), n, CODE[dtype], target.stream())
    target.sync()
    assert_bits_equal(to_numpy(ta, dtype), O.vector_add(a, b, dtype), "accumulate")
    assert_bits_equal(to_numpy(tb, dtype), b, "src untouched")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shift", [(0, 0, 0), (1, 1, 1), (3, 3, 3), (1, 2, 3), (0, 1, 0)])
def test_add_any_alignment(target, dtype, shift):
    """Operands that start off a 16-byte boundary: common misalignment takes the
    peeled vector path, different misalignments the element path."""
    import torch
    n = 5000
    print(f"add alignment dtype={dtype} shift={shift}", flush=True)
    a, b = make_inputs(2, n + 8, dtype, seed=5)
    ta, tb = to_torch(a, dtype, target.device), to_torch(b, dtype, target.device)
    td = torch.zeros(n + 16, dtype=ta.dtype, device=target.device)
    sd, sa, sb = shift
    es = ta.element_size()
    target.native.add(td.data_ptr() + sd * es, ta.data_ptr() + sa * es, tb.data_ptr() + sb * es, n, CODE[dtype],
               target.stream())
    target.sync()
    got = to_numpy(td, dtype)
    assert_bits_equal(got[sd:sd + n], O.vector_add(a[sa:sa + n], b[sb:sb + n], dtype), "add")
    assert not got[:sd].any() and not got[sd + n:].any(), "wrote outside the destination"


@pytest.mark.parametrize("dtype", DTYPES)
def test_bf16_and_f32_special_values(target, dtype):
    """Infinities, NaN, signed zeros, denormals and rounding ties go through the
    same bits as the oracle."""
    import torch
    if dtype == O.F32:
        vals = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, 1e-38,
                         1.0 + 2 ** -23, 2 ** -24, 16777216.0], dtype=np.float32)
    else:
        # every bf16 exponent with a few mantissas, plus specials
        pats = [0x0000, 0x8000, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x7FC0, 0x0001, 0x8001, 0x7F7F, 0x0080,
                0x3F81, 0x3B80, 0x4B80, 0x3FFF, 0x4000, 0x3C00, 0x3C01]
        vals = np.array(pats, dtype=np.uint16)
    a = np.repeat(vals, vals.size)
    b = np.tile(vals, vals.size)
    ta, tb = to_torch(a, dtype, target.device), to_torch(b, dtype, target.device)
    target.native.accumulate(ta.data_ptr(), tb.data_ptr(), a.size, CODE[dtype], target.stream())
    target.sync()
    assert_bits_equal(to_numpy(ta, dtype), O.vector_add(a, b, dtype), "special values")


def test_bf16_add_all_exponent_pairs(target):
    """All 2^16 bf16 patterns against 64 partners spanning the exponent range."""
    import torch
    a = np.arange(65536, dtype=np.uint16)
    partners = np.concatenate([np.arange(0, 65536, 2048, dtype=np.uint16) | np.uint16(0x55),
                               np.arange(0, 65536, 2048, dtype=np.uint16) | np.uint16(0x2A)])
    A = np.tile(a, partners.size)
    Bv = np.repeat(partners, a.size)
    ta, tb = to_torch(A, O.BF16, target.device), to_torch(Bv, O.BF16, target.device)
    target.native.accumulate(ta.data_ptr(), tb.data_ptr(), A.size, 1, target.stream())
    target.sync()
    assert_bits_equal(to_numpy(ta, O.BF16), O.vector_add(A, Bv, O.BF16), "bf16 exhaustive")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("count,n", [(1, 1000), (5, 4099), (64, 777)])
def test_add_batched(target, dtype, count, n):
    import torch
    print(f"add_batched dtype={dtype} count={count} n={n}", flush=True)
    a = make_inputs(count, n, dtype, seed=1)
    b = make_inputs(count, n, dtype, seed=100)
    ta = [to_torch(x, dtype, target.device) for x in a]
    tb = [to_torch(x, dtype, target.device) for x in b]
    td = [torch.zeros_like(t) for t in ta]
    target.native.add_batched([t.data_ptr() for t in td], [t.data_ptr() for t in ta], [t.data_ptr() for t in tb],
                       n, CODE[dtype], target.stream())
    target.sync()
    for s in range(count):
        assert_bits_equal(to_numpy(td[s], dtype), O.vector_add(a[s], b[s], dtype), f"segment {s}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [2, 3, 4, 7, 8, 16, 32, 64])
@pytest.mark.parametrize("order", ["ring", "halving"])
def test_reduce_kway_matches_sequential_hops(target, dtype, k, order):
    """The fused reduce equals k-1 oracle hops in the schedule's order."""
    import torch
    if order == "halving" and k & (k - 1):
        pytest.skip("halving order needs a power of two")
    n = 3001
    first = (k // 3) % k
    print(f"reduce_kway dtype={dtype} k={k} order={order} first={first}", flush=True)
    shards = make_inputs(k, n, dtype, seed=7)
    ts = [to_torch(x, dtype, target.device) for x in shards]
    out = torch.zeros_like(ts[0])
    target.native.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, CODE[dtype],
                       0 if order == "ring" else 1, first, True, target.stream())
    target.sync()
    if order == "ring":
        want = shards[first]
        for t in range(1, k):
            want = O.vector_add(want, shards[(first + t) % k], dtype)
    else:
        v = [shards[first ^ m] for m in range(k)]
        h = k // 2
        while h >= 1:
            for m in range(h):
                v[m] = O.vector_add(v[m], v[m + h], dtype)
            h //= 2
        want = v[0]
    assert_bits_equal(to_numpy(out, dtype), want, "reduce_kway")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("order,k", [("ring", 5), ("ring", 17), ("halving", 4), ("halving", 16)])
@pytest.mark.parametrize("out_shift", [0, 3])
def test_reduce_kway_shards_at_any_alignment(target, dtype, order, k, out_shift):
    """Every shard at its own element alignment (the fold reads 16-byte vectors
    wherever they lie), the output aligned (vector stores) or not (elements)."""
    import torch
    n = 70001
    shards = make_inputs(k, n, dtype, seed=60 + k)
    shifts = [(3 * q + 1) % 8 for q in range(k)]
    bufs = [to_torch(np.concatenate([np.zeros(sh, x.dtype), x, np.zeros(8 - sh, x.dtype)]), dtype, target.device)
            for x, sh in zip(shards, shifts)]
    ts = [b[sh:sh + n] for b, sh in zip(bufs, shifts)]
    out_big = torch.zeros(n + 8, dtype=ts[0].dtype, device=target.device)
    out = out_big[out_shift:out_shift + n]
    first = 2 % k
    target.native.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, CODE[dtype],
                              0 if order == "ring" else 1, first, True, target.stream())
    target.sync()
    if order == "ring":
        want = shards[first]
        for t in range(1, k):
            want = O.vector_add(want, shards[(first + t) % k], dtype)
    else:
        v = [shards[first ^ m] for m in range(k)]
        h = k // 2
        while h >= 1:
            for m in range(h):
                v[m] = O.vector_add(v[m], v[m + h], dtype)
            h //= 2
        want = v[0]
    assert_bits_equal(to_numpy(out.clone(), dtype), want, "fold of unaligned shards")
    assert not out_big[:out_shift].float().abs().sum() and not out_big[out_shift + n:].float().abs().sum()


def test_reduce_kway_bf16_single_rounding(target):
    """per_hop_round=0: fp32 partial sums, one rounding at the end (within 1 ulp
    of the per-hop result per hop; here checked exactly against numpy)."""
    import torch
    k, n = 8, 4099
    shards = make_inputs(k, n, O.BF16, seed=3)
    ts = [to_torch(x, O.BF16, target.device) for x in shards]
    out = torch.zeros_like(ts[0])
    target.native.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, 1, 0, 0, False,
                       target.stream())
    target.sync()
    acc = O.bf16_to_f32(shards[0])
    for t in range(1, k):
        acc = (acc + O.bf16_to_f32(shards[t])).astype(np.float32)
    assert_bits_equal(to_numpy(out, O.BF16), O.f32_to_bf16(acc), "single rounding")


@pytest.mark.parametrize("sizes", [[0], [1], [15, 16, 17], [4096, 1, 70000, 0, 33], [5] * 64])
@pytest.mark.parametrize("shift", [0, 1, 4])
def test_copy_batched_ragged(target, sizes, shift):
    import torch
    print(f"copy_batched sizes={sizes[:5]} shift={shift}", flush=True)
    rng = np.random.default_rng(0)
    srcs = [rng.integers(0, 256, s + 8, dtype=np.uint8) for s in sizes]
    ts = [torch.from_numpy(x).to(target.device) for x in srcs]
    td = [torch.full((s + 32,), 0xA5, dtype=torch.uint8, device=target.device) for s in sizes]
    target.native.copy_batched([t.data_ptr() + 16 + shift for t in td], [t.data_ptr() + shift for t in ts], sizes,
                        target.stream())
    target.sync()
    for s, src, dst in zip(sizes, srcs, td):
        got = dst.cpu().numpy()
        assert np.array_equal(got[16 + shift:16 + shift + s], src[shift:shift + s])
        assert (got[:16 + shift] == 0xA5).all() and (got[16 + shift + s:] == 0xA5).all()


def test_copy_mismatched_alignment(target):
    import torch
    rng = np.random.default_rng(1)
    src = rng.integers(0, 256, 10007, dtype=np.uint8)
    ts = torch.from_numpy(src).to(target.device)
    for ds, ss in [(1, 2), (4, 8), (3, 0), (0, 5)]:
        n = 9990
        td = torch.full((n + 32,), 0x5A, dtype=torch.uint8, device=target.device)
        target.native.copy_batched([td.data_ptr() + ds], [ts.data_ptr() + ss], [n], target.stream())
        target.sync()
        got = td.cpu().numpy()
        assert np.array_equal(got[ds:ds + n], src[ss:ss + n]), (ds, ss)
        assert (got[:ds] == 0x5A).all() and (got[ds + n:] == 0x5A).all()


@pytest.mark.parametrize("rows,cols,m", [(2, 4, 64), (4, 2, 6), (8, 8, 4096 + 16), (1, 5, 3), (3, 1, 10)])
def test_block_transpose(target, rows, cols, m):
    import torch
    x = np.random.default_rng(2).integers(0, 256, rows * cols * m, dtype=np.uint8)
    tx = torch.from_numpy(x).to(target.device)
    ty = torch.zeros_like(tx)
    target.native.block_transpose(ty.data_ptr(), tx.data_ptr(), rows, cols, m, target.stream())
    target.sync()
    assert np.array_equal(ty.cpu().numpy(), O.block_transpose(x, rows, cols))
    want = tx.view(rows, cols, -1).transpose(0, 1).reshape(-1)
    assert torch.equal(ty, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P", [2, 4, 8])
def test_rh_round_is_the_pairwise_half_add(target, dtype, P):
    """One round in place on the work buffers against the two branches of the
    reference written out with numpy slices."""
    import torch
    B = 517
    bufs = make_inputs(P, P * B, dtype, seed=9)
    tb = [to_torch(x, dtype, target.device) for x in bufs]
    cur = [x.copy() for x in bufs]
    rounds = P.bit_length() - 1
    for rnd in range(rounds):
        target.native.rh_round([t.data_ptr() for t in tb], None, None, P, B, rnd, CODE[dtype],
                        target.stream())
        target.sync()
        group = P >> rnd
        half = group // 2
        count = half * B
        snap = [c.copy() for c in cur]
        for r in range(P):
            start = (r // group) * group * B
            if r % group < half:
                p = r + half
                cur[r][start:start + count] = O.vector_add(snap[r][start:start + count],
                                                           snap[p][start:start + count], dtype)
            else:
                p = r - half
                cur[r][start + count:start + 2 * count] = O.vector_add(
                    snap[r][start + count:start + 2 * count], snap[p][start + count:start + 2 * count], dtype)
        for r in range(P):
            assert_bits_equal(to_numpy(tb[r], dtype), cur[r], f"round {rnd} rank {r}")


def test_invalid_arguments_return_codes(target):
    """Errors come back as codes + messages; nothing is launched."""
    from pccl._native import NativeError
    with pytest.raises(NativeError, match="unknown dtype"):
        target.native.accumulate(16, 16, 4, 7)
    with pytest.raises(NativeError, match="Unknown algorithm specified for reduce_scatter_mpi: tree"):
        target.native.reduce_scatter_virtual([16], [16], None, 4, 0, "tree")
    with pytest.raises(NativeError, match="power-of-two"):
        target.native.reduce_scatter_virtual([16] * 3, [16] * 3, [16] * 3, 4, 0, "recursive")


def test_probe_streams(target):
    """The read probe leaves the buffer alone; the write probe fills it with bf16 1.0."""
    import torch
    n = 70_000
    buf = torch.arange(n, dtype=torch.int32, device=target.device)
    before = buf.clone()
    target.native.probe_stream(0, buf.data_ptr(), n * 4, target.stream())
    target.sync()
    assert torch.equal(buf, before)
    target.native.probe_stream(1, buf.data_ptr(), n * 4, target.stream())
    target.sync()
    assert bool((buf.view(torch.int16) == 0x3F80).all())
    from pccl._native import NativeError
    with pytest.raises(NativeError, match="kind must be"):
        target.native.probe_stream(2, buf.data_ptr(), n * 4, target.stream())


@pytest.mark.parametrize("unroll", [1, 2, 4, 8])
@pytest.mark.parametrize("nt", [0, 1])
@pytest.mark.parametrize("grid_cap", [0, 3, 64])
def test_every_launch_tuning_gives_the_same_bits(target, unroll, nt, grid_cap):
    """Unroll depth, non-temporal hints and a capped (grid-stride) launch change
    speed only."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = {k: lib.get_tuning(k) for k in ("unroll", "unroll_copy", "nt_load", "nt_store", "grid_cap")}
    try:
        lib.set_tuning("unroll", unroll)
        lib.set_tuning("unroll_copy", unroll)
        lib.set_tuning("nt_load", nt)
        lib.set_tuning("nt_store", nt)
        lib.set_tuning("grid_cap", grid_cap)
        P, B = 4, 9001
        for dtype in DTYPES:
            ins = make_inputs(P, P * B, dtype, seed=17)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            for alg, ref in (("ring", O.ring_reduce_scatter), ("recursive", O.recursive_halving_reduce_scatter)):
                want = ref(ins, dtype)
                for mode in ("steps", "fused", "faithful"):
                    t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
                    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
                    target.sync()
                    for r in range(P):
                        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"{alg}/{mode}/{dtype} rank {r}")
            g_out = [torch.zeros(P * P * B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
            for mode in ("steps", "fused"):
                kernels.all_gather_ranks(g_out, t_in, "recursive", mode)
                target.sync()
                assert_bits_equal(to_numpy(g_out[P - 1], dtype), np.concatenate(ins), f"all_gather {mode}")
    finally:
        for k, v in saved.items():
            lib.set_tuning(k, v)


@pytest.mark.parametrize("grid_cap", [0, 7])
def test_ragged_collectives_and_capped_grids(target, grid_cap):
    """Ragged blocks (the general kernels) through every collective, with one
    workgroup per tile and with a grid capped to a few workgroups that stride
    over the tiles."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = lib.get_tuning("grid_cap")
    try:
        lib.set_tuning("grid_cap", grid_cap)
        P, B = 4, 150_001
        for dtype in DTYPES:
            ins = make_inputs(P, P * B, dtype, seed=23)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            for alg, ref in (("ring", O.ring_reduce_scatter), ("recursive", O.recursive_halving_reduce_scatter)):
                want = ref(ins, dtype)
                for mode in ("steps", "fused", "faithful"):
                    t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
                    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
                    target.sync()
                    for r in range(P):
                        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"{alg}/{mode}/{dtype} rank {r}")
            g_in = [t[:B + 3] for t in t_in]
            for alg in ("recursive", "ring"):
                for mode in ("steps", "fused"):
                    g_out = [torch.zeros(P * (B + 3), dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
                    kernels.all_gather_ranks(g_out, g_in, alg, mode)
                    target.sync()
                    for r in range(P):
                        assert_bits_equal(to_numpy(g_out[r], dtype), np.concatenate([x[:B + 3] for x in ins]),
                                          f"all_gather {alg}/{mode} rank {r}")
            # 2-D grid and the block transpose
            want2 = O.reduce_scatter_2d(ins, 2, 2, dtype, "ring")
            for mode in ("steps", "fused"):
                t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
                kernels.reduce_scatter_2d_ranks(t_out, t_in, 2, 2, "ring", mode)
                target.sync()
                for r in range(P):
                    assert_bits_equal(to_numpy(t_out[r], dtype), want2[r], f"2d/{mode}/{dtype} rank {r}")
        src = torch.arange(3 * 5 * 100_003, dtype=torch.int32, device=target.device).view(torch.uint8)
        dst = torch.zeros_like(src)
        kernels.block_transpose(dst, src, 3, 5)
        target.sync()
        want_t = src.view(torch.int32).view(3, 5, 100_003).transpose(0, 1).reshape(-1)
        assert torch.equal(dst.view(torch.int32), want_t)
    finally:
        lib.set_tuning("grid_cap", saved)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8])
def test_copy_chunk_mapping_covers_every_byte(target, unroll):
    """The vectors of a copying thread come from 4 KiB chunks 8 apart: every
    length around the boundaries of chunks and of groups of 8 tiles, aligned or
    not, is copied completely and nothing else is written."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = lib.get_tuning("unroll_copy")
    chunk = 4096
    lengths = sorted({c * chunk + d for c in (0, 1, 7, 8, 9, 15, 16, 17, 8 * unroll - 1, 8 * unroll, 8 * unroll + 1,
                                              16 * unroll + 3) for d in (-17, -16, -1, 0, 1, 16, 33) if c * chunk + d > 0})
    try:
        lib.set_tuning("unroll_copy", unroll)
        for shift_d, shift_s in ((0, 0), (16, 0), (3, 3), (5, 9)):
            srcs, dsts, want = [], [], []
            for i, n in enumerate(lengths):
                g = torch.Generator().manual_seed(i)
                s = torch.randint(0, 256, (n + 64,), dtype=torch.uint8, generator=g).to(target.device)
                d = torch.full((n + 64,), 0xEE, dtype=torch.uint8, device=target.device)
                srcs.append(s[shift_s:shift_s + n]); dsts.append(d[shift_d:shift_d + n]); want.append((d, s))
            kernels.copy_batched(dsts, srcs)
            target.sync()
            for (d, s), n in zip(want, lengths):
                assert torch.equal(d[shift_d:shift_d + n], s[shift_s:shift_s + n]), f"length {n} shifts {shift_d},{shift_s}"
                assert bool((d[:shift_d] == 0xEE).all()) and bool((d[shift_d + n:] == 0xEE).all()), f"length {n}"
    finally:
        lib.set_tuning("unroll_copy", saved)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,order", [(8, "ring"), (16, "ring"), (8, "halving"), (16, "halving"), (32, "halving"),
                                     (64, "halving")])
def test_reduce_kway_special_values(target, dtype, k, order):
    """Infinities, NaNs of any payload, signed zeros, denormals and the largest
    finite values folded by the fused reduce give the oracle's bits in every
    code path (fp32 lanes, packed bf16 partial sums)."""
    import torch
    rng = np.random.default_rng(99 + k)
    n = 5000
    if dtype == O.F32:
        pool = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 1e-38,
                         1.0 + 2 ** -23, 2 ** -24, 16777216.0, 0.5, -0.25], dtype=np.float32)
        shards = [rng.choice(pool, n, p=None).astype(np.float32) for _ in range(k)]
        # mostly ordinary values, so that specials meet finite partial sums as well
        for s in shards:
            keep = rng.random(n) < 0.9
            s[keep] = rng.standard_normal(int(keep.sum())).astype(np.float32)
    else:
        pool = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x7FC0, 0x7FA1, 0xFFFF, 0x0001, 0x8001,
                         0x7F7F, 0xFF7F, 0x0080, 0x3F81, 0x3B80, 0x4B80, 0x3FFF], dtype=np.uint16)
        shards = [rng.choice(pool, n).astype(np.uint16) for _ in range(k)]
        for s in shards:
            keep = rng.random(n) < 0.9
            s[keep] = O.f32_to_bf16(rng.standard_normal(int(keep.sum())).astype(np.float32))
    first = 5 % k
    ts = [to_torch(x, dtype, target.device) for x in shards]
    out = torch.zeros_like(ts[0])
    target.native.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, CODE[dtype],
                              0 if order == "ring" else 1, first, True, target.stream())
    target.sync()
    with np.errstate(all="ignore"):
        if order == "ring":
            want = shards[first]
            for t in range(1, k):
                want = O.vector_add(want, shards[(first + t) % k], dtype)
        else:
            v = [shards[first ^ m] for m in range(k)]
            h = k // 2
            while h >= 1:
                for m in range(h):
                    v[m] = O.vector_add(v[m], v[m + h], dtype)
                h //= 2
            want = v[0]
    got = to_numpy(out, dtype)
    if dtype == O.F32:
        # which payload and sign a sum of two different NaNs carries is left open by
        # IEEE 754 and differs between processors: NaN must meet NaN, all else bit for bit
        assert np.array_equal(np.isnan(got), np.isnan(want))
        got, want = np.where(np.isnan(got), np.float32(0), got), np.where(np.isnan(want), np.float32(0), want)
    assert_bits_equal(got, want, "reduce_kway special values")


def _fold_want(shards, dtype, order, first):
    k = len(shards)
    if order == "ring":
        want = shards[first]
        for t in range(1, k):
            want = O.vector_add(want, shards[(first + t) % k], dtype)
        return want
    v = [shards[first ^ m] for m in range(k)]
    h = k // 2
    while h >= 1:
        for m in range(h):
            v[m] = O.vector_add(v[m], v[m + h], dtype)
        h //= 2
    return v[0]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fold_rows", [1, 0])
def test_lean_and_general_fold_kernels_agree(target, dtype, fold_rows):
    """Aligned ring-order folds over up to 16 shards of streams from HBM go to the
    lean kernel on a 2-D grid (fold_rows = 1, the default; forced at test sizes by
    the one-wave and non-temporal settings), everything else to the general
    kernel: both must give the oracle's bits, flat and as whole reduce_scatters."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = {k: lib.get_tuning(k) for k in ("wg_kway", "nt_load", "nt_store", "lds_pad_kway", "fold_rows")}
    try:
        for key, val in (("wg_kway", 64), ("nt_load", 1), ("nt_store", 1), ("fold_rows", fold_rows)):
            lib.set_tuning(key, val)
        per_vec = 4 if dtype == O.F32 else 8
        for k, nvec, pad in ((2, 64, 0), (3, 65, 0), (4, 1, 7168), (5, 200, 0), (8, 129, 8192), (12, 63, 0), (16, 70, 9216), (17, 64, 0)):
            lib.set_tuning("lds_pad_kway", pad)
            n = nvec * per_vec
            shards = make_inputs(k, n, dtype, seed=300 + k)
            ts = [to_torch(x, dtype, target.device) for x in shards]
            out = torch.zeros(n, dtype=ts[0].dtype, device=target.device)
            first = (2 * k // 3) % k
            print(f"lean fold dtype={dtype} fold_rows={fold_rows} k={k} n={n}", flush=True)
            lib.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, CODE[dtype], 0, first, True, target.stream())
            target.sync()
            assert_bits_equal(to_numpy(out, dtype), _fold_want(shards, dtype, "ring", first), f"k={k}")
        lib.set_tuning("lds_pad_kway", 0)
        for P, B in ((3, 64 * per_vec), (8, 67 * per_vec), (16, 3 * per_vec)):
            ins = make_inputs(P, P * B, dtype, seed=77 + P)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
            print(f"lean fold reduce_scatter dtype={dtype} fold_rows={fold_rows} P={P} B={B}", flush=True)
            kernels.reduce_scatter_ranks(t_out, t_in, "ring", "fused")
            target.sync()
            want = O.ring_reduce_scatter(ins, dtype)
            for r in range(P):
                assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"P={P} rank {r}")
            t_io = [t.clone() for t in t_in]                       # in place: output r is block r of input r
            kernels.reduce_scatter_ranks([t_io[r][r * B:(r + 1) * B] for r in range(P)], t_io, "ring", "fused")
            target.sync()
            for r in range(P):
                assert_bits_equal(to_numpy(t_io[r][r * B:(r + 1) * B].clone(), dtype), want[r], f"in place P={P} rank {r}")
        # a grid beyond the shards of one launch: one fold per node (16 shards), then one per local rank (8)
        intra, inter, m = 16, 8, 4 * per_vec
        W = intra * inter
        ins = make_inputs(W, W * m, dtype, seed=900)
        t_in = [to_torch(x, dtype, target.device) for x in ins]
        t_out = [torch.zeros(m, dtype=t_in[0].dtype, device=target.device) for _ in range(W)]
        print(f"lean fold 2-D {intra}x{inter} dtype={dtype} fold_rows={fold_rows}", flush=True)
        kernels.reduce_scatter_2d_ranks(t_out, t_in, intra, inter, "ring", "fused")
        target.sync()
        want = O.reduce_scatter_2d(ins, intra, inter, dtype, "ring")
        for w in range(W):
            assert_bits_equal(to_numpy(t_out[w], dtype), want[w], f"2-D rank {w}")
    finally:
        for key, val in saved.items():
            lib.set_tuning(key, val)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("order", ["ring", "halving"])
def test_one_wave_fold_gives_the_same_bits(target, dtype, order):
    """The fused reduce with one-wave workgroups and paired loads (what streams
    from HBM get; forced here at test sizes): every k, shards at any alignment,
    whole reduce_scatters flat and on a grid."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = {k: lib.get_tuning(k) for k in ("wg_kway", "nt_load", "nt_store", "lds_pad_kway")}
    try:
        lib.set_tuning("wg_kway", 64)
        lib.set_tuning("nt_load", 1)
        lib.set_tuning("nt_store", 1)
        for pad in (0, 8192):
            lib.set_tuning("lds_pad_kway", pad)
            for k in (2, 3, 4, 7, 8, 16, 17, 32, 64):
                if order == "halving" and k & (k - 1):
                    continue
                n = 3001 if k < 32 else 1037
                shards = make_inputs(k, n, dtype, seed=100 + k)
                shifts = [(3 * q + 1) % 8 if pad else 0 for q in range(k)]      # second pass: every shard at its own alignment
                bufs = [to_torch(np.concatenate([np.zeros(sh, x.dtype), x, np.zeros(8 - sh, x.dtype)]), dtype, target.device)
                        for x, sh in zip(shards, shifts)]
                ts = [b[sh:sh + n] for b, sh in zip(bufs, shifts)]
                out_big = torch.zeros(n + 8, dtype=ts[0].dtype, device=target.device)
                out = out_big[(3 if pad else 0):][:n]
                first = (k // 3) % k
                print(f"one-wave fold dtype={dtype} order={order} k={k} pad={pad}", flush=True)
                lib.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, CODE[dtype], 0 if order == "ring" else 1,
                                first, True, target.stream())
                target.sync()
                assert_bits_equal(to_numpy(out.clone(), dtype), _fold_want(shards, dtype, order, first), f"k={k} pad={pad}")
        alg = "ring" if order == "ring" else "recursive"
        for P, B in ((4, 9001), (8, 515)):
            ins = make_inputs(P, P * B, dtype, seed=31 + P)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            want = (O.ring_reduce_scatter if order == "ring" else O.recursive_halving_reduce_scatter)(ins, dtype)
            t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
            kernels.reduce_scatter_ranks(t_out, t_in, alg, "fused")
            target.sync()
            for r in range(P):
                assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"{alg} P={P} rank {r}")
            want2 = O.reduce_scatter_2d(ins, 2, P // 2, dtype, alg)
            kernels.reduce_scatter_2d_ranks(t_out, t_in, 2, P // 2, alg, "fused")
            target.sync()
            for r in range(P):
                assert_bits_equal(to_numpy(t_out[r], dtype), want2[r], f"2-D {alg} 2x{P // 2} rank {r}")
        # the two-level ring order issues its loads in pairs across the borders of the groups: group sizes
        # that are even, odd and larger than the number of groups, blocks of whole vectors and ragged ones
        for intra, inter, m in (((4, 2, 520), (3, 2, 77), (2, 3, 1024), (5, 3, 9), (8, 8, 131), (3, 5, 64), (7, 1, 33), (1, 6, 40))
                                if order == "ring" else ()):
            W = intra * inter
            ins = make_inputs(W, W * m, dtype, seed=500 + W)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            t_out = [torch.zeros(m, dtype=t_in[0].dtype, device=target.device) for _ in range(W)]
            print(f"one-wave fold 2-D ring {intra}x{inter} m={m} dtype={dtype}", flush=True)
            kernels.reduce_scatter_2d_ranks(t_out, t_in, intra, inter, "ring", "fused")
            target.sync()
            want2 = O.reduce_scatter_2d(ins, intra, inter, dtype, "ring")
            for w in range(W):
                assert_bits_equal(to_numpy(t_out[w], dtype), want2[w], f"2-D ring {intra}x{inter} rank {w}")
    finally:
        for k, v in saved.items():
            lib.set_tuning(k, v)


@pytest.mark.parametrize("add_rows", [0, 1])
def test_lean_and_general_add_kernels_agree(target, add_rows):
    """Aligned contiguous adds go to the lean one-wave kernels, everything else
    (and everything when add_rows = 0) to the general ones."""
    import torch
    from pccl import kernels
    lib = target.native
    saved = {k: lib.get_tuning(k) for k in ("add_rows",)}
    try:
        lib.set_tuning("add_rows", add_rows)
        P, B = 4, 150_000          # blocks of whole vectors: the aligned path
        for dtype in DTYPES:
            ins = make_inputs(P, P * B, dtype, seed=29)
            t_in = [to_torch(x, dtype, target.device) for x in ins]
            for alg, ref in (("ring", O.ring_reduce_scatter), ("recursive", O.recursive_halving_reduce_scatter)):
                want = ref(ins, dtype)
                for mode in ("steps", "faithful"):
                    t_out = [torch.zeros(B, dtype=t_in[0].dtype, device=target.device) for _ in range(P)]
                    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
                    target.sync()
                    for r in range(P):
                        assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"{alg}/{mode}/{dtype} rank {r}")
            a, b = ins[0], ins[1]
            ta, tb = to_torch(a, dtype, target.device), to_torch(b, dtype, target.device)
            kernels.accumulate(ta, tb)
            target.sync()
            assert_bits_equal(to_numpy(ta, dtype), O.vector_add(a, b, dtype), "accumulate")
    finally:
        for k, v in saved.items():
            lib.set_tuning(k, v)
