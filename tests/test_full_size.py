"""Parity at the full sizes of the benchmark workloads (GPU only).

The numpy oracle cannot chew 4 GiB per test, but every collective here is
element-wise across ranks: output position i of block j depends only on
position j*B + i of every rank's input.  So the oracle is run on WINDOWS of the
full-size problem (start, end, unaligned middle of every block) and compared
bit for bit with the same windows of the GPU result; on top of that come
size-independent properties: the three execution modes (three different kernel
paths) agree on every byte, integer inputs give exact totals, all_gather equals
torch.cat, and 64-bit indexing is exercised beyond 2^32 bytes."""
import numpy as np
import pytest

from helpers import assert_bits_equal, to_numpy
from oracle import pccl_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MiB = 1 << 20


def _torch_dtype(dtype):
    import torch
    return {O.F32: torch.float32, O.BF16: torch.bfloat16, O.F16: torch.float16}[dtype]


def _gen(n, dtype, seed, std=1.0, kind="normal"):
    import torch
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    td = _torch_dtype(dtype)
    out = torch.empty(n, dtype=td, device=DEV)
    chunk = 1 << 26
    for i in range(0, n, chunk):
        m = min(chunk, n - i)
        if kind == "normal":
            x = torch.randn(m, generator=g, device=DEV) * std
        elif kind == "uniform":
            x = torch.rand(m, generator=g, device=DEV) * 2 - 1
        else:   # small integers
            x = torch.randint(-8, 9, (m,), generator=g, device=DEV).float()
        out[i:i + m] = x.to(td)
    return out


def _windows(B, w=4099):
    w = min(w, B)
    starts = sorted({0, max(0, B - w), max(0, min(B - w, B // 2 + 13)), max(0, min(B - w, (B // 3) | 1))})
    return [(s, w) for s in starts]


def _check_rs_windows(outs, ins, P, B, dtype, alg):
    ref = O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter
    for s, w in _windows(B):
        sub = [np.concatenate([to_numpy(ins[k][j * B + s:j * B + s + w], dtype) for j in range(P)]) for k in range(P)]
        want = ref(sub, dtype)
        for r in range(P):
            assert_bits_equal(to_numpy(outs[r][s:s + w], dtype), want[r], f"{alg} rank {r} window {s}")


def _same_bits(a, b):
    import torch
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


def test_config1_ring_p4_fp32_64mib_full_oracle():
    """Config 1 at full size, whole outputs against the oracle."""
    import torch
    from pccl import kernels
    P, n = 4, 16 * MiB
    B = n // P
    ins = [_gen(n, O.F32, 1234 + r, kind="uniform") for r in range(P)]
    want = O.ring_reduce_scatter([to_numpy(t, O.F32) for t in ins], O.F32)
    for mode in ("steps", "fused", "faithful"):
        print(f"cfg1 mode={mode}", flush=True)
        outs = [torch.zeros(B, device=DEV) for _ in range(P)]
        kernels.reduce_scatter_ranks(outs, ins, "ring", mode)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_numpy(outs[r], O.F32), want[r], f"{mode} rank {r}")


def test_config2_ring_p8_bf16_512mib_per_rank():
    """Config 2: 7 hops with bf16 rounding at every hop, 4 GiB of inputs."""
    import torch
    from pccl import kernels
    P, n = 8, 256 * MiB
    B = n // P
    ins = [_gen(n, O.BF16, 77 + r, std=1e-2) for r in range(P)]
    results = {}
    for mode in ("steps", "fused", "faithful"):
        print(f"cfg2 mode={mode}", flush=True)
        outs = [torch.zeros(B, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
        kernels.reduce_scatter_ranks(outs, ins, "ring", mode)
        torch.cuda.synchronize()
        results[mode] = outs
    _check_rs_windows(results["steps"], ins, P, B, O.BF16, "ring")
    for r in range(P):
        assert _same_bits(results["steps"][r], results["fused"][r]), f"fused differs, rank {r}"
        assert _same_bits(results["steps"][r], results["faithful"][r]), f"faithful differs, rank {r}"
    # per-hop rounding is visible: the fp32-accumulate variant gives other bits somewhere
    single = torch.zeros(B, dtype=torch.bfloat16, device=DEV)
    kernels.reduce_kway(single, [t[:B] for t in ins], "ring", 1, per_hop_round=False)
    torch.cuda.synchronize()
    assert not _same_bits(single, results["fused"][0])


def test_config2_integer_inputs_exact_totals():
    import torch
    from pccl import kernels
    P, n = 8, 64 * MiB
    B = n // P
    ins = [_gen(n, O.BF16, 5 + r, kind="int") for r in range(P)]
    total = torch.zeros(n, device=DEV)
    for t in ins:
        total += t.float()
    for alg in ("ring", "recursive"):
        for mode in ("steps", "fused"):
            outs = [torch.zeros(B, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
            kernels.reduce_scatter_ranks(outs, ins, alg, mode)
            torch.cuda.synchronize()
            for r in range(P):
                assert torch.equal(outs[r].float(), total[r * B:(r + 1) * B]), (alg, mode, r)


def test_config3_halving_round_512mib_halves():
    """Round 0 of P=64 with 1 GiB per rank, as one pair of ranks adds its
    strided halves; and the whole P=64 collective at a smaller block."""
    import torch
    from pccl import _native, kernels
    B = 256 * MiB                       # elements per half
    lib = _native.load()
    ins = [_gen(2 * B, O.BF16, 900 + r) for r in range(2)]
    work = [t.clone() for t in ins]
    lib.rh_round([w.data_ptr() for w in work], None, None, 2, B, 0, _native.BF16, kernels.stream_handle())
    torch.cuda.synchronize()
    for s, w in _windows(B):
        lo = O.vector_add(to_numpy(ins[0][s:s + w], O.BF16), to_numpy(ins[1][s:s + w], O.BF16), O.BF16)
        hi = O.vector_add(to_numpy(ins[1][B + s:B + s + w], O.BF16), to_numpy(ins[0][B + s:B + s + w], O.BF16), O.BF16)
        assert_bits_equal(to_numpy(work[0][s:s + w], O.BF16), lo, "lower rank")
        assert_bits_equal(to_numpy(work[1][B + s:B + s + w], O.BF16), hi, "upper rank")
    # the halves a rank sent away are untouched
    assert _same_bits(work[0][B:], ins[0][B:]) and _same_bits(work[1][:B], ins[1][:B])
    del work, ins
    # all 64 ranks, 6 rounds, 1 Mi-element blocks (128 MiB per rank, 8 GiB of inputs)
    P, Bs = 64, 1 * MiB
    ins = [_gen(P * Bs, O.BF16, 3000 + r) for r in range(P)]
    outs_s = [torch.zeros(Bs, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
    outs_f = [torch.zeros(Bs, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
    kernels.reduce_scatter_ranks(outs_s, ins, "recursive", "steps")
    kernels.reduce_scatter_ranks(outs_f, ins, "recursive", "fused")
    torch.cuda.synchronize()
    _check_rs_windows(outs_s, ins, P, Bs, O.BF16, "recursive")
    for r in range(P):
        assert _same_bits(outs_s[r], outs_f[r]), r


@pytest.mark.parametrize("alg,mode", [("ring", "steps"), ("recursive", "steps"), ("ring", "fused")])
def test_config4_all_gather_p16_128mib_shards(alg, mode):
    """2 GiB outputs (beyond the reference's int byte counts), all 16 materialised."""
    import torch
    from pccl import kernels
    P, n = 16, 64 * MiB
    print(f"cfg4 alg={alg} mode={mode}", flush=True)
    ins = [_gen(n, O.BF16, 40 + r) for r in range(P)]
    outs = [torch.empty(P * n, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
    for o in outs:
        o.view(torch.int16).fill_(0x5A5A)
    kernels.all_gather_ranks(outs, ins, alg, mode)
    torch.cuda.synchronize()
    cat = torch.cat(ins)
    for r in range(P):
        assert _same_bits(outs[r], cat), f"rank {r}"


@pytest.mark.parametrize("P,shard_bytes", [(64, 8 * MiB), (3, 300 * MiB + 5), (2, (1 << 32) + 4099), (5, 2 * MiB)])
def test_time_blocked_gather_shapes(P, shard_bytes):
    """The fused all_gather at shapes around its strips: many short shards (one
    strip per shard), ragged byte counts, a shard longer than 2^32 bytes, and
    the shortest shard the time-blocked kernel is chosen for."""
    import torch
    from pccl import kernels
    print(f"time-blocked gather P={P} shard={shard_bytes}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(P)
    ins = [torch.randint(0, 256, (shard_bytes,), dtype=torch.uint8, device=DEV, generator=g) for _ in range(P)]
    outs = [torch.full((P * shard_bytes,), 0x5A, dtype=torch.uint8, device=DEV) for _ in range(P)]
    kernels.all_gather_ranks(outs, ins, "ring", "fused")
    torch.cuda.synchronize()
    for r in range(P):
        for k in range(P):
            assert torch.equal(outs[r][k * shard_bytes:(k + 1) * shard_bytes], ins[k]), (r, k)


def test_config4_uneven_shards_padded_to_256_bytes():
    import torch
    from pccl import kernels
    P, n = 16, 64 * MiB
    rng = np.random.default_rng(4)
    lens = [int(n - rng.integers(0, n // 8)) for _ in range(P)]
    lens[7] |= 1                                   # an odd element count
    ins = [_gen(l, O.BF16, 60 + r) for r, l in enumerate(lens)]
    nbytes = [2 * l for l in lens]
    off = kernels.padded_offsets(nbytes, 256)
    total = off[-1] + (nbytes[-1] + 255) // 256 * 256
    outs = [torch.full((total,), 0xA5, dtype=torch.uint8, device=DEV) for _ in range(P)]
    kernels.all_gather_uneven_ranks(outs, ins, align=256)
    torch.cuda.synchronize()
    for r in (0, 5, 15):
        for k in range(P):
            assert torch.equal(outs[r][off[k]:off[k] + nbytes[k]], ins[k].view(torch.uint8)), (r, k)
            end = off[k + 1] if k + 1 < P else total
            assert bool((outs[r][off[k] + nbytes[k]:end] == 0xA5).all()), f"padding after shard {k} touched"
    assert all(_same_bits(outs[0], outs[r]) for r in range(1, P))


def test_config5_fused_32way_equals_31_hops():
    """One pass over 32 fp32 shards = 31 launches of the accumulate kernel, bit for bit."""
    import torch
    from pccl import kernels
    k, n = 32, 32 * MiB
    shards = [_gen(n, O.F32, 500 + r) for r in range(k)]
    fused = torch.empty(n, device=DEV)
    kernels.reduce_kway(fused, shards, "ring", first=1)
    acc = shards[1].clone()
    for t in range(1, k):
        kernels.accumulate(acc, shards[(1 + t) % k])
    torch.cuda.synchronize()
    assert _same_bits(fused, acc)
    for s, w in _windows(n):
        want = to_numpy(shards[1][s:s + w], O.F32)
        for t in range(1, k):
            want = O.vector_add(want, to_numpy(shards[(1 + t) % k][s:s + w], O.F32), O.F32)
        assert_bits_equal(to_numpy(fused[s:s + w], O.F32), want, f"window {s}")
    # halving order on the same shards: other association, same value up to rounding
    tree = torch.empty(n, device=DEV)
    kernels.reduce_kway(tree, shards, "halving", first=0)
    torch.cuda.synchronize()
    assert torch.allclose(tree, fused, rtol=1e-4, atol=1e-5)
    assert not _same_bits(tree, fused)


@pytest.mark.parametrize("nbytes", [4 * 1024, 16 * 1024, 64 * 1024, 256 * 1024, 1024 * 1024])
def test_small_messages_bf16(nbytes):
    """The sizes of the latency sweep (4 KiB .. 1 MiB)."""
    import torch
    from pccl import kernels
    n = nbytes // 2
    a, b = _gen(n, O.BF16, 1), _gen(n, O.BF16, 2)
    want = O.vector_add(to_numpy(a, O.BF16), to_numpy(b, O.BF16), O.BF16)
    kernels.accumulate(a, b)
    c = torch.empty_like(a)
    kernels.copy(c, a)
    torch.cuda.synchronize()
    assert_bits_equal(to_numpy(a, O.BF16), want)
    assert _same_bits(c, a)


def test_indexing_beyond_4gib():
    """One segment longer than 2^32 bytes: sizes and offsets are 64-bit end to end."""
    import torch
    from pccl import kernels
    n = (1 << 31) + 12345                         # bf16 elements: 4 GiB + 24690 bytes
    a = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    b = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    a.view(torch.int16).fill_(0x3F80)             # 1.0
    b.view(torch.int16).fill_(0x4000)             # 2.0
    tail = _gen(50000, O.BF16, 9)
    a[-50000:] = tail
    kernels.accumulate(a, b)
    torch.cuda.synchronize()
    assert bool((a[:1 << 20].view(torch.int16) == 0x4040).all())           # 3.0 at the start
    mid = (1 << 31) - 100000
    assert bool((a[mid:mid + 50000].view(torch.int16) == 0x4040).all())     # ... up to the random tail
    # the tail window [2^31 - 37655, 2^31 + 12345) straddles byte offset 2^32
    want = O.vector_add(to_numpy(tail, O.BF16), np.full(50000, 0x4000, np.uint16), O.BF16)
    assert_bits_equal(to_numpy(a[-50000:], O.BF16), want, "window across the 4 GiB line")


@pytest.mark.parametrize("alg,P,dtype", [("ring", 4, O.BF16), ("ring", 16, O.BF16), ("ring", 6, O.F32), ("ring", 16, O.F32),
                                         ("ring", 24, O.F32), ("recursive", 8, O.F32), ("recursive", 16, O.F32),
                                         ("recursive", 8, O.BF16), ("ring", 8, O.F16), ("recursive", 8, O.F16),
                                         ("recursive", 32, O.BF16), ("ring", 3, O.F32)])
def test_fused_reduce_at_streaming_sizes_equals_the_steps(alg, P, dtype):
    """From 288 MiB of traffic on the fused reduce runs with fewer workgroups per
    CU, a number chosen by shard count, element type and order: every such choice
    gives the bits of the per-step replay, and exact totals on integer inputs."""
    import torch
    from pccl import kernels
    es = 4 if dtype == O.F32 else 2
    td = _torch_dtype(dtype)
    B = (1024 * MiB // es // P // P) // 128 * 128 + 8          # about 1 GiB of inputs, blocks not a multiple of a tile
    ins = [_gen(P * B, dtype, 900 + r, kind="int") for r in range(P)]
    total = torch.zeros(P * B, device=DEV)
    for t in ins:
        total += t.float()
    outs = {}
    for mode in ("steps", "fused"):
        print(f"{alg} P={P} {dtype} mode={mode}", flush=True)
        outs[mode] = [torch.zeros(B, dtype=td, device=DEV) for _ in range(P)]
        kernels.reduce_scatter_ranks(outs[mode], ins, alg, mode)
        torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(outs["fused"][r].float(), total[r * B:(r + 1) * B]), f"totals, rank {r}"
        assert _same_bits(outs["fused"][r], outs["steps"][r]), f"rank {r}"
    del ins, total
    ins = [_gen(P * B, dtype, 950 + r) for r in range(P)]
    for mode in ("steps", "fused"):
        kernels.reduce_scatter_ranks(outs[mode], ins, alg, mode)
        torch.cuda.synchronize()
    for r in range(P):
        assert _same_bits(outs["fused"][r], outs["steps"][r]), f"random inputs, rank {r}"
    _check_rs_windows(outs["fused"], ins, P, B, dtype, alg)


@pytest.mark.parametrize("intra,inter,dtype", [(4, 2, O.F32), (4, 2, O.BF16), (4, 4, O.BF16), (4, 2, O.F16), (3, 2, O.F32),
                                               (16, 8, O.BF16)])
def test_fused_two_level_reduce_at_streaming_sizes_equals_the_steps(intra, inter, dtype):
    import torch
    from pccl import kernels
    W = intra * inter
    es = 4 if dtype == O.F32 else 2
    td = _torch_dtype(dtype)
    m = (1024 * MiB // es // W // W) // 128 * 128 + 8
    ins = [_gen(W * m, dtype, 700 + r) for r in range(W)]
    outs = {}
    for mode in ("steps", "fused"):
        print(f"2-D ring {intra}x{inter} {dtype} mode={mode}", flush=True)
        outs[mode] = [torch.zeros(m, dtype=td, device=DEV) for _ in range(W)]
        kernels.reduce_scatter_2d_ranks(outs[mode], ins, intra, inter, "ring", mode)
        torch.cuda.synchronize()
    for w in range(W):
        assert _same_bits(outs["fused"][w], outs["steps"][w]), f"rank {w}"
    s, n = m // 2 + 5, 2053
    sub = [np.concatenate([to_numpy(ins[k][j * m + s:j * m + s + n], dtype) for j in range(W)]) for k in range(W)]
    want = O.reduce_scatter_2d(sub, intra, inter, dtype, "ring")
    for w in range(W):
        assert_bits_equal(to_numpy(outs["fused"][w][s:s + n], dtype), want[w], f"window, rank {w}")
