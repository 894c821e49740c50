"""float16 as a third element type, end to end: the reference's Python algorithms
add whatever torch dtype they are given (pccl/reduce_scatter.py:24,83,95,158), and
ZeRO hands them float16 gradients through pccl/patch_deepspeed.py:42-59.  Every
hop is RNE_f16(float(a) + float(b)), checked bit for bit against the oracle, whose
arithmetic tests/test_oracle.py pins against torch's CPU float16 add.  NaN results
are stored as 0x7E00 by the kernels and by the oracle; which payload another
implementation would keep is unpinned."""
import numpy as np
import pytest

from helpers import assert_bits_equal, make_inputs, to_numpy, to_torch
from oracle import pccl_oracle as O

F16 = 2      # PCCL_HIP_F16


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 1024, 4097, 300_001])
def test_accumulate(target, n):
    a, b = make_inputs(2, n, O.F16, seed=3)
    ta, tb = to_torch(a, O.F16, target.device), to_torch(b, O.F16, target.device)
    target.native.accumulate(ta.data_ptr(), tb.data_ptr(), n, F16, target.stream())
    target.sync()
    assert_bits_equal(to_numpy(ta, O.F16), O.vector_add(a, b, O.F16), f"n={n}")


def test_every_bit_pattern_against_every_exponent(target):
    """All 65 536 patterns against 78 partners (every exponent, zeros, infinities,
    subnormals, the largest finite values, NaNs) through the lean kernel, the general
    kernel (operands one element apart in alignment) and the fused reduce."""
    import torch
    a = np.arange(65536, dtype=np.uint16)
    partners = np.concatenate([np.arange(0, 65536, 1024, dtype=np.uint16) | np.uint16(0x135),
                               np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF,
                                         0x3C00, 0x3C01, 0x7E00, 0x7D01], np.uint16)])
    A, B = np.tile(a, partners.size), np.repeat(partners, a.size)
    want = O.vector_add(A, B, O.F16)
    ta, tb = to_torch(A, O.F16, target.device), to_torch(B, O.F16, target.device)
    out = torch.zeros_like(ta)
    target.native.add(out.data_ptr(), ta.data_ptr(), tb.data_ptr(), A.size, F16, target.stream())
    target.sync()
    assert_bits_equal(to_numpy(out, O.F16), want, "lean add")
    big = torch.zeros(A.size + 8, dtype=torch.float16, device=target.device)
    big[1:A.size + 1] = ta
    out.zero_()
    target.native.add(out.data_ptr(), big[1:].data_ptr(), tb.data_ptr(), A.size, F16, target.stream())
    target.sync()
    assert_bits_equal(to_numpy(out, O.F16), want, "general add")
    out.zero_()
    target.native.reduce_kway(out.data_ptr(), [ta.data_ptr(), tb.data_ptr()], A.size, F16, 0, 0, True, target.stream())
    target.sync()
    assert_bits_equal(to_numpy(out, O.F16), want, "two-way fold")


@pytest.mark.parametrize("order", ["ring", "halving"])
@pytest.mark.parametrize("k", [2, 3, 8, 16, 17, 64])
def test_reduce_kway(target, order, k):
    import torch
    if order == "halving" and k & (k - 1):
        pytest.skip("halving order needs a power of two")
    n, first = 3001, (k // 3) % k
    shards = make_inputs(k, n, O.F16, seed=11)
    ts = [to_torch(x, O.F16, target.device) for x in shards]
    out = torch.zeros_like(ts[0])
    lib = target.native
    saved = {key: lib.get_tuning(key) for key in ("wg_kway", "nt_load", "nt_store")}
    try:
        for wg in (256, 64):               # 64: the one-wave workgroups that streams from HBM get
            lib.set_tuning("wg_kway", wg); lib.set_tuning("nt_load", 1); lib.set_tuning("nt_store", 1)
            out.zero_()
            lib.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, F16, 0 if order == "ring" else 1, first,
                            True, target.stream())
            target.sync()
            if order == "ring":
                want = shards[first]
                for t in range(1, k):
                    want = O.vector_add(want, shards[(first + t) % k], O.F16)
            else:
                v = [shards[first ^ m] for m in range(k)]
                h = k // 2
                while h >= 1:
                    for m in range(h):
                        v[m] = O.vector_add(v[m], v[m + h], O.F16)
                    h //= 2
                want = v[0]
            assert_bits_equal(to_numpy(out, O.F16), want, f"{order} k={k} wg={wg}")
    finally:
        for key, v in saved.items():
            lib.set_tuning(key, v)


def test_reduce_kway_single_rounding(target):
    """per_hop_round = 0: fp32 partial sums, one rounding at the end."""
    import torch
    k, n = 8, 4099
    shards = make_inputs(k, n, O.F16, seed=13)
    ts = [to_torch(x, O.F16, target.device) for x in shards]
    out = torch.zeros_like(ts[0])
    target.native.reduce_kway(out.data_ptr(), [t.data_ptr() for t in ts], n, F16, 0, 0, False, target.stream())
    target.sync()
    acc = O.f16_to_f32(shards[0])
    for t in range(1, k):
        acc = (acc + O.f16_to_f32(shards[t])).astype(np.float32)
    assert_bits_equal(to_numpy(out, O.F16), O.f32_to_f16(acc), "single rounding")


@pytest.mark.parametrize("alg,P", [("ring", 4), ("ring", 7), ("recursive", 8)])
@pytest.mark.parametrize("mode", ["steps", "fused", "faithful"])
@pytest.mark.parametrize("B", [1030, 1024])          # ragged blocks (general kernels) and whole vectors (lean kernels)
def test_reduce_scatter(target, alg, P, mode, B):
    import torch
    from pccl import kernels
    ins = make_inputs(P, P * B, O.F16, seed=17)
    t_in = [to_torch(x, O.F16, target.device) for x in ins]
    t_out = [torch.zeros(B, dtype=torch.float16, device=target.device) for _ in range(P)]
    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode)
    target.sync()
    want = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, O.F16)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r], O.F16), want[r], f"{alg}/{mode} rank {r}")


@pytest.mark.parametrize("alg", ["ring", "recursive"])
@pytest.mark.parametrize("mode", ["steps", "fused"])
def test_grid_and_per_rank_api(target, alg, mode):
    """reduce_scatter_2D on a 4 x 2 grid in one call, and the reference-shaped
    per-rank calls with use_pccl_cpp_backend on and off (the Python twin adds
    float16 through the same accumulate kernel)."""
    import torch
    import pccl
    from pccl import kernels
    intra, inter, m = 4, 2, 515
    W = intra * inter
    ins = make_inputs(W, W * m, O.F16, seed=23)
    t_in = [to_torch(x, O.F16, target.device) for x in ins]
    t_out = [torch.zeros(m, dtype=torch.float16, device=target.device) for _ in range(W)]
    kernels.reduce_scatter_2d_ranks(t_out, t_in, intra, inter, alg, mode)
    target.sync()
    want = O.reduce_scatter_2d(ins, intra, inter, O.F16, alg)
    for w in range(W):
        assert_bits_equal(to_numpy(t_out[w], O.F16), want[w], f"grid rank {w}")
    flat = (O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter)(ins, O.F16)
    for cpp in (True, False):
        outs = [torch.zeros(m, dtype=torch.float16, device=target.device) for _ in range(W)]
        world = pccl.VirtualWorld(W, target.device)
        world.run(lambda comm: pccl._reduce_scatter(outs[comm.Get_rank()], t_in[comm.Get_rank()], group=comm,
                                                    use_rh=alg == "recursive", use_pccl_cpp_backend=cpp))
        target.sync()
        for w in range(W):
            assert_bits_equal(to_numpy(outs[w], O.F16), flat[w], f"per-rank cpp={cpp} rank {w}")
