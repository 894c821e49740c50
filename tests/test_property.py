"""Randomised shapes on the CPU build: any P, block length, dtype, algorithm,
mode and operand misalignment must give the oracle's bits."""
import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings, strategies as st

from helpers import assert_bits_equal, make_inputs, to_numpy, to_torch
from oracle import pccl_oracle as O

SETTINGS = dict(max_examples=60, deadline=None,
                suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])


@settings(**SETTINGS)
@given(P=st.integers(1, 12), B=st.integers(1, 3000), bf16=st.booleans(), rec=st.booleans(),
       mode=st.sampled_from(["steps", "fused", "faithful"]), shift=st.integers(0, 7), seed=st.integers(0, 2 ** 16))
def test_reduce_scatter_random_shapes(cpu, P, B, bf16, rec, mode, shift, seed):
    import torch
    from pccl import kernels
    if rec:
        P = 1 << (P % 4)                                   # 1, 2, 4, 8
    dtype = O.BF16 if bf16 else O.F32
    td = torch.bfloat16 if bf16 else torch.float32
    ins = make_inputs(P, P * B, dtype, seed=seed)
    # every rank's buffers start `shift` elements into a larger allocation
    big_in = [torch.zeros(P * B + 8, dtype=td) for _ in range(P)]
    big_out = [torch.zeros(B + 8, dtype=td) for _ in range(P)]
    t_in, t_out = [], []
    for r in range(P):
        v = big_in[r][shift:shift + P * B]
        v.copy_(to_torch(ins[r], dtype, "cpu"))
        t_in.append(v)
        t_out.append(big_out[r][(shift * 3) % 8:(shift * 3) % 8 + B])
    kernels.reduce_scatter_ranks(t_out, t_in, "recursive" if rec else "ring", mode)
    want = (O.recursive_halving_reduce_scatter if rec else O.ring_reduce_scatter)(ins, dtype)
    for r in range(P):
        assert_bits_equal(to_numpy(t_out[r].clone(), dtype), want[r], f"rank {r}")
        lo = (shift * 3) % 8
        assert not big_out[r][:lo].float().abs().sum() and not big_out[r][lo + B:].float().abs().sum()


@settings(**SETTINGS)
@given(P=st.integers(1, 12), blk=st.integers(1, 5000), rec=st.booleans(), mode=st.sampled_from(["steps", "fused"]),
       shift=st.integers(0, 15), seed=st.integers(0, 2 ** 16))
def test_all_gather_random_shapes(cpu, P, blk, rec, mode, shift, seed):
    import torch
    from pccl import kernels
    if rec:
        P = 1 << (P % 4)
    rng = np.random.default_rng(seed)
    ins = [rng.integers(0, 256, blk, dtype=np.uint8) for _ in range(P)]
    big = [torch.from_numpy(np.concatenate([np.zeros(shift, np.uint8), x])) for x in ins]
    t_in = [b[shift:] for b in big]
    outs_big = [torch.full((P * blk + 16,), 0xA5, dtype=torch.uint8) for _ in range(P)]
    t_out = [o[(shift * 5) % 16:(shift * 5) % 16 + P * blk] for o in outs_big]
    kernels.all_gather_ranks(t_out, t_in, "recursive" if rec else "ring", mode)
    cat = np.concatenate(ins)
    for r in range(P):
        lo = (shift * 5) % 16
        got = outs_big[r].numpy()
        assert np.array_equal(got[lo:lo + P * blk], cat)
        assert (got[:lo] == 0xA5).all() and (got[lo + P * blk:] == 0xA5).all()


@settings(**SETTINGS)
@given(intra=st.integers(1, 5), inter=st.integers(1, 5), m=st.integers(1, 700), bf16=st.booleans(), rec=st.booleans(),
       mode=st.sampled_from(["steps", "fused"]), seed=st.integers(0, 2 ** 16))
def test_2d_random_shapes(cpu, intra, inter, m, bf16, rec, mode, seed):
    import torch
    from pccl import kernels
    if rec:
        intra, inter = 1 << (intra % 3), 1 << (inter % 3)
    dtype = O.BF16 if bf16 else O.F32
    td = torch.bfloat16 if bf16 else torch.float32
    W = intra * inter
    alg = "recursive" if rec else "ring"
    ins = make_inputs(W, W * m, dtype, seed=seed)
    t_in = [to_torch(x, dtype, "cpu") for x in ins]
    t_out = [torch.zeros(m, dtype=td) for _ in range(W)]
    kernels.reduce_scatter_2d_ranks(t_out, t_in, intra, inter, alg, mode)
    want = O.reduce_scatter_2d(ins, intra, inter, dtype, alg)
    for w in range(W):
        assert_bits_equal(to_numpy(t_out[w], dtype), want[w], f"rank {w}")
    g_out = [torch.zeros(W * m, dtype=td) for _ in range(W)]
    kernels.all_gather_2d_ranks(g_out, t_out, intra, inter, alg, mode)
    for w in range(W):
        assert_bits_equal(to_numpy(g_out[w], dtype), np.concatenate(want), f"gather rank {w}")
