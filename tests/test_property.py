"""Randomised shapes on the CPU build: any P, block length, dtype, algorithm,
mode and operand misalignment must give the oracle's bits."""
import numpy as np
from hypothesis import HealthCheck, assume, given, settings, strategies as st

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


@settings(**SETTINGS)
@given(P=st.integers(1, 9), nmax=st.integers(1, 40000), strip=st.sampled_from([-1, 1, 2, 5, 160]),
       unroll=st.sampled_from([0, 1, 2, 4, 8]), in_shift=st.integers(0, 15), out_shift=st.integers(0, 15),
       gap=st.integers(0, 33), seed=st.integers(0, 2 ** 16))
def test_time_blocked_gather_random_shapes(cpu, P, nmax, strip, unroll, in_shift, out_shift, gap, seed):
    """The time-blocked placement kernel on shards of random (also zero) lengths at
    random byte alignments of sources, outputs and offsets: every shard lands where
    it should and nothing else is touched."""
    import torch
    lib = cpu.native
    keys = ("gather_strip", "gather_strip_from", "unroll_gather")
    saved = {k: lib.get_tuning(k) for k in keys}
    rng = np.random.default_rng(seed)
    nbytes = [int(x) for x in rng.integers(0, nmax + 1, P)]
    shards = [rng.integers(0, 256, n, dtype=np.uint8) for n in nbytes]
    off, o = [], 0
    for n in nbytes:
        off.append(o)
        o += n + gap                                   # byte offsets of any alignment, `gap` untouched bytes between
    total = o
    assume(total > 0)                                  # a zero-length output tensor has no address to pass
    big_in = [torch.from_numpy(np.concatenate([np.zeros(in_shift, np.uint8), s])) for s in shards]
    t_in = [b[in_shift:] for b in big_in]
    big_out = [torch.full((total + 32,), 0xA5, dtype=torch.uint8) for _ in range(P)]
    t_out = [b[out_shift:out_shift + total] for b in big_out]
    try:
        lib.set_tuning("gather_strip", strip)
        lib.set_tuning("gather_strip_from", 0)
        lib.set_tuning("unroll_gather", unroll)
        lib.all_gather_uneven_virtual([t.data_ptr() for t in t_out], [t.data_ptr() if t.numel() else 0 for t in t_in],
                                      nbytes, off, 0)
    finally:
        for k, v in saved.items():
            lib.set_tuning(k, v)
    want = np.full(total + 32, 0xA5, np.uint8)
    for k in range(P):
        want[out_shift + off[k]:out_shift + off[k] + nbytes[k]] = shards[k]
    for r in range(P):
        assert np.array_equal(big_out[r].numpy(), want), f"rank {r}"


@settings(**SETTINGS)
@given(n=st.integers(1, 20000), bf16=st.booleans(), sd=st.integers(0, 7), sa=st.integers(0, 7), sb=st.integers(0, 7),
       k=st.integers(2, 9), seed=st.integers(0, 2 ** 16))
def test_differently_aligned_operands(cpu, n, bf16, sd, sa, sb, k, seed):
    """dst, a and b (and the shards of a fold) each at its own element alignment:
    aligned vector stores, sources read wherever they lie; the oracle's bits and
    nothing written outside dst."""
    import torch
    lib = cpu.native
    dtype = O.BF16 if bf16 else O.F32
    code = 1 if bf16 else 0
    td = torch.bfloat16 if bf16 else torch.float32
    xs = make_inputs(k, n, dtype, seed=seed)
    bufs = [torch.zeros(n + 8, dtype=td) for _ in range(k)]
    shifts = [(sa + 3 * q) % 8 for q in range(k)]
    shifts[1] = sb
    views = []
    for q in range(k):
        v = bufs[q][shifts[q]:shifts[q] + n]
        v.copy_(to_torch(xs[q], dtype, "cpu"))
        views.append(v)
    out_big = torch.zeros(n + 8, dtype=td)
    out = out_big[sd:sd + n]
    lib.add(out.data_ptr(), views[0].data_ptr(), views[1].data_ptr(), n, code, 0)
    assert_bits_equal(to_numpy(out.clone(), dtype), O.vector_add(xs[0], xs[1], dtype), "add")
    assert not out_big[:sd].float().abs().sum() and not out_big[sd + n:].float().abs().sum()
    out_big.zero_()
    lib.reduce_kway(out.data_ptr(), [v.data_ptr() for v in views], n, code, 0, 0, True, 0)
    want = xs[0]
    for q in range(1, k):
        want = O.vector_add(want, xs[q], dtype)
    assert_bits_equal(to_numpy(out.clone(), dtype), want, "fold")
    assert not out_big[:sd].float().abs().sum() and not out_big[sd + n:].float().abs().sum()
