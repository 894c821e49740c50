"""pccl_hip_reduce_scatter_virtual_noalloc: the per-step reduce_scatter whose
work buffers are the library's built-in scratch array.  Called through the C ABI
and compared bit for bit with pccl_hip_reduce_scatter_virtual (per-step mode,
caller-owned work buffers) and with the oracle, on two calls in a row, the
second with a smaller input (the scratch keeps the first call's contents)."""
import pytest

from helpers import assert_bits_equal, make_inputs, to_numpy, to_torch
from oracle import pccl_oracle as O


def _run_both(target, P, B, dtype, algorithm, seed):
    import torch
    from pccl import _native
    lib = target.native
    xs = make_inputs(P, P * B, dtype, seed=seed)
    tdt = torch.float32 if dtype == O.F32 else torch.bfloat16
    code = _native.F32 if dtype == O.F32 else _native.BF16
    ins = [to_torch(x, dtype, target.device) for x in xs]
    want_outs = [torch.zeros(B, dtype=tdt, device=target.device) for _ in range(P)]
    got_outs = [torch.zeros(B, dtype=tdt, device=target.device) for _ in range(P)]
    work = [torch.empty(P * B, dtype=tdt, device=target.device) for _ in range(P)] if P > 2 else None
    st = target.stream()
    lib.reduce_scatter_virtual([t.data_ptr() for t in want_outs], [t.data_ptr() for t in ins],
                               None if work is None else [t.data_ptr() for t in work], B, code, algorithm,
                               _native.MODE_STEPS, st)
    lib.reduce_scatter_virtual_noalloc([t.data_ptr() for t in got_outs], [t.data_ptr() for t in ins], B, code,
                                       algorithm, st)
    target.sync()
    ref = (O.ring_reduce_scatter if algorithm == "ring" else O.recursive_halving_reduce_scatter)(xs, dtype)
    for r in range(P):
        what = f"{algorithm} P={P} B={B} {dtype} rank {r}"
        assert_bits_equal(to_numpy(got_outs[r], dtype), to_numpy(want_outs[r], dtype), what + " (vs caller-owned work)")
        assert_bits_equal(to_numpy(got_outs[r], dtype), ref[r], what + " (vs oracle)")


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
@pytest.mark.parametrize("algorithm", ["ring", "recursive"])
def test_noalloc_matches_caller_owned_work_twice(target, algorithm, dtype):
    print(f"noalloc {algorithm} {dtype} on {target.name}", flush=True)
    # first call: 8 ranks, ragged block; second call, right after: smaller input
    _run_both(target, 8, 4099, dtype, algorithm, seed=11)
    _run_both(target, 4, 515, dtype, algorithm, seed=12)


def test_noalloc_largest_shape_that_fits(target):
    """8 ranks x 8 blocks of 128 Ki fp32: 8 slices of 4 MiB = the whole 32 MiB array."""
    from pccl import _native
    assert 8 * 8 * (128 << 10) * 4 == _native.NOALLOC_SCRATCH_BYTES
    B = (128 << 10) if target.device != "cpu" else 64     # the CPU build runs thread by thread: keep it short
    _run_both(target, 8, B, O.F32, "ring", seed=13)


def test_noalloc_small_rank_counts(target):
    for P in (1, 2, 3):
        _run_both(target, P, 130, O.BF16, "ring", seed=20 + P)


def test_noalloc_refuses_what_does_not_fit():
    """Validation happens on the host before any device call, so this runs without a GPU."""
    from pccl import _native
    lib = _native.load()
    E = _native.NativeError
    with pytest.raises(E, match="built-in scratch"):
        lib.reduce_scatter_virtual_noalloc([64] * 8, [64] * 8, (128 << 10) + 64, _native.F32, "ring")
    with pytest.raises(E, match="built-in scratch"):
        lib.reduce_scatter_virtual_noalloc([64] * 4, [64] * 4, 1 << 40, _native.BF16, "ring")
    with pytest.raises(E, match=r"P = 65 outside"):
        lib.reduce_scatter_virtual_noalloc([64] * 65, [64] * 65, 8, _native.F32, "ring")
    with pytest.raises(E, match="Unknown algorithm specified for reduce_scatter_mpi: tree"):
        lib.reduce_scatter_virtual_noalloc([64] * 4, [64] * 4, 8, _native.F32, "tree")
    with pytest.raises(E, match="power-of-two"):
        lib.reduce_scatter_virtual_noalloc([64] * 6, [64] * 6, 8, _native.F32, "recursive")
    # nothing to do: accepted without touching the device
    lib.reduce_scatter_virtual_noalloc([64] * 4, [64] * 4, 0, _native.F32, "ring")


@pytest.mark.gpu
@pytest.mark.parametrize("algorithm", ["ring", "recursive"])
def test_noalloc_replays_from_a_graph(algorithm):
    """What the entry point is for: captured into a HIP graph (the set-up call
    was made outside the capture), it replays with eager work between the
    replays and gives the oracle's bits on fresh inputs every time."""
    import torch
    from pccl import _native, kernels
    lib = _native.load()
    dev = "cuda:0"
    P, B, dtype = 8, 4096 + 24, O.BF16
    t_in = [to_torch(x, dtype, dev) for x in make_inputs(P, P * B, dtype, seed=11)]
    t_out = [torch.zeros(B, dtype=torch.bfloat16, device=dev) for _ in range(P)]
    outs, ins = [t.data_ptr() for t in t_out], [t.data_ptr() for t in t_in]
    lib.reduce_scatter_virtual_noalloc(outs, ins, B, _native.BF16, algorithm, kernels.stream_handle())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lib.reduce_scatter_virtual_noalloc(outs, ins, B, _native.BF16, algorithm, kernels.stream_handle())
    ref = O.ring_reduce_scatter if algorithm == "ring" else O.recursive_halving_reduce_scatter
    for rep in range(3):
        fresh = make_inputs(P, P * B, dtype, seed=100 + rep)
        for t, x in zip(t_in, fresh):
            t.copy_(to_torch(x, dtype, dev))
        for o in t_out:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = ref(fresh, dtype)
        for r in range(P):
            assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"replay {rep} rank {r}")
