"""Stream handling: work goes to the caller's current stream, and a whole
collective (launches only, no allocation, no memset) can be captured in a HIP
graph and replayed."""
import pytest

from helpers import assert_bits_equal, make_inputs, to_numpy, to_torch
from oracle import pccl_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_work_follows_the_current_stream():
    import torch
    from pccl import kernels
    side = torch.cuda.Stream()
    n = 1 << 22
    a, b = make_inputs(2, n, O.BF16, seed=3)
    ta, tb = to_torch(a, O.BF16, DEV), to_torch(b, O.BF16, DEV)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        assert kernels.stream_handle() == side.cuda_stream
        kernels.accumulate(ta, tb)
        done = torch.cuda.Event()
        done.record(side)
    done.synchronize()
    assert_bits_equal(to_numpy(ta, O.BF16), O.vector_add(a, b, O.BF16))


@pytest.mark.parametrize("alg,mode", [("ring", "steps"), ("recursive", "steps"), ("ring", "fused")])
def test_collective_replays_from_a_graph(alg, mode):
    """Capture once, replay several times with eager work and synchronisation in
    between; every replay must reproduce the eager result on fresh inputs."""
    import torch
    from pccl import kernels
    P, B, dtype = 8, 4096 + 24, O.BF16
    ins = make_inputs(P, P * B, dtype, seed=11)
    t_in = [to_torch(x, dtype, DEV) for x in ins]
    t_out = [torch.zeros(B, dtype=torch.bfloat16, device=DEV) for _ in range(P)]
    work = [torch.empty_like(t) for t in t_in]
    # warm up outside the capture
    kernels.reduce_scatter_ranks(t_out, t_in, alg, mode, work)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kernels.reduce_scatter_ranks(t_out, t_in, alg, mode, work)
    ref = O.ring_reduce_scatter if alg == "ring" else O.recursive_halving_reduce_scatter
    for rep in range(4):
        fresh = make_inputs(P, P * B, dtype, seed=100 + rep)
        for t, x in zip(t_in, fresh):
            t.copy_(to_torch(x, dtype, DEV))          # eager work between replays
        for o in t_out:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = ref(fresh, dtype)
        for r in range(P):
            assert_bits_equal(to_numpy(t_out[r], dtype), want[r], f"replay {rep} rank {r}")


def test_all_gather_replays_from_a_graph():
    import torch
    from pccl import kernels
    P, n = 8, 5000
    t_in = [torch.randn(n, device=DEV) for _ in range(P)]
    t_out = [torch.zeros(P * n, device=DEV) for _ in range(P)]
    kernels.all_gather_ranks(t_out, t_in, "recursive", "steps")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kernels.all_gather_ranks(t_out, t_in, "recursive", "steps")
    for rep in range(3):
        for t in t_in:
            t.normal_()
        for o in t_out:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        cat = torch.cat(t_in)
        for r in range(P):
            assert torch.equal(t_out[r], cat), (rep, r)
