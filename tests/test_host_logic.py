"""Host-side logic: virtual communicators, rendezvous, process-group grid,
argument checks of the extension entry points, dispatch precedence.  CPU only;
where data has to move it goes through the CPU build of the library."""
import threading

import pytest

from oracle import pccl_oracle as O


# ---- ProcessGroups grid --------------------------------------------------------

@pytest.mark.parametrize("intra,inter,grids", [(2, 2, 1), (4, 2, 1), (2, 4, 1), (2, 2, 2), (8, 1, 1), (1, 8, 1)])
def test_process_groups_membership_matches_mpi_colours(intra, inter, grids):
    """Virtual ProcessGroups reproduce the groups the reference gets from
    Split(rank // intra) and Split(rank % intra + (rank // (intra*inter)) * intra)."""
    import pccl
    world_size = intra * inter * grids
    world = pccl.VirtualWorld(world_size, "cpu")
    inner, outer = O.grid_groups(world_size, intra, inter)
    for r in range(world_size):
        pg = pccl.ProcessGroups(intra, inter, inner_group_backend="mpi", outer_group_backend="mpi", comm=world.comm(r))
        assert list(pg.get_inner_group().world_ranks) == inner[r]
        assert list(pg.get_outer_group().world_ranks) == outer[r]
        assert pg.get_world_size() == [intra, inter]
        assert pg.get_rank() == [inner[r].index(r), outer[r].index(r)]
        assert pg.get_rank(0) == inner[r].index(r) and pg.get_world_size(1) == inter
        with pytest.raises(ValueError):
            pg.get_rank(2)
        assert "VIRTUAL" in repr(pg)


def test_process_groups_argument_errors():
    import pccl
    world = pccl.VirtualWorld(6, "cpu")
    with pytest.raises(ValueError, match="must be divisible"):
        pccl.ProcessGroups(4, 1, comm=world.comm(0))
    with pytest.raises(ValueError, match="Unsupported inner_group_backend"):
        pccl.ProcessGroups(2, 3, inner_group_backend="gloo", comm=world.comm(0))
    with pytest.raises(ValueError, match="Unsupported outer_group_backend"):
        pccl.ProcessGroups(2, 3, outer_group_backend="ucx", comm=world.comm(0))
    with pytest.raises(AssertionError, match="pytorch distributed should be initialized"):
        pccl.ProcessGroups(2, 3)


def test_split_follows_mpi_semantics():
    import pccl
    world = pccl.VirtualWorld(6, "cpu")

    def main(comm):
        r = comm.Get_rank()
        sub = comm.Split(r % 2, key=-r)          # two colours, reversed order inside each
        return sub.world_ranks, sub.Get_rank(), sub.Get_size()

    res = world.run(main)
    assert res[0] == ((4, 2, 0), 2, 3)
    assert res[5] == ((5, 3, 1), 0, 3)
    assert res[2] == ((4, 2, 0), 1, 3)


# ---- rendezvous and error propagation --------------------------------------------

def test_collective_outside_spmd_is_refused(cpu):
    import torch
    import pccl
    world = pccl.VirtualWorld(2, "cpu")
    with pytest.raises(pccl.VirtualRankError, match="collective over 2 virtual ranks"):
        pccl.reduce_scatter_mpi(torch.zeros(4), torch.zeros(8), world.comm(0), "ring")
    with pytest.raises(pccl.VirtualRankError, match="needs VirtualWorld.run"):
        world.comm(0).Sendrecv(torch.zeros(4), 1, 0, torch.zeros(4), 1, 0)


def test_one_failing_rank_releases_the_others(cpu):
    import torch
    import pccl
    world = pccl.VirtualWorld(4, "cpu")

    def main(comm):
        if comm.Get_rank() == 2:
            raise KeyError("rank 2 broke")
        pccl.reduce_scatter_mpi(torch.zeros(4), torch.zeros(16), comm, "ring")

    with pytest.raises(KeyError, match="rank 2 broke"):
        world.run(main)
    # the world is usable again afterwards
    outs = [torch.zeros(4) for _ in range(4)]
    ins = [torch.arange(16, dtype=torch.float32) for _ in range(4)]
    world.run(lambda c: pccl.reduce_scatter_mpi(outs[c.Get_rank()], ins[c.Get_rank()], c, "ring"))
    for r in range(4):
        assert torch.equal(outs[r], 4 * torch.arange(16, dtype=torch.float32)[4 * r:4 * r + 4])


def test_mismatched_collectives_are_reported(cpu):
    import torch
    import pccl
    world = pccl.VirtualWorld(2, "cpu")

    def main(comm):
        alg = "ring" if comm.Get_rank() == 0 else "recursive"
        pccl.reduce_scatter_mpi(torch.zeros(4), torch.zeros(8), comm, alg)

    with pytest.raises(pccl.VirtualRankError):
        world.run(main)


def test_sendrecv_ring_moves_data(cpu):
    import torch
    import pccl
    P = 5
    world = pccl.VirtualWorld(P, "cpu")

    def main(comm):
        r = comm.Get_rank()
        send = torch.full((7,), float(r))
        recv = torch.zeros(7)
        for tag in range(3):                      # repeated exchanges reuse the mailboxes
            comm.Sendrecv(send, (r + 1) % P, tag, recv, (r - 1) % P, tag)
            send = recv.clone()
        return recv

    res = world.run(main)
    for r in range(P):
        assert torch.equal(res[r], torch.full((7,), float((r - 3) % P)))


# ---- the extension entry points keep the reference's checks ------------------------

def test_reduce_scatter_mpi_checks(cpu):
    """Order and wording of pccl/src/pccl.cpp:16-45,83."""
    import torch
    import pccl
    comm = pccl.VirtualWorld(1, "cpu").comm(0)
    c4 = pccl.VirtualWorld(4, "cpu").comm(0)
    f = torch.zeros
    with pytest.raises(RuntimeError, match="output tensor must be contiguous"):
        pccl.reduce_scatter_mpi(f(8)[::2], f(4), comm)
    with pytest.raises(RuntimeError, match="input tensor must be contiguous"):
        pccl.reduce_scatter_mpi(f(4), f(8)[::2], comm)
    with pytest.raises(RuntimeError, match="output tensor must be 1D"):
        pccl.reduce_scatter_mpi(f(2, 2), f(4), comm)
    with pytest.raises(RuntimeError, match="input tensor must be 1D"):
        pccl.reduce_scatter_mpi(f(4), f(2, 2), comm)
    with pytest.raises(RuntimeError, match="Input tensor size must be divisible by number of processes"):
        pccl.reduce_scatter_mpi(f(2), f(10), c4)
    with pytest.raises(RuntimeError, match="Output tensor must have block_size elements"):
        pccl.reduce_scatter_mpi(f(3), f(8), c4)
    with pytest.raises(RuntimeError, match="Input tensor must be of type float"):
        pccl.reduce_scatter_mpi(f(2, dtype=torch.int32), f(8, dtype=torch.int32), c4)
    with pytest.raises(RuntimeError, match="Output tensor must be of type float"):
        pccl.reduce_scatter_mpi(f(2, dtype=torch.float64), f(8), c4)
    with pytest.raises(RuntimeError, match="Unknown algorithm specified for reduce_scatter_mpi: tree"):
        pccl.reduce_scatter_mpi(f(2), f(8), c4, "tree")
    with pytest.raises(TypeError):
        pccl.reduce_scatter_mpi(f(2), f(8), object())


def test_all_gather_mpi_checks(cpu):
    """pccl/src/pccl.cpp:92-116,140."""
    import torch
    import pccl
    c4 = pccl.VirtualWorld(4, "cpu").comm(0)
    f = torch.zeros
    with pytest.raises(RuntimeError, match="output tensor must be contiguous"):
        pccl.all_gather_mpi(f(16)[::2], f(2), c4)
    with pytest.raises(RuntimeError, match="input tensor must be 1D"):
        pccl.all_gather_mpi(f(8), f(2, 1), c4)
    with pytest.raises(RuntimeError, match="Input and output tensors must have the same dtype"):
        pccl.all_gather_mpi(f(8), f(2, dtype=torch.bfloat16), c4)
    with pytest.raises(RuntimeError, match="Output tensor must have total_elem elements"):
        pccl.all_gather_mpi(f(9), f(2), c4)
    with pytest.raises(RuntimeError, match="Unknown algorithm specified for all_gather_mpi: tree"):
        pccl.all_gather_mpi(f(8), f(2), c4, "tree")


def test_dispatch_rejects_unknown_group_types(cpu):
    import torch
    import pccl
    with pytest.raises(TypeError, match="Unsupported group type"):
        pccl._reduce_scatter(torch.zeros(2), torch.zeros(4), group="mpi")
    with pytest.raises(TypeError, match="Unsupported group type"):
        pccl._all_gather(torch.zeros(4), torch.zeros(2), group=42)


def test_async_is_refused_where_the_reference_refuses_it(cpu):
    import torch
    import pccl
    comm = pccl.VirtualWorld(1, "cpu").comm(0)
    with pytest.raises(AssertionError, match="Non-blocking operations not supported"):
        pccl.recursive_halving_reduce_scatter_mpi(torch.zeros(4), torch.zeros(4), comm, async_op=True)
    with pytest.raises(AssertionError, match="non-blocking primitives not supported"):
        pccl.ring_reduce_scatter_mpi(torch.zeros(4), torch.zeros(4), comm, async_op=True)
    with pytest.raises(AssertionError, match="non-blocking primitives not supported"):
        pccl.recursive_doubling_allgather_mpi(torch.zeros(4), torch.zeros(4), comm, async_op=True)
    with pytest.raises(AssertionError, match="Non blocking version not implemented"):
        pccl.reduce_scatter_2D(torch.zeros(4), torch.zeros(4), group=None, async_op=True)
    with pytest.raises(AssertionError, match="Non blocking version not implemented"):
        pccl.all_gather_2D(torch.zeros(4), torch.zeros(4), group=None, async_op=True)


def test_native_backend_wins_over_directly_call_mpi(cpu, monkeypatch):
    """pccl/reduce_scatter.py:184 is tested before :191."""
    import torch
    import pccl
    from pccl import ext
    seen = []
    monkeypatch.setattr(ext, "reduce_scatter_mpi", lambda o, i, g, alg: seen.append(alg))
    comm = pccl.VirtualWorld(1, "cpu").comm(0)
    pccl._reduce_scatter(torch.zeros(4), torch.zeros(4), group=comm, directly_call_mpi=True,
                         use_rh=True, use_pccl_cpp_backend=True)
    pccl._reduce_scatter(torch.zeros(4), torch.zeros(4), group=comm, directly_call_mpi=True,
                         use_rh=False, use_pccl_cpp_backend=True)
    assert seen == ["recursive", "ring"]


def test_python_algorithm_accepts_another_op(cpu):
    """op= is honoured (pccl/reduce_scatter.py:24): max instead of add."""
    import torch
    import pccl
    P, B = 4, 6
    world = pccl.VirtualWorld(P, "cpu")
    g = torch.Generator().manual_seed(0)
    ins = [torch.randn(P * B, generator=g) for _ in range(P)]
    outs = [torch.zeros(B) for _ in range(P)]
    world.run(lambda c: pccl.recursive_halving_reduce_scatter_mpi(outs[c.Get_rank()], ins[c.Get_rank()], c,
                                                                 op=torch.maximum))
    want = torch.stack(ins).max(dim=0).values
    for r in range(P):
        assert torch.equal(outs[r], want[r * B:(r + 1) * B])


def test_build_kernels_build_loads_the_library():
    from pccl import build_kernels, _native
    lib = build_kernels.build()
    assert lib.version() == _native.ABI_VERSION and build_kernels.BUILT


def test_threads_share_nothing_but_the_rendezvous(cpu):
    """Two independent worlds can run at the same time."""
    import torch
    import pccl
    res = {}

    def drive(tag, P):
        world = pccl.VirtualWorld(P, "cpu")
        outs = [torch.zeros(3) for _ in range(P)]
        ins = [torch.full((3 * P,), float(r + 1)) for r in range(P)]
        world.run(lambda c: pccl._reduce_scatter(outs[c.Get_rank()], ins[c.Get_rank()], group=c,
                                                 use_pccl_cpp_backend=True))
        res[tag] = outs

    ts = [threading.Thread(target=drive, args=(i, 2 + i)) for i in range(3)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    for i in range(3):
        P = 2 + i
        for o in res[i]:
            assert torch.equal(o, torch.full((3,), float(P * (P + 1) // 2)))


def test_rank_slab_layout():
    """Buffers of the virtual ranks carved from one allocation: equal strides of
    the longest buffer (rounded to 256 bytes) plus the skew, no overlap."""
    import torch
    from pccl import kernels
    bufs = kernels.rank_slab(4, [100, 7, 0, 100], torch.bfloat16, "cpu", skew_bytes=512)
    assert [b.numel() for b in bufs] == [100, 7, 0, 100] and all(b.dtype == torch.bfloat16 for b in bufs)
    stride = 256 + 512
    assert bufs[1].data_ptr() - bufs[0].data_ptr() == stride
    assert bufs[3].data_ptr() - bufs[0].data_ptr() == 3 * stride
    for r, b in enumerate(bufs):
        b.fill_(float(r))
    assert all(bool((b == float(r)).all()) for r, b in enumerate(bufs))
    same = kernels.rank_slab(3, 64, torch.float32, "cpu", skew_bytes=0)
    assert same[1].data_ptr() - same[0].data_ptr() == 256
    with pytest.raises(ValueError):
        kernels.rank_slab(2, 8, torch.float32, "cpu", skew_bytes=100)
    with pytest.raises(ValueError):
        kernels.rank_slab(2, [8], torch.float32, "cpu")
