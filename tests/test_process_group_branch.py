"""The torch.distributed branch of the dispatchers (group=None or a
ProcessGroup: pccl/all_gather.py:107-112, pccl/all_reduce.py:31-35 of the
reference) delegates to torch.distributed.  Two CPU processes over gloo on
127.0.0.1; the GPU path is not involved."""
import os
import socket
import sys


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _rank_main(rank, world, port, queue):
    import torch
    import torch.distributed as dist
    sys.path.insert(0, os.path.join(ROOT, "sc2025-pccl-reproducer_amd"))
    import pccl
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=world)
    try:
        shard = torch.arange(5, dtype=torch.float32) + 10 * rank
        out = torch.zeros(5 * world)
        pccl._all_gather(out, shard, group=None)                     # default group
        sub = dist.new_group(list(range(world)))
        out2 = torch.zeros(5 * world)
        pccl._all_gather(out2, shard, group=sub)                     # an explicit ProcessGroup
        t = torch.full((4,), float(rank + 1))
        pccl._all_reduce(t, group=None)
        queue.put((rank, out.tolist(), out2.tolist(), t.tolist()))
    finally:
        dist.destroy_process_group()


def test_dispatchers_delegate_to_torch_distributed():
    import torch.multiprocessing as mp
    world, port = 2, _free_port()
    ctx = mp.get_context("spawn")
    queue = ctx.Queue()
    procs = [ctx.Process(target=_rank_main, args=(r, world, port, queue)) for r in range(world)]
    for p in procs:
        p.start()
    results = [queue.get(timeout=120) for _ in range(world)]
    for p in procs:
        p.join(timeout=60)
        assert p.exitcode == 0
    want = [float(x) for r in range(world) for x in range(10 * r, 10 * r + 5)]
    for rank, out, out2, t in results:
        assert out == want and out2 == want, rank
        assert t == [3.0] * 4, rank
