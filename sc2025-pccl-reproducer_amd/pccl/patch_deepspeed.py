"""Route DeepSpeed's collectives through PCCL (pccl/patch_deepspeed.py:95-126).

`patch_deepspeed(intra_node_pg_size, comm=...)` swaps five methods of
`deepspeed.comm.torch.TorchBackend`, exactly the ones the reference swaps:
world-group SUM collectives go to the hierarchical PCCL path (recursive
halving / doubling, native backend), everything else falls through to the
saved originals.  With virtual ranks every rank is a thread of one process, so
the process groups are kept per thread; the class is patched once.

DeepSpeed is imported when the function is called; without it the call raises.
"""
from __future__ import annotations

import threading
from typing import Optional

import torch
import torch.distributed as dist

from .all_gather import all_gather_2D
from .all_reduce import _all_reduce
from .build_kernels import build
from .process_groups import ProcessGroups
from .reduce_scatter import reduce_scatter_2D
from .virtual import VirtualComm

_tls = threading.local()
_patch_lock = threading.Lock()


def get_heir_pg() -> ProcessGroups:
    pg = getattr(_tls, "pg", None)
    assert pg is not None, "did you call the patch_deepspeed function?"
    return pg


class dummy_request:
    """What the patched methods return for async_op=True: the work is already
    enqueued in stream order (pccl/patch_deepspeed.py:18-23)."""

    def wait(self):
        pass


def _world() -> Optional[VirtualComm]:
    return getattr(_tls, "world", None)


def is_global_pg(group) -> bool:
    """True for the group spanning all ranks (pccl/patch_deepspeed.py:26-27)."""
    world = _world()
    if world is not None:       # virtual ranks: None or the world communicator itself
        return group is None or group is world or (
            isinstance(group, VirtualComm) and group.world_ranks == world.world_ranks)
    return (group is None) or (group == dist.group.WORLD) or (dist.get_world_size(group) == dist.get_world_size())


def _is_sum(op) -> bool:
    return op == dist.ReduceOp.SUM or getattr(op, "name", None) == "SUM"


def patched_all_gather(self, output_tensor, input_tensor, group=None, async_op=False):
    if is_global_pg(group):
        all_gather_2D(output_tensor, input_tensor, group=get_heir_pg(), async_op=False, use_rd=True,
                      use_pccl_cpp_backend=True)
        if async_op:
            return dummy_request()
    else:
        return self.old_all_gather_into_tensor(output_tensor, input_tensor, group, async_op)


def patched_reduce_scatter(self, output_tensor, input_tensor, op=dist.ReduceOp.SUM, group=None, async_op=False):
    if is_global_pg(group) and _is_sum(op):
        reduce_scatter_2D(output_tensor, input_tensor, group=get_heir_pg(), async_op=False, use_rh=True,
                          use_pccl_cpp_backend=True)
        if async_op:
            return dummy_request()
    else:
        return self.old_reduce_scatter_tensor(output_tensor, input_tensor, op, group, async_op)


def patched_all_reduce(self, tensor, op=dist.ReduceOp.SUM, group=None, async_op=False):
    world = _world()
    if world is not None and is_global_pg(group) and _is_sum(op):
        # the reference hands this to MPI_Allreduce (pccl/patch_deepspeed.py:61-70), whose
        # summation order is the MPI library's; here: halving reduce_scatter + doubling all_gather
        _all_reduce(tensor, group=world, use_rh_and_rd=True)
        if async_op:
            return dummy_request()
    else:
        return self.old_all_reduce(tensor, op, group, async_op)


def patched_broadcast(self, tensor, src, group=None, async_op=False):
    world = _world()
    if world is not None and is_global_pg(group):
        world.Bcast(tensor, root=src)
        if async_op:
            return dummy_request()
    else:
        return self.old_broadcast(tensor, src, group, async_op)


def patched_barrier(self, group=None, async_op=False, device_ids=None):
    world = _world()
    if world is not None and is_global_pg(group):
        if torch.cuda.is_available():
            torch.cuda.synchronize()
        world.Barrier()
        if async_op:
            return dummy_request()
    else:
        return self.old_barrier(group, async_op, device_ids)


def patch_deepspeed(intra_node_pg_size: int, comm: Optional[VirtualComm] = None):
    """Patch DeepSpeed's TorchBackend for the calling rank.

    comm: this rank's world communicator of virtual ranks; required.  The
    reference's own setting (no comm: torch.distributed initialised, one
    process per GPU, an mpi4py outer group, pccl/patch_deepspeed.py:95-110)
    needs real ranks on several GPUs, which this build does not drive: it is
    refused here, at patch time, rather than at the first collective."""
    if comm is None:
        raise RuntimeError("patch_deepspeed: this build runs on virtual ranks only; pass comm=<this rank's "
                           "pccl.VirtualComm> (VirtualWorld(P).run(...) hands one to every rank)")
    if not isinstance(comm, VirtualComm):
        raise TypeError(f"patch_deepspeed: comm must be a pccl.VirtualComm, got {type(comm)}")
    try:
        from deepspeed.comm.torch import TorchBackend
    except ImportError as e:
        raise RuntimeError("patch_deepspeed needs the deepspeed package") from e
    world_size = comm.Get_size()
    assert world_size % intra_node_pg_size == 0
    build()
    _tls.world = comm
    _tls.pg = ProcessGroups(intra_node_pg_size, world_size // intra_node_pg_size,
                            inner_group_backend="mpi", outer_group_backend="mpi", comm=comm)
    with _patch_lock:
        if getattr(TorchBackend, "_pccl_patched", False):
            return
        TorchBackend.old_all_gather_into_tensor = TorchBackend.all_gather_into_tensor
        TorchBackend.all_gather_into_tensor = patched_all_gather
        TorchBackend.old_reduce_scatter_tensor = TorchBackend.reduce_scatter_tensor
        TorchBackend.reduce_scatter_tensor = patched_reduce_scatter
        TorchBackend.old_all_reduce = TorchBackend.all_reduce
        TorchBackend.all_reduce = patched_all_reduce
        TorchBackend.old_broadcast = TorchBackend.broadcast
        TorchBackend.broadcast = patched_broadcast
        TorchBackend.old_barrier = TorchBackend.barrier
        TorchBackend.barrier = patched_barrier
        TorchBackend._pccl_patched = True
