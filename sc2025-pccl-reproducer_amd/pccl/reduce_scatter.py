"""reduce_scatter on process groups or virtual ranks (pccl/reduce_scatter.py).

Public names and keyword arguments are the reference's.  `group` may be a
torch.distributed ProcessGroup (delegated to torch.distributed, RCCL on ROCm)
or a `VirtualComm`.  On virtual ranks:

  use_pccl_cpp_backend=True   the native path: the ranks meet and ONE batched
                              HIP launch per step serves all of them
                              (pccl.ext.reduce_scatter_mpi);
  use_pccl_cpp_backend=False  the reference's Python algorithms, rank by rank:
                              every Sendrecv is a device copy and every
                              `op(buf, recv)` one launch of the accumulate kernel.

Both give the same bits: the summation order is fixed by the algorithm.
"""
from __future__ import annotations

import math
from typing import Optional, Union

import torch
import torch.distributed as dist

from . import ext, kernels
from .process_groups import ProcessGroups
from .request import Request
from .virtual import VirtualComm


def _reduce_into(dst: torch.Tensor, recv: torch.Tensor, op):
    """dst = op(dst, recv).  torch.add maps onto the accumulate kernel
    (pccl/src/common.cu:5-19); any other callable is applied as given."""
    if op is torch.add and dst.dtype in (torch.float32, torch.bfloat16, torch.float16):
        kernels.accumulate(dst, recv)
    else:
        dst.copy_(op(dst, recv))


def _clone(t: torch.Tensor) -> torch.Tensor:
    out = torch.empty_like(t)
    kernels.copy(out, t)
    return out


def _world_comm(group):
    if group is None:
        raise RuntimeError("no default communicator: pass group=<VirtualComm> "
                           "(the reference defaults to MPI.COMM_WORLD)")
    return group


def recursive_halving_reduce_scatter_mpi(output_tensor: torch.Tensor,
                                         input_tensor: torch.Tensor,
                                         group: Optional[VirtualComm] = None,
                                         async_op: bool = False,
                                         op=torch.add):
    """Recursive-halving reduce_scatter, one rank's part (pccl/reduce_scatter.py:20-98).

    P must be a power of two.  In round r the rank keeps the half of its active
    blocks that contains its own block, sends the other half to the partner at
    distance `half` and adds what the partner sent."""
    assert not async_op, "Non-blocking operations not supported"
    comm = _world_comm(group)
    rank, size = comm.Get_rank(), comm.Get_size()
    total_elems = input_tensor.numel()
    assert total_elems % size == 0, "Input tensor size must be divisible by number of processes"
    block_size = total_elems // size
    # the reference silently assumes a power of two (int(log2 P) rounds); fail instead of mis-reducing
    assert size & (size - 1) == 0, "recursive halving needs a power-of-two number of processes"
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    buf = _clone(input_tensor.view(-1))           # active region, shrinks every round
    rounds = int(math.log2(size))
    for r in range(rounds):
        half = buf.numel() // block_size // 2
        count = half * block_size
        recv_buf = torch.empty(count, dtype=buf.dtype, device=buf.device)
        if (rank % (size >> r)) < (size >> (r + 1)):
            partner = (rank + half) % size
            send_data, keep = _clone(buf[count:]), buf[:count]
        else:
            partner = (rank - half) % size
            send_data, keep = _clone(buf[:count]), buf[count:]
        comm.Sendrecv(sendbuf=send_data, dest=partner, sendtag=r,
                      recvbuf=recv_buf, source=partner, recvtag=r)
        _reduce_into(keep, recv_buf, op)
        buf = keep
    kernels.copy(output_tensor.view(-1), buf.view(-1))


def ring_reduce_scatter_mpi(output_tensor: torch.Tensor,
                            input_tensor: torch.Tensor,
                            group: Optional[VirtualComm] = None,
                            async_op: bool = False,
                            op=torch.add):
    """Ring reduce_scatter, one rank's part (pccl/reduce_scatter.py:102-161):
    P-1 steps of send block (rank-step-1), receive from the left, reduce into
    block (rank-step-2); the result is block `rank`."""
    assert not async_op, "non-blocking primitives not supported"
    comm = _world_comm(group)
    rank, size = comm.Get_rank(), comm.Get_size()
    assert input_tensor.dim() == 1, "input tensor should be 1D"
    assert output_tensor.dim() == 1, "output tensor should be 1D"
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    buf = _clone(input_tensor).view(size, -1)
    block_size = buf.size(1)
    tmp = torch.empty(block_size, dtype=buf.dtype, device=buf.device)
    dest, source = (rank + 1) % size, (rank - 1 + size) % size
    for step in range(size - 1):
        send_idx = (rank - step - 1) % size
        recv_idx = (rank - step - 2) % size
        send_data = _clone(buf[send_idx])
        comm.Sendrecv(sendbuf=send_data, dest=dest, sendtag=0,
                      recvbuf=tmp, source=source, recvtag=0)
        _reduce_into(buf[recv_idx], tmp, op)
    kernels.copy(output_tensor, buf[rank])


def _reduce_scatter(
    output_tensor: torch.Tensor,
    input_tensor: torch.Tensor,
    group: Optional[Union[dist.ProcessGroup, VirtualComm]] = None,
    async_op: bool = False,
    directly_call_mpi: bool = False,
    use_rh: bool = False,
    use_pccl_cpp_backend: bool = False,
) -> Optional[Request]:
    """Dispatch on the group type with the reference's precedence
    (pccl/reduce_scatter.py:164-203): the native backend wins over
    `directly_call_mpi`, which wins over the Python algorithms."""
    if group is None or isinstance(group, dist.ProcessGroup):
        request = dist.reduce_scatter_tensor(output_tensor, input_tensor, group=group, async_op=async_op)
    elif isinstance(group, VirtualComm):
        if use_pccl_cpp_backend:
            request = ext.reduce_scatter_mpi(output_tensor, input_tensor, group,
                                             "recursive" if use_rh else "ring")
        elif not directly_call_mpi:
            if use_rh:
                request = recursive_halving_reduce_scatter_mpi(output_tensor, input_tensor, group, async_op)
            else:
                request = ring_reduce_scatter_mpi(output_tensor, input_tensor, group, async_op)
        else:
            request = group.Reduce_scatter_block(input_tensor, output_tensor)
    else:
        raise TypeError(
            f"Unsupported group type: {type(group)}. "
            "Expected torch.distributed.ProcessGroup or pccl.virtual.VirtualComm."
        )
    return request


def reduce_scatter_2D(output_tensor: torch.Tensor,
                      input_tensor: torch.Tensor,
                      group: Optional[ProcessGroups] = None,
                      async_op: bool = False,
                      use_rh: bool = False,
                      use_pccl_cpp_backend: bool = False):
    """Hierarchical reduce_scatter (pccl/reduce_scatter.py:205-235): permute the
    input [inter, intra, m] -> [intra, inter, m], reduce_scatter inside the
    node, then across nodes."""
    assert not async_op, "Non blocking version not implemented"
    assert input_tensor.dim() == 1 and output_tensor.dim() == 1, "all_gather_2D only admits 1D tensors"
    intra_node_group_size, inter_node_group_size = group.get_world_size()

    if use_pccl_cpp_backend and getattr(group, "virtual_world", None) is not None:
        # virtual ranks, native backend: both levels and the permutation in one
        # batched call, nothing materialised in between
        ext.reduce_scatter_2d(output_tensor, input_tensor, group, "recursive" if use_rh else "ring")
        return

    input_permuted = torch.empty_like(input_tensor)
    kernels.block_transpose(input_permuted, input_tensor, inter_node_group_size, intra_node_group_size)

    output_intermediate = torch.empty(input_permuted.size(0) // intra_node_group_size,
                                      device=input_tensor.device, dtype=input_tensor.dtype)
    _reduce_scatter(output_intermediate, input_permuted, group.get_inner_group(), async_op=False,
                    use_rh=use_rh, use_pccl_cpp_backend=use_pccl_cpp_backend)
    _reduce_scatter(output_tensor, output_intermediate, group.get_outer_group(), async_op=False,
                    use_rh=use_rh, use_pccl_cpp_backend=use_pccl_cpp_backend)
