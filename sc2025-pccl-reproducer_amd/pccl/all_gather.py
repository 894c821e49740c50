"""all_gather on process groups or virtual ranks (pccl/all_gather.py).

Same names and keyword arguments as the reference.  On a `VirtualComm`:
`use_rd=True` runs recursive doubling -- natively batched with
`use_pccl_cpp_backend=True` (pccl.ext.all_gather_mpi), rank by rank otherwise;
`use_rd=False` is the path the reference hands to MPI_Allgather / Iallgather
(pccl/all_gather.py:124-128): here one fused placement launch.
"""
from __future__ import annotations

from typing import Optional, Union

import torch
import torch.distributed as dist

from . import ext, kernels
from .process_groups import ProcessGroups
from .request import Request, StreamRequest
from .virtual import VirtualComm


def recursive_doubling_allgather_mpi(output_tensor: torch.Tensor,
                                     input_tensor: torch.Tensor,
                                     group: Optional[VirtualComm] = None,
                                     async_op: bool = False):
    """Recursive-doubling all_gather, one rank's part (pccl/all_gather.py:14-95).
    P must be a power of two; block i of the output is rank i's input."""
    assert not async_op, "non-blocking primitives not supported"
    if group is None:
        raise RuntimeError("no default communicator: pass group=<VirtualComm>")
    comm = group
    rank, size = comm.Get_rank(), comm.Get_size()
    block_size = input_tensor.numel()
    assert output_tensor.numel() == size * block_size, "Output tensor has incorrect size"
    assert size & (size - 1) == 0, "recursive doubling needs a power-of-two number of processes"
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    kernels.copy(output_tensor[rank * block_size:(rank + 1) * block_size], input_tensor.view(-1))
    seg_size = 1
    while seg_size < size:
        partner = rank ^ seg_size
        group_start = (rank // (2 * seg_size)) * (2 * seg_size)
        if rank < partner:
            send_offset = group_start * block_size
            recv_offset = (group_start + seg_size) * block_size
        else:
            send_offset = (group_start + seg_size) * block_size
            recv_offset = group_start * block_size
        count = seg_size * block_size
        tmp = torch.empty(count, dtype=output_tensor.dtype, device=output_tensor.device)
        comm.Sendrecv(sendbuf=output_tensor[send_offset:send_offset + count], dest=partner, sendtag=0,
                      recvbuf=tmp, source=partner, recvtag=0)
        kernels.copy(output_tensor[recv_offset:recv_offset + count], tmp)
        seg_size *= 2


def _all_gather(
    output_tensor: torch.Tensor,
    input_tensor: torch.Tensor,
    group: Optional[Union[dist.ProcessGroup, VirtualComm]] = None,
    async_op: bool = False,
    use_rd: bool = False,
    use_pccl_cpp_backend: bool = False
) -> Optional[Request]:
    """Dispatch on the group type (pccl/all_gather.py:98-134)."""
    if group is None or isinstance(group, dist.ProcessGroup):
        request = dist.all_gather_into_tensor(output_tensor, input_tensor, group, async_op)
    elif isinstance(group, VirtualComm):
        if use_rd:
            if use_pccl_cpp_backend:
                request = ext.all_gather_mpi(output_tensor, input_tensor, group, "recursive")
            else:
                request = recursive_doubling_allgather_mpi(output_tensor, input_tensor, group, async_op)
        else:
            group.Allgather(input_tensor, output_tensor)
            # the non-blocking flavour returns a handle on the enqueued work
            request = Request(StreamRequest()) if async_op else None
    else:
        raise TypeError(
            f"Unsupported group type: {type(group)}. "
            "Expected torch.distributed.ProcessGroup or pccl.virtual.VirtualComm."
        )
    return request


def all_gather_2D(output_tensor: torch.Tensor,
                  input_tensor: torch.Tensor,
                  group: Optional[ProcessGroups] = None,
                  async_op: bool = False,
                  use_rd: bool = False,
                  use_pccl_cpp_backend: bool = False):
    """Hierarchical all_gather (pccl/all_gather.py:136-159): gather across
    nodes, gather inside the node, then undo the [intra, inter, m] layout."""
    assert not async_op, "Non blocking version not implemented"
    assert input_tensor.dim() == 1 and output_tensor.dim() == 1, "all_gather_2D only admits 1D tensors"
    intra_node_group_size, inter_node_group_size = group.get_world_size()

    if use_pccl_cpp_backend and getattr(group, "virtual_world", None) is not None:
        # virtual ranks, native backend: both levels and the un-permutation in one batched call
        ext.all_gather_2d(output_tensor, input_tensor, group, "recursive" if use_rd else "ring")
        return

    output_intermediate = torch.empty(input_tensor.size(0) * inter_node_group_size,
                                      device=input_tensor.device, dtype=input_tensor.dtype)
    _all_gather(output_intermediate, input_tensor, group.get_outer_group(), async_op=False,
                use_rd=use_rd, use_pccl_cpp_backend=use_pccl_cpp_backend)

    gathered = torch.empty_like(output_tensor)
    _all_gather(gathered, output_intermediate, group.get_inner_group(), async_op=False,
                use_rd=use_rd, use_pccl_cpp_backend=use_pccl_cpp_backend)
    # un-permute straight into the caller's tensor: one pass instead of the
    # reference's reshape-copy followed by copy_ (pccl/all_gather.py:158-159)
    kernels.block_transpose(output_tensor, gathered, intra_node_group_size, inter_node_group_size)
