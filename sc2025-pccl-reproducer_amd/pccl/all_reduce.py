"""all_reduce as reduce_scatter followed by all_gather (pccl/src/yacl.cpp:146-177,
pccl/all_reduce.py:21-55).  In place on `input_tensor`, like the reference."""
from __future__ import annotations

from typing import Optional, Union

import torch
import torch.distributed as dist

from .all_gather import _all_gather
from .reduce_scatter import _reduce_scatter
from .request import Request
from .virtual import VirtualComm


def _all_reduce(
    input_tensor: torch.Tensor,
    group: Optional[Union[dist.ProcessGroup, VirtualComm]] = None,
    async_op: bool = False,
    use_rh_and_rd: bool = False,
    use_yacl: bool = False,
    directly_call_mpi: bool = False,
    *,
    use_pccl_cpp_backend: bool = True,
) -> Optional[Request]:
    """The reference's signature (pccl/all_reduce.py:21-28) plus a keyword-only
    backend switch.  On virtual ranks:

    * `directly_call_mpi=True`: what the reference hands to MPI_Allreduce
      (pccl/all_reduce.py:46-49); a vendor MPI leaves the summation order open,
      here it is the ring order (Reduce_scatter_block + Allgather of the
      virtual communicator, one fused launch each);
    * otherwise reduce_scatter + all_gather with the ring schedules, or with
      recursive halving + doubling when `use_rh_and_rd` is set: the composition
      the reference reaches through `use_yacl=True` (pccl/src/yacl.cpp:146-177).
      The reference does nothing at all when neither `use_yacl` nor
      `directly_call_mpi` is given (pccl/all_reduce.py:40-44); that is not
      reproduced, the flag is accepted and the reduction always happens."""
    del use_yacl
    if group is None or isinstance(group, dist.ProcessGroup):
        return dist.all_reduce(input_tensor, group=group, async_op=async_op)
    if not isinstance(group, VirtualComm):
        raise TypeError(
            f"Unsupported group type: {type(group)}. "
            "Expected torch.distributed.ProcessGroup or pccl.virtual.VirtualComm."
        )
    assert not async_op, "Non blocking version not implemented"
    size = group.Get_size()
    if input_tensor.dim() != 1 or input_tensor.numel() % size:
        raise RuntimeError("Input tensor size must be divisible by number of processes")
    block = torch.empty(input_tensor.numel() // size, dtype=input_tensor.dtype, device=input_tensor.device)
    if directly_call_mpi:
        group.Reduce_scatter_block(input_tensor, block)
        group.Allgather(block, input_tensor)
        return None
    _reduce_scatter(block, input_tensor, group, use_rh=use_rh_and_rd, use_pccl_cpp_backend=use_pccl_cpp_backend)
    if use_rh_and_rd:
        _all_gather(input_tensor, block, group, use_rd=True, use_pccl_cpp_backend=use_pccl_cpp_backend)
    else:
        _all_gather(input_tensor, block, group, use_rd=False)
    return None
