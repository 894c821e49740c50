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
    use_pccl_cpp_backend: bool = True,
) -> Optional[Request]:
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
    _reduce_scatter(block, input_tensor, group, use_rh=use_rh_and_rd, use_pccl_cpp_backend=use_pccl_cpp_backend)
    if use_rh_and_rd:
        _all_gather(input_tensor, block, group, use_rd=True, use_pccl_cpp_backend=use_pccl_cpp_backend)
    else:
        _all_gather(input_tensor, block, group, use_rd=False)
    return None
