"""The two entry points of the reference's compiled extension, on virtual ranks.

`reduce_scatter_mpi(output, input, comm, algorithm)` and
`all_gather_mpi(output, input, comm, algorithm)` keep the names, argument order,
checks and messages of pccl/src/pccl.cpp:11-85 and :87-142.  Each virtual rank
calls them with its own tensors and communicator handle; the ranks meet, and
the last one to arrive enqueues the batched HIP launches for the whole
collective (include/pccl_hip.h: pccl_hip_reduce_scatter_virtual /
pccl_hip_all_gather_virtual).  Like the reference they return None with the
work queued on the current stream.

Deviation kept on purpose: reduce_scatter accepts bfloat16 and float16 as well as
float32 (the reference's extension rejects everything but float, pccl.cpp:42-45;
its Python algorithms are what run the 16-bit types).
"""
from __future__ import annotations

import torch

from . import kernels
from .virtual import VirtualComm


def _check_comm(py_comm):
    if not isinstance(py_comm, VirtualComm):
        raise TypeError(f"expected a pccl.virtual.VirtualComm, got {type(py_comm)}")


def reduce_scatter_mpi(output_tensor: torch.Tensor, input_tensor: torch.Tensor, py_comm,
                       algorithm: str = "recursive") -> None:
    # the checks of pccl/src/pccl.cpp:16-45, in the same order
    if not output_tensor.is_contiguous():
        raise RuntimeError("output tensor must be contiguous.")
    if not input_tensor.is_contiguous():
        raise RuntimeError("input tensor must be contiguous.")
    if output_tensor.dim() != 1:
        raise RuntimeError("output tensor must be 1D")
    if input_tensor.dim() != 1:
        raise RuntimeError("input tensor must be 1D")
    _check_comm(py_comm)
    size = py_comm.Get_size()
    total_elems = input_tensor.numel()
    if total_elems % size != 0:
        raise RuntimeError("Input tensor size must be divisible by number of processes")
    block_size = total_elems // size
    if output_tensor.numel() != block_size:
        raise RuntimeError("Output tensor must have block_size elements (input tensor numel()/world_size)")
    if input_tensor.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise RuntimeError("Input tensor must be of type float")
    if output_tensor.dtype != input_tensor.dtype:
        raise RuntimeError("Output tensor must be of type float")
    if algorithm not in ("recursive", "ring"):
        raise RuntimeError(f"Unknown algorithm specified for reduce_scatter_mpi: {algorithm}")
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    def launch(payloads):
        kernels.reduce_scatter_ranks([p[0] for p in payloads], [p[1] for p in payloads], algorithm)

    py_comm._collective(f"reduce_scatter_mpi[{algorithm}]", (output_tensor, input_tensor), launch)


def all_gather_mpi(output_tensor: torch.Tensor, input_tensor: torch.Tensor, py_comm,
                   algorithm: str = "recursive") -> None:
    # the checks of pccl/src/pccl.cpp:92-116,140
    if not output_tensor.is_contiguous():
        raise RuntimeError("output tensor must be contiguous.")
    if not input_tensor.is_contiguous():
        raise RuntimeError("input tensor must be contiguous.")
    if output_tensor.dim() != 1:
        raise RuntimeError("output tensor must be 1D")
    if input_tensor.dim() != 1:
        raise RuntimeError("input tensor must be 1D")
    if input_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("Input and output tensors must have the same dtype.")
    _check_comm(py_comm)
    size = py_comm.Get_size()
    if output_tensor.numel() != input_tensor.numel() * size:
        raise RuntimeError("Output tensor must have total_elem elements (input tensor numel() *world_size)")
    if algorithm not in ("recursive", "ring"):
        # the reference knows "recursive" only (pccl.cpp:126,140); "ring" is this build's schedule
        raise RuntimeError(f"Unknown algorithm specified for all_gather_mpi: {algorithm}")
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    def launch(payloads):
        kernels.all_gather_ranks([p[0] for p in payloads], [p[1] for p in payloads], algorithm)

    py_comm._collective(f"all_gather_mpi[{algorithm}]", (output_tensor, input_tensor), launch)


def _run_grids(payloads, intra, inter, launch_grid):
    """Split the world into its independent intra*inter grids (consecutive
    ranks, pccl/process_groups.py:97-98) and launch each."""
    per = intra * inter
    for g0 in range(0, len(payloads), per):
        part = payloads[g0:g0 + per]
        launch_grid([p[0] for p in part], [p[1] for p in part])


def reduce_scatter_2d(output_tensor: torch.Tensor, input_tensor: torch.Tensor, groups, algorithm: str) -> None:
    """Native path of reduce_scatter_2D on virtual ranks: every rank of the world
    communicator brings its tensors; the last one enqueues the batched launches
    (include/pccl_hip.h: pccl_hip_reduce_scatter_2d_virtual)."""
    intra, inter = groups.grid_shape
    world = groups.virtual_world
    if input_tensor.numel() % (intra * inter):
        raise RuntimeError("Input tensor size must be divisible by number of processes")
    if output_tensor.numel() != input_tensor.numel() // (intra * inter):
        raise RuntimeError("Output tensor must have block_size elements (input tensor numel()/world_size)")
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    def launch(payloads):
        _run_grids(payloads, intra, inter,
                   lambda outs, ins: kernels.reduce_scatter_2d_ranks(outs, ins, intra, inter, algorithm))

    world._collective(f"reduce_scatter_2D[{algorithm}]", (output_tensor, input_tensor), launch)


def all_gather_2d(output_tensor: torch.Tensor, input_tensor: torch.Tensor, groups, algorithm: str) -> None:
    """Native path of all_gather_2D on virtual ranks (pccl_hip_all_gather_2d_virtual)."""
    intra, inter = groups.grid_shape
    world = groups.virtual_world
    if input_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("Input and output tensors must have the same dtype.")
    if output_tensor.numel() != input_tensor.numel() * intra * inter:
        raise RuntimeError("Output tensor must have total_elem elements (input tensor numel() *world_size)")
    kernels.check_device_tensor(input_tensor, "input")
    kernels.check_device_tensor(output_tensor, "output")

    def launch(payloads):
        _run_grids(payloads, intra, inter,
                   lambda outs, ins: kernels.all_gather_2d_ranks(outs, ins, intra, inter, algorithm))

    world._collective(f"all_gather_2D[{algorithm}]", (output_tensor, input_tensor), launch)
