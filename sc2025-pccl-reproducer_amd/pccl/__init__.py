"""pccl -- MI355X-native per-GPU compute of PCCL's collectives.

Same import surface as the reference package (pccl/__init__.py:1-3), plus the
two functions of its compiled extension (`import pccl as pccl_cpp;
pccl_cpp.reduce_scatter_mpi(...)`, pccl/reduce_scatter.py:185-189) and the
virtual-rank machinery that stands in for MPI on one GPU.
"""
from .process_groups import ProcessGroups
from .all_gather import all_gather_2D, _all_gather, recursive_doubling_allgather_mpi
from .reduce_scatter import (reduce_scatter_2D, _reduce_scatter, recursive_halving_reduce_scatter_mpi,
                             ring_reduce_scatter_mpi)
from .all_reduce import _all_reduce
from .ext import reduce_scatter_mpi, all_gather_mpi
from .request import Request, StreamRequest
from .virtual import VirtualWorld, VirtualComm, VirtualRankError
from . import kernels, build_kernels

__all__ = [
    "ProcessGroups", "all_gather_2D", "_all_gather", "recursive_doubling_allgather_mpi",
    "reduce_scatter_2D", "_reduce_scatter", "recursive_halving_reduce_scatter_mpi",
    "ring_reduce_scatter_mpi", "_all_reduce", "reduce_scatter_mpi", "all_gather_mpi",
    "Request", "StreamRequest", "VirtualWorld", "VirtualComm", "VirtualRankError",
    "kernels", "build_kernels",
]
