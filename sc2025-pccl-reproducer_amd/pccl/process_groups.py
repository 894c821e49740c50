"""2-D grid of process groups (pccl/process_groups.py:6-263).

`ProcessGroups(intra, inter)` arranges the world as
`arange(world).reshape(num_grids, inter, intra)` (pccl/process_groups.py:97-98):
the inner group of a rank is its row (ranks of one node), the outer group its
column.  With `comm=` a `VirtualComm`, both groups are communicators of virtual
ranks on one GPU and no torch.distributed / MPI state is touched; the group
membership is the one the reference obtains from the MPI colours
`rank // intra` (:118) and `rank % intra + (rank // (intra*inter)) * intra` (:137).
Without `comm` the reference's behaviour is kept: torch.distributed must be
initialised, "nccl" groups come from `dist.new_group` (RCCL on ROCm) and "mpi"
groups from mpi4py, if that is installed.
"""
from __future__ import annotations

from typing import List, Optional, Union

import numpy as np
import torch.distributed as dist

from .virtual import VirtualComm


def grid_members(world_size: int, rank: int, intra_group_size: int, inter_group_size: int):
    """World ranks of `rank`'s inner and outer group, in group-rank order."""
    if world_size % (intra_group_size * inter_group_size) != 0:
        raise ValueError(
            f"world_size ({world_size}) must be divisible by (intra_group_size * inter_group_size) "
            f"({intra_group_size * inter_group_size} = {intra_group_size * inter_group_size})."
        )
    num_2d_grids = world_size // (intra_group_size * inter_group_size)
    grid = np.arange(world_size).reshape(num_2d_grids, inter_group_size, intra_group_size)
    g, j, i = np.argwhere(grid == rank)[0]
    return [int(x) for x in grid[g, j, :]], [int(x) for x in grid[g, :, i]]


class ProcessGroups:
    """Inner (intra-node) and outer (inter-node) groups of the current rank."""

    def __init__(
        self,
        intra_group_size: int,
        inter_group_size: int,
        inner_group_backend: str = "nccl",
        outer_group_backend: str = "mpi",
        comm: Optional[VirtualComm] = None,
    ):
        if comm is None:
            assert dist.is_initialized(), "pytorch distributed should be initialized by the user"
        # virtual ranks: the communicator spanning every grid, and the grid shape,
        # let the 2-D collectives batch all groups of a level into one launch
        self.virtual_world = comm
        self.grid_shape = (intra_group_size, inter_group_size)
        self.inner_group, self.outer_group = self.create_2D_grid(
            intra_group_size=intra_group_size,
            inter_group_size=inter_group_size,
            inner_group_backend=inner_group_backend,
            outer_group_backend=outer_group_backend,
            comm=comm,
        )

    @staticmethod
    def create_2D_grid(
        intra_group_size: int,
        inter_group_size: int,
        inner_group_backend: str = "nccl",
        outer_group_backend: str = "mpi",
        comm: Optional[VirtualComm] = None,
    ) -> List[Union["dist.ProcessGroup", VirtualComm]]:
        valid_backends = ["mpi", "nccl"]
        if inner_group_backend not in valid_backends:
            raise ValueError(f"Unsupported inner_group_backend '{inner_group_backend}'. Choose 'mpi' or 'nccl'.")
        if outer_group_backend not in valid_backends:
            raise ValueError(f"Unsupported outer_group_backend '{outer_group_backend}'. Choose 'mpi' or 'nccl'.")

        if comm is not None:
            # virtual ranks: both levels are communicators on one GPU
            if not isinstance(comm, VirtualComm):
                raise TypeError("comm must be a pccl.virtual.VirtualComm")
            rank, world_size = comm.Get_rank(), comm.Get_size()
            inner, outer = grid_members(world_size, rank, intra_group_size, inter_group_size)
            base = comm.world_ranks
            world = comm.world
            return [world.subcomm([base[r] for r in inner], base[rank]),
                    world.subcomm([base[r] for r in outer], base[rank])]

        if not dist.is_initialized():
            raise RuntimeError("torch.distributed is not initialized. Please initialize it before creating groups.")
        rank = dist.get_rank()
        world_size = dist.get_world_size()
        if world_size % (intra_group_size * inter_group_size) != 0:
            raise ValueError(
                f"world_size ({world_size}) must be divisible by (intra_group_size * inter_group_size) "
                f"({intra_group_size * inter_group_size} = {intra_group_size * inter_group_size})."
            )
        num_2d_grids = world_size // (intra_group_size * inter_group_size)
        grid = np.arange(world_size).reshape(num_2d_grids, inter_group_size, intra_group_size)

        def mpi_world():
            try:
                from mpi4py import MPI
            except ImportError as e:
                raise RuntimeError("the 'mpi' backend needs mpi4py; pass comm=VirtualComm for virtual ranks") from e
            return MPI.COMM_WORLD

        inner_group = outer_group = None
        if inner_group_backend == "nccl":
            # every rank must take part in every new_group call
            for i in range(num_2d_grids):
                for j in range(inter_group_size):
                    ranks = [int(x) for x in grid[i, j, :]]
                    this_group = dist.new_group(ranks=ranks, backend="nccl")
                    if rank in ranks:
                        inner_group = this_group
        else:
            inner_group = mpi_world().Split(rank // intra_group_size)

        if outer_group_backend == "nccl":
            for i in range(num_2d_grids):
                for j in range(intra_group_size):
                    ranks = [int(x) for x in grid[i, :, j]]
                    this_group = dist.new_group(ranks=ranks, backend="nccl")
                    if rank in ranks:
                        outer_group = this_group
        else:
            color = rank % intra_group_size + (rank // (intra_group_size * inter_group_size)) * intra_group_size
            outer_group = mpi_world().Split(color)

        if inner_group is None:
            raise RuntimeError("Failed to create the inner group for the current process.")
        if outer_group is None:
            raise RuntimeError("Failed to create the outer group for the current process.")
        return [inner_group, outer_group]

    def get_rank(self, group_index: Optional[int] = None) -> Union[int, List[int]]:
        if group_index is None:
            return [self._get_rank_internal(self.inner_group), self._get_rank_internal(self.outer_group)]
        elif group_index == 0:
            return self._get_rank_internal(self.inner_group)
        elif group_index == 1:
            return self._get_rank_internal(self.outer_group)
        raise ValueError("group_index must be 0 (inner) or 1 (outer).")

    def get_world_size(self, group_index: Optional[int] = None) -> Union[int, List[int]]:
        if group_index is None:
            return [self._get_world_size_internal(self.inner_group),
                    self._get_world_size_internal(self.outer_group)]
        elif group_index == 0:
            return self._get_world_size_internal(self.inner_group)
        elif group_index == 1:
            return self._get_world_size_internal(self.outer_group)
        raise ValueError("group_index must be 0 (inner) or 1 (outer) or None (for both).")

    @staticmethod
    def _get_rank_internal(group) -> int:
        if isinstance(group, dist.ProcessGroup):
            return dist.get_rank(group=group)
        if hasattr(group, "Get_rank"):
            return group.Get_rank()
        raise TypeError("Unsupported group type.")

    @staticmethod
    def _get_world_size_internal(group) -> int:
        if isinstance(group, dist.ProcessGroup):
            return dist.get_world_size(group=group)
        if hasattr(group, "Get_size"):
            return group.Get_size()
        raise TypeError("Unsupported group type.")

    def get_inner_group(self):
        return self.inner_group

    def get_outer_group(self):
        return self.outer_group

    def __repr__(self) -> str:
        def name(g):
            if isinstance(g, VirtualComm):
                return "VIRTUAL"
            return "NCCL" if isinstance(g, dist.ProcessGroup) else "MPI"
        return (f"<ProcessGroups inner_group_backend={name(self.inner_group)}, "
                f"outer_group_backend={name(self.outer_group)}>")
