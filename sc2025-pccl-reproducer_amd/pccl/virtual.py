"""Virtual ranks: P ranks of a PCCL job inside one process on one GPU.

The reference runs one process per GPU and moves data between them with
MPI_Sendrecv (pccl/src/reduce_scatter.cpp:67-69,140-142; pccl/all_gather.py:85-87).
Here every rank's buffers live in the same GPU's HBM, so a message is a
device-to-device copy (or, in the batched kernels, a direct read of the
partner's buffer) and a communicator is plain bookkeeping.

`VirtualComm` offers the slice of the mpi4py communicator interface that the
reference's code uses -- Get_rank / Get_size / Sendrecv / Barrier / Split /
Allgather / Reduce_scatter_block -- so the per-rank functions of this package
keep the reference's signatures.  Two ways to drive the ranks:

  * SPMD: `VirtualWorld(P).run(fn)` starts one Python thread per rank and calls
    `fn(comm)` in each, exactly like `mpirun -np P`; collective calls meet in a
    rendezvous and the last rank to arrive enqueues ONE batched launch for all;
  * driver: hand the per-rank tensors of all ranks to `pccl.kernels.*_ranks`
    (or the `VirtualWorld` helpers) from a single thread.

All work is enqueued on the calling thread's current torch stream (by default
every thread shares the device's default stream, which orders the ranks' work).
"""
from __future__ import annotations

import threading
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import kernels

# A rank that waits this long for its peers is reported instead of hanging.
RENDEZVOUS_TIMEOUT_S = 120.0


class VirtualRankError(RuntimeError):
    pass


class _Rendezvous:
    """All `size` ranks deposit a payload; the last one runs `action(payloads)`
    for everybody; every rank returns (or raises) together."""

    def __init__(self, size: int):
        self.size = size
        self.cv = threading.Condition()
        self.slots: List[object] = [None] * size
        self.present = [False] * size
        self.count = 0
        self.generation = 0
        self.kind = None
        self.outcome: Dict[int, Tuple[object, Optional[BaseException]]] = {}
        self.aborted: Optional[BaseException] = None

    def abort(self, exc: Optional[BaseException]):
        """Wake every waiting rank (exc) or re-arm the meeting point (None)."""
        with self.cv:
            self.aborted = exc
            if exc is None:
                self.slots = [None] * self.size
                self.present = [False] * self.size
                self.count = 0
            self.cv.notify_all()

    def arrive(self, rank: int, kind: str, payload, action: Callable[[list], object]):
        with self.cv:
            if self.present[rank]:
                raise VirtualRankError(
                    f"rank {rank} entered '{kind}' again before the other ranks of the communicator "
                    "made the call; drive virtual ranks from VirtualWorld.run() (one thread per rank)")
            if self.count and self.kind != kind:
                raise VirtualRankError(f"rank {rank} called '{kind}' while other ranks are in '{self.kind}'")
            gen = self.generation
            self.kind = kind
            self.slots[rank] = payload
            self.present[rank] = True
            self.count += 1
            if self.count == self.size:
                result, err = None, None
                try:
                    result = action(list(self.slots))
                except BaseException as e:  # delivered to every rank
                    err = e
                self.outcome[gen] = (result, err)
                self.outcome.pop(gen - 2, None)
                self.slots = [None] * self.size
                self.present = [False] * self.size
                self.count = 0
                self.generation += 1
                self.cv.notify_all()
            else:
                if self.size > 1 and not _in_spmd():
                    # a lone caller would wait for ever
                    self.slots[rank] = None
                    self.present[rank] = False
                    self.count -= 1
                    raise VirtualRankError(
                        f"'{kind}' is collective over {self.size} virtual ranks: call it from "
                        "VirtualWorld.run() (one thread per rank) or use the *_ranks driver functions")
                ok = self.cv.wait_for(lambda: self.generation != gen or self.aborted is not None,
                                      timeout=RENDEZVOUS_TIMEOUT_S)
                if self.generation == gen:
                    self.slots[rank] = None
                    self.present[rank] = False
                    self.count -= 1
                    if not ok:
                        raise VirtualRankError(f"rank {rank}: timed out in '{kind}' waiting for the other ranks")
                    raise VirtualRankError(f"rank {rank}: '{kind}' abandoned because another rank failed")
            result, err = self.outcome[gen]
        if err is not None:
            raise err
        return result


_tls = threading.local()


def _in_spmd() -> bool:
    return getattr(_tls, "spmd", False)


class _Group:
    """Shared state of one communicator: its world ranks and its meeting points."""

    def __init__(self, world: "VirtualWorld", ranks: Tuple[int, ...]):
        self.world = world
        self.ranks = ranks
        self.size = len(ranks)
        self.rendezvous = _Rendezvous(self.size)
        # point-to-point mailboxes: (src, dst, tag) -> tensor
        self.mail: Dict[Tuple[int, int, int], torch.Tensor] = {}
        self.mail_cv = threading.Condition()
        self.aborted: Optional[BaseException] = None

    def abort(self, exc: Optional[BaseException]):
        self.rendezvous.abort(exc)
        with self.mail_cv:
            self.aborted = exc
            if exc is None:
                self.mail.clear()
            self.mail_cv.notify_all()


class VirtualComm:
    """One rank's handle on a communicator of virtual ranks (an mpi4py.MPI.Comm
    stand-in for the calls the reference makes)."""

    def __init__(self, group: _Group, rank: int):
        self._group = group
        self._rank = rank

    # -- mpi4py surface ------------------------------------------------------
    def Get_rank(self) -> int:
        return self._rank

    def Get_size(self) -> int:
        return self._group.size

    @property
    def world(self) -> "VirtualWorld":
        return self._group.world

    @property
    def world_ranks(self) -> Tuple[int, ...]:
        """World rank of every member, in group-rank order."""
        return self._group.ranks

    def Barrier(self):
        self._group.rendezvous.arrive(self._rank, "Barrier", None, lambda _: None)

    def Split(self, color: int = 0, key: int = 0) -> "VirtualComm":
        """MPI_Comm_split: ranks with the same colour form a new communicator,
        ordered by (key, old rank) (pccl/process_groups.py:119,138)."""
        def action(payloads):
            by_colour: Dict[int, List[Tuple[int, int]]] = {}
            for old, (c, k) in enumerate(payloads):
                by_colour.setdefault(c, []).append((k, old))
            out = [None] * len(payloads)
            for members in by_colour.values():
                members.sort()
                ranks = tuple(self._group.ranks[old] for _, old in members)
                g = self._group.world._group_for(ranks)
                for new, (_, old) in enumerate(members):
                    out[old] = VirtualComm(g, new)
            return out
        return self._group.rendezvous.arrive(self._rank, "Split", (int(color), int(key)), action)[self._rank]

    def Sendrecv(self, sendbuf: torch.Tensor, dest: int, sendtag: int = 0, recvbuf: torch.Tensor = None,
                 source: int = 0, recvtag: int = 0):
        """Blocking send to `dest` + receive from `source`: the message is one
        device-to-device copy enqueued by the receiver."""
        g = self._group
        me = self._rank
        if not (0 <= dest < g.size and 0 <= source < g.size):
            raise VirtualRankError("Sendrecv: peer rank outside the communicator")
        if dest == me and source == me:
            kernels.copy(recvbuf.view(-1), sendbuf.view(-1))
            return
        if not _in_spmd():
            raise VirtualRankError("Sendrecv between virtual ranks needs VirtualWorld.run() (one thread per rank)")
        kernels.check_device_tensor(sendbuf, "sendbuf")
        kernels.check_device_tensor(recvbuf, "recvbuf")
        out_key = (me, dest, int(sendtag))
        in_key = (source, me, int(recvtag))
        with g.mail_cv:
            if out_key in g.mail:
                raise VirtualRankError("Sendrecv: a message with this (source, dest, tag) is still pending")
            g.mail[out_key] = sendbuf
            g.mail_cv.notify_all()
            g.mail_cv.wait_for(lambda: in_key in g.mail or g.aborted is not None, timeout=RENDEZVOUS_TIMEOUT_S)
            if in_key not in g.mail:
                g.mail.pop(out_key, None)
                raise VirtualRankError(f"rank {me}: Sendrecv gave up waiting for rank {source}")
            msg = g.mail[in_key]
        if msg.numel() * msg.element_size() != recvbuf.numel() * recvbuf.element_size():
            raise VirtualRankError("Sendrecv: message and receive buffer sizes differ")
        kernels.copy(recvbuf.view(-1), msg.view(-1))
        with g.mail_cv:
            del g.mail[in_key]            # consumed: the sender may reuse its buffer
            g.mail_cv.notify_all()
            g.mail_cv.wait_for(lambda: out_key not in g.mail or g.aborted is not None,
                               timeout=RENDEZVOUS_TIMEOUT_S)
            if out_key in g.mail:
                g.mail.pop(out_key, None)
                raise VirtualRankError(f"rank {me}: Sendrecv gave up waiting for rank {dest} to receive")

    def Allgather(self, sendbuf: torch.Tensor, recvbuf: torch.Tensor):
        """MPI_Allgather (pccl/all_gather.py:128): direct placement of every
        shard into every output in one launch."""
        def action(payloads):
            kernels.all_gather_ranks([p[1] for p in payloads], [p[0] for p in payloads], "ring", "fused")
        self._group.rendezvous.arrive(self._rank, "Allgather", (sendbuf, recvbuf), action)

    def Reduce_scatter_block(self, sendbuf: torch.Tensor, recvbuf: torch.Tensor):
        """MPI_Reduce_scatter_block (pccl/reduce_scatter.py:197).  The summation
        order of a vendor MPI is not defined by the reference; this one uses
        the ring order in a single fused pass."""
        def action(payloads):
            kernels.reduce_scatter_ranks([p[1] for p in payloads], [p[0] for p in payloads], "ring", "fused")
        self._group.rendezvous.arrive(self._rank, "Reduce_scatter_block", (sendbuf, recvbuf), action)

    def Bcast(self, buf: torch.Tensor, root: int = 0):
        """MPI_Bcast (pccl/patch_deepspeed.py:80): the root's buffer is copied
        into every other rank's buffer in one launch."""
        def action(payloads):
            src = payloads[root]
            others = [p for i, p in enumerate(payloads) if i != root]
            if others:
                kernels.copy_batched([o.view(-1) for o in others], [src.view(-1)] * len(others))
        if not 0 <= root < self._group.size:
            raise VirtualRankError("Bcast: root outside the communicator")
        self._group.rendezvous.arrive(self._rank, "Bcast", buf, action)

    def Free(self):
        pass

    # -- batched collectives used by the native path ---------------------------
    def _collective(self, kind: str, payload, action: Callable[[list], object]):
        return self._group.rendezvous.arrive(self._rank, kind, payload, action)

    def __repr__(self):
        return f"<VirtualComm rank={self._rank} size={self._group.size} ranks={self._group.ranks}>"


class VirtualWorld:
    """P virtual ranks on one GPU."""

    def __init__(self, size: int, device: Optional[torch.device] = None):
        if size < 1:
            raise ValueError("world size must be positive")
        self.size = size
        self.device = torch.device(device) if device is not None else torch.device("cuda", 0)
        self._groups: Dict[Tuple[int, ...], _Group] = {}
        self._lock = threading.Lock()
        self._world_group = self._group_for(tuple(range(size)))

    def _group_for(self, ranks: Tuple[int, ...]) -> _Group:
        with self._lock:
            g = self._groups.get(ranks)
            if g is None:
                g = self._groups[ranks] = _Group(self, ranks)
            return g

    def _abort_all(self, exc: Optional[BaseException]):
        with self._lock:
            groups = list(self._groups.values())
        for g in groups:
            g.abort(exc)

    def comm(self, rank: int) -> VirtualComm:
        """COMM_WORLD as seen by `rank`."""
        if not 0 <= rank < self.size:
            raise ValueError("rank outside the world")
        return VirtualComm(self._world_group, rank)

    def comms(self) -> List[VirtualComm]:
        return [self.comm(r) for r in range(self.size)]

    def subcomm(self, ranks: Sequence[int], rank: int) -> VirtualComm:
        """The communicator made of world ranks `ranks` (in that order) as seen
        by world rank `rank`; every member gets a handle on the same group."""
        ranks = tuple(int(r) for r in ranks)
        return VirtualComm(self._group_for(ranks), ranks.index(rank))

    def run(self, fn: Callable, *args, **kwargs) -> list:
        """Call fn(comm, *args, **kwargs) once per rank, each in its own thread,
        like `mpirun -np P`.  Returns the per-rank results; the first exception
        of any rank is re-raised after all threads have ended."""
        results = [None] * self.size
        errors: List[Optional[BaseException]] = [None] * self.size
        dev = self.device
        self._abort_all(None)          # re-arm every meeting point

        def body(r):
            _tls.spmd = True
            try:
                if dev.type == "cuda":
                    torch.cuda.set_device(dev)
                results[r] = fn(self.comm(r), *args, **kwargs)
            except BaseException as e:
                errors[r] = e
                self._abort_all(e)     # peers waiting for this rank give up now
            finally:
                _tls.spmd = False

        threads = [threading.Thread(target=body, args=(r,), name=f"vrank{r}", daemon=True)
                   for r in range(self.size)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        # report the root cause, not the peers that merely timed out waiting
        primary = [e for e in errors if e is not None and not isinstance(e, VirtualRankError)]
        anyerr = primary or [e for e in errors if e is not None]
        if anyerr:
            raise anyerr[0]
        return results
