"""Torch-facing wrappers of the HIP kernels in libpccl_hip.so.

PyTorch-ROCm is used for what the reference uses it for: device memory and the
current stream (pccl/src/reduce_scatter.cpp:29,116; pccl/src/all_gather.cpp:28).
Every function validates its tensors on the host, takes raw device addresses
and enqueues on `torch.cuda.current_stream()`.  Nothing here computes on the
CPU: tensors that are not on the GPU are rejected.
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence

import torch

from . import _native
from ._native import (BF16, F16, F32, MODE_FAITHFUL, MODE_FUSED, MODE_STEPS, ORDER_HALVING,
                      ORDER_RING, MAX_RANKS, MAX_VIRTUAL_RANKS)

_MODES = {"steps": MODE_STEPS, "fused": MODE_FUSED, "faithful": MODE_FAITHFUL}


# How a whole collective runs when the caller does not say: one fused launch.
# It gives the bits of the per-step replay of the same algorithm in a third to
# half of the time (P = 8 ring reduce_scatter of 512 MiB per rank on MI355X:
# 0.74 ms against 1.77 ms per step; 64-rank halving: 10.4 against 31.9 ms).
DEFAULT_MODE = "fused"


def mode_code(mode) -> int:
    """'steps' | 'fused' | 'faithful' (or None = $PCCL_VIRTUAL_MODE, default fused)."""
    if mode is None:
        mode = os.environ.get("PCCL_VIRTUAL_MODE", DEFAULT_MODE)
    if isinstance(mode, int):
        if mode not in _MODES.values():
            raise ValueError(f"unknown mode {mode}")
        return mode
    try:
        return _MODES[str(mode)]
    except KeyError:
        raise ValueError(f"unknown mode {mode!r}; expected one of {sorted(_MODES)}") from None


def dtype_code(dtype: torch.dtype) -> int:
    """Element type of the reduction kernels.  The reference's extension takes
    float32 only (pccl/src/pccl.cpp:42-45); bfloat16 and float16 are what its
    Python algorithms add with torch.add (pccl/reduce_scatter.py:24,83,95,158)."""
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float16:
        return F16
    raise RuntimeError("Input tensor must be of type float (float32, bfloat16 or float16)")


# the raw handle of torch's current stream without building a Stream object (a
# third of the cost; this runs once per call of a launch-bound small collective)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def stream_handle() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def check_device_tensor(t: torch.Tensor, name: str):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must reside on the GPU (got device {t.device}); "
                           "the HIP kernels have no CPU fallback")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} tensor must be contiguous.")


def _same_device(tensors: Sequence[torch.Tensor]):
    dev = tensors[0].device
    for t in tensors:
        if t.device != dev:
            raise RuntimeError("all virtual ranks must live on one GPU")


def _ptrs(tensors: Optional[Sequence[torch.Tensor]]):
    return None if tensors is None else [t.data_ptr() for t in tensors]


# ---------------------------------------------------------------------------
# element kernels
# ---------------------------------------------------------------------------

def accumulate(dst: torch.Tensor, src: torch.Tensor):
    """dst += src  (pccl/src/common.cu:5-19)."""
    check_device_tensor(dst, "dst"); check_device_tensor(src, "src")
    if dst.dtype != src.dtype or dst.numel() != src.numel():
        raise RuntimeError("accumulate: dst and src must have the same dtype and size")
    _native.load().accumulate(dst.data_ptr(), src.data_ptr(), dst.numel(), dtype_code(dst.dtype),
                              stream_handle())


def add(dst: torch.Tensor, a: torch.Tensor, b: torch.Tensor):
    """dst = a + b (dst may be a or b)."""
    for t, n in ((dst, "dst"), (a, "a"), (b, "b")):
        check_device_tensor(t, n)
    if not (dst.dtype == a.dtype == b.dtype) or not (dst.numel() == a.numel() == b.numel()):
        raise RuntimeError("add: operands must have the same dtype and size")
    _native.load().add(dst.data_ptr(), a.data_ptr(), b.data_ptr(), dst.numel(), dtype_code(dst.dtype),
                       stream_handle())


def add_batched(dst: Sequence[torch.Tensor], a: Sequence[torch.Tensor], b: Sequence[torch.Tensor]):
    """dst[s] = a[s] + b[s] for every segment s in one launch."""
    if not (len(dst) == len(a) == len(b)):
        raise ValueError("dst, a, b must have the same number of segments")
    if not dst:
        return
    n, dt = dst[0].numel(), dst[0].dtype
    for group, nm in ((dst, "dst"), (a, "a"), (b, "b")):
        for t in group:
            check_device_tensor(t, nm)
            if t.numel() != n or t.dtype != dt:
                raise RuntimeError("add_batched: all segments must have the same dtype and size")
    _native.load().add_batched(_ptrs(dst), _ptrs(a), _ptrs(b), n, dtype_code(dt), stream_handle())


def copy(dst: torch.Tensor, src: torch.Tensor):
    """Byte copy dst <- src (same number of bytes)."""
    copy_batched([dst], [src])


def copy_batched(dst: Sequence[torch.Tensor], src: Sequence[torch.Tensor]):
    """dst[s] <- src[s] (bytes) for every segment in one launch."""
    if len(dst) != len(src):
        raise ValueError("dst and src must have the same number of segments")
    nbytes = []
    for d, s in zip(dst, src):
        check_device_tensor(d, "dst"); check_device_tensor(s, "src")
        nb = d.numel() * d.element_size()
        if nb != s.numel() * s.element_size():
            raise RuntimeError("copy_batched: segment sizes differ")
        nbytes.append(nb)
    lib = _native.load()
    for i in range(0, len(dst), MAX_RANKS):
        lib.copy_batched(_ptrs(dst[i:i + MAX_RANKS]), _ptrs(src[i:i + MAX_RANKS]),
                         nbytes[i:i + MAX_RANKS], stream_handle())


def reduce_kway(out: torch.Tensor, shards: Sequence[torch.Tensor], order: str = "ring", first: int = 0,
                per_hop_round: bool = True):
    """out = sum of the shards, added in the order of a schedule, in one pass.

    order 'ring': shards first, first+1, ... (mod k) as a left fold;
    order 'halving': the butterfly of recursive halving rooted at `first`."""
    # a call on the same tensor objects replays the checked arguments of the first (see _PLANS below)
    key = ("kway", order, first, bool(per_hop_round), id(out), *map(id, shards))
    if shards and _plan_lookup(key, (out,), shards):
        return
    check_device_tensor(out, "out")
    for s in shards:
        check_device_tensor(s, "shard")
        if s.dtype != out.dtype or s.numel() != out.numel():
            raise RuntimeError("reduce_kway: shards must match the output's dtype and size")
    code = {"ring": ORDER_RING, "halving": ORDER_HALVING}.get(order)
    if code is None:
        raise ValueError(f"unknown order {order!r}")
    lib = _native.load()
    table = _native._ptr_table(_ptrs(shards))
    args = (out.data_ptr(), table, len(shards), out.numel(), dtype_code(out.dtype), code, first,
            1 if per_hop_round else 0)
    fn = lib._lib.pccl_hip_reduce_kway
    if fn(*args, stream_handle()):
        raise _native.NativeError(lib.last_error())
    _plan_store(key, lib, fn, args, (table,), (out,), shards)


def block_transpose(dst: torch.Tensor, src: torch.Tensor, rows: int, cols: int):
    """dst = src.view(rows, cols, -1).transpose(0, 1).reshape(-1)
    (pccl/reduce_scatter.py:226, pccl/all_gather.py:158)."""
    check_device_tensor(dst, "dst"); check_device_tensor(src, "src")
    nb = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != nb or dst.dtype != src.dtype:
        raise RuntimeError("block_transpose: dst and src must have the same dtype and size")
    if rows * cols == 0 or src.numel() % (rows * cols):
        raise RuntimeError("block_transpose: size must be divisible by rows*cols")
    if dst.data_ptr() == src.data_ptr() and nb:
        raise RuntimeError("block_transpose: dst must not alias src")
    _native.load().block_transpose(dst.data_ptr(), src.data_ptr(), rows, cols, nb // (rows * cols),
                                   stream_handle())


# ---------------------------------------------------------------------------
# whole collectives over a list of virtual ranks (group-rank order)
# ---------------------------------------------------------------------------

# A collective called again on the SAME tensor objects skips the per-tensor
# checks and the building of the pointer tables: the argument pack of the first,
# fully checked call is kept and replayed (a P = 8 reduce_scatter of 1 MiB costs
# 16 us of host time through the checks against 4 us of GPU time).  An entry is
# keyed by the identities of the tensors; it holds no reference to them and is
# dropped when one of them dies, so an identity cannot come back as another
# tensor while its entry exists.  A replay still compares what the C call
# depends on for EVERY tensor of the call, work buffers included: its current
# address (storage swapped under the same object by set_() or .data), its
# length (resize_()), its element type and that it is still contiguous.  Calls
# whose work buffers come from the allocator per call are not kept.
_PLANS = {}
_PLANS_MAX = 512


class _Plan:
    __slots__ = ("lib", "fn", "args", "state", "tables", "finals", "__weakref__")


def _plan_drop(key):
    ent = _PLANS.pop(key, None)
    if ent is not None:
        for f in ent.finals:          # the other tensors of the entry need not report their death any more
            f.detach()


def _plan_state(*groups):
    """What a recorded argument pack depends on, per tensor of the call."""
    return [(t.data_ptr(), t.numel(), t.dtype, t.is_contiguous()) for g in groups for t in g]


def _plan_lookup(key, tensors_a, tensors_b, extra=()):
    ent = _PLANS.get(key)
    if ent is None:
        return False
    if ent.lib is _native._loaded and ent.state == _plan_state(tensors_a, tensors_b, extra):
        if ent.fn(*ent.args, stream_handle()):
            raise _native.NativeError(ent.lib.last_error())
        return True
    _plan_drop(key)
    return False


def _plan_store(key, lib, fn, args, tables, tensors_a, tensors_b, extra=()):
    import weakref
    if len(_PLANS) >= _PLANS_MAX:
        for k in list(_PLANS):
            _plan_drop(k)
    ent = _Plan()
    ent.lib, ent.fn, ent.args, ent.tables = lib, fn, args, tables
    ent.state = _plan_state(tensors_a, tensors_b, extra)
    ent.finals = [weakref.finalize(t, _plan_drop, key) for t in (*tensors_a, *tensors_b, *extra)]
    _PLANS[key] = ent


def reduce_scatter_ranks(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor],
                         algorithm: str = "ring", mode=None,
                         work: Optional[Sequence[torch.Tensor]] = None) -> None:
    """reduce_scatter over P = len(inputs) virtual ranks in one call.

    inputs[r] holds P*B elements, outputs[r] receives block r of the sum with
    the summation order of `algorithm` ('ring': pccl/src/reduce_scatter.cpp:101-155,
    'recursive': :16-99).  Workspaces are taken from torch's caching allocator
    when the mode needs them, as the reference's shim does (pccl/src/pccl.cpp:58-73)."""
    P = len(inputs)
    if len(outputs) != P or P < 1:
        raise ValueError("need one output per input rank")
    m = mode_code(mode)          # the resolved mode: None follows $PCCL_VIRTUAL_MODE as it is now
    key = ("rs", algorithm, m, *map(id, outputs), *map(id, inputs), None, *(() if work is None else map(id, work)))
    if _plan_lookup(key, outputs, inputs, () if work is None else work):
        return
    if P > MAX_VIRTUAL_RANKS:
        raise RuntimeError(f"at most {MAX_VIRTUAL_RANKS} virtual ranks per communicator")
    for t in inputs:
        check_device_tensor(t, "input")
    for t in outputs:
        check_device_tensor(t, "output")
    _same_device(list(inputs) + list(outputs))
    total = inputs[0].numel()
    dt = inputs[0].dtype
    if total % P:
        raise RuntimeError("Input tensor size must be divisible by number of processes")
    B = total // P
    for i, o in zip(inputs, outputs):
        if i.numel() != total or i.dtype != dt:
            raise RuntimeError("all ranks must pass inputs of the same dtype and size")
        if o.numel() != B:
            raise RuntimeError("Output tensor must have block_size elements (input tensor numel()/world_size)")
        if o.dtype != dt:
            raise RuntimeError("Output tensor must be of type float (same dtype as the input)")
    need_work = _needs_work(m, P, algorithm)
    own_work = need_work and work is None
    if own_work:
        work = [torch.empty_like(inputs[r]) for r in range(P)]
    if work is not None:
        for w in work:
            check_device_tensor(w, "work")
            if w.numel() < total or w.dtype != dt:
                raise RuntimeError("work buffers must have the input's dtype and size")
    lib = _native.load()
    tables = (_native._ptr_table(_ptrs(outputs)), _native._ptr_table(_ptrs(inputs)),
              _native._ptr_table(_ptrs(work)) if need_work else None)
    args = (*tables, P, B, dtype_code(dt), algorithm.encode(), m)
    fn = lib._lib.pccl_hip_reduce_scatter_virtual
    if fn(*args, stream_handle()):
        raise _native.NativeError(lib.last_error())
    if not own_work:
        _plan_store(key, lib, fn, args, tables, outputs, inputs, () if work is None else work)


def _needs_work(m: int, P: int, algorithm: str) -> bool:
    """Whether pccl_hip_reduce_scatter_virtual wants work buffers: the faithful
    and per-step modes, and the fused halving order beyond the ranks of one
    launch (its first rounds run step by step)."""
    return ((m == MODE_FAITHFUL and P > 1) or (m == MODE_STEPS and P > 2)
            or (m == MODE_FUSED and P > MAX_RANKS and algorithm == "recursive"))


class CollectivePlan:
    """A collective on fixed buffers, validated once: calling the plan only
    makes the C call (no per-call checks, tables or allocations), which is what
    a launch-bound small-message loop wants.  The plan keeps its tensors alive."""

    def __init__(self, fn, args, keep):
        self._fn, self._args, self._keep = fn, args, keep

    def __call__(self):
        rc = self._fn(*self._args, stream_handle())
        if rc:
            raise _native.NativeError(_native.load().last_error())


def plan_reduce_scatter(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor],
                        algorithm: str = "ring", mode=None,
                        work: Optional[Sequence[torch.Tensor]] = None) -> CollectivePlan:
    """Validate like reduce_scatter_ranks, then return a callable that replays
    the collective on the same buffers."""
    P = len(inputs)
    m = mode_code(mode)
    total = inputs[0].numel()
    if _needs_work(m, P, algorithm):
        if work is None:
            work = [torch.empty_like(inputs[r]) for r in range(P)]
    else:
        work = None
    # one checked run; raises on any inconsistency
    reduce_scatter_ranks(outputs, inputs, algorithm, m, work)
    lib = _native.load()
    tabs = [_native._ptr_table(_ptrs(outputs)), _native._ptr_table(_ptrs(inputs)), _native._ptr_table(_ptrs(work))]
    args = (tabs[0], tabs[1], tabs[2], P, total // P, dtype_code(inputs[0].dtype), algorithm.encode(), m)
    return CollectivePlan(lib._lib.pccl_hip_reduce_scatter_virtual, args,
                          (list(outputs), list(inputs), None if work is None else list(work), tabs))


def plan_all_gather(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor],
                    algorithm: str = "recursive", mode=None) -> CollectivePlan:
    """Validate like all_gather_ranks, then return a callable that replays it."""
    m = mode_code(mode)
    all_gather_ranks(outputs, inputs, algorithm, m)
    lib = _native.load()
    tabs = [_native._ptr_table(_ptrs(outputs)), _native._ptr_table(_ptrs(inputs))]
    args = (tabs[0], tabs[1], len(inputs), inputs[0].numel() * inputs[0].element_size(), algorithm.encode(), m)
    return CollectivePlan(lib._lib.pccl_hip_all_gather_virtual, args, (list(outputs), list(inputs), tabs))


def all_gather_ranks(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor],
                     algorithm: str = "recursive", mode=None) -> None:
    """all_gather over P virtual ranks: outputs[r] = cat(inputs) for every r
    ('recursive': pccl/src/all_gather.cpp:15-69; 'ring': this build's schedule)."""
    P = len(inputs)
    if len(outputs) != P or P < 1:
        raise ValueError("need one output per input rank")
    m = mode_code(mode)
    key = ("ag", algorithm, m, *map(id, outputs), *map(id, inputs))
    if _plan_lookup(key, outputs, inputs):
        return
    if P > MAX_VIRTUAL_RANKS:
        raise RuntimeError(f"at most {MAX_VIRTUAL_RANKS} virtual ranks per communicator")
    for t in inputs:
        check_device_tensor(t, "input")
    for t in outputs:
        check_device_tensor(t, "output")
    _same_device(list(inputs) + list(outputs))
    blk = inputs[0].numel()
    dt = inputs[0].dtype
    for i, o in zip(inputs, outputs):
        if i.numel() != blk or i.dtype != dt:
            raise RuntimeError("all ranks must pass shards of the same dtype and size")
        if o.dtype != dt:
            raise RuntimeError("Input and output tensors must have the same dtype.")
        if o.numel() != blk * P:
            raise RuntimeError("Output tensor must have total_elem elements (input tensor numel() *world_size)")
    lib = _native.load()
    tables = (_native._ptr_table(_ptrs(outputs)), _native._ptr_table(_ptrs(inputs)))
    args = (*tables, P, blk * inputs[0].element_size(), algorithm.encode(), m)
    fn = lib._lib.pccl_hip_all_gather_virtual
    if fn(*args, stream_handle()):
        raise _native.NativeError(lib.last_error())
    _plan_store(key, lib, fn, args, tables, outputs, inputs)


# Distance added between the buffers of successive virtual ranks when they are
# carved from one allocation.  Many buffers of equal power-of-two size laid end
# to end put the same offset of every rank at a large power-of-two stride, the
# worst layout for the fused reduce on MI355X (a 64-rank ring fold of 1 GiB
# inputs: 5.2 TB/s at stride 1 GiB, 6.2-6.9 TB/s with 4 KiB ... 2 MiB more per
# rank; 32 ranks of 512 MiB: 5.7 against 6.4).  With 8 or 16 ranks the plain
# layout is as good or 2-3 % better, so this is for 32 ranks and more; 516 KiB
# was within 4 % of the best skew for every shape measured.
RANK_SKEW_BYTES = 516 * 1024


def rank_slab(P: int, numel, dtype: torch.dtype, device, skew_bytes: int = RANK_SKEW_BYTES) -> List[torch.Tensor]:
    """Buffers for P virtual ranks from ONE allocation: rank r's buffer of
    numel[r] (or numel) elements starts r * (longest buffer rounded up to
    256 bytes + skew_bytes) into it."""
    lens = [int(numel)] * P if isinstance(numel, int) else [int(n) for n in numel]
    if len(lens) != P or P < 1:
        raise ValueError("need one length per rank")
    if skew_bytes < 0 or skew_bytes % 256:
        raise ValueError("skew_bytes must be a non-negative multiple of 256")
    es = torch.empty(0, dtype=dtype).element_size()
    stride = (max(lens) * es + 255) // 256 * 256 + skew_bytes
    slab = torch.empty(P * stride, dtype=torch.uint8, device=device)
    return [slab[r * stride:r * stride + lens[r] * es].view(dtype) for r in range(P)]


def padded_offsets(nbytes: Sequence[int], align: int = 256) -> List[int]:
    """Byte offset of each shard when every shard is padded to `align` bytes."""
    off, out = 0, []
    for nb in nbytes:
        out.append(off)
        off += (nb + align - 1) // align * align
    return out


def all_gather_uneven_ranks(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor],
                            dst_off: Optional[Sequence[int]] = None, align: int = 256) -> List[int]:
    """all_gather of shards of different lengths: shard k lands at byte offset
    dst_off[k] (default: each shard padded to `align` bytes) of every output.
    Bytes between shards are left untouched.  Returns the offsets used.
    Not a reference feature (it requires equal shards, pccl/src/pccl.cpp:111-116)."""
    P = len(inputs)
    if len(outputs) != P or P < 1:
        raise ValueError("need one output per input rank")
    for t in inputs:
        check_device_tensor(t, "input")
    for t in outputs:
        check_device_tensor(t, "output")
    _same_device(list(inputs) + list(outputs))
    nbytes = [t.numel() * t.element_size() for t in inputs]
    if dst_off is None:
        dst_off = padded_offsets(nbytes, align)
    if len(dst_off) != P:
        raise ValueError("need one offset per shard")
    spans = sorted((int(o), int(o) + nb) for o, nb in zip(dst_off, nbytes))
    for (_, e0), (s1, _) in zip(spans, spans[1:]):
        if s1 < e0:
            raise RuntimeError("all_gather_uneven: shards overlap in the output")
    end = max((int(o) + nb for o, nb in zip(dst_off, nbytes)), default=0)
    for o in outputs:
        if o.numel() * o.element_size() < end:
            raise RuntimeError("all_gather_uneven: output too small for the shard layout")
    _native.load().all_gather_uneven_virtual(_ptrs(outputs), _ptrs(inputs), nbytes, list(dst_off),
                                             stream_handle())
    return list(dst_off)


# ---------------------------------------------------------------------------
# 2-D (hierarchical) collectives over intra*inter virtual ranks, world order
# ---------------------------------------------------------------------------

def _check_2d(outputs, inputs, intra, inter):
    W = intra * inter
    if intra < 1 or inter < 1 or len(inputs) != W or len(outputs) != W:
        raise ValueError("need intra*inter inputs and outputs, in world-rank order")
    if W > MAX_VIRTUAL_RANKS:
        raise RuntimeError(f"at most {MAX_VIRTUAL_RANKS} virtual ranks per 2-D grid")
    for t in inputs:
        check_device_tensor(t, "input")
    for t in outputs:
        check_device_tensor(t, "output")
    _same_device(list(inputs) + list(outputs))
    return W


def reduce_scatter_2d_ranks(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor], intra: int,
                            inter: int, algorithm: str = "recursive", mode=None) -> None:
    """reduce_scatter_2D for a whole grid of intra*inter virtual ranks (rank
    w = node*intra + local) in one call: the input permutation of
    pccl/reduce_scatter.py:226 is read in place by the first inner step, and one
    launch per step serves every inner (then every outer) group."""
    W = _check_2d(outputs, inputs, intra, inter)
    total, dt = inputs[0].numel(), inputs[0].dtype
    if total % W:
        raise RuntimeError("Input tensor size must be divisible by number of processes")
    m = total // W
    for i, o in zip(inputs, outputs):
        if i.numel() != total or i.dtype != dt:
            raise RuntimeError("all ranks must pass inputs of the same dtype and size")
        if o.numel() != m or o.dtype != dt:
            raise RuntimeError("Output tensor must have block_size elements (input tensor numel()/world_size)")
    code = mode_code(mode)
    if code == MODE_FAITHFUL:
        code = MODE_STEPS
    work = mid = None
    if code == MODE_FUSED and W > MAX_RANKS and max(intra, inter) > MAX_RANKS:
        code = MODE_STEPS                 # the fused mode folds at most MAX_RANKS ranks per level; same bits step by step
    if code == MODE_STEPS and (intra > 2 or inter > 2):
        work = [torch.empty_like(inputs[w]) for w in range(W)]
    # the intermediates between the levels: the per-step mode, and the fused mode beyond the shards of one
    # launch (one fold per node, then one per local rank)
    if (code == MODE_STEPS or W > MAX_RANKS) and intra > 1 and inter > 1:
        mid = [torch.empty(inter * m, dtype=dt, device=inputs[0].device) for _ in range(W)]
    _native.load().reduce_scatter_2d_virtual(_ptrs(outputs), _ptrs(inputs), _ptrs(work), _ptrs(mid), intra, inter,
                                             m, dtype_code(dt), algorithm, code, stream_handle())


def all_gather_2d_ranks(outputs: Sequence[torch.Tensor], inputs: Sequence[torch.Tensor], intra: int,
                        inter: int, algorithm: str = "recursive", mode=None) -> None:
    """all_gather_2D for a whole grid of intra*inter virtual ranks in one call;
    the inner stage writes through the un-permutation of pccl/all_gather.py:158-159."""
    W = _check_2d(outputs, inputs, intra, inter)
    n, dt = inputs[0].numel(), inputs[0].dtype
    for i, o in zip(inputs, outputs):
        if i.numel() != n or i.dtype != dt:
            raise RuntimeError("all ranks must pass shards of the same dtype and size")
        if o.dtype != dt:
            raise RuntimeError("Input and output tensors must have the same dtype.")
        if o.numel() != n * W:
            raise RuntimeError("Output tensor must have total_elem elements (input tensor numel() *world_size)")
    code = mode_code(mode)
    if code == MODE_FAITHFUL:
        code = MODE_STEPS
    mid = None
    if code == MODE_STEPS and intra > 1 and inter > 1:
        mid = [torch.empty(inter * n, dtype=dt, device=inputs[0].device) for _ in range(W)]
    _native.load().all_gather_2d_virtual(_ptrs(outputs), _ptrs(inputs), _ptrs(mid), intra, inter,
                                         n * inputs[0].element_size(), algorithm, code, stream_handle())
