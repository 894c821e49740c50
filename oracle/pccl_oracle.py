"""CPU oracle for the per-GPU compute of PCCL's collectives (numpy).

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module: it exists so that tests, the smoke check and the CPU-baseline leg of the
benchmark can compare the HIP kernels with an independent restatement of the
reference's algorithms.  It never touches a GPU.

Every function simulates P ranks in one process.  A rank owns its own numpy
buffers; an MPI_Sendrecv between ranks is modelled as "snapshot every send
buffer of the step, then deliver", which is what simultaneous blocking
Sendrecvs guarantee.  The schedules follow the reference line by line:

  vector_add                          pccl/src/common.cu:5-10 (fp32);
                                      torch.add on bf16 / fp16 tensors for the
                                      16-bit types (pccl/reduce_scatter.py:24,83,95,158)
  ring_reduce_scatter                 pccl/src/reduce_scatter.cpp:101-155,
                                      pccl/reduce_scatter.py:102-161
  recursive_halving_reduce_scatter    pccl/src/reduce_scatter.cpp:16-99,
                                      pccl/reduce_scatter.py:20-98
  recursive_doubling_all_gather       pccl/src/all_gather.cpp:15-69,
                                      pccl/all_gather.py:14-95
  ring_all_gather                     schedule defined by this build (the
                                      reference delegates to MPI_Allgather,
                                      pccl/all_gather.py:124-128); the result
                                      is the concatenation either way
  grid_groups                         pccl/process_groups.py:97-98,118,137
  reduce_scatter_2d / all_gather_2d   pccl/reduce_scatter.py:205-235,
                                      pccl/all_gather.py:136-159

Data types: "f32" arrays are numpy float32; "bf16" and "f16" arrays are numpy
uint16 holding the bfloat16 / binary16 bit patterns.

Pinning (see tests/test_oracle.py): the fp32 add is numpy's IEEE binary32 add;
the bf16 add is checked against torch's CPU bfloat16 add over every exponent
pair and against an independent integer rounding; the f16 add against torch's CPU
float16 add over all 65 536 patterns and against the exactly rounded float64 sum; the schedules are checked
against closed-form summation orders (left fold from rank j+1, XOR butterfly;
for the 2-D collectives the inner order inside every node, then the outer order
across the nodes), against exact integer sums, against P = 2 reducing to one add, against the C
restatement in pccl_oracle.c, and against the committed vectors in
tests/golden/.  The reference ships no golden vectors of its own.
"""
from __future__ import annotations

import numpy as np

F32 = "f32"
BF16 = "bf16"
F16 = "f16"


# --------------------------------------------------------------------------
# element arithmetic
# --------------------------------------------------------------------------

def bf16_to_f32(u: np.ndarray) -> np.ndarray:
    """Widen bfloat16 bit patterns (uint16) to float32: exact."""
    u = np.ascontiguousarray(u, dtype=np.uint16)
    return (u.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 to bfloat16 bit patterns, round-to-nearest-even.

    NaN maps to the canonical quiet NaN 0x7FC0, as c10::BFloat16 does on the
    host.  This is the rounding torch applies to the fp32 sum in torch.add on
    bfloat16 operands."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    rounded = ((bits + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    return np.where(np.isnan(x), np.uint16(0x7FC0), rounded).astype(np.uint16)


def f16_to_f32(u: np.ndarray) -> np.ndarray:
    """Widen binary16 bit patterns (uint16) to float32: exact."""
    return np.ascontiguousarray(u, dtype=np.uint16).view(np.float16).astype(np.float32)


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    """Round float32 to binary16 bit patterns, round-to-nearest-even (numpy's
    conversion; values beyond 65504 + half an ulp become infinity).  NaN maps to
    the canonical quiet NaN 0x7E00."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        h = x.astype(np.float16).view(np.uint16)
    return np.where(np.isnan(x), np.uint16(0x7E00), h).astype(np.uint16)


def vector_add(a: np.ndarray, b: np.ndarray, dtype: str) -> np.ndarray:
    """a[i] + b[i] in the arithmetic of `dtype` (one hop of any schedule).

    f32: one IEEE-754 binary32 RNE add (pccl/src/common.cu:8).
    bf16: RNE_bf16(float(a) + float(b)), the fp32 sum itself RNE.
    f16:  RNE_f16(float(a) + float(b)); binary32 has 24 >= 2*11+2 significand
          bits, so this is the correctly rounded binary16 sum."""
    if dtype == F32:
        with np.errstate(over="ignore", invalid="ignore"):
            return (np.asarray(a, np.float32) + np.asarray(b, np.float32)).astype(np.float32)
    if dtype == BF16:
        with np.errstate(over="ignore", invalid="ignore"):
            s = bf16_to_f32(a) + bf16_to_f32(b)
        return f32_to_bf16(s)
    if dtype == F16:
        with np.errstate(over="ignore", invalid="ignore"):
            s = f16_to_f32(a) + f16_to_f32(b)
        return f32_to_f16(s)
    raise ValueError(f"unknown dtype {dtype!r}")


def _check_inputs(inputs, dtype):
    P = len(inputs)
    if P < 1:
        raise ValueError("need at least one rank")
    want = np.float32 if dtype == F32 else np.uint16
    n = inputs[0].size
    for x in inputs:
        if x.dtype != want or x.ndim != 1 or x.size != n:
            raise ValueError("inputs must be equal-length 1-D arrays of the oracle dtype")
    return P, n


# --------------------------------------------------------------------------
# reduce_scatter
# --------------------------------------------------------------------------

def ring_reduce_scatter(inputs, dtype=F32):
    """Ring reduce_scatter over P simulated ranks.

    inputs[r]: rank r's P*B elements.  Returns outputs[r] (B elements).
    Per rank: buf = copy(input); for step in 0..P-2 send block
    (r-step-1) mod P to r+1, receive a block from r-1 into tmp, and
    buf[(r-step-2) mod P] += tmp; output = buf[r]
    (pccl/src/reduce_scatter.cpp:119-152)."""
    P, n = _check_inputs(inputs, dtype)
    if n % P:
        raise ValueError("Input tensor size must be divisible by number of processes")
    B = n // P
    buf = [x.copy().reshape(P, B) for x in inputs]
    for step in range(P - 1):
        # every rank posts its send block first ...
        sent = [buf[r][(r - step - 1) % P].copy() for r in range(P)]
        # ... and then reduces what its left neighbour sent
        for r in range(P):
            tmp = sent[(r - 1) % P]
            recv_idx = (r - step - 2) % P
            buf[r][recv_idx] = vector_add(buf[r][recv_idx], tmp, dtype)
    return [buf[r][r].copy() for r in range(P)]


def recursive_halving_reduce_scatter(inputs, dtype=F32):
    """Recursive-halving reduce_scatter, P a power of two.

    Round r: group = P >> r, half = current_blocks / 2, count = half * B.
    Ranks with (rank % group) < group/2 keep the lower half and add the
    partner's (rank + half) lower half to it; the others keep the upper half
    and add the partner's (rank - half) upper half
    (pccl/src/reduce_scatter.cpp:50-89).  Natural order: rank i ends with
    block i."""
    P, n = _check_inputs(inputs, dtype)
    if n % P:
        raise ValueError("Input tensor size must be divisible by number of processes")
    if P & (P - 1):
        raise ValueError("recursive halving needs a power-of-two number of ranks")
    B = n // P
    rounds = P.bit_length() - 1
    cur = [x.copy() for x in inputs]          # the active region of each rank
    blocks = P
    for r in range(rounds):
        group = P >> r
        half = blocks // 2
        count = half * B
        lower = [(k % group) < (group // 2) for k in range(P)]
        sent = [cur[k][count:2 * count].copy() if lower[k] else cur[k][:count].copy()
                for k in range(P)]
        nxt = []
        for k in range(P):
            if lower[k]:
                partner = (k + half) % P
                nxt.append(vector_add(cur[k][:count], sent[partner], dtype))
            else:
                partner = (k - half + P) % P
                nxt.append(vector_add(cur[k][count:2 * count], sent[partner], dtype))
        cur = nxt
        blocks = half
    return [c[:B].copy() for c in cur]


# --------------------------------------------------------------------------
# all_gather (typeless: works on bytes)
# --------------------------------------------------------------------------

def _as_bytes(x):
    return np.ascontiguousarray(x).view(np.uint8).reshape(-1)


def recursive_doubling_all_gather(inputs, fill=0xA5):
    """Recursive-doubling all_gather in bytes, P a power of two.

    out[r*blk:(r+1)*blk] = input; seg = 1; while seg < P: partner = r ^ seg,
    group_start = (r // (2 seg)) * 2 seg; the lower rank of the pair sends
    [group_start, +seg) and receives [group_start+seg, +seg), the upper rank
    the mirror image; seg *= 2 (pccl/src/all_gather.cpp:31-66).
    Returns the P outputs as uint8 arrays.  `fill` pre-fills the outputs so a
    byte that no step wrote is visible."""
    P = len(inputs)
    if P & (P - 1):
        raise ValueError("recursive doubling needs a power-of-two number of ranks")
    shards = [_as_bytes(x) for x in inputs]
    blk = shards[0].size
    if any(s.size != blk for s in shards):
        raise ValueError("shards must have equal size")
    out = [np.full(P * blk, fill, np.uint8) for _ in range(P)]
    for r in range(P):
        out[r][r * blk:(r + 1) * blk] = shards[r]
    seg = 1
    while seg < P:
        plan = []
        for r in range(P):
            partner = r ^ seg
            gs = (r // (2 * seg)) * (2 * seg)
            if r < partner:
                send_off, recv_off = gs * blk, (gs + seg) * blk
            else:
                send_off, recv_off = (gs + seg) * blk, gs * blk
            plan.append((partner, send_off, recv_off))
        cnt = seg * blk
        sent = [out[r][plan[r][1]:plan[r][1] + cnt].copy() for r in range(P)]
        for r in range(P):
            partner, _, recv_off = plan[r]
            out[r][recv_off:recv_off + cnt] = sent[partner]
        seg *= 2
    return out


def ring_all_gather(inputs, fill=0xA5):
    """Ring all_gather in bytes (any P): the mirror of the ring reduce_scatter.

    out[r] block r = input; step s = 0..P-2: rank r sends block (r - s) mod P
    to r+1 and receives block (r - s - 1) mod P from r-1."""
    P = len(inputs)
    shards = [_as_bytes(x) for x in inputs]
    blk = shards[0].size
    if any(s.size != blk for s in shards):
        raise ValueError("shards must have equal size")
    out = [np.full(P * blk, fill, np.uint8) for _ in range(P)]
    for r in range(P):
        out[r][r * blk:(r + 1) * blk] = shards[r]
    for s in range(P - 1):
        sent = []
        for r in range(P):
            j = (r - s) % P
            sent.append(out[r][j * blk:(j + 1) * blk].copy())
        for r in range(P):
            j = (r - s - 1) % P
            out[r][j * blk:(j + 1) * blk] = sent[(r - 1) % P]
    return out


def uneven_all_gather(inputs, dst_off, total_bytes, fill=0xA5):
    """Build-defined uneven all_gather: shard k (any byte length) lands at byte
    offset dst_off[k] of every rank's output; bytes outside the shards keep
    `fill`.  Not a reference feature (pccl/src/pccl.cpp:111-116 requires equal
    shards)."""
    P = len(inputs)
    shards = [_as_bytes(x) for x in inputs]
    out = [np.full(total_bytes, fill, np.uint8) for _ in range(P)]
    for r in range(P):
        for k in range(P):
            out[r][dst_off[k]:dst_off[k] + shards[k].size] = shards[k]
    return out


# --------------------------------------------------------------------------
# 2-D (hierarchical) collectives
# --------------------------------------------------------------------------

def grid_groups(world, intra, inter):
    """Group membership of ProcessGroups (pccl/process_groups.py:97-138).

    Returns (inner, outer): inner[rank] / outer[rank] are the lists of world
    ranks in that rank's inner / outer group, in group-rank order.  Built from
    the MPI colours: inner colour = rank // intra (:118); outer colour =
    rank % intra + (rank // (intra*inter)) * intra (:137); Split orders the
    members of one colour by world rank."""
    if world % (intra * inter):
        raise ValueError("world_size must be divisible by intra_group_size * inter_group_size")
    inner_colour = [r // intra for r in range(world)]
    outer_colour = [r % intra + (r // (intra * inter)) * intra for r in range(world)]
    inner = [[q for q in range(world) if inner_colour[q] == inner_colour[r]] for r in range(world)]
    outer = [[q for q in range(world) if outer_colour[q] == outer_colour[r]] for r in range(world)]
    return inner, outer


def block_transpose(x, rows, cols):
    """x.view(rows, cols, -1).transpose(0, 1).reshape(-1)."""
    return np.ascontiguousarray(x.reshape(rows, cols, -1).transpose(1, 0, 2)).reshape(-1)


def reduce_scatter_2d(inputs, intra, inter, dtype=F32, algorithm="recursive"):
    """reduce_scatter_2D over world = intra*inter ranks with both levels on the
    hand-written algorithm (`ring` or `recursive`), i.e. ProcessGroups with
    inner and outer backend "mpi" (pccl/reduce_scatter.py:205-235):
    permute input [inter, intra, m] -> [intra, inter, m]; reduce_scatter in the
    inner group; reduce_scatter of the intermediate in the outer group."""
    world = intra * inter
    if len(inputs) != world:
        raise ValueError("need intra*inter ranks")
    rs = ring_reduce_scatter if algorithm == "ring" else recursive_halving_reduce_scatter
    inner, outer = grid_groups(world, intra, inter)
    permuted = [block_transpose(x, inter, intra) for x in inputs]
    mid = [None] * world
    for r in range(world):
        g = inner[r]
        if g[0] == r:
            outs = rs([permuted[q] for q in g], dtype)
            for q, o in zip(g, outs):
                mid[q] = o
    out = [None] * world
    for r in range(world):
        g = outer[r]
        if g[0] == r:
            outs = rs([mid[q] for q in g], dtype)
            for q, o in zip(g, outs):
                out[q] = o
    return out


def all_gather_2d(inputs, intra, inter, algorithm="recursive"):
    """all_gather_2D over world = intra*inter ranks (pccl/all_gather.py:136-159):
    all_gather in the outer group, all_gather of the intermediate in the inner
    group, then the un-permute [intra, inter, m] -> [inter, intra, m].
    Returns uint8 arrays."""
    world = intra * inter
    if len(inputs) != world:
        raise ValueError("need intra*inter ranks")
    ag = ring_all_gather if algorithm == "ring" else recursive_doubling_all_gather
    inner, outer = grid_groups(world, intra, inter)
    mid = [None] * world
    for r in range(world):
        g = outer[r]
        if g[0] == r:
            outs = ag([inputs[q] for q in g])
            for q, o in zip(g, outs):
                mid[q] = o
    out = [None] * world
    for r in range(world):
        g = inner[r]
        if g[0] == r:
            outs = ag([mid[q] for q in g])
            for q, o in zip(g, outs):
                out[q] = block_transpose(o, intra, inter)
    return out


def all_reduce(inputs, dtype=F32, algorithm="recursive"):
    """all_reduce = reduce_scatter followed by all_gather of the result blocks
    (pccl/src/yacl.cpp:146-177).  Returns one array per rank."""
    rs = ring_reduce_scatter if algorithm == "ring" else recursive_halving_reduce_scatter
    ag = ring_all_gather if algorithm == "ring" else recursive_doubling_all_gather
    blocks = rs(inputs, dtype)
    gathered = ag(blocks)
    want = np.float32 if dtype == F32 else np.uint16
    return [g.view(want).copy() for g in gathered]
