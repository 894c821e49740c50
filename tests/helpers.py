"""Test helpers: seeded inputs, torch <-> oracle conversions, closed forms."""
import numpy as np

from oracle import pccl_oracle as O


def make_inputs(P, n, dtype, seed=0, dist="normal", scale=1.0):
    """P arrays of n elements in oracle representation (f32 -> float32,
    bf16 -> uint16 bit patterns); rank r uses seed + r."""
    out = []
    for r in range(P):
        rng = np.random.default_rng(seed + r)
        if dist == "normal":
            x = rng.standard_normal(n, dtype=np.float32) * np.float32(scale)
        elif dist == "uniform":
            x = (rng.random(n, dtype=np.float32) * 2 - 1) * np.float32(scale)
        elif dist == "int":      # small integers: every summation order is exact
            x = rng.integers(-8, 9, n).astype(np.float32)
        else:
            raise ValueError(dist)
        out.append(x if dtype == O.F32 else O.f32_to_bf16(x) if dtype == O.BF16 else O.f32_to_f16(x))
    return out


def to_torch(x, dtype, device):
    import torch
    x = np.array(x, copy=True)            # never share memory with the oracle's inputs
    if dtype == O.F32:
        return torch.from_numpy(x).to(device)
    return torch.from_numpy(x.view(np.int16)).to(device).view(torch.bfloat16 if dtype == O.BF16 else torch.float16)


def to_numpy(t, dtype):
    import torch
    if dtype == O.F32:
        return t.detach().cpu().numpy()
    return t.detach().view(torch.int16).cpu().numpy().view(np.uint16)


def bits(x):
    return np.ascontiguousarray(x).view(np.uint8)


def assert_bits_equal(got, want, what=""):
    g, w = bits(got), bits(want)
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    if not np.array_equal(g, w):
        bad = np.flatnonzero(g != w)
        raise AssertionError(f"{what}: {bad.size} differing bytes, first at byte {bad[0]}")


# ---- closed forms, written independently of the oracle's simulations -------

def ring_closed_form(inputs, dtype):
    """Block j = ((x_{j+1} + x_{j+2}) + ...) + x_j, indices mod P: the left fold
    in rank order that the ring performs on block j."""
    P = len(inputs)
    B = inputs[0].size // P
    outs = []
    for j in range(P):
        acc = inputs[(j + 1) % P][j * B:(j + 1) * B]
        for t in range(2, P + 1):
            acc = O.vector_add(acc, inputs[(j + t) % P][j * B:(j + 1) * B], dtype)
        outs.append(np.array(acc, copy=True))
    return outs


def halving_closed_form(inputs, dtype):
    """Block j = T_L(j)[j] with T_0(k) = x_k, T_{t+1}(k) = T_t(k) + T_t(k ^ (P >> (t+1)))."""
    P = len(inputs)
    B = inputs[0].size // P
    L = P.bit_length() - 1
    outs = []
    for j in range(P):
        T = [inputs[k][j * B:(j + 1) * B] for k in range(P)]
        for t in range(L):
            d = P >> (t + 1)
            T = [O.vector_add(T[k], T[k ^ d], dtype) for k in range(P)]
        outs.append(np.array(T[j], copy=True))
    return outs


def _fold_in_schedule_order(xs, j, algorithm, dtype):
    """What block j of a reduce_scatter over len(xs) ranks holds when rank k
    contributed xs[k]: the ring's left fold from rank j+1, or the XOR butterfly."""
    P = len(xs)
    if algorithm == "ring":
        acc = xs[(j + 1) % P]
        for t in range(2, P + 1):
            acc = O.vector_add(acc, xs[(j + t) % P], dtype)
        return np.array(acc, copy=True)
    T = list(xs)
    for t in range(P.bit_length() - 1):
        d = P >> (t + 1)
        T = [O.vector_add(T[k], T[k ^ d], dtype) for k in range(P)]
    return np.array(T[j], copy=True)


def grid_closed_form(inputs, intra, inter, dtype, algorithm):
    """reduce_scatter_2D in closed form: world rank w = node * intra + local ends
    with block w of the total, summed first over the locals of every node in the
    inner schedule's order for block `local`, then over the nodes in the outer
    schedule's order for block `node`."""
    W = intra * inter
    m = inputs[0].size // W
    outs = []
    for w in range(W):
        node, local = divmod(w, intra)
        per_node = [_fold_in_schedule_order([inputs[n * intra + l][w * m:(w + 1) * m] for l in range(intra)],
                                            local, algorithm, dtype) for n in range(inter)]
        outs.append(_fold_in_schedule_order(per_node, node, algorithm, dtype))
    return outs

