"""The reference's own vectorAdd (pccl/src/common.hip, compiled for gfx950 into
oracle/_ref by `make -C oracle ref`) run beside the library's accumulate on the
same GPU: same bits, and what each sustains."""
import ctypes
import os

import numpy as np
import pytest

from conftest import ROOT

REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libref_common.so")
# void vectorAdd(float* a, const float* b, int n, hipStream_t stream)   (pccl/include/common_hip.h:21)
REF_SYMBOL = "_Z9vectorAddPfPKfiP12ihipStream_t"

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ref_vector_add():
    if not os.path.exists(REF_LIB):
        pytest.skip("oracle/_ref/libref_common.so not built (the reference was not mounted at build time)")
    fn = getattr(ctypes.CDLL(REF_LIB), REF_SYMBOL)
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    return fn


@pytest.mark.parametrize("n", [1, 255, 256, 257, 4099, (1 << 20) + 3])
def test_accumulate_equals_the_references_kernel(ref_vector_add, n):
    """pccl_hip_accumulate (fp32) and the reference's vectorAddKernel
    (pccl/src/common.hip:7-21) give the same bits, special values included."""
    import torch
    from pccl import kernels
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 2 ** -24], np.float32)
    k = min(n, specials.size * specials.size)
    a[:k] = np.repeat(specials, specials.size)[:k]
    b[:k] = np.tile(specials, specials.size)[:k]
    dev = torch.device("cuda", 0)
    mine, theirs = torch.from_numpy(a).to(dev), torch.from_numpy(a).to(dev)
    tb = torch.from_numpy(b).to(dev)
    stream = torch.cuda.current_stream().cuda_stream
    kernels.accumulate(mine, tb)
    ref_vector_add(theirs.data_ptr(), tb.data_ptr(), n, stream)
    torch.cuda.synchronize()
    assert torch.equal(mine.view(torch.int32), theirs.view(torch.int32))


def test_throughput_beside_the_references_kernel(ref_vector_add, capsys):
    """The same 256 MiB fp32 accumulate through both kernels, 20 timed calls
    each after 5 warm-ups (the reference's timing convention)."""
    import torch
    from pccl import kernels
    dev = torch.device("cuda", 0)
    n = 64 << 20
    a = torch.randn(n, device=dev)
    b = torch.randn(n, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(20):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / 20

    t_ref = timed(lambda: ref_vector_add(a.data_ptr(), b.data_ptr(), n, stream))
    t_lib = timed(lambda: kernels.accumulate(a, b))
    gbs = lambda ms: 3 * n * 4 / ms / 1e6
    with capsys.disabled():
        print(f"\n256 MiB fp32 accumulate on this GPU: reference vectorAddKernel {t_ref:.4f} ms = {gbs(t_ref):.0f} GB/s, "
              f"pccl_hip_accumulate {t_lib:.4f} ms = {gbs(t_lib):.0f} GB/s", flush=True)
    # a loose sanity bound only: the throughput claim belongs to bench.py, not to a correctness suite
    assert t_lib < 1.5 * t_ref, "the library's kernel is far slower than the reference's one-element-per-thread kernel"


NAN_PATTERNS = np.array([0x7FC00001, 0xFFC00002, 0x7F800003, 0xFF800004, 0x7FE12345, 0x7FC00000, 0xFFFFFFFF,
                         0x3F800000, 0x7F800000, 0xFF800000, 0x00000000], dtype=np.uint32)


def _nan_operands(k, n, seed):
    """k operands of n fp32 values: every ordered pair of the patterns above in
    operands 0 and 1, random draws of them (one in four) among ordinary values
    elsewhere, so that NaNs of different payloads meet at every hop."""
    rng = np.random.default_rng(seed)
    ops = []
    for q in range(k):
        x = rng.standard_normal(n).astype(np.float32).view(np.uint32)
        pick = rng.random(n) < 0.25
        x[pick] = rng.choice(NAN_PATTERNS, int(pick.sum()))
        ops.append(x)
    m = NAN_PATTERNS.size
    ops[0][:m * m] = np.repeat(NAN_PATTERNS, m)
    ops[1][:m * m] = np.tile(NAN_PATTERNS, m)
    return ops


def _dev(x):
    import torch
    return torch.from_numpy(x.view(np.int32).copy()).to("cuda:0")


def _bits(t):
    return t.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("n", [121, 4096 + 121])
def test_two_nans_keep_the_payload_the_references_kernel_keeps(ref_vector_add, n):
    """a[i] = a[i] + b[i] with BOTH operands NaN: IEEE 754 leaves the surviving
    payload open, the reference's compiled kernel keeps b's.  accumulate and the
    three-address add (scalar and vector paths) give the same bits."""
    import torch
    from pccl import _native
    lib = _native.load()
    a, b = _nan_operands(2, n, 5)
    st = torch.cuda.current_stream().cuda_stream
    theirs, tb = _dev(a), _dev(b)
    ref_vector_add(theirs.data_ptr(), tb.data_ptr(), n, st)
    mine = _dev(a)
    lib.accumulate(mine.data_ptr(), tb.data_ptr(), n, _native.F32, st)
    ta, three = _dev(a), _dev(np.zeros_like(a))
    lib.add(three.data_ptr(), ta.data_ptr(), tb.data_ptr(), n, _native.F32, st)
    torch.cuda.synchronize()
    want = _bits(theirs)
    both = np.isnan(a.view(np.float32)) & np.isnan(b.view(np.float32)) & (a != b)
    assert both.sum() >= 30                               # the case in question is really there
    assert np.array_equal(_bits(mine), want)
    assert np.array_equal(_bits(three), want)


@pytest.mark.parametrize("P", [4, 8, 16])
def test_ring_order_with_nans_equals_hops_of_the_references_kernel(ref_vector_add, P):
    """Block j of a ring reduce_scatter rebuilt hop by hop with the reference's
    own kernel -- rank j+t adds the running sum it received into a copy of its
    block, vectorAdd(own, received), pccl/src/reduce_scatter.cpp:145 -- against
    the per-step and the fused mode of the library: same bits, NaN payloads
    included (which the CPU oracle cannot pin: a host add keeps other payloads)."""
    import torch
    from pccl import kernels
    B = 1000
    ins = _nan_operands(P, P * B, 40 + P)
    t_in = [_dev(x).view(torch.float32) for x in ins]
    st = torch.cuda.current_stream().cuda_stream
    want = []
    for j in range(P):
        running = t_in[(j + 1) % P][j * B:(j + 1) * B].clone()
        for t in range(2, P + 1):
            own = t_in[(j + t) % P][j * B:(j + 1) * B].clone()
            ref_vector_add(own.data_ptr(), running.data_ptr(), B, st)
            running = own
        want.append(running)
    for mode in ("steps", "fused", "faithful"):
        outs = [torch.zeros(B, device="cuda:0") for _ in range(P)]
        kernels.reduce_scatter_ranks(outs, t_in, "ring", mode)
        torch.cuda.synchronize()
        for j in range(P):
            assert np.array_equal(_bits(outs[j].view(torch.int32)), _bits(want[j].view(torch.int32))), (mode, j)


@pytest.mark.parametrize("P", [4, 8, 16, 32, 64])
def test_halving_order_with_nans_equals_rounds_of_the_references_kernel(ref_vector_add, P):
    """Recursive halving rebuilt with the reference's kernel: in every round a
    rank adds its partner's half into its own, vectorAdd(own, received)
    (pccl/src/reduce_scatter.cpp:71,84-85); per-step and fused mode agree with
    it bit for bit, NaN payloads included."""
    import torch
    from pccl import kernels
    B = 300 if P <= 16 else 40
    ins = _nan_operands(P, P * B, 70 + P)
    t_in = [_dev(x).view(torch.float32) for x in ins]
    st = torch.cuda.current_stream().cuda_stream
    bufs = [t.clone() for t in t_in]
    group = P
    while group > 1:
        half = group // 2
        count = half * B
        old = [b.clone() for b in bufs]                     # what every rank sends this round
        for r in range(P):
            lower = (r % group) < half
            partner = r + half if lower else r - half
            off = (r // group) * group * B + (0 if lower else count)
            own = bufs[r][off:off + count]
            ref_vector_add(own.data_ptr(), old[partner][off:off + count].data_ptr(), count, st)
        group = half
    for mode in ("steps", "fused", "faithful"):
        outs = [torch.zeros(B, device="cuda:0") for _ in range(P)]
        kernels.reduce_scatter_ranks(outs, t_in, "recursive", mode)
        torch.cuda.synchronize()
        for r in range(P):
            assert np.array_equal(_bits(outs[r].view(torch.int32)), _bits(bufs[r][r * B:(r + 1) * B].view(torch.int32))), (mode, r)
