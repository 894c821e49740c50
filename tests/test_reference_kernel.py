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
    assert t_lib < t_ref, "the library's kernel must not be slower than the reference's"
