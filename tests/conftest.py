"""Shared fixtures.  Tests marked `gpu` need a real MI355X and call the HIP
library through its C ABI; everything else runs on the CPU."""
import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "sc2025-pccl-reproducer_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # without a GPU, skip GPU tests instead of failing in the first HIP call
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import pccl_oracle
    return pccl_oracle


@pytest.fixture(scope="session")
def liboracle():
    """The C restatement (oracle/pccl_oracle.c) through ctypes; built on demand."""
    path = os.path.join(ROOT, "oracle", "build", "liboracle.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    lib = ctypes.CDLL(path)
    vp, sz, i = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.oracle_ring_reduce_scatter.argtypes = [vp, vp, i, sz, i]
    lib.oracle_rh_reduce_scatter.argtypes = [vp, vp, i, sz, i]
    lib.oracle_rd_all_gather.argtypes = [vp, vp, i, sz]
    lib.oracle_ring_all_gather.argtypes = [vp, vp, i, sz]
    lib.oracle_vector_add.argtypes = [vp, vp, sz, i]
    lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
    return lib


CSRC = os.path.join(PKG_PARENT, "csrc")
EMUL_SO = os.path.join(ROOT, "tests", "build", "libpccl_hip_cpu.so")
HOST_CLANG = "/opt/rocm/lib/llvm/bin/clang++"


def build_cpu_library(out=EMUL_SO, extra_flags=(), opt="-O1"):
    """Compile the UNCHANGED library source for the host with the stand-in
    <hip/hip_runtime.h> of tests/hip_cpu_shim: each launch then runs the kernel
    thread by thread on the CPU.  Used to check indexing and the host-side
    schedules without a GPU; never loaded by the product package."""
    srcs = [os.path.join(CSRC, "pccl_hip.hip"), os.path.join(CSRC, "pccl_kernels.h"),
            os.path.join(ROOT, "include", "pccl_hip.h"),
            os.path.join(ROOT, "tests", "hip_cpu_shim", "hip", "hip_runtime.h")]
    if os.path.exists(out) and all(os.path.getmtime(out) >= os.path.getmtime(s) for s in srcs):
        return out
    if not os.path.exists(HOST_CLANG):
        pytest.skip("host clang++ of the ROCm toolchain not found")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    cmd = [HOST_CLANG, "-x", "c++", "-std=c++17", opt, "-g", "-fPIC", "-shared", *extra_flags,
           "-I", os.path.join(ROOT, "tests", "hip_cpu_shim"), "-I", os.path.join(ROOT, "include"),
           "-I", CSRC, "-o", out, srcs[0]]
    subprocess.run(cmd, check=True, capture_output=True)
    return out


class Target:
    """Where a parity test runs: the HIP library on cuda:0, or the CPU build of
    the same source on host memory."""

    def __init__(self, name, device, lib):
        self.name, self.device, self.native = name, device, lib

    def sync(self):
        if self.device != "cpu":
            import torch
            torch.cuda.synchronize()

    def stream(self):
        if self.device == "cpu":
            return 0
        import torch
        return torch.cuda.current_stream().cuda_stream


def _cpu_target(monkeypatch):
    from pccl import _native, kernels
    lib = _native.NativeLib(build_cpu_library())

    def check_host_tensor(t, name):
        if not t.is_contiguous():
            raise RuntimeError(f"{name} tensor must be contiguous.")

    monkeypatch.setattr(_native, "_loaded", lib)
    monkeypatch.setattr(kernels, "check_device_tensor", check_host_tensor)
    monkeypatch.setattr(kernels, "stream_handle", lambda: 0)
    return Target("cpu-build", "cpu", lib)


@pytest.fixture(params=[pytest.param("hip", marks=pytest.mark.gpu), "cpu-build"])
def target(request, monkeypatch):
    """Parity tests run twice: on the GPU through libpccl_hip.so (marked gpu),
    and on the CPU build of the same source (indexing and schedules)."""
    if request.param == "hip":
        from pccl import _native
        # the product library: must already be in the tree; missing = error, not skip
        return Target("hip", "cuda:0", _native.load())
    return _cpu_target(monkeypatch)


@pytest.fixture
def cpu(monkeypatch):
    """The CPU build only (host-logic tests)."""
    return _cpu_target(monkeypatch)
