"""Bounds check of every kernel without a GPU: the library source compiled for
the host with AddressSanitizer, driven over exact-size buffers."""
import glob
import os
import subprocess
import sys

import pytest

from conftest import EMUL_SO, HOST_CLANG, ROOT, build_cpu_library


def test_kernels_stay_in_bounds_under_address_sanitizer():
    runtimes = glob.glob("/opt/rocm/lib/llvm/lib/clang/*/lib/linux/libclang_rt.asan-x86_64.so")
    if not os.path.exists(HOST_CLANG) or not runtimes:
        pytest.skip("no host clang++ with a shared AddressSanitizer runtime")
    lib = build_cpu_library(out=EMUL_SO.replace(".so", "_asan.so"),
                            extra_flags=("-fsanitize=address", "-shared-libasan", "-fno-omit-frame-pointer"))
    env = dict(os.environ, LD_PRELOAD=runtimes[0], ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:exitcode=86")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "asan_check.py"), lib],
                       capture_output=True, text=True, env=env, timeout=900)
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-4000:])
    assert "ASAN CHECK OK" in p.stdout
