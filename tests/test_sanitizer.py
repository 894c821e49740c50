"""Bounds and undefined-behaviour check of every kernel without a GPU: the
library source compiled for the host with AddressSanitizer and
UndefinedBehaviorSanitizer (one unoptimised build with both, which compiles in
a third of the time of two optimised ones), driven over exact-size buffers."""
import glob
import os
import subprocess
import sys

import pytest

from conftest import EMUL_SO, HOST_CLANG, ROOT, build_cpu_library


@pytest.fixture(scope="module")
def sanitizer_run():
    runtimes = glob.glob("/opt/rocm/lib/llvm/lib/clang/*/lib/linux/libclang_rt.asan-x86_64.so")
    if not os.path.exists(HOST_CLANG) or not runtimes:
        pytest.skip("no host clang++ with a shared AddressSanitizer runtime")
    lib = build_cpu_library(out=EMUL_SO.replace(".so", "_san.so"), opt="-O0",
                            extra_flags=("-fsanitize=address,undefined", "-fno-sanitize=vptr", "-shared-libsan",
                                         "-fno-omit-frame-pointer"))
    env = dict(os.environ, LD_PRELOAD=runtimes[0], ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:exitcode=86",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=0")
    return subprocess.run([sys.executable, os.path.join(ROOT, "tests", "asan_check.py"), lib],
                          capture_output=True, text=True, env=env, timeout=900)


def test_kernels_stay_in_bounds_under_address_sanitizer(sanitizer_run):
    p = sanitizer_run
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-4000:])
    assert "AddressSanitizer" not in p.stderr, p.stderr[-4000:]
    assert "ASAN CHECK OK" in p.stdout


def test_kernels_show_no_undefined_behaviour(sanitizer_run):
    """Misaligned vector accesses, shifts and integer overflow in the index
    arithmetic would print a runtime error."""
    p = sanitizer_run
    assert "runtime error" not in p.stderr, p.stderr[-4000:]
    assert "ASAN CHECK OK" in p.stdout
