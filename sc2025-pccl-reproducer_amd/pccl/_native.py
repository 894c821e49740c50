"""ctypes binding of libpccl_hip.so (C ABI: include/pccl_hip.h).

This is the Python side of the boundary that the reference crosses with
`import pccl as pccl_cpp` into its JIT-built pybind11 module
(pccl/reduce_scatter.py:185, pccl/all_gather.py:116, pccl/src/pccl.cpp:145-148).
Everything here works on plain integers (device addresses, sizes, a stream
handle); torch never appears, so the same class binds any build of the library.

There is no fallback: if the shared library is missing, `load()` raises.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional, Sequence

F32 = 0
BF16 = 1
F16 = 2

ORDER_RING = 0
ORDER_HALVING = 1

MODE_STEPS = 0
MODE_FUSED = 1
MODE_FAITHFUL = 2

MAX_RANKS = 64            # segments / shards of one launch
MAX_VIRTUAL_RANKS = 4096  # per-step modes of the 1-D collectives
NOALLOC_SCRATCH_BYTES = 32 << 20   # built-in work space of reduce_scatter_virtual_noalloc
ABI_VERSION = 1

LIB_NAME = "libpccl_hip.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

_vp = ctypes.c_void_p
_sz = ctypes.c_size_t
_int = ctypes.c_int
_vpp = ctypes.POINTER(ctypes.c_void_p)
_szp = ctypes.POINTER(ctypes.c_size_t)

# name -> (restype, argtypes); must list every symbol include/pccl_hip.h declares
SIGNATURES = {
    "pccl_hip_version": (_int, []),
    "pccl_hip_last_error": (ctypes.c_char_p, []),
    "pccl_hip_dtype_size": (_sz, [_int]),
    "pccl_hip_accumulate": (_int, [_vp, _vp, _sz, _int, _vp]),
    "pccl_hip_add": (_int, [_vp, _vp, _vp, _sz, _int, _vp]),
    "pccl_hip_add_batched": (_int, [_vpp, _vpp, _vpp, _int, _sz, _int, _vp]),
    "pccl_hip_rh_round": (_int, [_vpp, _vpp, _vpp, _int, _sz, _int, _int, _vp]),
    "pccl_hip_reduce_kway": (_int, [_vp, _vpp, _int, _sz, _int, _int, _int, _int, _vp]),
    "pccl_hip_copy_batched": (_int, [_vpp, _vpp, _szp, _int, _vp]),
    "pccl_hip_gather_place": (_int, [_vp, _vpp, _szp, _szp, _int, _vp]),
    "pccl_hip_block_transpose": (_int, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "pccl_hip_reduce_scatter_virtual": (_int, [_vpp, _vpp, _vpp, _int, _sz, _int, ctypes.c_char_p, _int, _vp]),
    "pccl_hip_reduce_scatter_virtual_noalloc": (_int, [_vpp, _vpp, _int, _sz, _int, ctypes.c_char_p, _vp]),
    "pccl_hip_all_gather_virtual": (_int, [_vpp, _vpp, _int, _sz, ctypes.c_char_p, _int, _vp]),
    "pccl_hip_all_gather_uneven_virtual": (_int, [_vpp, _vpp, _szp, _szp, _int, _vp]),
    "pccl_hip_reduce_scatter_2d_virtual": (_int, [_vpp, _vpp, _vpp, _vpp, _int, _int, _sz, _int, ctypes.c_char_p,
                                                  _int, _vp]),
    "pccl_hip_all_gather_2d_virtual": (_int, [_vpp, _vpp, _vpp, _int, _int, _sz, ctypes.c_char_p, _int, _vp]),
    "pccl_hip_probe_stream": (_int, [_int, _vp, _sz, _vp]),
    "pccl_hip_probe_mix": (_int, [_vpp, _int, _vpp, _int, _sz, _int, _int, _vp]),
    "pccl_hip_set_tuning": (_int, [ctypes.c_char_p, ctypes.c_long]),
    "pccl_hip_get_tuning": (ctypes.c_long, [ctypes.c_char_p]),
    "pccl_hip_launch_count": (ctypes.c_ulonglong, []),
}


def _ptr_table(addrs: Optional[Sequence[int]]):
    if addrs is None:
        return None
    return (ctypes.c_void_p * len(addrs))(*[int(a) if a else None for a in addrs])


def _size_table(vals: Sequence[int]):
    return (ctypes.c_size_t * len(vals))(*[int(v) for v in vals])


class NativeError(RuntimeError):
    """A call into libpccl_hip.so returned a failure code."""


class NativeLib:
    """One loaded build of the C-ABI library."""

    def __init__(self, path: str = LIB_PATH):
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} not found: the HIP library has not been built. "
                "Run `make -C sc2025-pccl-reproducer_amd/csrc` (or pccl.build_kernels.build()) first; "
                "there is no fallback implementation.")
        self.path = path
        self._lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self._lib, name)   # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        got = self._lib.pccl_hip_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{path}: ABI version {got}, this package needs {ABI_VERSION}")

    # -- helpers ---------------------------------------------------------
    def _check(self, rc: int):
        if rc != 0:
            msg = self._lib.pccl_hip_last_error().decode("utf-8", "replace")
            raise NativeError(msg or f"libpccl_hip error {rc}")

    def last_error(self) -> str:
        return self._lib.pccl_hip_last_error().decode("utf-8", "replace")

    def version(self) -> int:
        return self._lib.pccl_hip_version()

    def dtype_size(self, dtype: int) -> int:
        return self._lib.pccl_hip_dtype_size(dtype)

    def set_tuning(self, key: str, value: int):
        self._check(self._lib.pccl_hip_set_tuning(key.encode(), int(value)))

    def launch_count(self) -> int:
        return int(self._lib.pccl_hip_launch_count())

    def get_tuning(self, key: str) -> int:
        return self._lib.pccl_hip_get_tuning(key.encode())

    # -- kernels (addresses are ints) --------------------------------------
    def accumulate(self, dst, src, n, dtype, stream=0):
        self._check(self._lib.pccl_hip_accumulate(dst, src, n, dtype, stream))

    def add(self, dst, a, b, n, dtype, stream=0):
        self._check(self._lib.pccl_hip_add(dst, a, b, n, dtype, stream))

    def add_batched(self, dst, a, b, n, dtype, stream=0):
        if not (len(dst) == len(a) == len(b)):
            raise ValueError("dst, a, b must have the same number of segments")
        self._check(self._lib.pccl_hip_add_batched(_ptr_table(dst), _ptr_table(a), _ptr_table(b),
                                                   len(dst), n, dtype, stream))

    def rh_round(self, bufs, src, outs, P, B, rnd, dtype, stream=0):
        self._check(self._lib.pccl_hip_rh_round(_ptr_table(bufs), _ptr_table(src), _ptr_table(outs),
                                                P, B, rnd, dtype, stream))

    def reduce_kway(self, out, shards, n, dtype, order=ORDER_RING, first=0, per_hop_round=True, stream=0):
        self._check(self._lib.pccl_hip_reduce_kway(out, _ptr_table(shards), len(shards), n, dtype, order,
                                                   first, 1 if per_hop_round else 0, stream))

    def copy_batched(self, dst, src, nbytes, stream=0):
        if not (len(dst) == len(src) == len(nbytes)):
            raise ValueError("dst, src, nbytes must have the same number of segments")
        self._check(self._lib.pccl_hip_copy_batched(_ptr_table(dst), _ptr_table(src), _size_table(nbytes),
                                                    len(dst), stream))

    def gather_place(self, out, shards, nbytes, dst_off, stream=0):
        self._check(self._lib.pccl_hip_gather_place(out, _ptr_table(shards), _size_table(nbytes),
                                                    _size_table(dst_off), len(shards), stream))

    def block_transpose(self, dst, src, rows, cols, m_bytes, stream=0):
        self._check(self._lib.pccl_hip_block_transpose(dst, src, rows, cols, m_bytes, stream))

    def reduce_scatter_virtual(self, outputs, inputs, work, B, dtype, algorithm, mode=MODE_STEPS, stream=0):
        P = len(inputs)
        self._check(self._lib.pccl_hip_reduce_scatter_virtual(
            _ptr_table(outputs), _ptr_table(inputs), _ptr_table(work), P, B, dtype,
            algorithm.encode(), mode, stream))

    def reduce_scatter_virtual_noalloc(self, outputs, inputs, B, dtype, algorithm, stream=0):
        """Per-step reduce_scatter whose work buffers are the library's built-in scratch."""
        self._check(self._lib.pccl_hip_reduce_scatter_virtual_noalloc(
            _ptr_table(outputs), _ptr_table(inputs), len(inputs), B, dtype, algorithm.encode(), stream))

    def all_gather_virtual(self, outputs, inputs, block_bytes, algorithm, mode=MODE_STEPS, stream=0):
        P = len(inputs)
        self._check(self._lib.pccl_hip_all_gather_virtual(
            _ptr_table(outputs), _ptr_table(inputs), P, block_bytes, algorithm.encode(), mode, stream))

    def all_gather_uneven_virtual(self, outputs, inputs, nbytes, dst_off, stream=0):
        P = len(inputs)
        self._check(self._lib.pccl_hip_all_gather_uneven_virtual(
            _ptr_table(outputs), _ptr_table(inputs), _size_table(nbytes), _size_table(dst_off), P, stream))


    def reduce_scatter_2d_virtual(self, outputs, inputs, work, mid, intra, inter, m, dtype, algorithm,
                                  mode=MODE_STEPS, stream=0):
        self._check(self._lib.pccl_hip_reduce_scatter_2d_virtual(
            _ptr_table(outputs), _ptr_table(inputs), _ptr_table(work), _ptr_table(mid), intra, inter, m, dtype,
            algorithm.encode(), mode, stream))

    def all_gather_2d_virtual(self, outputs, inputs, mid, intra, inter, block_bytes, algorithm,
                              mode=MODE_STEPS, stream=0):
        self._check(self._lib.pccl_hip_all_gather_2d_virtual(
            _ptr_table(outputs), _ptr_table(inputs), _ptr_table(mid), intra, inter, block_bytes,
            algorithm.encode(), mode, stream))


    def probe_stream(self, kind, buf, nbytes, stream=0):
        self._check(self._lib.pccl_hip_probe_stream(kind, buf, nbytes, stream))


    def probe_mix(self, reads, writes, nbytes, shape=0, vectors=4, stream=0):
        self._check(self._lib.pccl_hip_probe_mix(_ptr_table(reads) if reads else None, len(reads),
                                                 _ptr_table(writes) if writes else None, len(writes), nbytes,
                                                 shape, vectors, stream))


_lock = threading.Lock()
_loaded: Optional[NativeLib] = None


def load() -> NativeLib:
    """The process-wide library instance; raises if it has not been built."""
    global _loaded
    with _lock:
        if _loaded is None:
            _loaded = NativeLib(LIB_PATH)
        return _loaded


def is_built() -> bool:
    return os.path.exists(LIB_PATH)
