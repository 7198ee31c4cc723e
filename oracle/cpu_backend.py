"""Backend object that runs kernel descriptors on the CPU oracle.

TEST INFRASTRUCTURE ONLY: it lets the same graphs that run on the GPU through
`descent_amd.Environment` run on `liboracle.so` for comparison.  Buffers are
numpy arrays; `Environment` drives it kernel by kernel with the reference's
buffer-lifetime algorithm (it offers no `make_schedule`).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

from descent_amd import _abi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.orc_run_kernel.restype = C.c_int
        _lib.orc_run_kernel.argtypes = [C.POINTER(_abi.CKernelDesc), C.POINTER(C.c_void_p), C.c_int, C.c_uint32]
        _lib.orc_pcg.restype = C.c_uint32
        _lib.orc_pcg.argtypes = [C.c_uint32]
        _lib.orc_rand_from_index.restype = C.c_float
        _lib.orc_rand_from_index.argtypes = [C.c_uint32, C.c_int32, C.c_uint32]
        _lib.orc_load_index.restype = C.c_int64
        _lib.orc_load_index.argtypes = [C.POINTER(_abi.CView), C.POINTER(C.c_int64)]
    return _lib


def run_kernel(kernel, arrays, rand_seed: int = 0) -> None:
    """Run one descriptor on float32 numpy arrays bound inputs-then-outputs."""
    mk = _abi.MarshalledKernel(kernel)
    for a in arrays:
        assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    ptrs = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    rc = lib().orc_run_kernel(C.byref(mk.desc), ptrs, len(arrays), rand_seed & 0xFFFFFFFF)
    if rc != 0:
        raise ValueError(f"oracle rejected kernel {kernel.label_name()}")


def load_index(view, coord) -> int:
    cv = _abi.c_view(view)
    cc = (C.c_int64 * 7)(*coord)
    return lib().orc_load_index(C.byref(cv), cc)


class CpuBackend:
    def __init__(self):
        lib()
        self.launches = []  # labels, in launch order

    def alloc(self, nbytes: int):
        return np.empty(max(1, nbytes // 4), dtype=np.float32)

    def free(self, handle) -> None:
        pass

    def write(self, handle, offset: int, data) -> None:
        raw = handle.view(np.uint8)
        data = np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data.view(np.uint8)
        raw[offset : offset + data.size] = data.reshape(-1)

    def fill_zero(self, handle, offset: int, nbytes: int) -> None:
        handle.view(np.uint8)[offset : offset + nbytes] = 0

    def read(self, handle, offset: int, nbytes: int) -> bytes:
        return handle.view(np.uint8)[offset : offset + nbytes].tobytes()

    def launch(self, kernel, handles, rand_seed: int) -> None:
        self.launches.append(kernel.label_name())
        run_kernel(kernel, handles, rand_seed)

    def sync(self) -> None:
        pass
