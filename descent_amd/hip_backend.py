"""ctypes binding of libdescent_hip.so (the C ABI in include/descent_hip.h) and
the backend object `Environment` drives.

There is no CPU fallback: if the library is missing, or no gfx950 device is
present, constructing `HipBackend` raises.
"""
from __future__ import annotations

import ctypes as C
import weakref
import os
from typing import List

import numpy as np

from . import _abi

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libdescent_hip.so")

_lib = None


class DescentHipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"descent_hip error {status} ({_abi.STATUS_NAMES[status] if 0 <= status < 7 else '?'}): {message}")
        self.status = status


def lib():
    """Loads the built library; raises if it has not been built (python -m descent_amd.csrc.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python {os.path.join(_CSRC, 'build.py')}` "
            "(there is no CPU fallback for the HIP backend)"
        )
    L = C.CDLL(LIB_PATH)
    vp, u64, sz, i32, u32 = C.c_void_p, C.c_uint64, C.c_size_t, C.c_int32, C.c_uint32
    sig = {
        "dsc_last_error": (C.c_char_p, []),
        "dsc_ctx_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
        "dsc_ctx_destroy": (C.c_int, [vp]),
        "dsc_ctx_caps": (C.c_int, [vp, C.POINTER(_abi.CCaps)]),
        "dsc_ctx_sync": (C.c_int, [vp]),
        "dsc_ctx_stream": (C.c_int, [vp, C.POINTER(vp)]),
        "dsc_fence_record": (C.c_int, [vp, C.POINTER(u64)]),
        "dsc_fence_wait": (C.c_int, [vp, u64]),
        "dsc_fence_query": (C.c_int, [vp, u64, C.POINTER(C.c_int)]),
        "dsc_buf_alloc": (C.c_int, [vp, sz, C.POINTER(u64)]),
        "dsc_buf_free": (C.c_int, [vp, u64]),
        "dsc_buf_info": (C.c_int, [vp, u64, C.POINTER(vp), C.POINTER(sz)]),
        "dsc_heap_stats": (C.c_int, [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
        "dsc_buf_write": (C.c_int, [vp, u64, sz, vp, sz]),
        "dsc_buf_fill_zero": (C.c_int, [vp, u64, sz, sz]),
        "dsc_buf_read": (C.c_int, [vp, u64, sz, vp, sz]),
        "dsc_buf_alloc_io": (C.c_int, [vp, sz, C.POINTER(u64)]),
        "dsc_host_alloc": (C.c_int, [vp, sz, C.POINTER(vp)]),
        "dsc_host_free": (C.c_int, [vp, vp]),
        "dsc_buf_write_async": (C.c_int, [vp, u64, sz, vp, sz, C.POINTER(u64)]),
        "dsc_buf_read_async": (C.c_int, [vp, u64, sz, vp, sz, C.POINTER(u64)]),
        "dsc_kernel_get": (C.c_int, [vp, C.POINTER(_abi.CKernelDesc), C.POINTER(vp)]),
        "dsc_kernel_buffer_count": (C.c_int, [vp]),
        "dsc_kernel_reference_group_count": (C.c_int64, [vp]),
        "dsc_kernel_label": (C.c_char_p, [vp]),
        "dsc_kernel_source": (C.c_char_p, [vp]),
        "dsc_kernel_launch": (C.c_int, [vp, vp, C.POINTER(u64), C.c_int, u32]),
        "dsc_codegen_source": (C.c_int, [C.POINTER(_abi.CKernelDesc), C.POINTER(vp)]),
        "dsc_codegen_compile": (C.c_int, [C.POINTER(_abi.CKernelDesc), C.c_char_p, C.POINTER(sz)]),
        "dsc_codegen_check_schedule": (C.c_int, [C.POINTER(_abi.CScheduleDesc), u32, C.c_char_p, C.POINTER(vp)]),
        "dsc_free_string": (None, [vp]),
        "dsc_cache_stats": (C.c_int, [C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
        "dsc_schedule_create": (C.c_int, [vp, C.POINTER(_abi.CScheduleDesc), u32, C.POINTER(vp)]),
        "dsc_schedule_destroy": (C.c_int, [vp, vp]),
        "dsc_schedule_run": (C.c_int, [vp, vp, C.POINTER(u64), u32]),
        "dsc_schedule_run_static": (C.c_int, [vp, vp, C.POINTER(u64), C.POINTER(u64), u32]),
        "dsc_schedule_launch_count": (C.c_int, [vp, C.POINTER(i32), C.POINTER(i32)]),
        "dsc_schedule_describe": (C.c_int, [vp, C.POINTER(vp)]),
        "dsc_schedule_dot": (C.c_int, [vp, C.POINTER(vp)]),
        "dsc_prof_markers": (C.c_int, [vp, C.c_int]),
        "dsc_prof_enable": (C.c_int, [vp, C.c_int]),
        "dsc_prof_reset": (C.c_int, [vp]),
        "dsc_prof_report": (C.c_int, [vp, C.c_int, C.POINTER(vp)]),
        "dsc_prof_query": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
        "dsc_prof_work": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double),
                                    C.POINTER(C.c_int64)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


EXPORTED_SYMBOLS = [
    "dsc_last_error", "dsc_ctx_create", "dsc_ctx_destroy", "dsc_ctx_caps", "dsc_ctx_sync", "dsc_ctx_stream",
    "dsc_fence_record", "dsc_fence_wait", "dsc_fence_query",
    "dsc_buf_alloc", "dsc_buf_free", "dsc_buf_info", "dsc_heap_stats", "dsc_buf_write", "dsc_buf_fill_zero",
    "dsc_buf_read", "dsc_buf_alloc_io", "dsc_host_alloc", "dsc_host_free", "dsc_buf_write_async", "dsc_buf_read_async", "dsc_kernel_get", "dsc_kernel_buffer_count", "dsc_kernel_reference_group_count",
    "dsc_kernel_label", "dsc_kernel_source", "dsc_kernel_launch", "dsc_codegen_source", "dsc_codegen_compile",
    "dsc_codegen_check_schedule", "dsc_free_string", "dsc_cache_stats", "dsc_schedule_create", "dsc_schedule_destroy",
    "dsc_schedule_run", "dsc_schedule_run_static", "dsc_schedule_launch_count", "dsc_schedule_describe", "dsc_schedule_dot", "dsc_prof_markers", "dsc_prof_enable", "dsc_prof_reset",
    "dsc_prof_report", "dsc_prof_query", "dsc_prof_work",
]


def check(status: int) -> None:
    if status != 0:
        raise DescentHipError(status, lib().dsc_last_error().decode(errors="replace"))


def _take_string(p: C.c_void_p) -> str:
    text = C.string_at(p).decode(errors="replace")
    lib().dsc_free_string(p)
    return text


# -- device-free code generation (CPU tests) -----------------------------------------------------------
def codegen_source(kernel) -> str:
    mk = _abi.MarshalledKernel(kernel)
    out = C.c_void_p()
    check(lib().dsc_codegen_source(C.byref(mk.desc), C.byref(out)))
    return _take_string(out)


def codegen_compile(kernel, arch: str = "gfx950") -> int:
    mk = _abi.MarshalledKernel(kernel)
    n = C.c_size_t()
    check(lib().dsc_codegen_compile(C.byref(mk.desc), arch.encode(), C.byref(n)))
    return n.value


def cache_stats():
    """(files used, hipRTC compilations, files refused and deleted) of the on-disk code-object cache, process-wide."""
    a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
    check(lib().dsc_cache_stats(C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


def schedule_flags(fused) -> int:
    """`fused`: True (all fusion), False (one launch per reference cluster), "generic-conv" (all fusion, but
    convolutions stay on the generic MatMul path instead of the dedicated kernels), "graph-replay"
    (all fusion, each run captured as a HIP graph and replayed when the buffers land on the same addresses), or
    "split-conv-grads" (all fusion, but a convolution's data and filter gradients stay two kernels)."""
    if fused == "generic-conv":
        return _abi.SCHEDULE_NO_CONV_KERNELS
    if fused == "graph-replay":
        return _abi.SCHEDULE_GRAPH_REPLAY
    if fused == "split-conv-grads":
        return _abi.SCHEDULE_SPLIT_CONV_GRADS
    return 0 if fused else _abi.SCHEDULE_NO_FUSION


def check_schedule(graph, fused=True, arch: str = "gfx950") -> str:
    """Plans and compiles every kernel of a graph's schedule without a GPU; returns the listing."""
    ms = _abi.MarshalledSchedule(graph)
    out = C.c_void_p()
    flags = schedule_flags(fused)
    check(lib().dsc_codegen_check_schedule(C.byref(ms.desc), flags, arch.encode(), C.byref(out)))
    return _take_string(out)


class HipSchedule:
    def __init__(self, backend: "HipBackend", graph, fused):
        self._backend = backend
        self._ms = _abi.MarshalledSchedule(graph)
        self.params = self._ms.params
        self._handle = C.c_void_p()
        flags = schedule_flags(fused)
        check(lib().dsc_schedule_create(backend._ctx, C.byref(self._ms.desc), flags, C.byref(self._handle)))
        self._slots = (C.c_uint64 * max(1, len(self.params)))()
        backend._schedules.add(self)

    def close(self) -> None:
        """dsc_schedule_destroy, while the context the schedule was created on is still alive (the backend closes its
        live schedules before it destroys the context): graph executables, the replay region and the spare buffers of
        a schedule that replays HIP graphs go back with it."""
        handle, self._handle = self._handle, C.c_void_p()
        if handle and self._backend._ctx:
            lib().dsc_schedule_destroy(self._backend._ctx, handle)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def run(self, handles: List[int], rand_seed: int) -> List[int]:
        for i, h in enumerate(handles):
            self._slots[i] = h or 0
        check(lib().dsc_schedule_run(self._backend._ctx, self._handle, self._slots, rand_seed & 0xFFFFFFFF))
        return [self._slots[i] or None for i in range(len(handles))]

    def run_static(self, handles: List[int], spare: List[int], rand_seed: int):
        """dsc_schedule_run_static: no device allocation; every written parameter goes into its slot's spare buffer and
        the two swap.  Returns (handles, spare) after the call."""
        spares = (C.c_uint64 * max(1, len(self.params)))()
        for i, h in enumerate(handles):
            self._slots[i] = h or 0
            spares[i] = spare[i] or 0
        check(lib().dsc_schedule_run_static(self._backend._ctx, self._handle, self._slots, spares, rand_seed & 0xFFFFFFFF))
        return [self._slots[i] or None for i in range(len(handles))], [spares[i] or None for i in range(len(handles))]

    def written_slots(self) -> List[int]:
        """Parameter slots a run writes (they need a spare buffer for run_static)."""
        d = self._ms.desc
        return sorted({d.outputs[i].param for i in range(d.n_outputs)})

    def launch_count(self):
        a, b = C.c_int32(), C.c_int32()
        check(lib().dsc_schedule_launch_count(self._handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    def describe(self) -> str:
        out = C.c_void_p()
        check(lib().dsc_schedule_describe(self._handle, C.byref(out)))
        return _take_string(out)

    def dot(self) -> str:
        """The fused schedule as a graphviz digraph."""
        out = C.c_void_p()
        check(lib().dsc_schedule_dot(self._handle, C.byref(out)))
        return _take_string(out)


class HipBackend:
    def __init__(self, device: int = 0):
        self._ctx = C.c_void_p()
        check(lib().dsc_ctx_create(device, C.byref(self._ctx)))
        self._kernels = {}
        self._pinned = {}
        self._schedules = weakref.WeakSet()

    def close(self):
        for schedule in list(self._schedules):
            schedule.close()
        if self._ctx:
            lib().dsc_ctx_destroy(self._ctx)
            self._ctx = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- memory ---------------------------------------------------------------------------------------
    def alloc(self, nbytes: int) -> int:
        h = C.c_uint64()
        check(lib().dsc_buf_alloc(self._ctx, nbytes, C.byref(h)))
        return h.value

    def alloc_io(self, nbytes: int) -> int:
        """A buffer from the device memory set aside for overlapped uploads."""
        h = C.c_uint64()
        check(lib().dsc_buf_alloc_io(self._ctx, nbytes, C.byref(h)))
        return h.value

    def free(self, handle: int) -> None:
        check(lib().dsc_buf_free(self._ctx, handle))

    def write(self, handle: int, offset: int, data) -> None:
        arr = np.ascontiguousarray(data) if isinstance(data, np.ndarray) else np.frombuffer(bytes(data), dtype=np.uint8)
        check(lib().dsc_buf_write(self._ctx, handle, offset, arr.ctypes.data, arr.nbytes))

    def fill_zero(self, handle: int, offset: int, nbytes: int) -> None:
        check(lib().dsc_buf_fill_zero(self._ctx, handle, offset, nbytes))

    def read(self, handle: int, offset: int, nbytes: int) -> bytes:
        out = np.empty(nbytes, dtype=np.uint8)
        check(lib().dsc_buf_read(self._ctx, handle, offset, out.ctypes.data, nbytes))
        return out.tobytes()

    # -- overlapped I/O (second stream) -----------------------------------------------------------------------
    def host_array(self, shape, dtype=np.float32) -> np.ndarray:
        """A numpy array over pinned host memory (dsc_host_alloc) that write_async / read_async use in place.
        The memory lives until host_release(array) or the backend is closed."""
        dtype = np.dtype(dtype)
        count = int(np.prod(shape)) if np.ndim(shape) else int(shape)
        nbytes = max(1, count * dtype.itemsize)
        p = C.c_void_p()
        check(lib().dsc_host_alloc(self._ctx, nbytes, C.byref(p)))
        raw = (C.c_uint8 * nbytes).from_address(p.value)
        arr = np.frombuffer(raw, dtype=dtype, count=count).reshape(shape)
        self._pinned[arr.ctypes.data] = p.value
        return arr

    def host_release(self, arr: np.ndarray) -> None:
        check(lib().dsc_host_free(self._ctx, self._pinned.pop(arr.ctypes.data)))

    def write_async(self, handle: int, offset: int, data: np.ndarray) -> int:
        """Upload on the copy stream; returns the fence after which a pinned `data` may be rewritten."""
        arr = np.ascontiguousarray(data)
        f = C.c_uint64()
        check(lib().dsc_buf_write_async(self._ctx, handle, offset, arr.ctypes.data, arr.nbytes, C.byref(f)))
        return f.value

    def read_async(self, handle: int, offset: int, out: np.ndarray) -> int:
        """Read-back into a host_array; the data is valid once the returned fence has finished."""
        f = C.c_uint64()
        check(lib().dsc_buf_read_async(self._ctx, handle, offset, out.ctypes.data, out.nbytes, C.byref(f)))
        return f.value

    def device_ptr(self, handle: int) -> int:
        p, n = C.c_void_p(), C.c_size_t()
        check(lib().dsc_buf_info(self._ctx, handle, C.byref(p), C.byref(n)))
        return p.value

    def heap_stats(self):
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        check(lib().dsc_heap_stats(self._ctx, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def caps(self) -> _abi.CCaps:
        caps = _abi.CCaps()
        check(lib().dsc_ctx_caps(self._ctx, C.byref(caps)))
        return caps

    def stream(self) -> int:
        p = C.c_void_p()
        check(lib().dsc_ctx_stream(self._ctx, C.byref(p)))
        return p.value or 0

    # -- kernels ----------------------------------------------------------------------------------------
    def kernel(self, kernel):
        k = self._kernels.get(kernel)
        if k is None:
            mk = _abi.MarshalledKernel(kernel)
            k = C.c_void_p()
            check(lib().dsc_kernel_get(self._ctx, C.byref(mk.desc), C.byref(k)))
            self._kernels[kernel] = k
        return k

    def kernel_source(self, kernel) -> str:
        return lib().dsc_kernel_source(self.kernel(kernel)).decode()

    def launch(self, kernel, handles, rand_seed: int) -> None:
        k = self.kernel(kernel)
        arr = (C.c_uint64 * len(handles))(*handles)
        check(lib().dsc_kernel_launch(self._ctx, k, arr, len(handles), rand_seed & 0xFFFFFFFF))

    def make_schedule(self, graph, fused=True) -> HipSchedule:
        return HipSchedule(self, graph, fused)

    def sync(self) -> None:
        check(lib().dsc_ctx_sync(self._ctx))

    # -- fences (device/fence.rs) -------------------------------------------------------------------------
    def fence_record(self) -> int:
        f = C.c_uint64()
        check(lib().dsc_fence_record(self._ctx, C.byref(f)))
        return f.value

    def fence_wait(self, fence: int) -> None:
        check(lib().dsc_fence_wait(self._ctx, fence))

    def fence_finished(self, fence: int) -> bool:
        out = C.c_int()
        check(lib().dsc_fence_query(self._ctx, fence, C.byref(out)))
        return bool(out.value)

    # -- timing -----------------------------------------------------------------------------------------
    def profile(self, enabled: bool) -> None:
        check(lib().dsc_prof_enable(self._ctx, 1 if enabled else 0))

    def markers(self, enabled: bool) -> None:
        """Wraps every launch in a ROCTx range named by the kernel's label (rocprofv3 --marker-trace)."""
        check(lib().dsc_prof_markers(self._ctx, 1 if enabled else 0))

    def profile_reset(self) -> None:
        check(lib().dsc_prof_reset(self._ctx))

    def timing_report(self, top_n: int = 5) -> str:
        out = C.c_void_p()
        check(lib().dsc_prof_report(self._ctx, top_n, C.byref(out)))
        return _take_string(out)

    def timing_query(self, prefix: str):
        avg, n = C.c_double(), C.c_int64()
        check(lib().dsc_prof_query(self._ctx, prefix.encode(), C.byref(avg), C.byref(n)))
        return avg.value, n.value

    def timing_work(self, prefix: str):
        """(total us, algorithmic bytes, algorithmic flops, launches) of the launches whose label starts with prefix."""
        us, nbytes, flops, n = C.c_double(), C.c_double(), C.c_double(), C.c_int64()
        check(lib().dsc_prof_work(self._ctx, prefix.encode(), C.byref(us), C.byref(nbytes), C.byref(flops), C.byref(n)))
        return us.value, nbytes.value, flops.value, n.value
