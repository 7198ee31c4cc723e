"""Environment: parameters, upload/download and graph execution.

Host-side mirror of src/environment.rs.  The device work is delegated to a
backend object:

    alloc(nbytes) -> handle        free(handle)
    write(handle, offset, bytes)   fill_zero(handle, offset, nbytes)
    read(handle, offset, nbytes) -> bytes
    launch(kernel_descriptor, [handles], rand_seed)
    sync()
    make_schedule(graph, fused) -> object with .run(param_handles, seed)   (optional)

`descent_amd.hip_backend.HipBackend` implements it over the C ABI of
libdescent_hip.so and is the default.  A backend that lacks `make_schedule`
is driven kernel by kernel with the reference's own buffer-lifetime algorithm
(`Environment._run_cluster_by_cluster`).
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import numpy as np

from .array import Parameter, Scope
from .graph import Graph
from .kernel import FillKernel
from .module import Initializer
from .shape import Shape


class ParameterWriter:
    """Sequential byte writer into a parameter's fresh buffer; whatever is left
    unwritten when it is closed is zero-filled (src/environment.rs:42-59,
    src/device/staging.rs:181-187)."""

    def __init__(self, backend, handle, nbytes: int):
        self._backend, self._handle, self._nbytes = backend, handle, nbytes
        self._pos = 0
        self._closed = False

    def write(self, data) -> int:
        buf = np.ascontiguousarray(data).view(np.uint8).reshape(-1) if isinstance(data, np.ndarray) else np.frombuffer(
            bytes(data), dtype=np.uint8
        )
        n = min(len(buf), self._nbytes - self._pos)
        if n:
            self._backend.write(self._handle, self._pos, buf[:n])
            self._pos += n
        return n

    def zero_fill(self) -> None:
        self.close()

    def close(self) -> None:
        if not self._closed:
            self._closed = True
            if self._pos < self._nbytes:
                self._backend.fill_zero(self._handle, self._pos, self._nbytes - self._pos)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Environment:
    def __init__(self, backend=None, use_schedule: bool = True, fused: bool = True):
        if backend is None:
            from .hip_backend import HipBackend

            backend = HipBackend()
        self.backend = backend
        self.use_schedule = use_schedule and hasattr(backend, "make_schedule")
        self.fused = fused
        self.parameters: List[Parameter] = []

    # -- parameters (src/environment.rs:126-229) --------------------------------
    def static_parameter(self, shape, name: str) -> Parameter:
        p = Parameter(self, shape, name, None)
        self.parameters.append(p)
        return p

    def trainable_parameter(self, shape, name: str, reset_to: Initializer) -> Parameter:
        p = Parameter(self, shape, name, reset_to)
        self.parameters.append(p)
        return p

    def writer(self, parameter: Parameter) -> ParameterWriter:
        """Frees the old buffer and allocates a new one (src/environment.rs:160-175)."""
        parameter.checked(self)
        self._fresh_buffer(parameter)
        return ParameterWriter(self.backend, parameter.buffer, parameter.shape.buffer_size())

    def _fresh_buffer(self, parameter: Parameter, io: bool = False) -> None:
        # The new buffer is taken before the old one is given back (the reference frees first): the old one is
        # still read by the step enqueued before this call, and an upload into other memory can run beside that step.
        old = parameter.buffer
        alloc = self.backend.alloc_io if io else self.backend.alloc
        parameter.buffer = alloc(parameter.shape.buffer_size())
        if old is not None:
            self.backend.free(old)

    def host_array(self, parameter: Parameter) -> np.ndarray:
        """Pinned host array of the parameter's shape for write_parameter_async / read_parameter_async."""
        parameter.checked(self)
        return self.backend.host_array(tuple(parameter.shape), np.float32)

    def write_parameter_async(self, parameter: Parameter, data: np.ndarray) -> int:
        """Like write_parameter, on the backend's copy stream: the upload overlaps with graph runs enqueued before
        it, later runs wait for it.  `data` from host_array() is read in place and must not be rewritten before
        the returned fence has finished (backend.fence_wait); other arrays are copied before the call returns."""
        parameter.checked(self)
        data = np.ascontiguousarray(data)
        if data.dtype not in (np.float32, np.uint32, np.int32):
            data = data.astype(np.float32)
        if data.nbytes != parameter.shape.buffer_size():
            raise ValueError(f"parameter {parameter.name!r} holds {parameter.shape.buffer_size()} bytes, got {data.nbytes}")
        self._fresh_buffer(parameter, io=True)
        return self.backend.write_async(parameter.buffer, 0, data)

    def read_parameter_async(self, parameter: Parameter, out: np.ndarray) -> int:
        """Starts a read-back of the parameter's current value into `out` (from host_array()) without blocking;
        `out` holds it once the returned fence has finished."""
        parameter.checked(self)
        if parameter.buffer is None:
            raise ValueError(f"parameter {parameter.name!r} has no value")
        if out.nbytes != parameter.shape.buffer_size():
            raise ValueError(f"parameter {parameter.name!r} holds {parameter.shape.buffer_size()} bytes, got {out.nbytes}")
        return self.backend.read_async(parameter.buffer, 0, out)

    def write_parameter(self, parameter: Parameter, data) -> None:
        data = np.ascontiguousarray(data)
        if data.dtype not in (np.float32, np.uint32, np.int32):
            data = data.astype(np.float32)
        with self.writer(parameter) as w:
            w.write(data)

    def static_parameter_with_data(self, shape, name: str, data) -> Parameter:
        p = self.static_parameter(shape, name)
        self.write_parameter(p, np.asarray(data, dtype=np.float32))
        return p

    def reader(self, parameter: Parameter) -> bytes:
        parameter.checked(self)
        if parameter.buffer is None:
            raise ValueError(f"parameter {parameter.name!r} has no value")
        return self.backend.read(parameter.buffer, 0, parameter.shape.buffer_size())

    def read_parameter_to_vec(self, parameter: Parameter) -> np.ndarray:
        return np.frombuffer(self.reader(parameter), dtype=np.float32).copy()

    def read_parameter(self, parameter: Parameter) -> np.ndarray:
        return self.read_parameter_to_vec(parameter).reshape(tuple(parameter.shape))

    def read_parameter_scalar(self, parameter: Parameter) -> float:
        return float(self.read_parameter_to_vec(parameter)[0])

    def save_parameters(self, path, parameters) -> int:
        """Writes the parameters' values to `path` as raw little-endian f32, in the order given and with no header --
        what piping each `reader()` (io::Read, src/environment.rs:63-67, 177-189) into one file gives.  Returns the
        number of bytes written."""
        total = 0
        with open(path, "wb") as f:
            for p in parameters:
                data = self.reader(p)
                f.write(data)
                total += len(data)
        return total

    def load_parameters(self, path, parameters) -> None:
        """Reads a file written by save_parameters back through `writer()` (io::Write, src/environment.rs:50-61).
        The file must hold exactly the listed parameters' bytes."""
        import os

        want = sum(p.shape.buffer_size() for p in parameters)
        have = os.path.getsize(path)
        if have != want:
            raise ValueError(f"{path}: {have} bytes, the parameters hold {want}")
        with open(path, "rb") as f:
            for p in parameters:
                with self.writer(p) as w:
                    w.write(np.frombuffer(f.read(p.shape.buffer_size()), dtype=np.float32))

    def reset_parameter(self, parameter: Parameter, rng: np.random.Generator) -> None:
        """src/environment.rs:190-202. The reference draws from ChaCha20 via the
        `rand` crate (Open01 + Box-Muller); that stream is not reproduced here,
        only the distributions: N(0, scale^2) and U(-scale, scale)."""
        init = parameter.reset_to
        n = parameter.shape.element_count()
        if init is None:
            raise ValueError("parameter has no initializer")
        if init.kind == "zero":
            self.writer(parameter).zero_fill()
        elif init.kind == "normal":
            self.write_parameter(parameter, (rng.standard_normal(n) * init.scale).astype(np.float32))
        else:
            self.write_parameter(parameter, ((rng.random(n) * 2.0 - 1.0) * init.scale).astype(np.float32))

    # -- graphs -------------------------------------------------------------------
    def scope(self) -> Scope:
        return Scope(self)

    def build_graph(self, f: Callable[[Scope], None]) -> Graph:
        scope = self.scope()
        f(scope)
        return scope.build_graph()

    def run(self, graph: Graph, rand_seed: int) -> None:
        """src/environment.rs:326-516"""
        rand_seed &= 0xFFFFFFFF
        if self.use_schedule:
            key = (id(self.backend), self.fused)
            cache = graph.__dict__.setdefault("_schedules", {})
            sched = cache.get(key)
            if sched is None:
                sched = cache[key] = self.backend.make_schedule(graph, self.fused)
            handles = [p.checked(self).buffer for p in sched.params]
            handles = sched.run(handles, rand_seed)
            for p, h in zip(sched.params, handles):
                p.buffer = h
        else:
            self._run_cluster_by_cluster(graph, rand_seed)

    def run_static(self, graph: Graph, rand_seed: int) -> None:
        """`run` through dsc_schedule_run_static: the step's intermediates live in the library's fixed scratch array
        and every parameter the graph writes alternates between its buffer and one spare buffer, allocated here the
        first time the parameter is written this way -- after that a step allocates no device memory at all."""
        rand_seed &= 0xFFFFFFFF
        key = (id(self.backend), self.fused)
        cache = graph.__dict__.setdefault("_schedules", {})
        sched = cache.get(key)
        if sched is None:
            sched = cache[key] = self.backend.make_schedule(graph, self.fused)
        written = set(sched.written_slots())
        spare = []
        for i, p in enumerate(sched.params):
            p.checked(self)
            if i in written:
                if p.__dict__.get("spare") is None:
                    p.spare = self.backend.alloc(p.shape.buffer_size())
                spare.append(p.spare)
            else:
                spare.append(None)
        handles, spare = sched.run_static([p.buffer for p in sched.params], spare, rand_seed)
        for i, (p, h) in enumerate(zip(sched.params, handles)):
            p.buffer = h
            if i in written:
                p.spare = spare[i]

    def _run_cluster_by_cluster(self, graph: Graph, rand_seed: int) -> None:
        be = self.backend
        ops = graph.ops
        inputs = [n for n in sorted(ops.nodes) if ops.nodes[n].op.kind == "Input"]
        outputs = [n for n in sorted(ops.nodes) if ops.nodes[n].op.kind == "Output"]
        input_params = {ops.nodes[n].op.a for n in inputs}
        output_params = {ops.nodes[n].op.a for n in outputs}

        usage: Dict[int, int] = {}
        buffer: Dict[int, object] = {}
        for cl in graph.clusters.values():
            for n in cl.inputs:
                usage[n] = usage.get(n, 0) + 1

        # a node that becomes a parameter's new value must survive its other uses
        for n in outputs:
            (src,) = ops.predecessors(n)
            usage[src] = usage.get(src, 0) + 1

        # inputs share the parameter's buffer, or take it when the parameter is rewritten
        for n in inputs:
            p = ops.nodes[n].op.a.checked(self)
            if p.buffer is None:
                raise ValueError(f"parameter {p.name!r} has no value")
            if p not in output_params:
                buffer[n] = p.buffer
                usage[n] = usage.get(n, 0) + 1
            else:
                buffer[n], p.buffer = p.buffer, None
        # parameters that are only written lose their old buffer
        for n in outputs:
            p = ops.nodes[n].op.a.checked(self)
            if p not in input_params and p.buffer is not None:
                be.free(p.buffer)
                p.buffer = None

        for cid in graph.clusters_sorted:
            cl = graph.clusters[cid]
            for n in cl.inputs:
                usage[n] -= 1
            for out in cl.outputs:
                shape = ops.nodes[out.node_id].shape
                if out.copy_from is None:
                    h = be.alloc(shape.buffer_size())
                else:
                    src = out.copy_from
                    if usage.get(src, 0) != 0:
                        raise NotImplementedError("deep copy of a still-used accumulator")  # environment.rs:441
                    if buffer.get(src) is not None:
                        h = buffer.pop(src)
                    elif ops.nodes[src].op.kind == "Literal":
                        h = be.alloc(shape.buffer_size())
                        be.launch(FillKernel(ops.nodes[src].op.a, shape.element_count()), [h], rand_seed)
                    else:
                        raise RuntimeError("cannot copy-on-write node")
                assert buffer.get(out.node_id) is None
                buffer[out.node_id] = h
            handles = [buffer[n] for n in cl.inputs] + [buffer[o.node_id] for o in cl.outputs]
            be.launch(cl.kernel, handles, rand_seed)
            for n in cl.inputs:
                if usage[n] == 0 and buffer.get(n) is not None:
                    be.free(buffer.pop(n))

        for n in outputs:
            p = ops.nodes[n].op.a
            (src,) = ops.predecessors(n)
            p.buffer = buffer.pop(src)

    def sync(self) -> None:
        self.backend.sync()

    def print_timings(self, label: str, top_n: int = 5) -> None:
        """src/environment.rs:518-520"""
        if hasattr(self.backend, "timing_report"):
            print(f"{label}:\n{self.backend.timing_report(top_n)}")
