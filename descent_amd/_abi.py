"""ctypes mirror of include/descent_hip.h and marshalling of kernel
descriptors / graphs into its POD structs."""
from __future__ import annotations

import ctypes as C
from typing import List, Sequence

from . import kernel as K
from .graph import Graph
from .shape import BROADCAST, Shape, View

MAX_DIM = 7

(OK, ERR_INVALID, ERR_OOM, ERR_HIP, ERR_COMPILE, ERR_UNSUPPORTED, ERR_NO_DEVICE) = range(7)
STATUS_NAMES = ("ok", "invalid", "out of memory", "hip", "compile", "unsupported", "no device")

KIND_FILL, KIND_PER_ELEMENT, KIND_REDUCE, KIND_MATMUL, KIND_UNPAD, KIND_W2I, KIND_SCATTER_ADD = range(7)
(PE_LOAD, PE_LITERAL_F32, PE_LITERAL_U32, PE_COORD, PE_RAND, PE_UNARY, PE_BINARY, PE_SELECT, PE_GATHER) = range(9)

SCHEDULE_NO_FUSION = 1
SCHEDULE_NO_CONV_KERNELS = 2
SCHEDULE_GRAPH_REPLAY = 4
SCHEDULE_SPLIT_CONV_GRADS = 8


class CShape(C.Structure):
    _fields_ = [("rank", C.c_int32), ("dims", C.c_int64 * MAX_DIM)]


class CView(C.Structure):
    _fields_ = [
        ("in_shape", CShape),
        ("in_offset", C.c_int64 * MAX_DIM),
        ("out_shape", CShape),
        ("map_axis", C.c_int32 * MAX_DIM),
        ("map_step", C.c_int64 * MAX_DIM),
    ]


class CPeOp(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("op", C.c_int32),
        ("args", C.c_int32 * 4),
        ("bits", C.c_uint32),
        ("input_index", C.c_int32),
        ("view_index", C.c_int32),
        ("axis", C.c_int32),
        ("gather_shape", CShape),
    ]


class CKernelDesc(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("shape", CShape),
        ("n_inputs", C.c_int32),
        ("inputs", C.POINTER(CView)),
        ("n_ops", C.c_int32),
        ("ops", C.POINTER(CPeOp)),
        ("n_outputs", C.c_int32),
        ("outputs", C.POINTER(C.c_int32)),
        ("n_builtin_views", C.c_int32),
        ("builtin_views", C.POINTER(CView)),
        ("fill_bits", C.c_uint32),
        ("reduce_op", C.c_int32),
        ("axis", C.c_int32),
        ("pad", C.c_int32),
        ("stride_w", C.c_int32),
        ("stride_h", C.c_int32),
        ("output_mode", C.c_int32),
    ]


class CCaps(C.Structure):
    _fields_ = [
        ("has_float_atomic_add", C.c_int32),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("device_memory_bytes", C.c_int64),
        ("arch", C.c_char * 32),
    ]


class CClusterOutput(C.Structure):
    _fields_ = [
        ("node", C.c_int32),
        ("copy_from", C.c_int32),
        ("copy_from_is_literal", C.c_int32),
        ("literal_bits", C.c_uint32),
    ]


class CCluster(C.Structure):
    _fields_ = [
        ("kernel", CKernelDesc),
        ("n_inputs", C.c_int32),
        ("inputs", C.POINTER(C.c_int32)),
        ("n_outputs", C.c_int32),
        ("outputs", C.POINTER(CClusterOutput)),
    ]


class CParamIO(C.Structure):
    _fields_ = [("node", C.c_int32), ("param", C.c_int32)]


class CScheduleDesc(C.Structure):
    _fields_ = [
        ("n_nodes", C.c_int32),
        ("node_elements", C.POINTER(C.c_int64)),
        ("n_clusters", C.c_int32),
        ("clusters", C.POINTER(CCluster)),
        ("n_inputs", C.c_int32),
        ("inputs", C.POINTER(CParamIO)),
        ("n_outputs", C.c_int32),
        ("outputs", C.POINTER(CParamIO)),
        ("n_params", C.c_int32),
    ]


def c_shape(shape: Sequence[int]) -> CShape:
    s = CShape()
    s.rank = len(shape)
    for i, d in enumerate(shape):
        s.dims[i] = d
    return s


def c_view(view: View) -> CView:
    v = CView()
    v.in_shape = c_shape(view.input_shape)
    for i, o in enumerate(view.input_offsets):
        v.in_offset[i] = o
    v.out_shape = c_shape(view.output_shape)
    for j, (axis, step) in enumerate(view.mapping):
        v.map_axis[j] = axis
        v.map_step[j] = step
    return v


def _view_array(views: Sequence[View]):
    arr = (CView * max(1, len(views)))()
    for i, v in enumerate(views):
        arr[i] = c_view(v)
    return arr


class MarshalledKernel:
    """A CKernelDesc plus the ctypes arrays it points into (kept alive here)."""

    def __init__(self, kernel):
        d = CKernelDesc()
        self.desc = d
        self._keep: List[object] = []
        views: Sequence[View] = ()
        if isinstance(kernel, K.FillKernel):
            d.kind = KIND_FILL
            d.shape = c_shape([kernel.element_count])
            d.fill_bits = kernel.value.bits
        elif isinstance(kernel, K.PerElementKernel):
            d.kind = KIND_PER_ELEMENT
            d.shape = c_shape([kernel.element_count])
            views = kernel.inputs
            builtin_views: List[View] = []
            ops = (CPeOp * max(1, len(kernel.ops)))()
            for i, op in enumerate(kernel.ops):
                o = ops[i]
                if isinstance(op, K.PeLoad):
                    o.kind, o.input_index = PE_LOAD, op.input_index
                elif isinstance(op, K.PeLiteral):
                    o.kind = PE_LITERAL_U32 if op.value.is_u32 else PE_LITERAL_F32
                    o.bits = op.value.bits
                elif isinstance(op, K.PeCoord):
                    o.kind, o.view_index = PE_COORD, len(builtin_views)
                    builtin_views.append(op.view)
                elif isinstance(op, K.PeRand):
                    o.kind, o.view_index, o.bits = PE_RAND, len(builtin_views), op.uid
                    builtin_views.append(op.view)
                elif isinstance(op, K.PeUnary):
                    o.kind, o.op = PE_UNARY, K.UNARY_OPS.index(op.op)
                    o.args[0] = op.arg
                elif isinstance(op, K.PeBinary):
                    o.kind, o.op = PE_BINARY, K.BINARY_OPS.index(op.op)
                    o.args[0], o.args[1] = op.args
                elif isinstance(op, K.PeSelect):
                    o.kind, o.op = PE_SELECT, K.COMPARE_MODES.index(op.compare_mode)
                    for j in range(4):
                        o.args[j] = op.args[j]
                elif isinstance(op, K.PeGather):
                    o.kind, o.input_index, o.axis = PE_GATHER, op.input_index, op.axis
                    o.args[0] = op.arg
                    o.gather_shape = c_shape(op.shape)
                else:
                    raise TypeError(f"unknown per-element op {op!r}")
            outs = (C.c_int32 * max(1, len(kernel.outputs)))(*kernel.outputs)
            bviews = _view_array(builtin_views)
            d.n_ops, d.ops = len(kernel.ops), ops
            d.n_outputs, d.outputs = len(kernel.outputs), outs
            d.n_builtin_views, d.builtin_views = len(builtin_views), bviews
            self._keep += [ops, outs, bviews]
        elif isinstance(kernel, K.ReduceKernel):
            d.kind = KIND_REDUCE
            d.shape = c_shape(kernel.shape)
            views = (kernel.input,)
            d.reduce_op = K.REDUCE_OPS.index(kernel.reduce_op)
            d.axis = kernel.axis
        elif isinstance(kernel, K.MatMulKernel):
            d.kind = KIND_MATMUL
            d.shape = c_shape(kernel.shape)
            views = (kernel.a, kernel.b)
            d.output_mode = kernel.output_mode
        elif isinstance(kernel, K.UnpadKernel):
            d.kind = KIND_UNPAD
            d.shape = c_shape(kernel.shape)
            views = (kernel.input,)
            d.axis, d.pad = kernel.axis, kernel.pad
        elif isinstance(kernel, K.WindowsToImageKernel):
            d.kind = KIND_W2I
            d.shape = c_shape(kernel.shape)
            views = (kernel.input,)
            d.stride_w, d.stride_h = kernel.stride
        elif isinstance(kernel, K.ScatterAddKernel):
            d.kind = KIND_SCATTER_ADD
            d.shape = c_shape(kernel.shape)
            views = (kernel.values, kernel.indices)
            d.axis = kernel.axis
        else:
            raise TypeError(f"unknown kernel {kernel!r}")
        arr = _view_array(views)
        d.n_inputs, d.inputs = len(views), arr
        self._keep.append(arr)


class MarshalledSchedule:
    """A CScheduleDesc for a whole Graph; `params` lists the Parameters in the
    slot order the params array of dsc_schedule_run uses."""

    def __init__(self, graph: Graph):
        ops = graph.ops
        self._keep: List[object] = []
        self.params = []
        slot = {}

        def slot_of(p):
            if p not in slot:
                slot[p] = len(self.params)
                self.params.append(p)
            return slot[p]

        n_nodes = ops.node_bound()
        elements = (C.c_int64 * max(1, n_nodes))()
        for nid, node in ops.nodes.items():
            elements[nid] = node.shape.element_count()

        clusters = (CCluster * max(1, len(graph.clusters_sorted)))()
        for i, cid in enumerate(graph.clusters_sorted):
            cl = graph.clusters[cid]
            mk = MarshalledKernel(cl.kernel)
            ins = (C.c_int32 * max(1, len(cl.inputs)))(*cl.inputs)
            outs = (CClusterOutput * max(1, len(cl.outputs)))()
            for j, o in enumerate(cl.outputs):
                outs[j].node = o.node_id
                outs[j].copy_from = -1 if o.copy_from is None else o.copy_from
                if o.copy_from is not None and ops.nodes[o.copy_from].op.kind == "Literal":
                    outs[j].copy_from_is_literal = 1
                    outs[j].literal_bits = ops.nodes[o.copy_from].op.a.bits
            c = clusters[i]
            c.kernel = mk.desc
            c.n_inputs, c.inputs = len(cl.inputs), ins
            c.n_outputs, c.outputs = len(cl.outputs), outs
            self._keep += [mk, ins, outs]

        in_nodes = [n for n in sorted(ops.nodes) if ops.nodes[n].op.kind == "Input"]
        out_nodes = [n for n in sorted(ops.nodes) if ops.nodes[n].op.kind == "Output"]
        ins = (CParamIO * max(1, len(in_nodes)))()
        for i, n in enumerate(in_nodes):
            ins[i].node, ins[i].param = n, slot_of(ops.nodes[n].op.a)
        outs = (CParamIO * max(1, len(out_nodes)))()
        for i, n in enumerate(out_nodes):
            (src,) = ops.predecessors(n)
            outs[i].node, outs[i].param = src, slot_of(ops.nodes[n].op.a)

        d = CScheduleDesc()
        d.n_nodes, d.node_elements = n_nodes, elements
        d.n_clusters, d.clusters = len(graph.clusters_sorted), clusters
        d.n_inputs, d.inputs = len(in_nodes), ins
        d.n_outputs, d.outputs = len(out_nodes), outs
        d.n_params = len(self.params)
        self.desc = d
        self._keep += [elements, clusters, ins, outs]
