"""Graph-building array API with "dual array" autodiff.

Host-side mirror of src/array.rs.  An `Array` is a handle to an op node; every
operator appends nodes to the owning `Scope`.  A `DualArray` pairs a value
with the node that will hold d(loss)/d(value); each forward op immediately
appends its backward ops (src/array.rs:794-1147).  Nothing here touches the
device: the result is an `OpGraph` that `Scope.build_graph` lowers to clusters.

u32 arrays share the class: the reference's `UArray` is the same node handle
with the u32 operator set (src/array.rs:14-18, 733-734), selected here by the
`is_u32` flag.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence, Tuple, Union

import numpy as np

from .graph import Graph, MOV, Op, OpGraph
from .kernel import Literal
from .shape import BATCHES, ROWS, Shape, View


def _axis(axis: int, shape: Shape) -> int:
    return shape.axis(axis)


class Array:
    __slots__ = ("node_id", "scope", "is_u32")

    def __init__(self, node_id: int, scope: "Scope", is_u32: bool = False):
        self.node_id = node_id
        self.scope = scope
        self.is_u32 = is_u32

    # -- plumbing ------------------------------------------------------------
    def _like(self, node_id: int) -> "Array":
        return Array(node_id, self.scope, self.is_u32)

    def _lift(self, value) -> "Array":
        """IntoArray / IntoUArray (src/array.rs:27-58)."""
        if isinstance(value, Array):
            return value
        if isinstance(value, DualArray):
            return value.value()
        if isinstance(value, Parameter):
            return self.scope.parameter_value(value)
        if self.is_u32:
            return self.scope.literal_u32(int(value))
        return self.scope.literal(float(value)).value()

    @property
    def shape(self) -> Shape:
        return self.scope.ops.nodes[self.node_id].shape

    def view(self, view: View) -> "Array":
        """A Mov node reading this array through `view` (src/array.rs:106-122)."""
        s = self.scope
        nid = s.ops.new_node(s.colour, view.output_shape, MOV)
        s.ops.add_edge(self.node_id, nid, 0, view)
        return self._like(nid)

    def broadcast(self, shape) -> "Array":
        return self.view(View.broadcast(self.shape, Shape(shape)))

    def _unary(self, name: str) -> "Array":
        s = self.scope
        return self._like(s.ops.new_node(s.colour, self.shape, Op("Unary", name), [self.node_id]))

    def _binary(self, rhs, name: str) -> "Array":
        rhs = self._lift(rhs)
        shape = self.shape.broadcast_with(rhs.shape)
        lhs_id = self.broadcast(shape).node_id
        rhs_id = rhs.broadcast(shape).node_id
        s = self.scope
        return self._like(s.ops.new_node(s.colour, shape, Op("Binary", name), [lhs_id, rhs_id]))

    def _keep_axis(self, axis: int, keep: bool) -> "Array":
        return self if keep else self.remove_axis(_axis(axis, self.shape))

    def reshape(self, shape) -> "Array":
        shape = Shape(shape)
        if shape.element_count() != self.shape.element_count():
            raise ValueError(f"cannot reshape {self.shape!r} to {shape!r}")
        s = self.scope
        return self._like(s.ops.new_node(s.colour, shape, MOV, [self.node_id]))

    def remove_axis(self, axis: int) -> "Array":
        return self.reshape(self.shape.remove_axis(axis))

    def insert_axis(self, axis: int) -> "Array":
        return self.reshape(self.shape.insert_axis(axis, 1))

    def limit_axis(self, axis: int, start: Optional[int] = None, end: Optional[int] = None) -> "Array":
        shape = self.shape
        axis = _axis(axis, shape)
        start = 0 if start is None else start
        end = shape[axis] if end is None else end
        return self.view(View.limited(shape, axis, start, end))

    def lock_axis(self, axis: int, coord: int, keep_axis: bool) -> "Array":
        axis = _axis(axis, self.shape)
        return self.limit_axis(axis, coord, coord + 1)._keep_axis(axis, keep_axis)

    def transpose(self) -> "Array":
        return self.view(self.shape.identity_view().transposed())

    def permute_axes(self, perm: Sequence[int]) -> "Array":
        return self.view(self.shape.identity_view().permute_axes(perm))

    # -- gradients -------------------------------------------------------------
    def with_empty_grad(self) -> Tuple["Array", "Array"]:
        """A source-less Mov that `accumulate` later wires up (src/array.rs:228-239)."""
        s = self.scope
        return self, Array(s.ops.new_node(s.colour, self.shape, MOV), s)

    def accumulate(self, src) -> None:
        """grad += src, by rewiring the Mov's single input (src/array.rs:617-650)."""
        src = self._lift(src)
        ops = self.scope.ops
        node = ops.nodes[self.node_id]
        if node.op != MOV:
            raise ValueError("accumulate target must be a gradient placeholder")
        if tuple(node.shape) != tuple(src.shape):
            raise ValueError(f"accumulate shape mismatch {node.shape!r} vs {src.shape!r}")
        in_edges = ops.in_edges(self.node_id)
        if in_edges:
            prev = ops.edges[in_edges[0]].src
            ops.remove_edge(in_edges[0])
            src_id = ops.new_node(self.scope.colour, src.shape, Op("Binary", "Add"), [prev, src.node_id])
        else:
            src_id = src.node_id
        ops.add_edge(src_id, self.node_id, 0, src.shape.identity_view())

    def _set_loss_grad_root(self) -> None:
        """d(loss)/d(loss) = 1/mini_batch (src/array.rs:652-672)."""
        shape = self.shape
        scale = self.scope.literal(float(np.float32(1.0) / np.float32(shape[0]))).value().broadcast(shape)
        ops = self.scope.ops
        assert ops.nodes[self.node_id].op == MOV and not ops.in_edges(self.node_id)
        ops.add_edge(scale.node_id, self.node_id, 0, shape.identity_view())

    def unbroadcast(self, shape: Shape) -> "Array":
        """Sum away broadcast axes (src/array.rs:241-262)."""
        out = self
        while len(out.shape) > len(shape):
            out = out.reduce_sum(0, False)
        assert len(out.shape) == len(shape)
        for index, (src, dst) in enumerate(zip(out.shape, shape)):
            if src != dst:
                assert dst == 1
                out = out.reduce_sum(index, True)
        return out

    # -- selection -------------------------------------------------------------
    def _select(self, mode: str, rhs, on_pass, on_fail) -> "Array":
        rhs, on_pass, on_fail = self._lift(rhs), self._lift(on_pass), self._lift(on_fail)
        shape = (
            self.shape.broadcast_with(rhs.shape).broadcast_with(on_pass.shape).broadcast_with(on_fail.shape)
        )
        ids = [a.broadcast(shape).node_id for a in (self, rhs, on_pass, on_fail)]
        s = self.scope
        return Array(s.ops.new_node(s.colour, shape, Op("Select", mode), ids), s)

    def select_eq(self, rhs, on_pass, on_fail) -> "Array":
        return self._select("Eq", rhs, on_pass, on_fail)

    def select_gt(self, rhs, on_pass, on_fail) -> "Array":
        return self._select("Gt", rhs, on_pass, on_fail)

    def coord(self, axis: int) -> "Array":
        """Index along `axis`, broadcastable against self (src/array.rs:369-374)."""
        shape = self.shape
        axis = _axis(axis, shape)
        return self.scope.coord(shape[axis]).value().reshape(shape.coord(axis))

    def one_hot(self, count: int) -> "Array":
        return self.scope.coord(count).value().select_eq(self, 1.0, 0.0)

    def concat(self, other, axis: int) -> "Array":
        """src/array.rs:299-324: select between two replicate-padded operands."""
        other = self._lift(other)
        shape = self.shape
        axis = _axis(axis, shape)
        length, other_length = shape[axis], other.shape[axis]
        out_shape = shape.resize_axis(axis, length + other_length)
        if tuple(out_shape) != tuple(other.shape.resize_axis(axis, length + other_length)):
            raise ValueError("concat operands differ outside the concat axis")
        coord = self.scope.coord(length + other_length).value().reshape(out_shape.coord(axis))
        return coord.select_gt(float(length - 1), other.pad(axis, length, 0), self.pad(axis, 0, other_length))

    # -- reductions ------------------------------------------------------------
    def _reduce(self, name: str, axis: int) -> "Array":
        shape = self.shape
        axis = _axis(axis, shape)
        if shape[axis] == 1:
            return self
        s = self.scope
        return Array(s.ops.new_node(s.colour, shape.reduce(axis), Op("Reduce", name, axis), [self.node_id]), s)

    def reduce_max(self, axis: int, keep_axis: bool) -> "Array":
        axis = _axis(axis, self.shape)
        return self._reduce("Max", axis)._keep_axis(axis, keep_axis)

    def reduce_sum(self, axis: int, keep_axis: bool) -> "Array":
        axis = _axis(axis, self.shape)
        return self._reduce("Sum", axis)._keep_axis(axis, keep_axis)

    def argmax(self, axis: int, keep_axis: bool) -> "Array":
        """Largest index among the maxima (src/array.rs:362-367)."""
        axis = _axis(axis, self.shape)
        coord_or_zero = self.select_eq(self.reduce_max(axis, True), self.coord(axis), 0.0)
        return coord_or_zero.reduce_max(axis, keep_axis)

    # -- gather / scatter ----------------------------------------------------------
    def gather(self, axis: int, indices: "Array") -> "Array":
        """src/array.rs:376-397"""
        (index_count,) = indices.shape
        values_shape = self.shape
        axis = _axis(axis, values_shape)
        shape = values_shape.resize_axis(axis, index_count)
        index = indices.reshape(shape.coord(axis)).broadcast(shape)
        s = self.scope
        return Array(s.ops.new_node(s.colour, shape, Op("Gather", axis), [self.node_id, index.node_id]), s)

    def scatter_add(self, values, axis: int, indices: "Array") -> "Array":
        """src/array.rs:398-425"""
        shape = self.shape
        values = self._lift(values)
        axis = _axis(axis, shape)
        (index_count,) = indices.shape
        if tuple(shape.resize_axis(axis, index_count)) != tuple(values.shape):
            raise ValueError("scatter_add values shape mismatch")
        s = self.scope
        return Array(
            s.ops.new_node(
                s.colour, shape, Op("ScatterAdd", axis), [self.node_id, values.node_id, indices.node_id]
            ),
            s,
        )

    # -- math --------------------------------------------------------------------
    def square(self):
        return self * self

    def sqrt(self):
        return self._unary("Sqrt")

    def exp(self):
        return self._unary("Exp")

    def log(self):
        return self._unary("Log")

    def sin(self):
        return self._unary("Sin")

    def cos(self):
        return self._unary("Cos")

    def sigmoid(self):
        return self.exp() / (self.exp() + 1.0)

    def tanh(self):
        a, b = self.exp(), (-self).exp()
        return (a - b) / (a + b)

    def pow(self, rhs):
        return self._binary(rhs, "Pow")

    def to_u32_bits(self) -> "Array":
        return Array(self.node_id, self.scope, True)

    def to_f32_bits(self) -> "Array":
        return Array(self.node_id, self.scope, False)

    def into_u32(self) -> "Array":
        return self._unary("FloatToUint").to_u32_bits()

    def into_f32(self) -> "Array":
        return self._unary("UintToFloat").to_f32_bits()

    def __add__(self, rhs):
        return self._binary(rhs, "UAdd" if self.is_u32 else "Add")

    def __radd__(self, lhs):
        return self._lift(lhs)._binary(self, "UAdd" if self.is_u32 else "Add")

    def __mul__(self, rhs):
        return self._binary(rhs, "UMul" if self.is_u32 else "Mul")

    def __rmul__(self, lhs):
        return self._lift(lhs)._binary(self, "UMul" if self.is_u32 else "Mul")

    def __sub__(self, rhs):
        return self._binary(rhs, "Sub")

    def __rsub__(self, lhs):
        return self._lift(lhs)._binary(self, "Sub")

    def __truediv__(self, rhs):
        return self._binary(rhs, "Div")

    def __rtruediv__(self, lhs):
        return self._lift(lhs)._binary(self, "Div")

    def __neg__(self):
        return self._unary("Neg")

    def __mod__(self, rhs):
        assert self.is_u32
        return self._binary(rhs, "URem")

    def __xor__(self, rhs):
        assert self.is_u32
        return self._binary(rhs, "UBitXor")

    # -- matmul / images -------------------------------------------------------------
    def matmul(self, rhs) -> "Array":
        lhs = self.insert_axis(0)
        rhs = self._lift(rhs).insert_axis(0)
        return lhs.batched_matmul(rhs, BATCHES).remove_axis(0)

    def batched_matmul(self, rhs: "Array", output_mode: int) -> "Array":
        """Split-K partials, then a sum over them (src/array.rs:500-520)."""
        s = self.scope
        shape = self.shape.batched_matmul(rhs.shape, output_mode)
        chunks = Array(s.ops.new_node(s.colour, shape, Op("MatMul", output_mode), [self.node_id, rhs.node_id]), s)
        out = chunks.reduce_sum(0, False)
        return out if output_mode == BATCHES else out.permute_axes([1, 0, 2])

    def pad(self, axis: int, before: int, after: int) -> "Array":
        if before + after == 0:
            return self
        shape = self.shape
        return self.view(shape.padded_view(_axis(axis, shape), before, after))

    def unpad(self, axis: int, pad: int) -> "Array":
        if pad == 0:
            return self
        shape = self.shape
        axis = _axis(axis, shape)
        s = self.scope
        return Array(s.ops.new_node(s.colour, shape.unpad(axis, pad), Op("Unpad", axis, pad), [self.node_id]), s)

    def pad_image(self, pad: int) -> "Array":
        return self.pad(-3, pad, pad).pad(-2, pad, pad)

    def unpad_image(self, pad: int) -> "Array":
        return self.unpad(-3, pad).unpad(-2, pad)

    def image_to_windows(self, filter_wh, stride_wh, groups: int) -> "Array":
        """A rank+3 strided view of [..., h, w, c] (src/array.rs:559-600)."""
        in_shape = self.shape
        n = len(in_shape)
        y_axis, x_axis, c_axis = n - 3, n - 2, n - 1
        out_shape = in_shape.image_to_windows(filter_wh, stride_wh, groups)
        group_nc = out_shape[-1]
        sw, sh = stride_wh
        ident = in_shape.identity_view()

        def stepped(axis, mult):
            a, st = ident.mapping[axis]
            return (a, st * mult) if a >= 0 else (a, st)

        mapping = list(ident.mapping[: len(out_shape) - 6])
        mapping += [
            stepped(y_axis, sh),
            stepped(x_axis, sw),
            stepped(c_axis, group_nc),
            ident.mapping[y_axis],
            ident.mapping[x_axis],
            ident.mapping[c_axis],
        ]
        return self.view(View(in_shape, ident.input_offsets, tuple(mapping), out_shape))

    def windows_to_image(self, stride_wh) -> "Array":
        s = self.scope
        shape = self.shape.windows_to_image(stride_wh)
        return Array(s.ops.new_node(s.colour, shape, Op("WindowsToImage", tuple(stride_wh)), [self.node_id]), s)


class DualArray:
    """(value, d loss / d value) pair (src/array.rs:20-25, 794-1147)."""

    __slots__ = ("value_node_id", "loss_grad_node_id", "scope")

    def __init__(self, value: Array, loss_grad: Array):
        self.value_node_id = value.node_id
        self.loss_grad_node_id = loss_grad.node_id
        self.scope = value.scope

    def value(self) -> Array:
        return Array(self.value_node_id, self.scope)

    def loss_grad(self) -> Array:
        return Array(self.loss_grad_node_id, self.scope)

    def into_inner(self) -> Tuple[Array, Array]:
        return self.value(), self.loss_grad()

    @property
    def shape(self) -> Shape:
        return self.value().shape

    def _lift(self, value) -> "DualArray":
        """IntoDualArray (src/array.rs:60-77)."""
        if isinstance(value, DualArray):
            return value
        if isinstance(value, Parameter):
            return self.scope.parameter(value)
        if isinstance(value, Array):
            raise TypeError("an Array has no gradient; wrap it explicitly")
        return self.scope.literal(float(value))

    def next_colour(self) -> "DualArray":
        self.scope.next_colour()
        return self

    def map(self, f: Callable[["DualArray"], "DualArray"]) -> "DualArray":
        return f(self)

    def apply(self, module, ctx) -> "DualArray":
        return module.eval(self, ctx)

    # -- elementwise ---------------------------------------------------------------
    def square(self):
        return self * self

    def sin(self):
        a, da = self.into_inner()
        b, db = a.sin().with_empty_grad()
        da.accumulate(db * a.cos())
        return DualArray(b, db)

    def tanh(self):
        a, da = self.into_inner()
        b, db = a.tanh().with_empty_grad()
        da.accumulate(db * 4.0 / ((2.0 * a).exp() + 2.0 + (-2.0 * a).exp()))
        return DualArray(b, db)

    def sigmoid(self):
        a, da = self.into_inner()
        b, db = a.sigmoid().with_empty_grad()
        da.accumulate(db * a.exp() / (a.exp() + 1.0).square())
        return DualArray(b, db)

    def leaky_relu(self, leakiness: float):
        """src/array.rs:860-867"""
        a, da = self.into_inner()
        b, db = a.select_gt(0.0, a, a * leakiness).with_empty_grad()
        da.accumulate(a.select_gt(0.0, db, db * leakiness))
        return DualArray(b, db)

    def pow(self, rhs):
        a, da = self.into_inner()
        b, db = self._lift(rhs).into_inner()
        c, dc = a.pow(b).with_empty_grad()
        da.accumulate((dc * b * a.pow(b - 1.0)).unbroadcast(a.shape))
        db.accumulate((dc * a.log() * c).unbroadcast(b.shape))
        return DualArray(c, dc)

    def select_eq(self, rhs, on_pass, on_fail):
        a, _ = self.into_inner()
        b, _ = self._lift(rhs).into_inner()
        p, dp = self._lift(on_pass).into_inner()
        f, df = self._lift(on_fail).into_inner()
        c, dc = a.select_eq(b, p, f).with_empty_grad()
        dp.accumulate(a.select_eq(b, dc, 0.0).unbroadcast(p.shape))
        df.accumulate(a.select_eq(b, 0.0, dc).unbroadcast(f.shape))
        return DualArray(c, dc)

    def __add__(self, rhs):
        rhs = self._lift(rhs)
        a, da = self.into_inner()
        b, db = rhs.into_inner()
        c, dc = (a + b).with_empty_grad()
        da.accumulate(dc.unbroadcast(a.shape))
        db.accumulate(dc.unbroadcast(b.shape))
        return DualArray(c, dc)

    def __sub__(self, rhs):
        rhs = self._lift(rhs)
        a, da = self.into_inner()
        b, db = rhs.into_inner()
        c, dc = (a - b).with_empty_grad()
        da.accumulate(dc.unbroadcast(a.shape))
        db.accumulate(-dc.unbroadcast(b.shape))
        return DualArray(c, dc)

    def __mul__(self, rhs):
        rhs = self._lift(rhs)
        a, da = self.into_inner()
        b, db = rhs.into_inner()
        c, dc = (a * b).with_empty_grad()
        da.accumulate((b * dc).unbroadcast(a.shape))
        db.accumulate((a * dc).unbroadcast(b.shape))
        return DualArray(c, dc)

    # -- structure -------------------------------------------------------------------
    def transpose(self):
        a, da = self.into_inner()
        b, db = a.transpose().with_empty_grad()
        da.accumulate(db.transpose())
        return DualArray(b, db)

    def reshape(self, shape):
        old = self.shape
        a, da = self.into_inner()
        b, db = a.reshape(shape).with_empty_grad()
        da.accumulate(db.reshape(old))
        return DualArray(b, db)

    def flatten(self):
        shape = self.shape
        return self.reshape([shape[0], Shape(shape[1:]).element_count()])

    def insert_axis(self, axis: int):
        a, da = self.into_inner()
        b, db = a.insert_axis(axis).with_empty_grad()
        da.accumulate(db.remove_axis(axis))
        return DualArray(b, db)

    def remove_axis(self, axis: int):
        a, da = self.into_inner()
        b, db = a.remove_axis(axis).with_empty_grad()
        da.accumulate(db.insert_axis(axis))
        return DualArray(b, db)

    def _keep_axis(self, axis: int, keep: bool):
        return self if keep else self.remove_axis(axis)

    def permute_axes(self, perm: Sequence[int]):
        inv = [0] * len(perm)
        for src, dst in enumerate(perm):
            inv[dst] = src
        a, da = self.into_inner()
        b, db = a.permute_axes(perm).with_empty_grad()
        da.accumulate(db.permute_axes(inv))
        return DualArray(b, db)

    def lock_axis(self, axis: int, coord: int, keep_axis: bool):
        """src/array.rs:928-940"""
        axis = _axis(axis, self.shape)
        a, da = self.into_inner()
        b, db = a.lock_axis(axis, coord, True).with_empty_grad()
        da.accumulate(a.coord(axis).select_eq(float(coord), db, 0.0))
        return DualArray(b, db)._keep_axis(axis, keep_axis)

    def concat(self, other, axis: int):
        other = self._lift(other)
        shape = self.shape
        axis = _axis(axis, shape)
        length = shape[axis]
        a, da = self.into_inner()
        b, db = other.into_inner()
        c, dc = a.concat(b, axis).with_empty_grad()
        da.accumulate(dc.limit_axis(axis, None, length))
        db.accumulate(dc.limit_axis(axis, length, None))
        return DualArray(c, dc)

    # -- reductions ------------------------------------------------------------------
    def _reduce(self, name: str, axis: int):
        """src/array.rs:1049-1059: max routes the gradient to every element
        equal to the maximum (ties receive it more than once)."""
        a, da = self.into_inner()
        b, db = a._reduce(name, axis).with_empty_grad()
        if name == "Max":
            da.accumulate(a.select_eq(b, db, 0.0))
        else:
            da.accumulate(db.broadcast(da.shape))
        return DualArray(b, db)

    def reduce_sum(self, axis: int, keep_axis: bool):
        axis = _axis(axis, self.shape)
        return self._reduce("Sum", axis)._keep_axis(axis, keep_axis)

    def reduce_max(self, axis: int, keep_axis: bool):
        axis = _axis(axis, self.shape)
        return self._reduce("Max", axis)._keep_axis(axis, keep_axis)

    # -- matmul / conv ---------------------------------------------------------------
    def batched_matmul(self, rhs: "DualArray", output_mode: int):
        """src/array.rs:869-878"""
        a, da = self.into_inner()
        b, db = rhs.into_inner()
        c, dc = a.batched_matmul(b, output_mode).with_empty_grad()
        da.accumulate(dc.batched_matmul(b.transpose(), BATCHES))
        db.accumulate(a.transpose().batched_matmul(dc, BATCHES))
        return DualArray(c, dc)

    def matmul(self, rhs):
        lhs = self.insert_axis(0)
        rhs = self._lift(rhs).insert_axis(0)
        return lhs.batched_matmul(rhs, BATCHES).remove_axis(0)

    def pad_image(self, pad: int):
        a, da = self.into_inner()
        b, db = a.pad_image(pad).with_empty_grad()
        da.accumulate(db.unpad_image(pad))
        return DualArray(b, db)

    def image_to_windows(self, filter_wh, stride_wh, groups: int):
        a, da = self.into_inner()
        b, db = a.image_to_windows(filter_wh, stride_wh, groups).with_empty_grad()
        da.accumulate(db.windows_to_image(stride_wh))
        return DualArray(b, db)

    def conv2d(self, filt, pad: int, stride_wh=(1, 1)):
        """NHWC input, filter [groups, oc/groups, fh, fw, ic/groups]; lowered to
        pad -> windows view -> batched matmul over groups in Rows mode
        (src/array.rs:989-1031)."""
        filt = self._lift(filt)
        padded = self.pad_image(pad)
        input_m, _, _, input_nc = padded.shape
        fg, foc, fh, fw, fic = filt.shape
        if input_nc != fg * fic:
            raise ValueError("conv2d channel mismatch")
        windows = padded.image_to_windows((fw, fh), stride_wh, fg)
        wm, oh, ow, wg, wfh, wfw, wnc = windows.shape
        assert (wm, wg, wfh, wfw, wnc) == (input_m, fg, fh, fw, fic)
        a = windows.reshape([input_m * oh * ow, fg, fh * fw * fic]).permute_axes([1, 0, 2])
        b = filt.reshape([fg, foc, fh * fw * fic])
        c = a.batched_matmul(b.transpose(), ROWS)
        return c.permute_axes([1, 0, 2]).reshape([input_m, oh, ow, fg * foc])

    def max_pool2d(self, filter_wh, stride_wh):
        """src/array.rs:1033-1047"""
        windows = self.image_to_windows(filter_wh, stride_wh, 1)
        m, oh, ow, g, fh, fw, nc = windows.shape
        return (
            windows.reshape([m * oh * ow * g, fh * fw, nc]).reduce_max(1, True).reshape([m, oh, ow, g * nc])
        )

    def set_loss(self) -> Array:
        self.loss_grad()._set_loss_grad_root()
        return self.value()


class Parameter:
    """Named device-resident tensor owned by an Environment
    (src/parameter.rs:28-73). `buffer` is the only device-facing field."""

    def __init__(self, owner, shape, name: str, reset_to=None):
        self.owner = owner
        self.shape = Shape(shape)
        self.name = name
        self.reset_to = reset_to
        self.buffer = None  # backend buffer handle or None

    def is_trainable(self) -> bool:
        return self.reset_to is not None

    def checked(self, owner) -> "Parameter":
        if self.owner is not owner:
            raise ValueError("parameter does not come from the same environment")  # src/parameter.rs:51-56
        return self

    def __repr__(self):
        return f"Parameter({self.name!r}, {self.shape!r})"


class Scope:
    """Collects ops for one graph (src/array.rs:1222-1442)."""

    def __init__(self, owner):
        self.owner = owner
        self.ops = OpGraph()
        self.colour = 0
        self._next_rand_uid = 0
        self._inputs = {}  # Parameter -> (value_node, grad_node or None)
        self._outputs = {}  # Parameter -> Output node id

    def next_colour(self):
        self.colour += 1

    def literal(self, value: float) -> DualArray:
        nid = self.ops.new_node(self.colour, [1], Op("Literal", Literal.f32(value)))
        return DualArray(*Array(nid, self).with_empty_grad())

    def literal_u32(self, value: int) -> Array:
        return Array(self.ops.new_node(self.colour, [1], Op("Literal", Literal.u32(value))), self, True)

    def coord(self, length: int) -> DualArray:
        nid = self.ops.new_node(self.colour, [length], Op("Coord"))
        return DualArray(*Array(nid, self).with_empty_grad())

    def rand(self, shape) -> DualArray:
        """Uniform [0,1] values; each call gets its own stream id
        (src/array.rs:1300-1317)."""
        uid = self._next_rand_uid
        self._next_rand_uid += 1
        nid = self.ops.new_node(self.colour, Shape(shape), Op("Rand", uid))
        return DualArray(*Array(nid, self).with_empty_grad())

    def _input(self, parameter: Parameter):
        parameter.checked(self.owner)
        if parameter not in self._inputs:
            value = self.ops.new_node(self.colour, parameter.shape, Op("Input", parameter))
            grad = self.ops.new_node(self.colour, parameter.shape, MOV)
            self._inputs[parameter] = (value, grad)
        return self._inputs[parameter]

    def parameter(self, parameter: Parameter) -> DualArray:
        value, grad = self._input(parameter)
        if grad is None:
            raise ValueError("parameter was already written in this scope; it has no gradient")
        return DualArray(Array(value, self), Array(grad, self))

    def parameter_value(self, parameter: Parameter) -> Array:
        return Array(self._input(parameter)[0], self)

    def write_parameter_value(self, parameter: Parameter, rhs: Array) -> None:
        """src/array.rs:1363-1392: later reads in this scope see `rhs`."""
        parameter.checked(self.owner)
        if tuple(parameter.shape) != tuple(rhs.shape):
            raise ValueError(f"write_parameter_value shape mismatch {parameter.shape!r} vs {rhs.shape!r}")
        nid = self.ops.new_node(self.colour, rhs.shape, Op("Output", parameter), [rhs.node_id])
        old = self._outputs.get(parameter)
        if old is not None:
            self.ops.remove_node(old)
        self._outputs[parameter] = nid
        self._inputs[parameter] = (rhs.node_id, None)

    def update_parameter_value(self, parameter: Parameter, f: Callable[[Array], Array]) -> Array:
        result = f(self.parameter_value(parameter))
        self.write_parameter_value(parameter, result)
        return result

    def accumulator(self, shape) -> Array:
        return Array(self.ops.new_node(self.colour, Shape(shape), MOV), self)

    def trainable_parameters(self) -> List[Parameter]:
        out = []
        for nid in sorted(self.ops.nodes):
            op = self.ops.nodes[nid].op
            if op.kind == "Input" and op.a.is_trainable():
                out.append(op.a)
        return out

    def build_graph(self) -> Graph:
        return Graph(self.ops.clone())
