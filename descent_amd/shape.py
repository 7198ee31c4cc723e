"""Shapes and views: the address algebra every kernel reads memory through.

Host-side mirror of the reference's `Shape` / `View` (src/shape.rs).  A `View`
describes how an op reads its argument: per input axis an offset plus a sum of
(step * output coordinate) terms, clamped to the input extent when the
reachable range leaves it (edge-replicate padding, src/shape.rs:374-379 and
:503-526).  Views are immutable value objects: equality and hashing are by
content because kernel descriptors are cache keys (src/kernel.rs:1037-1056).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Optional, Sequence, Tuple

MAX_DIM = 7  # src/shape.rs:10
MATMUL_MAX_K_SIZE = 1024  # src/op.rs:74

BATCHES = 0  # MatMulOutputMode::Batches (src/op.rs:76-80)
ROWS = 1  # MatMulOutputMode::Rows


def div_round_up(a: int, b: int) -> int:
    return (a + b - 1) // b


class Shape(tuple):
    """Dense row-major extent, 1..MAX_DIM axes, all > 0 (src/shape.rs:40-48)."""

    def __new__(cls, dims: Iterable[int]):
        dims = tuple(int(d) for d in dims)
        if not dims or len(dims) > MAX_DIM:
            raise ValueError(f"shape rank must be 1..{MAX_DIM}, got {dims}")
        if any(d <= 0 for d in dims):
            raise ValueError(f"shape extents must be positive, got {dims}")
        return super().__new__(cls, dims)

    def __repr__(self):
        return "[" + ", ".join(str(d) for d in self) + "]"

    # -- basic queries -----------------------------------------------------
    def axis(self, index: int) -> int:
        """Negative indices address from the end (src/shape.rs:174-177)."""
        a = index + len(self) if index < 0 else index
        if not 0 <= a < len(self):
            raise IndexError(f"axis {index} out of range for {self!r}")
        return a

    def element_count(self) -> int:
        n = 1
        for d in self:
            n *= d
        return n

    def buffer_size(self) -> int:
        return 4 * self.element_count()

    def strides(self) -> Tuple[int, ...]:
        out = []
        s = 1
        for d in reversed(self):
            out.append(s)
            s *= d
        return tuple(reversed(out))

    # -- derived shapes ----------------------------------------------------
    def _replace(self, axis: int, value: int) -> "Shape":
        d = list(self)
        d[axis] = value
        return Shape(d)

    def prefix_ones_to_len(self, n: int) -> "Shape":
        return Shape((1,) * max(0, n - len(self)) + tuple(self))

    def broadcast_with(self, rhs: "Shape") -> "Shape":
        """numpy-style broadcast of two shapes (src/shape.rs:73-92)."""
        n = max(len(self), len(rhs))
        a, b = self.prefix_ones_to_len(n), rhs.prefix_ones_to_len(n)
        out = []
        for x, y in zip(a, b):
            if x == 1:
                out.append(y)
            elif y == 1 or x == y:
                out.append(x)
            else:
                raise ValueError(f"cannot broadcast {self!r} with {rhs!r}")
        return Shape(out)

    def batched_matmul(self, rhs: "Shape", output_mode: int) -> "Shape":
        """[b,m,k] x [b,k,n] -> [r,b,m,n] or [r,m,b,n], r = ceil(k/1024)
        split-K partials (src/shape.rs:94-104)."""
        if len(self) != 3 or len(rhs) != 3:
            raise ValueError("batched_matmul needs rank-3 operands")
        b0, m, k0 = self
        b1, k1, n = rhs
        if b0 != b1 or k0 != k1:
            raise ValueError(f"matmul shape mismatch {self!r} x {rhs!r}")
        r = div_round_up(k0, MATMUL_MAX_K_SIZE)
        return Shape((r, b0, m, n)) if output_mode == BATCHES else Shape((r, m, b0, n))

    def pad(self, axis: int, before: int, after: int) -> "Shape":
        return self._replace(axis, self[axis] + before + after)

    def unpad(self, axis: int, pad: int) -> "Shape":
        return self._replace(axis, self[axis] - 2 * pad)

    def reduce(self, axis: int) -> "Shape":
        return self._replace(axis, 1)

    def resize_axis(self, axis: int, length: int) -> "Shape":
        return self._replace(axis, length)

    def coord(self, axis: int) -> "Shape":
        """All ones except `axis` (src/shape.rs:193-198)."""
        return Shape(d if i == axis else 1 for i, d in enumerate(self))

    def insert_axis(self, axis: int, length: int) -> "Shape":
        d = list(self)
        d.insert(axis, length)
        return Shape(d)

    def remove_axis(self, axis: int) -> "Shape":
        d = list(self)
        del d[axis]
        return Shape(d)

    def image_to_windows(self, filter_wh, stride_wh, groups: int) -> "Shape":
        """[..., h, w, c] -> [..., oh, ow, groups, fh, fw, c/groups]
        (src/shape.rs:120-141). Tuples are (w, h) as in the reference."""
        if len(self) < 3:
            raise ValueError("image_to_windows needs [..., h, w, c]")
        prefix, (in_h, in_w, in_nc) = tuple(self[:-3]), self[-3:]
        if in_nc % groups:
            raise ValueError("channels not divisible by groups")
        fw, fh = filter_wh
        sw, sh = stride_wh
        out_w = (in_w - fw) // sw + 1
        out_h = (in_h - fh) // sh + 1
        if (out_w - 1) * sw != in_w - fw or (out_h - 1) * sh != in_h - fh:
            raise ValueError("filter/stride do not tile the image exactly")
        return Shape(prefix + (out_h, out_w, groups, fh, fw, in_nc // groups))

    def windows_to_image(self, stride_wh) -> "Shape":
        """Inverse of image_to_windows (src/shape.rs:143-156)."""
        if len(self) < 6:
            raise ValueError("windows_to_image needs [..., oh, ow, g, fh, fw, c]")
        prefix = tuple(self[:-6])
        out_h, out_w, groups, fh, fw, group_nc = self[-6:]
        sw, sh = stride_wh
        return Shape(prefix + ((out_h - 1) * sh + fh, (out_w - 1) * sw + fw, groups * group_nc))

    def identity_view(self) -> "View":
        return View.identity(self)

    def padded_view(self, axis: int, before: int, after: int) -> "View":
        return View.padded(self, axis, before, after)


BROADCAST = -1  # AxisMapping::Broadcast (src/shape.rs:322-325)


def _mapping(axis: int, length: int) -> Tuple[int, int]:
    """AxisMapping::new (src/shape.rs:334-341): a length-1 axis never steps."""
    return (axis, 1) if length > 1 else (BROADCAST, 0)


@dataclass(frozen=True)
class View:
    """src/shape.rs:354-360. `mapping[j] = (input_axis, step)` or
    `(BROADCAST, 0)` for each output axis j."""

    input_shape: Shape
    input_offsets: Tuple[int, ...]
    mapping: Tuple[Tuple[int, int], ...]
    output_shape: Shape

    def __post_init__(self):
        assert len(self.input_offsets) == len(self.input_shape)
        assert len(self.mapping) == len(self.output_shape)

    # -- constructors ------------------------------------------------------
    @staticmethod
    def identity(shape: Shape) -> "View":
        shape = Shape(shape)
        return View(shape, (0,) * len(shape), tuple(_mapping(i, d) for i, d in enumerate(shape)), shape)

    @staticmethod
    def padded(shape: Shape, axis: int, before: int, after: int) -> "View":
        """Negative offset + clamp = replicate padding (src/shape.rs:374-379)."""
        v = View.identity(shape)
        off = list(v.input_offsets)
        off[axis] = -before
        return View(v.input_shape, tuple(off), v.mapping, v.output_shape.pad(axis, before, after))

    @staticmethod
    def limited(shape: Shape, axis: int, start: int, end: int) -> "View":
        """Sub-range [start, end) of one axis (src/shape.rs:381-401)."""
        v = View.identity(shape)
        off = list(v.input_offsets)
        off[axis] = start
        mp = list(v.mapping)
        mp[axis] = _mapping(axis, end - start)
        return View(v.input_shape, tuple(off), tuple(mp), v.output_shape.resize_axis(axis, end - start))

    @staticmethod
    def broadcast(input_shape: Shape, output_shape: Shape) -> "View":
        """src/shape.rs:578-602."""
        input_shape, output_shape = Shape(input_shape), Shape(output_shape)
        if len(input_shape) > len(output_shape):
            raise ValueError(f"cannot broadcast {input_shape!r} to {output_shape!r}")
        lead = len(output_shape) - len(input_shape)
        mp = [(BROADCAST, 0)] * lead
        for i, (src, dst) in enumerate(zip(input_shape, output_shape[lead:])):
            if src == dst:
                mp.append(_mapping(i, src))
            elif src == 1:
                mp.append((BROADCAST, 0))
            else:
                raise ValueError(f"cannot broadcast {input_shape!r} to {output_shape!r}")
        return View(input_shape, (0,) * len(input_shape), tuple(mp), output_shape)

    @staticmethod
    def try_from_reshape(input_shape: Shape, output_shape: Shape) -> Optional["View"]:
        """A reshape that only inserts/removes length-1 axes is a view
        (src/shape.rs:421-455)."""
        if tuple(input_shape) == tuple(output_shape):
            return View.identity(input_shape)
        mp = []
        for in_axis, in_len in enumerate(input_shape):
            if in_len == 1:
                continue
            while True:
                if len(mp) >= len(output_shape):
                    return None
                out_len = output_shape[len(mp)]
                if out_len == in_len:
                    mp.append(_mapping(in_axis, in_len))
                    break
                if out_len != 1:
                    return None
                mp.append((BROADCAST, 0))
        while len(mp) < len(output_shape):
            assert output_shape[len(mp)] == 1
            mp.append((BROADCAST, 0))
        return View(Shape(input_shape), (0,) * len(input_shape), tuple(mp), Shape(output_shape))

    # -- queries -----------------------------------------------------------
    def is_identity(self) -> bool:
        return self == View.identity(self.output_shape)

    def is_contiguous(self) -> bool:
        """Same linear element order as the input (src/shape.rs:403-419)."""
        if self.input_shape.element_count() != self.output_shape.element_count():
            return False
        if any(self.input_offsets):
            return False
        in_strides = self.input_shape.strides()
        for (axis, step), out_stride in zip(self.mapping, self.output_shape.strides()):
            if axis != BROADCAST and in_strides[axis] * step != out_stride:
                return False
        return True

    def _span(self, input_axis: int) -> Tuple[int, int]:
        lo = hi = self.input_offsets[input_axis]
        for (axis, step), length in zip(self.mapping, self.output_shape):
            if axis == input_axis:
                d = (length - 1) * step
                lo += min(d, 0)
                hi += max(d, 0)
        return lo, hi

    def input_needs_clamp(self, input_axis: int) -> bool:
        """src/shape.rs:503-526."""
        lo, hi = self._span(input_axis)
        return lo < 0 or hi > self.input_shape[input_axis] - 1

    def _input_axis_mapping_count(self, input_axis: int) -> int:
        return sum(1 for axis, _ in self.mapping if axis == input_axis)

    def _can_pad_output(self, output_axis: int) -> bool:
        """src/shape.rs:467-488."""
        axis, step = self.mapping[output_axis]
        if axis == BROADCAST:
            return True
        if self._input_axis_mapping_count(axis) != 1:
            return False
        base = self.input_offsets[axis]
        d = (self.output_shape[output_axis] - 1) * step
        return base + min(d, 0) <= 0 and self.input_shape[axis] - 1 <= base + max(d, 0)

    def _can_combine_with(self, view: "View") -> bool:
        """src/shape.rs:490-496."""
        return tuple(self.output_shape) == tuple(view.input_shape) and all(
            self._can_pad_output(a) or not view.input_needs_clamp(a) for a in range(len(self.output_shape))
        )

    def _can_reshape_to(self, view: "View") -> bool:
        return self.is_contiguous() and self.output_shape.element_count() == view.input_shape.element_count()

    def can_view_through(self, view: "View", can_reshape: bool) -> bool:
        """src/shape.rs:528-530."""
        return self._can_combine_with(view) or (can_reshape and self._can_reshape_to(view))

    def through(self, view: "View", can_reshape: bool) -> "View":
        """Compose: read `self`'s output through `view` (src/shape.rs:532-567)."""
        if not self._can_combine_with(view):
            assert can_reshape and self._can_reshape_to(view)
            return view
        off = list(self.input_offsets)
        for (axis, step), o in zip(self.mapping, view.input_offsets):
            if axis != BROADCAST:
                off[axis] += step * o
        mp = []
        for axis, step in view.mapping:
            if axis == BROADCAST:
                mp.append((BROADCAST, 0))
            else:
                ia, istep = self.mapping[axis]
                mp.append((BROADCAST, 0) if ia == BROADCAST else (ia, istep * step))
        return View(self.input_shape, tuple(off), tuple(mp), view.output_shape)

    def transposed(self) -> "View":
        n = len(self.mapping)
        assert n >= 2
        perm = list(range(n))
        perm[-2], perm[-1] = perm[-1], perm[-2]
        return self.permute_axes(perm)

    def permute_axes(self, perm: Sequence[int]) -> "View":
        """src/shape.rs:627-635."""
        return View(
            self.input_shape,
            self.input_offsets,
            tuple(self.mapping[i] for i in perm),
            Shape(self.output_shape[i] for i in perm),
        )

    def load_in_columns_hint(self) -> bool:
        """src/shape.rs:614-625 (only a load-order hint for the reference's
        matmul shader; kept for descriptor completeness)."""
        if len(self.mapping) < 2:
            return False
        oa, os_ = self.mapping[-2]
        ia, is_ = self.mapping[-1]
        if oa == BROADCAST or ia == BROADCAST:
            return False
        if oa == ia:
            return abs(os_) < abs(is_)
        return oa > ia

    # -- evaluation (host side; used by tests and the interpreter) -----------
    def load_index(self, coord: Sequence[int]) -> int:
        """Linear input element read for one output coordinate
        (src/kernel.rs:89-133 generate_load_coord / generate_load_index)."""
        strides = self.input_shape.strides()
        total = 0
        for axis in range(len(self.input_shape)):
            c = self.input_offsets[axis]
            for (a, step), oc in zip(self.mapping, coord):
                if a == axis:
                    c += step * oc
            if self.input_needs_clamp(axis):
                c = min(max(c, 0), self.input_shape[axis] - 1)
            total += c * strides[axis]
        return total
