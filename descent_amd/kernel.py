"""Kernel descriptors: the seven kinds of device work a graph lowers to.

Host-side mirror of `GenericKernel` and its variants (src/kernel.rs:146-886).
A descriptor is a hashable value; equal descriptors share one compiled kernel
(src/kernel.rs:1037-1056).  Code generation and launch live behind the C ABI;
these classes only carry the data and the reference's reporting helpers
(`label_name`, `group_count`, `buffer_count`, src/kernel.rs:135-143).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass
from typing import Tuple, Union

from .shape import Shape, View, div_round_up, BATCHES, ROWS

# ---- op vocabularies (src/op.rs:22-70); values match include/descent_hip.h ----
UNARY_OPS = ("Mov", "Neg", "Sqrt", "Exp", "Log", "Sin", "Cos", "FloatToUint", "UintToFloat")
BINARY_OPS = ("Add", "Sub", "Mul", "Div", "Pow", "UAdd", "UMul", "URem", "UBitXor")
COMPARE_MODES = ("Eq", "Gt")
REDUCE_OPS = ("Max", "Sum")


def f32_bits(value: float) -> int:
    return struct.unpack("<I", struct.pack("<f", value))[0]


def bits_f32(bits: int) -> float:
    return struct.unpack("<f", struct.pack("<I", bits & 0xFFFFFFFF))[0]


@dataclass(frozen=True)
class Literal:
    """src/op.rs:22-26: an f32 value or a u32 bit pattern, stored as bits."""

    is_u32: bool
    bits: int

    @staticmethod
    def f32(value: float) -> "Literal":
        if value != value:
            raise ValueError("literal must not be NaN")  # NotNan<f32>
        return Literal(False, f32_bits(value))

    @staticmethod
    def u32(value: int) -> "Literal":
        return Literal(True, value & 0xFFFFFFFF)

    def __repr__(self):
        return f"U32({self.bits})" if self.is_u32 else f"F32({bits_f32(self.bits)!r})"


# ---- per-element ops (src/kernel.rs:8-35) -------------------------------------
@dataclass(frozen=True)
class PeLoad:
    input_index: int


@dataclass(frozen=True)
class PeLiteral:
    value: Literal


@dataclass(frozen=True)
class PeCoord:
    view: View


@dataclass(frozen=True)
class PeRand:
    uid: int
    view: View


@dataclass(frozen=True)
class PeUnary:
    op: str
    arg: int


@dataclass(frozen=True)
class PeBinary:
    op: str
    args: Tuple[int, int]


@dataclass(frozen=True)
class PeSelect:
    compare_mode: str
    args: Tuple[int, int, int, int]


@dataclass(frozen=True)
class PeGather:
    shape: Shape
    axis: int
    input_index: int
    arg: int


PeOp = Union[PeLoad, PeLiteral, PeCoord, PeRand, PeUnary, PeBinary, PeSelect, PeGather]


# ---- kernels -----------------------------------------------------------------
@dataclass(frozen=True)
class FillKernel:
    """src/kernel.rs:146-193"""

    value: Literal
    element_count: int

    def buffer_count(self):
        return 1

    def group_count(self):
        return div_round_up(self.element_count, 64)

    def label_name(self):
        return f"Fill({self.value!r}) {self.element_count}"


@dataclass(frozen=True)
class PerElementKernel:
    """src/kernel.rs:196-383"""

    element_count: int
    inputs: Tuple[View, ...]
    outputs: Tuple[int, ...]
    ops: Tuple[PeOp, ...]

    def buffer_count(self):
        return len(self.inputs) + len(self.outputs)

    def group_count(self):
        return div_round_up(self.element_count, 64)

    def label_name(self):
        return f"PerElement ({len(self.ops)} ops) [{self.element_count}]"


@dataclass(frozen=True)
class MatMulKernel:
    """src/kernel.rs:386-557. `shape` is [r,b,m,n] (Batches) or [r,m,b,n]
    (Rows) with r split-K partials."""

    shape: Shape
    output_mode: int
    a: View
    b: View

    @property
    def m(self):
        return self.a.output_shape[-2]

    @property
    def n(self):
        return self.b.output_shape[-1]

    @property
    def k(self):
        return self.a.output_shape[-1]

    @property
    def k_chunk_count(self):
        return self.shape[0]

    @property
    def batch_count(self):
        return self.shape[1 if self.output_mode == BATCHES else 2]

    def buffer_count(self):
        return 3

    def group_count(self):
        return self.batch_count * self.k_chunk_count * div_round_up(self.m, 16) * div_round_up(self.n, 16)

    def label_name(self):
        return f"MatMul (k={self.k}) {self.shape!r}"


@dataclass(frozen=True)
class ReduceKernel:
    """src/kernel.rs:560-642"""

    shape: Shape
    input: View
    reduce_op: str
    axis: int

    @property
    def k(self):
        return self.input.output_shape[self.axis]

    def buffer_count(self):
        return 2

    def group_count(self):
        return div_round_up(self.shape.element_count(), 64)

    def label_name(self):
        return f"Reduce (k={self.k}) {self.shape!r}"


@dataclass(frozen=True)
class UnpadKernel:
    """src/kernel.rs:645-710"""

    shape: Shape
    input: View
    axis: int
    pad: int

    def buffer_count(self):
        return 2

    def group_count(self):
        return div_round_up(self.shape.element_count(), 64)

    def label_name(self):
        return f"Unpad {self.shape!r}"


@dataclass(frozen=True)
class WindowsToImageKernel:
    """src/kernel.rs:713-810. `stride` is (w, h)."""

    shape: Shape
    input: View
    stride: Tuple[int, int]

    def buffer_count(self):
        return 2

    def group_count(self):
        return div_round_up(self.shape.element_count(), 64)

    def label_name(self):
        return f"WindowsToImage {self.shape!r}"


@dataclass(frozen=True)
class ScatterAddKernel:
    """src/kernel.rs:813-874"""

    shape: Shape
    values: View
    axis: int
    indices: View

    def buffer_count(self):
        return 3

    def group_count(self):
        return div_round_up(self.values.output_shape.element_count(), 64)

    def label_name(self):
        return f"ScatterAdd {self.values.output_shape!r}"


GenericKernel = Union[
    FillKernel, PerElementKernel, MatMulKernel, ReduceKernel, UnpadKernel, WindowsToImageKernel, ScatterAddKernel
]
