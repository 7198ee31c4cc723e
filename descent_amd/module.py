"""Layer building blocks; every one lowers to array ops.

Host-side mirror of src/module.rs (Dense :37-90, Conv2D :92-215, MaxPool2D
:217-224, MaxBlurPool2D :226-252, Dropout :254-279).  Images are NHWC, conv
filters are [groups, oc/groups, fh, fw, ic/groups], dense weights [in, out].
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

from .array import DualArray, Parameter


@dataclass(frozen=True)
class Initializer:
    """src/parameter.rs:10-26"""

    kind: str  # "zero" | "normal" | "uniform"
    scale: float = 0.0

    @staticmethod
    def zero():
        return Initializer("zero")

    @staticmethod
    def rand_normal(scale: float):
        return Initializer("normal", float(np.float32(scale)))

    @staticmethod
    def rand_uniform(scale: float):
        return Initializer("uniform", float(np.float32(scale)))

    @staticmethod
    def for_relu(fan_in: int):
        return Initializer.rand_normal(float(np.sqrt(np.float32(2.0) / np.float32(fan_in))))

    @staticmethod
    def for_siren(fan_in: int, is_first_layer: bool):
        scale = np.sqrt(np.float32(6.0) / np.float32(fan_in)) * np.float32(30.0 if is_first_layer else 1.0)
        return Initializer.rand_uniform(float(scale))


@dataclass(frozen=True)
class EvalContext:
    is_training: bool


class Module:
    def eval(self, x: DualArray, ctx: EvalContext) -> DualArray:
        raise NotImplementedError

    def train(self, x: DualArray) -> DualArray:
        return self.eval(x, EvalContext(True))

    def test(self, x: DualArray) -> DualArray:
        return self.eval(x, EvalContext(False))


class Dense(Module):
    def __init__(self, env, n_in: int, n_out: int, w_initializer=None, b_initializer=None):
        self.w = env.trainable_parameter([n_in, n_out], "w", w_initializer or Initializer.for_relu(n_in))
        self.b = env.trainable_parameter([n_out], "b", b_initializer or Initializer.zero())

    def eval(self, x, ctx):
        return x.next_colour().matmul(self.w) + self.b


class Conv2D(Module):
    def __init__(self, env, in_channels, out_channels, filter_w, filter_h, pad=0, stride=(1, 1), groups=1,
                 is_blur=False):
        fic, foc = in_channels // groups, out_channels // groups
        if fic * groups != in_channels or foc * groups != out_channels:
            raise ValueError("channels not divisible by groups")
        shape = [groups, foc, filter_h, filter_w, fic]
        if is_blur:
            # fixed 3x3 binomial filter per channel (src/module.rs:141-167)
            assert [foc, filter_h, filter_w, fic] == [1, 3, 3, 1]
            self.f = env.static_parameter(shape, "f")
            self.b = env.static_parameter([out_channels], "b")
            taps = np.array([1, 2, 1, 2, 4, 2, 1, 2, 1], dtype=np.float32) / np.float32(16.0)
            env.write_parameter(self.f, np.tile(taps, groups))
            env.writer(self.b).zero_fill()
        else:
            self.f = env.trainable_parameter(shape, "f", Initializer.for_relu(filter_h * filter_w * fic))
            self.b = env.trainable_parameter([out_channels], "b", Initializer.zero())
        self.pad = pad
        self.stride = tuple(stride)

    def eval(self, x, ctx):
        return x.next_colour().conv2d(self.f, self.pad, self.stride) + self.b


class MaxPool2D(Module):
    def eval(self, x, ctx):
        return x.next_colour().max_pool2d((2, 2), (2, 2))


class MaxBlurPool2D(Module):
    def __init__(self, env, channels: int):
        self.blur = Conv2D(env, channels, channels, 3, 3, pad=1, stride=(2, 2), groups=channels, is_blur=True)

    def eval(self, x, ctx):
        return self.blur.eval(x.next_colour().max_pool2d((2, 2), (1, 1)), ctx)


class Dropout(Module):
    """Inverted dropout from the counter-based generator; forward and backward
    evaluate the same Rand node so the masks agree (src/module.rs:254-279)."""

    def __init__(self, amount: float):
        self.amount = amount

    def eval(self, x, ctx):
        if not ctx.is_training:
            return x
        scope = x.scope
        scope.next_colour()
        rv = scope.rand(x.shape).value()
        a, da = x.into_inner()
        survivor_scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(self.amount)))
        b, db = rv.select_gt(self.amount, survivor_scale * a, 0.0).with_empty_grad()
        da.accumulate(rv.select_gt(self.amount, survivor_scale * db, 0.0))
        return DualArray(b, db)


class LSTMCell(Module):
    """Unrolled over the time axis (-2) (src/module.rs:281-363)."""

    class _Weight:
        def __init__(self, env, prefix, n_in, n_out):
            self.input = env.trainable_parameter([n_in, n_out], f"{prefix}_wi", Initializer.rand_normal(0.01))
            self.hidden = env.trainable_parameter([n_out, n_out], f"{prefix}_wh", Initializer.rand_normal(0.01))
            self.bias = env.trainable_parameter([n_out], f"{prefix}_b", Initializer.zero())

        def eval(self, x, hidden):
            y = x.matmul(self.input)
            if hidden is not None:
                y = y + hidden.matmul(self.hidden)
            return y + self.bias

    def __init__(self, env, n_in, n_out):
        self.forget_gate = self._Weight(env, "forget", n_in, n_out)
        self.input_gate = self._Weight(env, "input", n_in, n_out)
        self.output_gate = self._Weight(env, "output", n_in, n_out)
        self.cell_input = self._Weight(env, "cell", n_in, n_out)

    def eval(self, x, ctx):
        steps = x.shape[-2]
        prev_cell = prev_hidden = None
        for i in range(steps):
            xi = x.next_colour().lock_axis(-2, i, False)
            input_gate = self.input_gate.eval(xi, prev_hidden).sigmoid()
            output_gate = self.output_gate.eval(xi, prev_hidden).sigmoid()
            cell_input = self.cell_input.eval(xi, prev_hidden).tanh()
            cell = input_gate * cell_input
            if prev_cell is not None:
                cell = cell + self.forget_gate.eval(xi, prev_hidden).sigmoid() * prev_cell
            prev_hidden = output_gate * cell.tanh()
            prev_cell = cell
        return prev_hidden
