"""Optimisers expressed as graph ops (mirror of src/optimizer.rs)."""
from __future__ import annotations

import math
from typing import List

import numpy as np

from .array import Parameter, Scope


def add_weight_decay_to_grad(scope: Scope, parameters: List[Parameter], weight_decay: float) -> None:
    """src/optimizer.rs:3-13"""
    if weight_decay == 0.0:
        return
    scope.next_colour()
    for p in parameters:
        w, g = scope.parameter(p).into_inner()
        g.accumulate(w * weight_decay)


class _Optimizer:
    def __init__(self):
        self.state: List[Parameter] = []

    def reset_state(self, env) -> None:
        for p in self.state:
            env.writer(p).zero_fill()


class StochasticGradientDescent(_Optimizer):
    """v <- momentum*v + g; theta <- theta - lr*v (src/optimizer.rs:23-52)."""

    def __init__(self, env, scope: Scope, parameters, learning_rate, momentum: float):
        super().__init__()
        scope.next_colour()
        lr = learning_rate
        for p in parameters:
            g = scope.parameter(p).loss_grad()
            if momentum == 0.0:
                scope.update_parameter_value(p, lambda theta: theta - _mul(lr, g))
            else:
                v_param = env.static_parameter(p.shape, "v")
                v = scope.update_parameter_value(v_param, lambda v: v * momentum + g)
                scope.update_parameter_value(p, lambda theta: theta - _mul(lr, v))
                self.state.append(v_param)
        self.reset_state(env)


class Adam(_Optimizer):
    """Bias-corrected step size alpha = lr*sqrt(1-b2^t)/(1-b1^t) with the powers
    taken as exp(ln(b)*t); epsilon is added outside the correction
    (src/optimizer.rs:66-104)."""

    def __init__(self, env, scope: Scope, parameters, learning_rate, beta1: float, beta2: float, epsilon: float):
        super().__init__()
        scope.next_colour()
        t_param = env.static_parameter([1], "t")
        t = scope.update_parameter_value(t_param, lambda t: t + 1.0)
        self.state.append(t_param)

        ln_b1 = float(np.log(np.float32(beta1)))
        ln_b2 = float(np.log(np.float32(beta2)))
        alpha = _mul(learning_rate, (1.0 - (ln_b2 * t).exp()).sqrt()) / (1.0 - (ln_b1 * t).exp())

        one_minus_b1 = float(np.float32(1.0) - np.float32(beta1))
        one_minus_b2 = float(np.float32(1.0) - np.float32(beta2))
        for p in parameters:
            m_param = env.static_parameter(p.shape, "m")
            v_param = env.static_parameter(p.shape, "v")
            g = scope.parameter(p).loss_grad()
            m = scope.update_parameter_value(m_param, lambda m: m * beta1 + g * one_minus_b1)
            v = scope.update_parameter_value(v_param, lambda v: v * beta2 + g * g * one_minus_b2)
            self.state += [m_param, v_param]
            scope.update_parameter_value(p, lambda theta: theta - alpha * m / (v.sqrt() + epsilon))
        self.reset_state(env)


def _mul(lhs, rhs):
    """`lr * x` where lr is a float or an Array (IntoArray for f32 puts the
    literal on the left, src/array.rs:724-729)."""
    return lhs * rhs
