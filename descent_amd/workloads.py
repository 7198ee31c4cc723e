"""The benchmark configurations as graphs: what the reference's examples assemble
(examples/fashion_mnist/main.rs:131-287, examples/image_fit/main.rs:52-275),
with synthetic seeded inputs uploaded as data.

Each builder returns a `Workload`: the environment, the train graph, the
parameters to feed and read back, and a callable that uploads one seeded
batch.  The same builder runs against any backend.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

import numpy as np

from .array import Parameter
from .environment import Environment
from .graph import Graph
from .loss import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss
from .module import Conv2D, Dense, Dropout, EvalContext, MaxPool2D, Module
from .optimizer import Adam, StochasticGradientDescent


@dataclass
class Workload:
    env: Environment
    graph: Graph
    inputs: Dict[str, Parameter]
    trainable: List[Parameter]
    state: List[Parameter]
    scalars: Dict[str, Parameter] = field(default_factory=dict)
    test_graph: Optional[Graph] = None

    def snapshot(self) -> Dict[str, np.ndarray]:
        """All trainable parameters, optimiser state and scalars, by name#index."""
        out = {}
        for i, p in enumerate(self.trainable):
            out[f"param{i}:{p.name}"] = self.env.read_parameter(p)
        for i, p in enumerate(self.state):
            out[f"state{i}:{p.name}"] = self.env.read_parameter(p)
        for k, p in self.scalars.items():
            out[k] = self.env.read_parameter(p)
        return out


class ConvNet(Module):
    """examples/fashion_mnist/main.rs:171-222 (max-pool variant)."""

    def __init__(self, env, c1=16, c2=32, hidden=128, classes=10, side=28):
        self.conv1 = Conv2D(env, 1, c1, 3, 3, pad=1)
        self.pool1 = MaxPool2D()
        self.conv2 = Conv2D(env, c1, c2, 3, 3, pad=1, groups=2)
        self.pool2 = MaxPool2D()
        self.fc1 = Dense(env, (side // 4) * (side // 4) * c2, hidden)
        self.fc2 = Dense(env, hidden, classes)

    def eval(self, x, ctx):
        x = x.apply(self.conv1, ctx).leaky_relu(0.01).apply(self.pool1, ctx)
        x = x.apply(self.conv2, ctx).leaky_relu(0.01).apply(self.pool2, ctx)
        x = x.flatten().apply(Dropout(0.5), ctx)
        return x.apply(self.fc1, ctx).leaky_relu(0.01).apply(self.fc2, ctx)


class Linear(Module):
    """examples/fashion_mnist/main.rs:131-147"""

    def __init__(self, env, n_in=784, classes=10):
        self.fc = Dense(env, n_in, classes)

    def eval(self, x, ctx):
        return x.flatten().apply(self.fc, ctx)


def _classifier_workload(env: Environment, module: Module, batch: int, side: int, optimizer: str,
                         rng: np.random.Generator, init: str = "he") -> Workload:
    """Train-graph assembly of examples/fashion_mnist/main.rs:235-287 (weight decay 0)."""
    x_param = env.static_parameter([batch, side, side, 1], "x")
    y_param = env.static_parameter([batch, 1], "y")
    loss_sum = env.static_parameter([1], "loss")
    accuracy_sum = env.static_parameter([1], "accuracy")

    scope = env.scope()
    x = module.train(scope.parameter(x_param))
    loss = softmax_cross_entropy_loss(x, y_param).set_loss()
    accuracy = softmax_cross_entropy_accuracy(x, y_param)
    scope.update_parameter_value(loss_sum, lambda s: s + loss.reduce_sum(0, False))
    scope.update_parameter_value(accuracy_sum, lambda s: s + accuracy.reduce_sum(0, False))
    parameters = scope.trainable_parameters()
    if optimizer == "adam":
        opt = Adam(env, scope, parameters, 1e-3, 0.9, 0.999, 1e-8)
    else:
        opt = StochasticGradientDescent(env, scope, parameters, 0.1, 0.9)
    graph = scope.build_graph()

    def test(scope):
        xt = module.test(scope.parameter(x_param))
        lt = softmax_cross_entropy_loss(xt, y_param).set_loss()
        at = softmax_cross_entropy_accuracy(xt, y_param)
        scope.update_parameter_value(loss_sum, lambda s: s + lt.reduce_sum(0, False))
        scope.update_parameter_value(accuracy_sum, lambda s: s + at.reduce_sum(0, False))

    test_graph = env.build_graph(test)

    for p in parameters:
        if init == "xavier" and len(p.shape) == 2:
            bound = np.sqrt(6.0 / (p.shape[0] + p.shape[1]))
            env.write_parameter(p, rng.uniform(-bound, bound, p.shape.element_count()).astype(np.float32))
        else:
            env.reset_parameter(p, rng)
    for p in (loss_sum, accuracy_sum):
        env.writer(p).zero_fill()
    env.write_parameter(x_param, rng.random(x_param.shape.element_count(), dtype=np.float32))
    env.write_parameter(y_param, rng.integers(0, 10, batch).astype(np.float32))
    return Workload(env, graph, {"x": x_param, "y": y_param}, parameters, opt.state,
                    {"loss": loss_sum, "accuracy": accuracy_sum}, test_graph)


def convnet(env: Environment, batch: int = 1000, seed: int = 3, side: int = 28) -> Workload:
    """ConvNet full training step with Adam (lr 1e-3): conv3x3 1->16 pad 1, leaky_relu, maxpool 2x2; conv3x3
    16->32 pad 1 groups 2, leaky_relu, maxpool; flatten; dropout 0.5; dense ->128 leaky_relu; dense ->10;
    softmax cross-entropy."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return _classifier_workload(env, ConvNet(env, side=side), batch, side, "adam", rng)


def linear_classifier(env: Environment, batch: int = 1000, seed: int = 1) -> Workload:
    """Single-layer softmax classifier, SGD momentum 0.9 lr 0.1, Xavier-uniform weights."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return _classifier_workload(env, Linear(env), batch, 28, "sgd", rng, init="xavier")


@dataclass
class MatmulWorkload:
    env: Environment
    graph: Graph
    a: Parameter
    b: Parameter
    bias: Parameter
    c: Parameter
    m: int
    n: int
    k: int

    @property
    def flops(self) -> float:
        return 2.0 * self.m * self.n * self.k


def matmul_epilogue(env: Environment, m: int, n: int, k: int, seed: int = 2, upload: bool = True) -> MatmulWorkload:
    """C = leaky_relu(A.B + bias, 0.01) through the array API; A, B, bias ~ N(0,1)."""
    a = env.static_parameter([m, k], "a")
    b = env.static_parameter([k, n], "b")
    bias = env.static_parameter([n], "bias")
    c = env.static_parameter([m, n], "c")

    def build(scope):
        z = scope.parameter_value(a).matmul(scope.parameter_value(b)) + scope.parameter_value(bias)
        scope.write_parameter_value(c, z.select_gt(0.0, z, z * 0.01))

    graph = env.build_graph(build)
    if upload:
        rng = np.random.Generator(np.random.PCG64(seed))
        env.write_parameter(a, rng.standard_normal(m * k, dtype=np.float32))
        env.write_parameter(b, rng.standard_normal(k * n, dtype=np.float32))
        env.write_parameter(bias, rng.standard_normal(n, dtype=np.float32))
    return MatmulWorkload(env, graph, a, b, bias, c, m, n, k)
