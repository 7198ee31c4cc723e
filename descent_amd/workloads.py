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
from .module import Conv2D, Dense, Dropout, EvalContext, MaxBlurPool2D, MaxPool2D, Module
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
    """examples/fashion_mnist/main.rs:171-222: the max-pool network, or with `blur_pool` the ConvBlurNet whose pools
    are a stride-1 max pool followed by a stride-2 depthwise blur (main.rs:187-199)."""

    def __init__(self, env, c1=16, c2=32, hidden=128, classes=10, side=28, blur_pool=False):
        self.conv1 = Conv2D(env, 1, c1, 3, 3, pad=1)
        self.pool1 = MaxBlurPool2D(env, c1) if blur_pool else MaxPool2D()
        self.conv2 = Conv2D(env, c1, c2, 3, 3, pad=1, groups=2)
        self.pool2 = MaxBlurPool2D(env, c2) if blur_pool else MaxPool2D()
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


class SingleLayer(Module):
    """examples/fashion_mnist/main.rs:146-169: one hidden layer with leaky_relu(0.01)."""

    def __init__(self, env, n_in=784, hidden_units=300, classes=10):
        self.fc1 = Dense(env, n_in, hidden_units)
        self.fc2 = Dense(env, hidden_units, classes)

    def eval(self, x, ctx):
        return x.flatten().apply(self.fc1, ctx).leaky_relu(0.01).apply(self.fc2, ctx)


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


def convnet(env: Environment, batch: int = 1000, seed: int = 3, side: int = 28, blur_pool: bool = False) -> Workload:
    """ConvNet full training step with Adam (lr 1e-3): conv3x3 1->16 pad 1, leaky_relu, maxpool 2x2; conv3x3
    16->32 pad 1 groups 2, leaky_relu, maxpool; flatten; dropout 0.5; dense ->128 leaky_relu; dense ->10;
    softmax cross-entropy.  `blur_pool` makes each pool a 2x2 stride-1 max pool and a fixed 3x3 stride-2 blur."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return _classifier_workload(env, ConvNet(env, side=side, blur_pool=blur_pool), batch, side, "adam", rng)


def single_layer_classifier(env: Environment, batch: int = 1000, seed: int = 2, side: int = 28, hidden_units: int = 300,
                            optimizer: str = "sgd") -> Workload:
    """The reference's single-hidden-layer classifier (side*side -> hidden_units -> 10)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return _classifier_workload(env, SingleLayer(env, side * side, hidden_units), batch, side, optimizer, rng)


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


# ---- image fit (examples/image_fit/main.rs) ----------------------------------------------------------------------
def positional_encoding(x, freq_count: int):
    """sin(x * 2^i * pi + {0, pi/2}) for i < freq_count: 2*freq_count features per input coordinate
    (examples/image_fit/main.rs:259-275)."""
    scope = x.scope
    pi32 = float(np.float32(np.pi))
    freq = scope.literal(2.0).pow(scope.coord(freq_count)) * pi32
    phase = scope.coord(2).reshape([2, 1]) * 0.5 * pi32
    shape = x.shape
    calc_shape = tuple(shape) + (1, 1)
    out_shape = tuple(shape[:-1]) + (shape[-1] * 2 * freq_count,)
    return (x.reshape(calc_shape) * freq + phase).sin().reshape(out_shape)


class ReluMlp(Module):
    """examples/image_fit/main.rs:52-87 (`Relu`; its activation is leaky_relu(0.01))."""

    def __init__(self, env, freq_count: int, hidden_units, n_in: int = 2, leakiness: float = 0.01):
        self.freq_count = freq_count
        self.leakiness = leakiness
        prev = n_in if freq_count == 0 else 2 * n_in * freq_count
        self.hidden = []
        for h in hidden_units:
            self.hidden.append(Dense(env, prev, h))
            prev = h
        self.final = Dense(env, prev, 3)

    def eval(self, x, ctx):
        if self.freq_count:
            x = positional_encoding(x, self.freq_count)
        for layer in self.hidden:
            x = x.apply(layer, ctx).leaky_relu(self.leakiness)
        return x.apply(self.final, ctx)


class Siren(Module):
    """examples/image_fit/main.rs:89-128: sin activations; omega_0 = 30 enters through the first layer's
    initialiser scale (src/parameter.rs:22-25)."""

    def __init__(self, env, hidden_units, n_in: int = 2):
        from .module import Initializer

        prev = n_in
        self.hidden = []
        for i, h in enumerate(hidden_units):
            self.hidden.append(Dense(env, prev, h, Initializer.for_siren(prev, i == 0), Initializer.rand_uniform(1.0)))
            prev = h
        self.final = Dense(env, prev, 3)

    def eval(self, x, ctx):
        for layer in self.hidden:
            x = x.apply(layer, ctx).sin()
        return x.apply(self.final, ctx)


HASH_PRIME = 1526263  # examples/image_fit/main.rs:139

# floor(16 * b^i), b = exp((ln 2048 - ln 16) / 15): the reference evaluates this in f32 and its top level can
# land on 2047 or 2048 depending on rounding (examples/image_fit/main.rs:222-228); the table is fixed here.
HASH_LEVEL_SIZES = (16, 22, 30, 42, 58, 80, 111, 153, 212, 294, 406, 561, 776, 1072, 1482, 2048)


class HashGrid(Module):
    """One level: bilinear interpolation of 4 gathered table entries; backward scatters into the table
    (examples/image_fit/main.rs:120-203)."""

    def __init__(self, env, grid_size: int, entry_count: int, values_per_entry: int):
        from .module import Initializer

        points = grid_size + 1
        full = points * points
        entry_count = min(entry_count, full)
        self.grid_size = grid_size
        self.stride = points if entry_count == full else HASH_PRIME
        self.t = env.trainable_parameter([entry_count, values_per_entry], "t", Initializer.rand_uniform(1.0e-4))

    def eval(self, x, ctx):
        from .array import DualArray

        scope = x.scope
        xv, _ = x.next_colour().into_inner()
        t, dt = scope.parameter(self.t).into_inner()
        entry_count = t.shape[0]
        stride = self.stride

        cf = (xv * 0.5 + 0.5) * float(self.grid_size)
        c = cf.into_u32()
        f = cf - c.into_f32()
        c0, c1 = c.lock_axis(-1, 0, False), c.lock_axis(-1, 1, False)
        f0, f1 = f.lock_axis(-1, 0, True), f.lock_axis(-1, 1, True)

        ia = ((c0 + 0) ^ (c1 * stride + 0)) % entry_count
        ib = ((c0 + 1) ^ (c1 * stride + 0)) % entry_count
        ic = ((c0 + 0) ^ (c1 * stride + stride)) % entry_count
        id_ = ((c0 + 1) ^ (c1 * stride + stride)) % entry_count

        ta, tb, tc, td = (t.gather(-2, i) for i in (ia, ib, ic, id_))
        g0, g1 = 1.0 - f0, 1.0 - f1
        wa, wb, wc, wd = g0 * g1, f0 * g1, g0 * f1, f0 * f1
        y, dy = (ta * wa + tb * wb + tc * wc + td * wd).with_empty_grad()
        dt.accumulate(
            scope.literal(0.0).value().broadcast(dt.shape)
            .scatter_add(dy * wa, -2, ia).scatter_add(dy * wb, -2, ib)
            .scatter_add(dy * wc, -2, ic).scatter_add(dy * wd, -2, id_)
        )
        return DualArray(y, dy)


class MultiHashGrid(Module):
    """examples/image_fit/main.rs:205-257: levels concatenated pairwise, then an MLP decoder."""

    def __init__(self, env, level_sizes, entry_count: int, hidden_units, values_per_entry: int = 2):
        self.grids = [HashGrid(env, g, entry_count, values_per_entry) for g in level_sizes]
        prev = len(self.grids) * values_per_entry
        self.hidden = []
        for h in hidden_units:
            self.hidden.append(Dense(env, prev, h))
            prev = h
        self.final = Dense(env, prev, 3)

    def eval(self, x, ctx):
        out = None
        for grid in self.grids:
            y = grid.eval(x, ctx)
            out = y if out is None else out.concat(y, -1)
        for layer in self.hidden:
            out = layer.eval(out, ctx).leaky_relu(0.01)
        return self.final.eval(out, ctx)


def sinusoid_image(points: np.ndarray, seed: int = 4) -> np.ndarray:
    """Target RGB in [0,1]: a seeded sum of 32 random 2-D sinusoids, clamped.  `points` is [m, 2] in [0,1]^2."""
    rng = np.random.Generator(np.random.PCG64(seed))
    freq = rng.uniform(-12.0, 12.0, (32, 2))
    phase = rng.uniform(0.0, 2 * np.pi, (32, 3))
    amp = rng.uniform(0.0, 0.25, (32, 3))
    arg = points.astype(np.float64) @ freq.T * (2 * np.pi)  # [m, 32]
    rgb = 0.5 + (np.sin(arg[:, :, None] + phase[None]) * amp[None]).sum(axis=1)
    return np.clip(rgb, 0.0, 1.0).astype(np.float32)


def _image_fit_workload(env: Environment, module: Module, points01: np.ndarray, rng, lr: float, betas, signed_inputs: bool) -> Workload:
    """Train-graph assembly of examples/image_fit/main.rs:303-332: L2 loss, Adam."""
    m = points01.shape[0]
    x_param = env.static_parameter([m, 2], "x")
    y_param = env.static_parameter([m, 3], "y")
    loss_sum = env.static_parameter([1], "loss")
    scope = env.scope()
    out = module.train(scope.parameter(x_param))
    loss = (out - y_param).square().reduce_sum(-1, True).set_loss()
    scope.update_parameter_value(loss_sum, lambda s: s + loss.reduce_sum(0, False))
    parameters = scope.trainable_parameters()
    opt = Adam(env, scope, parameters, lr, betas[0], betas[1], 1e-8)
    graph = scope.build_graph()
    for p in parameters:
        env.reset_parameter(p, rng)
    env.writer(loss_sum).zero_fill()
    x = (points01 * 2.0 - 1.0) if signed_inputs else points01
    env.write_parameter(x_param, x.astype(np.float32))
    env.write_parameter(y_param, sinusoid_image(points01))
    return Workload(env, graph, {"x": x_param, "y": y_param}, parameters, opt.state, {"loss": loss_sum})


def coordinate_mlp(env: Environment, side: int = 512, variant: str = "relu-pe", hidden=(256, 256, 256, 256),
                   freq_count: int = 16, seed: int = 5, leakiness: float = 0.01) -> Workload:
    """Coordinate MLP image fit: every point of a side x side grid in [0,1]^2; "relu-pe" = positional encoding
    (freq_count sin/cos pairs per axis) + leaky_relu(0.01) hidden layers, "siren" = sin activations; Adam lr 1e-3."""
    rng = np.random.Generator(np.random.PCG64(seed))
    axis = (np.arange(side, dtype=np.float64) + 0.5) / side
    pts = np.stack(np.meshgrid(axis, axis, indexing="xy"), axis=-1).reshape(-1, 2)
    module = Siren(env, hidden) if variant == "siren" else ReluMlp(env, freq_count, hidden, leakiness=leakiness)
    # the SIREN consumes coordinates in [-1, 1] as the reference feeds them (examples/image_fit/main.rs:372-375)
    return _image_fit_workload(env, module, pts, rng, 1e-3, (0.9, 0.999), signed_inputs=variant == "siren")


def hash_grid_fit(env: Environment, batch: int = 1 << 18, levels=HASH_LEVEL_SIZES, entry_count: int = 1 << 19,
                  hidden=(64, 64), seed: int = 6) -> Workload:
    """Multi-level hash encoding image fit: `batch` uniform points of [0,1]^2 (fed as 2u-1, the domain the
    reference's HashGrid maps back with x*0.5+0.5), 2 features per entry, tables U(+-1e-4), decoder MLP with
    leaky_relu(0.01), L2 loss, Adam lr 1e-3."""
    rng = np.random.Generator(np.random.PCG64(seed))
    pts = rng.random((batch, 2)) * (1.0 - 1e-6)
    module = MultiHashGrid(env, levels, entry_count, hidden)
    return _image_fit_workload(env, module, pts, rng, 1e-3, (0.9, 0.999), signed_inputs=True)
