"""Differential test of the convolution / pooling side of the schedule: seeded random small conv nets (filter size,
stride, padding, groups, channel counts, pooling and batch drawn per seed; geometries the workloads never use) trained
for two SGD-with-momentum steps on the GPU with all fusion, with one launch per reference cluster, and on the CPU
oracle.  Every parameter and momentum buffer after the steps must agree to relative L2 <= 1e-4, the accuracy count
exactly: the steps cover conv forward (implicit GEMM), both conv gradients (dedicated and generic paths, whichever
the geometry allows), max-pool forward/backward, the bias reductions and the fused softmax cross-entropy."""
import numpy as np
import pytest

from conftest import rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _draw_net(rng):
    side = int(rng.choice([8, 10, 12, 14, 18]))
    cin = int(rng.choice([1, 2, 3, 4]))
    batch = int(rng.choice([2, 5, 16, 33]))
    blocks = []
    h, c = side, cin
    for _ in range(int(rng.integers(1, 4))):
        for _attempt in range(20):
            f = int(rng.choice([1, 2, 3, 5]))
            stride = int(rng.choice([1, 1, 2]))
            pad = int(rng.choice([0, 1, 2]))
            groups = int(rng.choice([1, 1, 2]))
            cout = int(rng.choice([2, 4, 6, 8, 16]))
            if c % groups or cout % groups:
                continue
            padded = h + 2 * pad
            if padded < f or (padded - f) % stride:
                continue
            out = (padded - f) // stride + 1
            if out < 2:
                continue
            pool = bool(rng.integers(0, 2)) and out % 2 == 0 and out >= 4
            blocks.append((c, cout, f, pad, stride, groups, pool))
            h, c = (out // 2 if pool else out), cout
            break
        if h < 4:
            break
    return side, cin, batch, blocks, h, c


def _run_case(env, seed, steps=2):
    from descent_amd.loss import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss
    from descent_amd.module import Conv2D, Dense, MaxPool2D, Module
    from descent_amd.optimizer import StochasticGradientDescent

    rng = np.random.default_rng(seed)
    side, cin, batch, blocks, h, c = _draw_net(rng)

    class Net(Module):
        def __init__(self):
            self.convs = [Conv2D(env, ci, co, f, f, pad=pad, stride=(st, st), groups=g) for (ci, co, f, pad, st, g, _) in blocks]
            self.pool = MaxPool2D()
            self.fc = Dense(env, h * h * c, 7)

        def eval(self, x, ctx):
            for conv, (_, _, _, _, _, _, pool) in zip(self.convs, blocks):
                x = x.apply(conv, ctx).leaky_relu(0.01)
                if pool:
                    x = x.apply(self.pool, ctx)
            return x.flatten().apply(self.fc, ctx)

    net = Net()
    x_param = env.static_parameter([batch, side, side, cin], "x")
    y_param = env.static_parameter([batch, 1], "y")
    acc_sum = env.static_parameter([1], "accuracy")
    scope = env.scope()
    z = net.train(scope.parameter(x_param))
    softmax_cross_entropy_loss(z, y_param).set_loss()
    acc = softmax_cross_entropy_accuracy(z, y_param)
    scope.update_parameter_value(acc_sum, lambda s: s + acc.reduce_sum(0, False))
    params = scope.trainable_parameters()
    opt = StochasticGradientDescent(env, scope, params, 0.05, 0.9)
    graph = scope.build_graph()
    for p in params:
        env.reset_parameter(p, rng)
    env.writer(acc_sum).zero_fill()
    env.write_parameter(x_param, rng.standard_normal((batch, side, side, cin), dtype=np.float32))
    env.write_parameter(y_param, rng.integers(0, 7, (batch, 1)).astype(np.float32))
    for i in range(steps):
        env.run(graph, 10 + i)
    out = {f"p{i}:{p.name}{list(p.shape)}": env.read_parameter(p) for i, p in enumerate(params)}
    out.update({f"v{i}": env.read_parameter(p) for i, p in enumerate(opt.state)})
    return graph, out, env.read_parameter(acc_sum), (side, cin, batch, blocks)


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_convnet_fused_unfused_oracle(hip_backend_session, seed):
    from descent_amd import Environment
    from oracle.cpu_backend import CpuBackend

    graph, fused, acc_f, net = _run_case(Environment(hip_backend_session, fused=True), 9100 + seed)
    _, plain, acc_p, _ = _run_case(Environment(hip_backend_session, fused=False), 9100 + seed)
    _, want, acc_w, _ = _run_case(Environment(CpuBackend()), 9100 + seed)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert np.array_equal(acc_p, acc_w) and np.array_equal(acc_f, acc_w), f"accuracy {acc_f} {acc_p} {acc_w} for {net}"
    for key in want:
        assert np.all(np.isfinite(want[key])), f"seed {seed}: the case itself overflows ({net})"
        assert rel_l2(plain[key], want[key]) <= TOL, f"seed {seed} {key}: unfused vs oracle {rel_l2(plain[key], want[key])} for {net}\n{listing}"
        assert rel_l2(fused[key], want[key]) <= TOL, f"seed {seed} {key}: fused vs oracle {rel_l2(fused[key], want[key])} for {net}\n{listing}"
