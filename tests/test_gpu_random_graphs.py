"""Differential test of the schedule's fusion passes: seeded random graphs through the array API, run on the GPU
with all fusion, on the GPU with one launch per reference cluster, and on the CPU oracle.

The graphs mix what the passes look for -- per-element chains, broadcasts of per-row values, reductions along
either axis (kept or dropped), transposes, matmuls with per-element consumers, selects -- in orders no workload
here contains, so a fusion that is only correct for the shapes of the ConvNet shows up.  Values stay O(1) by
construction (every op is followed by a scale or a squash), so relative L2 <= 1e-4 per output is meaningful."""
import numpy as np
import pytest

from conftest import rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _build_case(env, seed):
    rng = np.random.default_rng(seed)
    m = int(rng.choice([3, 17, 64, 130, 1000]))
    n = int(rng.choice([2, 10, 33, 64, 100]))
    p = int(rng.choice([1, 8, 50]))
    data = {
        "a": rng.standard_normal((m, n), dtype=np.float32),
        "b": rng.standard_normal((m, n), dtype=np.float32),
        "w": rng.standard_normal((n, p), dtype=np.float32),
        "row": rng.standard_normal((m, 1), dtype=np.float32),
        "col": rng.standard_normal((n,), dtype=np.float32),
    }
    params = {k: env.static_parameter_with_data(list(v.shape), k, v) for k, v in data.items()}
    n_ops = int(rng.integers(4, 14))
    plan = [(int(rng.integers(0, 12)), int(rng.integers(0, 1 << 30)), int(rng.integers(0, 1 << 30))) for _ in range(n_ops)]
    n_out = int(rng.integers(1, 4))
    out_picks = [int(rng.integers(0, 1 << 30)) for _ in range(n_out)]
    outputs = []

    def build(s):
        pool = [s.parameter_value(params["a"]), s.parameter_value(params["b"])]
        w, row, col = s.parameter_value(params["w"]), s.parameter_value(params["row"]), s.parameter_value(params["col"])

        def same_shape(x, pick):
            cands = [y for y in pool if tuple(y.shape) == tuple(x.shape)]
            return cands[pick % len(cands)]

        for op, i, j in plan:
            x = pool[i % len(pool)]
            shape = tuple(x.shape)
            if op == 0:
                y = x + same_shape(x, j) * 0.5
            elif op == 1:
                y = x * same_shape(x, j) * 0.5
            elif op == 2:
                y = (x * 0.3).exp() * 0.5
            elif op == 3:
                y = x.select_gt(0.0, x, x * 0.1)
            elif op == 4:  # softmax along the last axis
                t = (x - x.reduce_max(-1, True)).exp()
                y = t / t.reduce_sum(-1, True)
            elif op == 5:
                y = x.reduce_sum(0, True) * (1.0 / shape[0]) + x * 0.5
            elif op == 6:
                y = x.sin()
            elif op == 7:
                y = x.transpose() if len(shape) == 2 else x
            elif op == 8:
                y = (x.matmul(w) * (1.0 / np.sqrt(n))) if shape == (m, n) else x.square() * 0.25
            elif op == 9:
                y = (x + row) if shape == (m, n) else ((x + col) if shape[-1] == n else x * 0.9)
            elif op == 10:
                y = x - x.reduce_sum(-1, True) * (1.0 / shape[-1])
            else:
                y = x.reduce_max(-1, False).reshape([shape[0], 1]) * 0.5 + x * 0.25 if len(shape) == 2 else x
            pool.append(y)
        taken = set()
        for k, pick in enumerate(out_picks):
            idx = len(pool) - 1 - (pick % min(4, len(pool)))
            if idx in taken or idx < 2:  # a node's buffer can become only one parameter's (environment.rs:506-515)
                continue
            taken.add(idx)
            # a distinct scale per output: two outputs never end up as one node (common subexpressions merge)
            y = pool[idx] * (1.0 + 0.125 * (k + 1))
            o = env.static_parameter(list(y.shape), f"out{k}")
            outputs.append(o)
            s.write_parameter_value(o, y)

    graph = env.build_graph(build)
    env.run(graph, seed & 0xFFFF)
    return graph, [env.read_parameter(o) for o in outputs]


@pytest.mark.parametrize("seed", list(range(40)))
def test_random_graph_fused_unfused_oracle(hip_backend_session, seed):
    from descent_amd import Environment
    from oracle.cpu_backend import CpuBackend

    fused_env = Environment(hip_backend_session, fused=True)
    plain_env = Environment(hip_backend_session, fused=False)
    cpu_env = Environment(CpuBackend())
    graph, fused = _build_case(fused_env, 7000 + seed)
    _, plain = _build_case(plain_env, 7000 + seed)
    _, want = _build_case(cpu_env, 7000 + seed)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert len(fused) == len(want) == len(plain)
    for k, (f, u, c) in enumerate(zip(fused, plain, want)):
        assert f.shape == c.shape
        assert np.all(np.isfinite(c)), f"seed {seed}: the case itself overflows"
        assert rel_l2(u, c) <= TOL, f"seed {seed} output {k}: unfused vs oracle {rel_l2(u, c)}\n{listing}"
        assert rel_l2(f, c) <= TOL, f"seed {seed} output {k}: fused vs oracle {rel_l2(f, c)}\n{listing}"
