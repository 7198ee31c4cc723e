"""Parity at the full sizes of the benchmark configurations, where the CPU oracle is too slow to run every step:
the fused schedule (what bench.py times) against the schedule with one launch per reference cluster, which shares no
fused kernel with it (no implicit GEMM, no conv-gradient kernel, no row fusion, no epilogues, no multi-part
launches) and is itself checked against the oracle at reduced size elsewhere.  The ConvNet at batch 1000 is also
checked against the oracle directly for one step."""
import numpy as np
import pytest

from conftest import rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _pair(be, build, steps, first_seed):
    from descent_amd import Environment

    out = []
    for fused in (True, False):
        env = Environment(be, fused=fused)
        w = build(env)
        for i in range(steps):
            env.run(w.graph, first_seed + i)
        out.append(w.snapshot())
        del w, env
    return out


def test_convnet_batch_1000_fused_unfused_and_oracle(hip_backend_session):
    from descent_amd import Environment, workloads
    from oracle.cpu_backend import CpuBackend

    fused, plain = _pair(hip_backend_session, lambda e: workloads.convnet(e, batch=1000, seed=3), 2, 50)
    for key in plain:
        if key == "accuracy":
            assert np.array_equal(fused[key], plain[key])
        else:
            assert rel_l2(fused[key], plain[key]) <= TOL, f"{key}: {rel_l2(fused[key], plain[key])}"
    cenv = Environment(CpuBackend())
    cw = workloads.convnet(cenv, batch=1000, seed=3)
    for i in range(2):
        cenv.run(cw.graph, 50 + i)
    want = cw.snapshot()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(fused[key], want[key])
        else:
            assert rel_l2(fused[key], want[key]) <= TOL, f"{key} vs oracle: {rel_l2(fused[key], want[key])}"


@pytest.mark.parametrize("variant", ["relu-pe", "siren"])
def test_coordinate_mlp_512_fused_unfused(hip_backend_session, variant):
    from descent_amd import workloads

    fused, plain = _pair(hip_backend_session, lambda e: workloads.coordinate_mlp(e, variant=variant), 2, 0)
    for key in plain:
        assert np.all(np.isfinite(plain[key])), key
        assert rel_l2(fused[key], plain[key]) <= TOL, f"{variant} {key}: {rel_l2(fused[key], plain[key])}"


def test_hash_grid_2p18_fused_unfused(hip_backend_session):
    """Both schedules scatter with float atomics in a different order, so the looser bound of the scatter-add tests
    applies to every tensor (all depend on the tables after the first step)."""
    from descent_amd import workloads

    fused, plain = _pair(hip_backend_session, lambda e: workloads.hash_grid_fit(e), 2, 0)
    for key in plain:
        assert np.all(np.isfinite(plain[key])), key
        assert rel_l2(fused[key], plain[key]) <= 1e-3, f"{key}: {rel_l2(fused[key], plain[key])}"
