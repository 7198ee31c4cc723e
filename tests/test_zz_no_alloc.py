"""dsc_schedule_run_static (the entry point that allocates no device memory: intermediates in the library's fixed
scratch array, written parameters in caller-provided spare buffers) against dsc_schedule_run on the same seeded
workloads, through the C ABI.  Both run the same kernels, so fp32 tensors must agree to the 1e-4 relative L2 bound of
the parity tests and arg-max derived outputs exactly; where no float atomics are involved they agree bit for bit."""
import numpy as np
import pytest

from conftest import rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _steps(be, build, static, steps, first_seed):
    from descent_amd import Environment

    be.profile(False)  # per-launch timing creates events, which the static run refuses to do
    env = Environment(be)
    w = build(env)
    live_before = arena_before = None
    for i in range(steps):
        if static:
            env.run_static(w.graph, first_seed + i)
            if i == 1:  # the spares exist after the first step: from here on nothing may be allocated
                live_before, _, arena_before = be.heap_stats()
        else:
            env.run(w.graph, first_seed + i)
    snap = w.snapshot()
    if static and steps > 2:
        live_after, _, arena_after = be.heap_stats()
        assert (live_after, arena_after) == (live_before, arena_before)
    listing = next(iter(w.graph.__dict__["_schedules"].values())).describe()
    for p in list(w.inputs.values()) + w.trainable + w.state + list(w.scalars.values()):
        for h in (p.buffer, p.__dict__.get("spare")):
            if h is not None:
                be.free(h)
        p.buffer = None
        p.spare = None
    return snap, listing


def _compare(got, want, exact, tol=TOL):
    assert got.keys() == want.keys()
    for key in want:
        if key == "accuracy" or exact:
            assert np.array_equal(got[key].view(np.uint32), want[key].view(np.uint32)), key
        else:
            assert rel_l2(got[key], want[key]) <= tol, (key, rel_l2(got[key], want[key]))


def test_static_run_matches_the_allocating_run_on_two_calls_in_a_row(hip_backend_session):
    """ConvNet train steps (Adam, dropout) at batch 64, then -- same process, same scratch array, which still holds the
    first workload's intermediates -- at batch 16: every parameter, optimiser state and scalar, three steps each."""
    from descent_amd import workloads

    be = hip_backend_session
    for batch, seed in ((64, 5), (16, 6)):
        build = lambda e: workloads.convnet(e, batch=batch, seed=seed)
        want, _ = _steps(be, build, False, 3, 900)
        got, listing = _steps(be, build, True, 3, 900)
        assert "static runs: at most" in listing, listing
        _compare(got, want, exact=True)


def test_static_run_places_prefilled_accumulators_and_scatter_chains(hip_backend_session):
    """The reduced hash grid: accumulators that start as a literal are filled by one launch at the start of the run and
    handed along their ScatterAdd chains; float atomics reorder sums, so the looser 1e-3 bound of that workload."""
    from descent_amd import workloads

    kw = dict(batch=8192, levels=(4, 16, 40, 100), entry_count=2048, hidden=(32,), seed=22)
    build = lambda e: workloads.hash_grid_fit(e, **kw)
    want, _ = _steps(hip_backend_session, build, False, 3, 0)
    got, _ = _steps(hip_backend_session, build, True, 3, 0)
    _compare(got, want, exact=False, tol=1e-3)


def test_static_run_refuses_what_does_not_fit_and_what_it_cannot_place(hip_backend_session):
    from descent_amd import Environment, workloads
    from descent_amd.hip_backend import DescentHipError

    be = hip_backend_session
    env = Environment(be)
    w = workloads.convnet(env, batch=8000, seed=3)  # conv1's pooled activations alone exceed the 64 MiB array
    before = {id(p): p.buffer for p in w.trainable + w.state}
    with pytest.raises(DescentHipError) as err:
        env.run_static(w.graph, 1)
    assert err.value.status == 5 and "static scratch array holds 67108864 bytes" in str(err.value), str(err.value)
    assert all(p.buffer == before[id(p)] for p in w.trainable + w.state)  # nothing was enqueued or swapped
    env.run(w.graph, 1)  # the allocating entry point still takes the same schedule
    be.sync()
    # a written slot without a spare, and a spare that is the parameter's own buffer
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    handles = [p.buffer for p in sched.params]
    with pytest.raises(DescentHipError):
        sched.run_static(handles, [None] * len(handles), 1)
    small = Environment(be)
    w2 = workloads.convnet(small, batch=16, seed=3)
    small.run_static(w2.graph, 1)
    sched2 = next(iter(w2.graph.__dict__["_schedules"].values()))
    handles = [p.buffer for p in sched2.params]
    with pytest.raises(DescentHipError):
        sched2.run_static(handles, list(handles), 2)
    be.sync()
