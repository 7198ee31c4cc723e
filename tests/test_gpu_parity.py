"""GPU parity: the HIP backend, called through the C ABI, against the CPU oracle on the same seeded inputs.

Tolerances (stated by the benchmark definition): relative L2 <= 1e-4 per fp32 tensor; exact for the reference's
known-answer tests (small integers) and for index/argmax style outputs."""
import numpy as np
import pytest

from conftest import rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-4


def _envs(hip_backend_session, **kw):
    from descent_amd import Environment
    from oracle.cpu_backend import CpuBackend

    return Environment(hip_backend_session, **kw), Environment(CpuBackend())


@pytest.mark.parametrize("mode", ["fused", "unfused", "kernel_by_kernel"])
def test_reference_known_answers(hip_backend_session, mode):
    import reference_cases
    from descent_amd import Environment

    for case in reference_cases.ALL:
        env = Environment(hip_backend_session, use_schedule=mode != "kernel_by_kernel", fused=mode == "fused")
        actual, expected = case(env)
        assert np.array_equal(actual, np.asarray(expected, np.float32)), f"{case.__name__} [{mode}]: {actual}"


MATMUL_SHAPES = [
    (1, 1, 1), (16, 16, 16), (33, 17, 9), (128, 128, 128), (100, 10, 784), (1000, 128, 784), (257, 130, 1030),
    (64, 300, 2100), (9, 16, 5000),
    # very short k with a wide output: the short-k kernel
    (20000, 64, 3), (5000, 256, 8), (70000, 16, 1),
    # small outputs over a long k: the tall-k kernel (ragged tiles, one tile, many tiles)
    (9, 16, 50000), (72, 16, 70000), (33, 50, 140000), (250, 3, 66000),
    # few columns, a moderate number of rows: the dot-product kernel (lanes share a row's k range)
    (1000, 10, 128), (1000, 10, 400), (300, 16, 100), (70, 3, 37), (5000, 1, 64), (64, 13, 315), (16383, 5, 33), (200, 2, 2048),
]


@pytest.mark.parametrize("m,n,k", MATMUL_SHAPES)
@pytest.mark.parametrize("fused", [True, False])
def test_matmul_epilogue_vs_oracle(hip_backend_session, m, n, k, fused):
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session, fused=fused)
    gw = workloads.matmul_epilogue(genv, m, n, k, seed=m + n + k)
    cw = workloads.matmul_epilogue(cenv, m, n, k, seed=m + n + k)
    genv.run(gw.graph, 1)
    cenv.run(cw.graph, 1)
    err = rel_l2(genv.read_parameter(gw.c), cenv.read_parameter(cw.c))
    assert err <= TOL, f"{m}x{n}x{k} fused={fused}: rel L2 {err}"


def _transposed_case(env, rng, m, n, k, ta, tb):
    a = env.static_parameter_with_data([k, m] if ta else [m, k], "a", rng.standard_normal(m * k, dtype=np.float32))
    b = env.static_parameter_with_data([n, k] if tb else [k, n], "b", rng.standard_normal(k * n, dtype=np.float32))
    c = env.static_parameter([m, n], "c")

    def build(s):
        av, bv = s.parameter_value(a), s.parameter_value(b)
        s.write_parameter_value(c, (av.transpose() if ta else av).matmul(bv.transpose() if tb else bv))

    env.run(env.build_graph(build), 0)
    return env.read_parameter(c)


@pytest.mark.parametrize("ta,tb", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(128, 64, 256), (100, 36, 77), (72, 16, 3000), (72, 16, 40000), (128, 10, 400), (100, 7, 50)])
def test_matmul_transposed_operands(hip_backend_session, ta, tb, m, n, k):
    genv, cenv = _envs(hip_backend_session)
    got = _transposed_case(genv, np.random.default_rng(5), m, n, k, ta, tb)
    want = _transposed_case(cenv, np.random.default_rng(5), m, n, k, ta, tb)
    assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k,tile,buffers,force", [
    (256, 256, 64, "32x32x16", None, None), (1024, 512, 128, "64x32x16", None, "64,32,16,2,1,8"), (1024, 1024, 128, "64x64x16", None, None),
    (1024, 1024, 1024, "64x64x64", None, None), (2048, 1024, 128, "128x64x16", None, "128,64,16,2,2,8"), (2048, 2048, 64, "128x128x16", None, None),
    (2048, 2048, 64, "128x128x16", "3", None), (4096, 2048, 64, "256x128x16", "2", None), (4096, 4096, 128, "256x256x32", "2", None),
    (4096, 4096, 48, "256x256x16", "3", None), (4096, 4096, 160, "256x256x32", None, None), (2048, 2048, 256, "128x128x32", None, None),
    (4096, 1024, 256, "128x64x32", None, "128,64,32,2,2,8"), (4096, 2048, 128, "256x128x32", None, None),
    # more tiles than workgroups: a workgroup's stream of k-tiles runs on into its next unit
    (2048, 3072, 64, "128x64x16", None, None), (2048, 3072, 64, "128x64x16", "3", None), (1024, 1536, 512, "64x64x64", None, None),
    (1024, 1536, 512, "64x64x64", "3", None), (8192, 4096, 48, "256x256x16", "3", None), (8192, 8192, 128, "256x256x32", None, None),
    (4096, 4096, 64, "256x256x16", None, None),
    # tiles that reach past M or N repeat the last row / the last four columns and store only what exists
    (1000, 1000, 512, "64x64x64", None, None), (1000, 1000, 512, "64x64x64", "3", None), (2500, 1100, 128, "128x128x32", None, "128,128,32,2,2,8"),
    (5000, 3000, 128, "256x256x32", None, "256,256,32,4,4,8"), (4100, 2052, 64, "256x128x16", None, "256,128,16,4,2,4"), (36, 20, 64, "32x32x16", None, None),
])
def test_matmul_tiles_loaded_straight_into_lds(hip_backend_session, monkeypatch, m, n, k, tile, buffers, force, ta, tb):
    """Whole-tile products take their k-tiles from memory straight into LDS: every tile shape, both operand
    layouts on either side, two and three tile buffers, against the oracle."""
    from descent_amd import hip_backend

    if buffers is None:
        monkeypatch.delenv("DSC_MM_DIRECT_LDS", raising=False)
    else:
        monkeypatch.setenv("DSC_MM_DIRECT_LDS", buffers)  # read when a kernel is generated; part of the kernel cache key
    if force is None:
        monkeypatch.delenv("DSC_MM_TILE", raising=False)
    else:
        monkeypatch.setenv("DSC_MM_TILE", force)  # a tile shape the choice by predicted rate does not take for this product
    genv, cenv = _envs(hip_backend_session)
    got = _transposed_case(genv, np.random.default_rng(m + k), m, n, k, ta, tb)
    want = _transposed_case(cenv, np.random.default_rng(m + k), m, n, k, ta, tb)
    assert rel_l2(got, want) <= TOL
    # the launch that ran is the one the listing describes
    a = genv.static_parameter([k, m] if ta else [m, k], "a")
    b = genv.static_parameter([n, k] if tb else [k, n], "b")
    c = genv.static_parameter([m, n], "c")

    def build(s):
        av, bv = s.parameter_value(a), s.parameter_value(b)
        s.write_parameter_value(c, (av.transpose() if ta else av).matmul(bv.transpose() if tb else bv))

    listing = hip_backend.check_schedule(genv.build_graph(build), fused=True)
    assert f"tile {tile} " in listing and f"A{2 if ta else 1} B{2 if tb else 1}" in listing, listing
    assert f"tiles straight into LDS x{buffers or 2}" in listing, listing


@pytest.mark.parametrize("m,n,k", [(2048, 1024, 128), (1000, 520, 256), (4096, 4096, 64), (300, 36, 64)])
def test_matmul_epilogue_with_a_per_element_and_a_per_column_operand(hip_backend_session, m, n, k):
    """The store path requests the epilogue's own operands ahead of its staging rounds: a bias (per column) and a mask
    (per element), on whole and on ragged products, against the oracle."""
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(m + n)
        a = env.static_parameter_with_data([m, k], "a", rng.standard_normal(m * k, dtype=np.float32))
        b = env.static_parameter_with_data([k, n], "b", rng.standard_normal(k * n, dtype=np.float32))
        bias = env.static_parameter_with_data([n], "bias", rng.standard_normal(n, dtype=np.float32))
        mask = env.static_parameter_with_data([m, n], "mask", rng.standard_normal(m * n, dtype=np.float32))
        c = env.static_parameter([m, n], "c")

        def build(s):
            z = s.parameter_value(a).matmul(s.parameter_value(b)) + s.parameter_value(bias)
            s.write_parameter_value(c, s.parameter_value(mask).select_gt(0.0, z, z * 0.01))

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(c), graph

    got, graph = run(genv)
    want, _ = run(cenv)
    assert rel_l2(got, want) <= TOL
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert int(listing.split()[0]) == 1 and "+epilogue" in listing and "tiles straight into LDS" in listing, listing


@pytest.mark.parametrize("m,n,k,tb,epilogue", [
    (16384, 3, 256, False, True), (20000, 5, 64, False, False), (40001, 16, 200, True, True), (16390, 2, 66, False, False),
    (262144, 3, 256, True, True), (70000, 1, 128, False, True),
])
def test_tall_products_with_long_contiguous_rows_and_few_columns(hip_backend_session, m, n, k, tb, epilogue):
    """The output layer of a coordinate network: many rows, each long and contiguous, a few columns.  Lanes share a
    row (every cache line requested once) and a workgroup walks several groups of rows with B staged once; row
    counts that end inside a group, k off the 16-byte grid, B in either layout, with and without a fused consumer."""
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(m + k)
        a = env.static_parameter_with_data([m, k], "a", rng.standard_normal(m * k, dtype=np.float32))
        b = env.static_parameter_with_data([n, k] if tb else [k, n], "b", rng.standard_normal(k * n, dtype=np.float32))
        bias = env.static_parameter_with_data([n], "bias", rng.standard_normal(n, dtype=np.float32))
        c = env.static_parameter([m, n], "c")

        def build(s):
            bv = s.parameter_value(b)
            z = s.parameter_value(a).matmul(bv.transpose() if tb else bv)
            if epilogue:
                z = z + s.parameter_value(bias)
                z = z.select_gt(0.0, z, z * 0.01)
            s.write_parameter_value(c, z)

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(c), graph

    got, graph = run(genv)
    want, _ = run(cenv)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert "dot products:" in listing and int(listing.split()[0]) == 1, listing
    assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("m,n,k", [(65536, 128, 2), (100000, 64, 3), (70000, 256, 4), (262144, 256, 3), (132072, 64, 3), (65536, 32, 3), (131072, 16, 3)])
def test_data_and_weight_gradient_of_a_layer_with_few_outputs_as_one_kernel(hip_backend_session, m, n, k):
    """dZ = (dY W^T) masked by the stored activation X, and dW = X^T dY: one kernel reads X once for both (the weight
    gradient's k chunks become the kernel's row chunks; the last chunk of a ragged row count is short)."""
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(m + n)
        dy = env.static_parameter_with_data([m, k], "dy", rng.standard_normal(m * k, dtype=np.float32))
        x = env.static_parameter_with_data([m, n], "x", rng.standard_normal(m * n, dtype=np.float32))
        w = env.static_parameter_with_data([n, k], "w", rng.standard_normal(n * k, dtype=np.float32))
        dz = env.static_parameter([m, n], "dz")
        dw = env.static_parameter([n, k], "dw")

        def build(s):
            d, xv = s.parameter_value(dy), s.parameter_value(x)
            p = d.matmul(s.parameter_value(w).transpose())
            s.write_parameter_value(dz, xv.select_gt(0.0, p, p * 0.01))
            s.write_parameter_value(dw, xv.transpose().matmul(d))

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(dz), env.read_parameter(dw), graph

    got_z, got_w, graph = run(genv)
    want_z, want_w, _ = run(cenv)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert "+the weight gradient X^T A over" in listing and int(listing.split()[0]) == 2, listing
    assert rel_l2(got_z, want_z) <= TOL
    assert rel_l2(got_w, want_w) <= TOL


@pytest.mark.parametrize("rows,m,n,force,buffers", [
    (16384, 128, 260, "64,64,16,1,1,8", None), (32768, 128, 132, "128,64,32,2,2,8", None), (16384, 256, 388, "256,256,32,4,4,8", None),
    (8192, 512, 512, None, None), (16384, 256, 256, None, "3"), (16384, 256, 256, "128,128,32,2,2,8", None),
])
def test_column_sums_from_tiles_loaded_straight_into_lds(hip_backend_session, monkeypatch, rows, m, n, force, buffers):
    """A weight gradient x^T dz with the bias gradient (the column sums of dz) taken from the B tiles as they pass
    through LDS: whole and ragged products, a thread's pieces on one and on both sides of the swapped row halves,
    two and three tile buffers, against the oracle."""
    if buffers is None:
        monkeypatch.delenv("DSC_MM_DIRECT_LDS", raising=False)
    else:
        monkeypatch.setenv("DSC_MM_DIRECT_LDS", buffers)
    if force is None:
        monkeypatch.delenv("DSC_MM_TILE", raising=False)
    else:
        monkeypatch.setenv("DSC_MM_TILE", force)
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(rows + n)
        x = env.static_parameter_with_data([rows, m], "x", rng.standard_normal(rows * m, dtype=np.float32))
        dz = env.static_parameter_with_data([rows, n], "dz", rng.standard_normal(rows * n, dtype=np.float32))
        dw = env.static_parameter([m, n], "dw")
        db = env.static_parameter([n], "db")

        def build(s):
            d = s.parameter_value(dz)
            s.write_parameter_value(db, d.reduce_sum(0, False) * 0.5)
            # (the sine keeps x a stored operand of the product and puts the product behind the sum in the schedule)
            s.write_parameter_value(dw, s.parameter_value(x).sin().transpose().matmul(d))

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(dw), env.read_parameter(db), graph

    got_w, got_b, graph = run(genv)
    want_w, want_b, _ = run(cenv)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert "+column sums of B" in listing and f"tiles straight into LDS x{buffers or 2}" in listing, listing
    if force is not None:
        bm, bn, bk = force.split(",")[:3]
        assert f"tile {bm}x{bn}x{bk} " in listing, listing
    assert rel_l2(got_w, want_w) <= TOL
    assert rel_l2(got_b, want_b) <= TOL


@pytest.mark.parametrize("case", ["k-chunks", "batches", "rows-mode", "batches-transposed"])
def test_direct_lds_tiles_over_k_chunks_and_batches(hip_backend_session, case):
    """The same path where a unit is a (k-chunk, batch, tile) triple: the reference's 1024-deep k-chunks written as
    separate partial products (cluster by cluster), and batched products in both output modes."""
    from descent_amd import hip_backend
    from descent_amd.array import BATCHES, ROWS

    fused = case != "k-chunks"
    genv, cenv = _envs(hip_backend_session, fused=fused)

    def run(env):
        rng = np.random.default_rng(11)
        if case == "k-chunks":
            m, n, k = 512, 512, 4096
            a = env.static_parameter_with_data([m, k], "a", rng.standard_normal(m * k, dtype=np.float32))
            b = env.static_parameter_with_data([k, n], "b", rng.standard_normal(k * n, dtype=np.float32))
            c = env.static_parameter([m, n], "c")
            build = lambda s: s.write_parameter_value(c, s.parameter_value(a).matmul(s.parameter_value(b)))
        else:
            g, m, n, k = 3, 1024, 512, 96
            tb = case == "batches-transposed"
            a = env.static_parameter_with_data([g, m, k], "a", rng.standard_normal(g * m * k, dtype=np.float32))
            b = env.static_parameter_with_data([g, n, k] if tb else [g, k, n], "b", rng.standard_normal(g * k * n, dtype=np.float32))
            c = env.static_parameter([g, m, n], "c")

            def build(s):
                bv = s.parameter_value(b)
                s.write_parameter_value(c, s.parameter_value(a).batched_matmul(bv.transpose() if tb else bv, ROWS if case == "rows-mode" else BATCHES))

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(c), graph

    got, graph = run(genv)
    want, _ = run(cenv)
    assert rel_l2(got, want) <= TOL
    listing = hip_backend.check_schedule(graph, fused=fused)
    assert "tiles straight into LDS" in listing, listing
    if case == "k-chunks":
        assert "chunks 4" in listing, listing


@pytest.mark.parametrize("rows,with_last", [(16384, True), (40000, True), (20000, False)])
def test_concat_chain_with_gathers_as_one_row_kernel(hip_backend_session, rows, with_last):
    """Four pieces of different widths joined by three concats, one of them gathered from a table through indices
    computed from a small array, another scaled: one launch that evaluates a row per thread.  Bit-exact against the
    oracle (nothing is summed)."""
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(rows)
        a = env.static_parameter_with_data([rows, 2], "a", rng.standard_normal(rows * 2, dtype=np.float32))
        t = env.static_parameter_with_data([1000, 3], "t", rng.standard_normal(3000, dtype=np.float32))
        i = env.static_parameter_with_data([rows], "i", rng.integers(0, 5000, rows).astype(np.float32))
        c = env.static_parameter_with_data([rows, 2], "c", rng.standard_normal(rows * 2, dtype=np.float32))
        d = env.static_parameter_with_data([rows, 5], "d", rng.standard_normal(rows * 5, dtype=np.float32))
        width = 12 if with_last else 7  # 7: rows that are not whole 16-byte pieces
        out = env.static_parameter([rows, width], "out")

        def build(s):
            index = (s.parameter_value(i).into_u32() * 7) % 1000
            gathered = s.parameter_value(t).gather(-2, index)
            joined = (s.parameter_value(a) * 2.0).concat(gathered, -1).concat(s.parameter_value(c) + 1.0, -1)
            if with_last:
                joined = joined.concat(s.parameter_value(d), -1)
            s.write_parameter_value(out, joined)

        graph = env.build_graph(build)
        env.run(graph, 0)
        return env.read_parameter(out), graph

    got, graph = run(genv)
    want, _ = run(cenv)
    assert np.array_equal(got, want)
    listing = next(iter(graph.__dict__["_schedules"].values())).describe()
    assert int(listing.split()[0]) == 1 and "a thread per row of %d columns" % (12 if with_last else 7) in listing, listing


@pytest.mark.parametrize("mode", ["fused", "unfused", "kernel_by_kernel"])
def test_convnet_train_steps_vs_oracle(hip_backend_session, mode):
    """Three Adam steps of the ConvNet at batch 16: every parameter, optimiser state and the loss/accuracy sums."""
    from descent_amd import Environment, workloads
    from oracle.cpu_backend import CpuBackend

    genv = Environment(hip_backend_session, use_schedule=mode != "kernel_by_kernel", fused=mode == "fused")
    cenv = Environment(CpuBackend())
    gw = workloads.convnet(genv, batch=16, seed=11)
    cw = workloads.convnet(cenv, batch=16, seed=11)
    for step in range(3):
        genv.run(gw.graph, 1000 + step)
        cenv.run(cw.graph, 1000 + step)
    got, want = gw.snapshot(), cw.snapshot()
    assert got.keys() == want.keys()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key  # argmax-derived: exact
        else:
            err = rel_l2(got[key], want[key])
            assert err <= TOL, f"{key} [{mode}]: rel L2 {err}"


@pytest.mark.parametrize("mode,batch", [("fused", 16), ("unfused", 16), ("fused", 64)])
def test_conv_blur_net_train_steps_vs_oracle(hip_backend_session, mode, batch):
    """Three Adam steps of the ConvBlurNet (examples/fashion_mnist/main.rs:187-199: every pool a 2x2 stride-1 max pool
    and a fixed 3x3 stride-2 depthwise blur, src/module.rs:219-246): parameters, optimiser state, loss and accuracy."""
    from descent_amd import Environment, workloads
    from oracle.cpu_backend import CpuBackend

    genv = Environment(hip_backend_session, fused=mode == "fused")
    cenv = Environment(CpuBackend())
    gw = workloads.convnet(genv, batch=batch, seed=19, blur_pool=True)
    cw = workloads.convnet(cenv, batch=batch, seed=19, blur_pool=True)
    for step in range(3):
        genv.run(gw.graph, 2000 + step)
        cenv.run(cw.graph, 2000 + step)
    got, want = gw.snapshot(), cw.snapshot()
    assert got.keys() == want.keys()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key
        else:
            err = rel_l2(got[key], want[key])
            assert err <= TOL, f"{key} [{mode}, batch {batch}]: rel L2 {err}"


def test_linear_classifier_steps_vs_oracle(hip_backend_session):
    """Config 1: single-layer softmax classifier, batch 1000, SGD momentum; 10 steps then one eval pass."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session)
    gw = workloads.linear_classifier(genv, batch=1000, seed=1)
    cw = workloads.linear_classifier(cenv, batch=1000, seed=1)
    for step in range(10):
        genv.run(gw.graph, step)
        cenv.run(cw.graph, step)
    genv.run(gw.test_graph, 99)
    cenv.run(cw.test_graph, 99)
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key
        else:
            assert rel_l2(got[key], want[key]) <= TOL, key


def test_large_matmul_sampled_rows(hip_backend_session):
    """4096^3 with the fused epilogue: 64 sampled rows against a float64 product (the oracle would take minutes)."""
    from descent_amd import Environment, workloads

    env = Environment(hip_backend_session)
    n = 4096
    w = workloads.matmul_epilogue(env, n, n, n, seed=7)
    env.run(w.graph, 0)
    c = env.read_parameter(w.c)
    a = env.read_parameter(w.a).astype(np.float64)
    b = env.read_parameter(w.b).astype(np.float64)
    bias = env.read_parameter(w.bias).astype(np.float64)
    rows = np.random.default_rng(0).choice(n, 64, replace=False)
    z = a[rows] @ b + bias
    want = np.where(z > 0, z, 0.01 * z)
    assert rel_l2(c[rows], want) <= TOL


@pytest.mark.parametrize("m,n,k", [(1000, 128, 784), (1000, 128, 1568), (777, 100, 600), (3000, 36, 516), (257, 200, 2048), (4099, 32, 1024)])
def test_matmul_with_k_split_inside_the_workgroups(hip_backend_session, m, n, k):
    """Small products over a moderate k run as one launch, the eight waves of a workgroup a slice of k each: ragged row
    and column counts, k that is no multiple of 16 or of the waves' slices, against a float64 product."""
    from descent_amd import Environment, workloads

    env = Environment(hip_backend_session)
    w = workloads.matmul_epilogue(env, m, n, k, seed=m + n + k)
    env.run(w.graph, 0)
    listing = next(iter(w.graph.__dict__["_schedules"].values())).describe()
    assert int(listing.split()[0]) == 1 and "k split over the 8 waves of a workgroup" in listing, listing
    a = env.read_parameter(w.a).astype(np.float64)
    b = env.read_parameter(w.b).astype(np.float64)
    z = a @ b + env.read_parameter(w.bias).astype(np.float64)
    assert rel_l2(env.read_parameter(w.c), np.where(z > 0, z, 0.01 * z)) <= 2e-6, listing


def test_heap_reuse_and_errors(hip_backend_session):
    from descent_amd.hip_backend import DescentHipError

    be = hip_backend_session
    live0, _, _ = be.heap_stats()
    hs = [be.alloc(1000 * (i + 1)) for i in range(8)]
    ptrs = [be.device_ptr(h) for h in hs]
    assert all(p % 256 == 0 for p in ptrs)
    assert len(set(ptrs)) == len(ptrs)
    for h in hs[::2]:
        be.free(h)
    for h in hs[1::2]:
        be.free(h)
    assert be.heap_stats()[0] == live0
    with pytest.raises(DescentHipError):
        be.free(hs[0])  # double free is reported, not undefined behaviour
    h = be.alloc(64)
    with pytest.raises(DescentHipError):
        be.read(h, 0, 128)  # range check
    be.write(h, 0, np.arange(16, dtype=np.float32))
    be.fill_zero(h, 32, 32)
    got = np.frombuffer(be.read(h, 0, 64), np.float32)
    assert np.array_equal(got, np.concatenate([np.arange(8, dtype=np.float32), np.zeros(8, np.float32)]))
    be.free(h)


def test_bias_gradient_rides_on_the_weight_gradient_matmul(hip_backend_session):
    """A 128x128 grid through two hidden layers of 256: dZ is [16384, 256], large enough for the schedule to take the
    bias gradients (column sums of dZ) out of the weight-gradient MatMuls that read dZ as their B operand, instead of
    a Reduce pass of its own.  Three Adam steps against the oracle."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session)
    kw = dict(side=128, variant="relu-pe", hidden=(256, 256), freq_count=4, seed=31)
    gw = workloads.coordinate_mlp(genv, **kw)
    cw = workloads.coordinate_mlp(cenv, **kw)
    for step in range(3):
        genv.run(gw.graph, step)
        cenv.run(cw.graph, step)
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    assert listing.count("+column sums of B") >= 2, listing
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        err = rel_l2(got[key], want[key])
        assert err <= TOL, f"{key}: rel L2 {err}"


@pytest.mark.parametrize("variant", ["relu-pe", "siren", "plain-relu"])
def test_coordinate_mlp_steps_vs_oracle(hip_backend_session, variant):
    """Config 4 at reduced size (64x64 grid, two hidden layers of 64): three Adam steps.  "plain-relu" is the leaky
    variant with slope 0: the schedule reads the sign of a pre-activation off the stored activation either way."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session)
    kw = dict(side=64, variant="relu-pe" if variant == "plain-relu" else variant, hidden=(64, 64), freq_count=8, seed=21,
              leakiness=0.0 if variant == "plain-relu" else 0.01)
    gw = workloads.coordinate_mlp(genv, **kw)
    cw = workloads.coordinate_mlp(cenv, **kw)
    for step in range(3):
        genv.run(gw.graph, step)
        cenv.run(cw.graph, step)
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        err = rel_l2(got[key], want[key])
        assert err <= TOL, f"{variant} {key}: rel L2 {err}"


def test_hash_grid_steps_vs_oracle(hip_backend_session):
    """Config 5 at reduced size: dense and hashed levels, bilinear gathers, float-atomic scatter-add.
    The atomic adds reorder fp32 sums, so the bound is the looser 1e-3 (relative L2) for every tensor here:
    the tables directly, everything else through them after the first step."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session)
    kw = dict(batch=8192, levels=(4, 16, 40, 100), entry_count=2048, hidden=(32,), seed=22)
    gw = workloads.hash_grid_fit(genv, **kw)
    cw = workloads.hash_grid_fit(cenv, **kw)
    for step in range(3):
        genv.run(gw.graph, step)
        cenv.run(cw.graph, step)
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        err = rel_l2(got[key], want[key])
        assert err <= 1e-3, f"{key}: rel L2 {err}"


def test_hash_grid_steps_vs_oracle_with_the_encoding_as_one_kernel(hip_backend_session):
    """Config 5 at a size where the planner's large-array passes apply: the corner indices and weights are evaluated
    by their readers (outputs of 256 KiB), the chain of concats and gathers is one row kernel (65536 rows), the
    hashed levels' ScatterAdd chains go through binned records of rows of two.  Same bound as the smaller case."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session)
    kw = dict(batch=1 << 16, levels=(16, 40, 100, 300), entry_count=1 << 14, hidden=(32,), seed=23)
    gw = workloads.hash_grid_fit(genv, **kw)
    cw = workloads.hash_grid_fit(cenv, **kw)
    for step in range(2):
        genv.run(gw.graph, step)
        cenv.run(cw.graph, step)
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    assert "a thread per row of 8 columns" in listing, listing
    assert "(target, two values) records" in listing, listing
    assert not any(line.split(": ")[1].startswith("PerElement (20 ops)") for line in listing.splitlines() if ": " in line), listing
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        err = rel_l2(got[key], want[key])
        assert err <= 1e-3, f"{key}: rel L2 {err}"


def test_gather_indices_are_bit_exact(hip_backend_session):
    """The hash index arithmetic (u32 xor / mul / rem on bit-cast floats) and the gathered values must match
    the oracle bit for bit."""
    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(3)
        pts = env.static_parameter_with_data([4096, 2], "x", rng.random((4096, 2), dtype=np.float32) * 2 - 1)
        table = env.static_parameter_with_data([2048, 2], "t", rng.standard_normal((2048, 2), dtype=np.float32))
        idx_out = env.static_parameter([4096], "i")
        val_out = env.static_parameter([4096, 2], "v")

        def build(s):
            cf = (s.parameter_value(pts) * 0.5 + 0.5) * 100.0
            c = cf.into_u32()
            c0, c1 = c.lock_axis(-1, 0, False), c.lock_axis(-1, 1, False)
            i = ((c0 + 1) ^ (c1 * 1526263 + 1526263)) % 2048
            s.write_parameter_value(idx_out, i.to_f32_bits())
            s.write_parameter_value(val_out, s.parameter_value(table).gather(-2, i))

        env.run(env.build_graph(build), 0)
        return env.read_parameter(idx_out).view(np.uint32), env.read_parameter(val_out)

    gi, gv = run(genv)
    ci, cv = run(cenv)
    assert np.array_equal(gi, ci) and gi.max() < 2048
    assert np.array_equal(gv.view(np.uint32), cv.view(np.uint32))


def _softmax_case(env, m, n, seed, quantised):
    """Logits as a trainable parameter: per-row loss, d loss / d logits and the per-row accuracy flag."""
    from descent_amd import Initializer
    from descent_amd.loss import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss

    rng = np.random.default_rng(seed)
    z = rng.standard_normal((m, n), dtype=np.float32) * 3
    if quantised:  # repeated maxima in a row: the arg-max tie rule decides the accuracy flag
        z = np.round(z)
    zp = env.trainable_parameter([m, n], "z", Initializer.zero())
    yp = env.static_parameter_with_data([m, 1], "y", rng.integers(0, n, (m, 1)).astype(np.float32))
    env.write_parameter(zp, z)
    loss_rows, acc_rows, dz = env.static_parameter([m, 1], "l"), env.static_parameter([m, 1], "a"), env.static_parameter([m, n], "dz")

    def build(s):
        zd = s.parameter(zp)
        loss = softmax_cross_entropy_loss(zd, yp).set_loss()
        s.write_parameter_value(loss_rows, loss)
        s.write_parameter_value(acc_rows, softmax_cross_entropy_accuracy(zd, yp))
        s.write_parameter_value(dz, zd.loss_grad())

    g = env.build_graph(build)
    env.run(g, 0)
    return g, env.read_parameter(loss_rows), env.read_parameter(acc_rows), env.read_parameter(dz)


@pytest.mark.parametrize("m,k,n", [(1000, 128, 10), (300, 64, 7), (5000, 200, 16), (65, 33, 3), (1000, 400, 10)])
def test_classifier_head_product_is_the_first_stage_of_the_row_fused_launch(hip_backend_session, m, k, n):
    """features x weights + bias -> softmax cross-entropy and accuracy: the small MatMul runs inside the row-fused launch
    (lanes of a row share its k range); loss rows, accuracy flags and the gradient of the logits against the oracle."""
    from descent_amd import Initializer
    from descent_amd.loss import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss

    genv, cenv = _envs(hip_backend_session)

    def run(env):
        rng = np.random.default_rng(m + k + n)
        x = env.static_parameter_with_data([m, k], "x", rng.standard_normal(m * k, dtype=np.float32))
        w = env.trainable_parameter([k, n], "w", Initializer.zero())
        env.write_parameter(w, rng.standard_normal(k * n, dtype=np.float32) * 0.3)
        b = env.static_parameter_with_data([n], "b", rng.standard_normal(n, dtype=np.float32))
        y = env.static_parameter_with_data([m, 1], "y", rng.integers(0, n, (m, 1)).astype(np.float32))
        loss_rows, acc_rows, dw = env.static_parameter([m, 1], "l"), env.static_parameter([m, 1], "a"), env.static_parameter([k, n], "dw")

        def build(s):
            wd = s.parameter(w)
            z = s.parameter(x).next_colour().matmul(wd) + s.parameter(b)
            loss = softmax_cross_entropy_loss(z, y).set_loss()
            s.write_parameter_value(loss_rows, loss)
            s.write_parameter_value(acc_rows, softmax_cross_entropy_accuracy(z, y))
            s.write_parameter_value(dw, wd.loss_grad())

        g = env.build_graph(build)
        env.run(g, 0)
        return g, env.read_parameter(loss_rows), env.read_parameter(acc_rows), env.read_parameter(dw)

    g, gl, ga, gdw = run(genv)
    _, cl, ca, cdw = run(cenv)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    assert "the first a MatMul over k=%d shared by the row's lanes" % k in listing, listing
    assert rel_l2(gl, cl) <= TOL and rel_l2(gdw, cdw) <= TOL
    # Arg-max outputs are exact.  The one admissible difference: the two paths add a logit's k terms in different
    # orders, so two logits of a row that lie closer than the rounding of those sums may swap places.  Every row
    # whose flag differs must be such a near-tie (top two float64 logits closer than k * 2^-23 * sum |x * w|, the
    # bound on the difference of two fp32 summation orders); every other row's flag is bit-equal by construction.
    rng = np.random.default_rng(m + k + n)
    x64 = rng.standard_normal(m * k, dtype=np.float32).reshape(m, k).astype(np.float64)
    w64 = (rng.standard_normal(k * n, dtype=np.float32) * 0.3).astype(np.float32).reshape(k, n).astype(np.float64)
    b64 = rng.standard_normal(n, dtype=np.float32).astype(np.float64)
    differing = np.flatnonzero(ga.ravel() != ca.ravel())
    assert len(differing) <= max(2, m // 500), differing
    for row in differing:
        z = x64[row] @ w64 + b64
        top = np.sort(z)[-2:]
        bound = k * 2.0 ** -23 * float(np.max((np.abs(x64[row])[:, None] * np.abs(w64)).sum(axis=0)))
        assert top[1] - top[0] <= bound, (row, top, bound)


@pytest.mark.parametrize("m,n", [(1000, 10), (37, 3), (64, 64), (5, 33), (4097, 2), (300, 17)])
@pytest.mark.parametrize("quantised", [False, True])
def test_softmax_cross_entropy_runs_as_one_row_fused_launch(hip_backend_session, m, n, quantised):
    genv, cenv = _envs(hip_backend_session)
    g, gl, ga, gdz = _softmax_case(genv, m, n, 31 + m + n, quantised)
    _, cl, ca, cdz = _softmax_case(cenv, m, n, 31 + m + n, quantised)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    assert "RowFused [%d, %d]" % (m, n) in listing and int(listing.split()[0]) <= 2, listing
    assert rel_l2(gl, cl) <= TOL and rel_l2(gdz, cdz) <= TOL
    assert np.array_equal(ga, ca)  # arg-max derived: exact, ties included


@pytest.mark.parametrize("fused", [True, "split-conv-grads", "generic-conv"])
def test_convnet_step_at_batch_64_vs_oracle(hip_backend_session, fused):
    """At this batch the convolution GEMMs are large enough for the row-per-thread kernels.  The data gradient of
    the second convolution runs either as the dedicated kernel (MatMul + reshape copy + WindowsToImage + both
    Unpads, image tile in LDS) or, with "generic-conv", as one MatMul over the padded image whose operands are
    fused producers.  Two Adam steps, every parameter and optimiser state."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session, fused=fused)
    gw = workloads.convnet(genv, batch=64, seed=13)
    cw = workloads.convnet(cenv, batch=64, seed=13)
    for step in range(2):
        genv.run(gw.graph, 500 + step)
        cenv.run(cw.graph, 500 + step)
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    if fused is True:
        assert "ConvBackward" in listing and "filter gradient mfma 16x16x4 5x1 tiles" in listing, listing
    elif fused == "split-conv-grads":
        assert "ConvDataGrad" in listing and "3x3 taps x 16 channels, border folds fused" in listing, listing
    else:
        assert "MatMul (k=144) [1, 16384, 2, 8]" in listing and "row-per-thread" in listing, listing
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key
        else:
            err = rel_l2(got[key], want[key])
            assert err <= TOL, f"{key}: rel L2 {err}"


def _scatter_chain_case(env, n, entries, links, seed):
    """`links` scatter-adds chained through one [entries, 2] accumulator, as the corner updates of one hash-grid
    level are: values [n, 2] ~ N(0,1), indices uniform."""
    rng = np.random.default_rng(seed)
    vals = [env.static_parameter_with_data([n, 2], f"v{i}", rng.standard_normal((n, 2), dtype=np.float32)) for i in range(links)]
    idxs = [env.static_parameter_with_data([n], f"i{i}", rng.integers(0, entries, n).astype(np.float32)) for i in range(links)]
    out = env.static_parameter([entries, 2], "acc")

    def build(s):
        acc = s.literal(0.0).value().broadcast([entries, 2])
        for v, i in zip(vals, idxs):
            acc = acc.scatter_add(s.parameter_value(v), 0, s.parameter_value(i).into_u32())
        s.write_parameter_value(out, acc)

    g = env.build_graph(build)
    env.run(g, 0)
    want = np.zeros((entries, 2), np.float64)
    for v, i in zip(vals, idxs):
        np.add.at(want, env.read_parameter(i).astype(np.int64), env.read_parameter(v).astype(np.float64))
    return g, env.read_parameter(out), want


@pytest.mark.parametrize("n,entries,links", [(131072, 289, 4), (65536, 3481, 2), (131072, 100000, 4), (70000, 3, 3), (262144, 12544, 4), (100001, 17000, 5)])
def test_scatter_add_chains_vs_float64(hip_backend_session, n, entries, links):
    """Float atomics reorder the sums, so the bound is the looser one stated for scatter-add: 1e-4 relative L2
    against a float64 accumulation, for the GPU (accumulators that fit LDS go through per-workgroup sums first) and
    for the oracle's serial fp32 sums alike."""
    genv, cenv = _envs(hip_backend_session)
    g, got, want = _scatter_chain_case(genv, n, entries, links, 40 + entries)
    _, oracle, _ = _scatter_chain_case(cenv, n, entries, links, 40 + entries)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    # the whole chain of scatter-adds is one launch (two when the values are binned by accumulator segment first),
    # the Fill that zeroes the accumulator and the bin counters another; the index conversions are evaluated by the
    # links themselves (their input, the index array, is small enough to stay in L2)
    assert "Multi (%d kernels: ScatterAdd" % links in listing, listing
    # accumulators with at least 16 values per entry, of up to 8192 floats (18432 when the chain has too few values
    # for the two-launch form): one LDS copy per workgroup takes every link
    lds_limit = 64 * 1024 if links * n * 2 >= 1 << 18 else 144 * 1024  # the LDS copy is kept in double
    if entries * 2 * 8 <= lds_limit and links * n * 2 >= 16 * entries * 2:
        assert "accumulator of %d floats kept in LDS" % (entries * 2) in listing, listing
        assert int(listing.split()[0]) == 2, listing
    elif links * n * 2 >= 1 << 18:
        # larger accumulators with enough values: records ordered by segment, then summed segment by segment in LDS
        assert "stage 1 of 2" in listing and "stage 2 of 2" in listing and "kept in LDS" not in listing, listing
        assert int(listing.split()[0]) == 3, listing
    else:
        assert "kept in LDS" not in listing and "stage 1 of 2" not in listing, listing
        assert int(listing.split()[0]) == 2, listing
    assert rel_l2(got, want) <= TOL
    assert rel_l2(oracle, want) <= TOL


def test_fences_order_work_like_the_reference_fence_set(hip_backend_session):
    """device/fence.rs:21-86: ids grow by one, waiting on one retires the older ones, unknown ids are errors."""
    from descent_amd import Environment, workloads
    from descent_amd.hip_backend import DescentHipError

    be = hip_backend_session
    env = Environment(be)
    w = workloads.matmul_epilogue(env, 1024, 1024, 1024, seed=3)
    fences = []
    for step in range(4):  # two steps in flight, as the reference keeps them (device/command_buffer.rs:64-123)
        env.run(w.graph, step)
        fences.append(be.fence_record())
        if len(fences) > 2:
            be.fence_wait(fences[-3])
            assert be.fence_finished(fences[-3])
    assert fences == list(range(fences[0], fences[0] + 4))
    be.fence_wait(fences[-1])
    assert all(be.fence_finished(f) for f in fences)
    with pytest.raises(DescentHipError):
        be.fence_wait(fences[-1] + 100)
    with pytest.raises(DescentHipError):
        be.fence_wait(0)


def test_graph_replay_matches_direct_launches_on_every_replay(hip_backend_session):
    """Ten ConvNet steps (batch 16, a new dropout seed each step) with HIP-graph replay against the same steps on
    the oracle, parameters compared after every step: replays after the first must see the new seed (it travels
    through a device cell) and the same buffers, with eager uploads and reads between them."""
    from descent_amd import workloads

    genv, cenv = _envs(hip_backend_session, fused="graph-replay")
    gw = workloads.convnet(genv, batch=16, seed=17)
    cw = workloads.convnet(cenv, batch=16, seed=17)
    for step in range(10):
        genv.run(gw.graph, 300 + step)
        cenv.run(cw.graph, 300 + step)
        got, want = gw.snapshot(), cw.snapshot()  # eager device-to-host reads between the replays
        for key in want:
            if key == "accuracy":
                assert np.array_equal(got[key], want[key]), (step, key)
            else:
                assert rel_l2(got[key], want[key]) <= TOL, (step, key, rel_l2(got[key], want[key]))
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    import re
    m = re.search(r"graph replays (\d+), captured (\d+), direct runs (\d+)", listing)
    assert m and int(m.group(1)) + int(m.group(2)) + int(m.group(3)) >= 10, listing
    # the schedule keeps its intermediates in a region of its own and lets every written parameter alternate between
    # its buffer and a spare, so a step's pointers repeat with period two: two captures, every other step a replay
    assert (int(m.group(1)), int(m.group(2)), int(m.group(3))) == (8, 2, 0), listing


def test_graph_replay_with_an_output_that_starts_without_a_buffer(hip_backend_session):
    """A written parameter that has no buffer before the first run (an output nobody uploaded to) leaves no old
    buffer behind to serve as the next run's spare: the schedule has to give that slot a new spare, or it would fall
    back to allocating runs for good.  Six runs of a chain of four products: two captures, four replays, every run's
    result against the oracle."""
    import re

    genv, cenv = _envs(hip_backend_session, fused="graph-replay")

    def make(env):
        rng = np.random.default_rng(77)
        a = env.static_parameter_with_data([256, 256], "a", rng.standard_normal((256, 256), dtype=np.float32))
        b = env.static_parameter_with_data([256, 256], "b", rng.standard_normal((256, 256), dtype=np.float32) / 16)
        out = env.static_parameter([256, 256], "out")  # never written from the host
        assert out.buffer is None

        def build(s):
            bv = s.parameter_value(b)
            c = s.parameter_value(a)
            for _ in range(4):
                c = c.matmul(bv)
            s.write_parameter_value(out, c)

        return env.build_graph(build), out

    gg, gout = make(genv)
    cg, cout = make(cenv)
    cenv.run(cg, 0)
    want = cenv.read_parameter(cout)
    for step in range(6):
        genv.run(gg, step)
        assert rel_l2(genv.read_parameter(gout), want) <= TOL, step
    listing = next(iter(gg.__dict__["_schedules"].values())).describe()
    assert int(listing.split()[0]) >= 4, listing
    m = re.search(r"graph replays (\d+), captured (\d+), direct runs (\d+)", listing)
    assert m and (int(m.group(1)), int(m.group(2)), int(m.group(3))) == (4, 2, 0), listing


@pytest.mark.parametrize("batch,side,hidden", [(1000, 28, 128), (333, 24, 300), (64, 28, 64)])
@pytest.mark.parametrize("switch", [None, "DSC_FUSE_ROWS_DGRAD", "DSC_FUSE_ROWS_OPERAND"])
def test_hidden_layer_classifier_head_in_one_row_fused_launch(hip_backend_session, monkeypatch, batch, side, hidden, switch):
    """The reference's single-hidden-layer classifier, three momentum steps: the row-fused launch of the head evaluates
    and stores the hidden activation (bias + leaky_relu over the first product's k chunks) and ends with the head's
    data gradient masked by it; each of the two can be switched off, and all three ways match the oracle."""
    from descent_amd import workloads

    if switch:
        monkeypatch.setenv(switch, "0")
    # (the first product's k stays split into chunks here: on the kernel that splits k inside its workgroups the hidden
    # activation is that kernel's epilogue and there is no cluster for the row-fused launch to take)
    monkeypatch.setenv("DSC_MM_KSPLIT", "0")
    genv, cenv = _envs(hip_backend_session)
    gw = workloads.single_layer_classifier(genv, batch=batch, side=side, hidden_units=hidden)
    cw = workloads.single_layer_classifier(cenv, batch=batch, side=side, hidden_units=hidden)
    for step in range(3):
        genv.run(gw.graph, 40 + step)
        cenv.run(cw.graph, 40 + step)
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    line = next(l for l in listing.splitlines() if "RowFused" in l)
    assert ("data gradient behind the last" in line) == (switch != "DSC_FUSE_ROWS_DGRAD"), listing
    assert ("fused producers>" in line) == (switch != "DSC_FUSE_ROWS_OPERAND"), listing
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key
        else:
            assert rel_l2(got[key], want[key]) <= TOL, (key, rel_l2(got[key], want[key]), listing)


@pytest.mark.parametrize("loaders", ["0", "1", "2"])
@pytest.mark.parametrize("batch,side", [(520, 28), (777, 20)])
def test_convnet_backward_with_and_without_loader_waves(hip_backend_session, monkeypatch, loaders, batch, side):
    """Two Adam steps of the ConvNet with the second convolution's backward kernel in its three forms: 256 threads that
    fill, multiply and fold in turn (0), loader waves with the pooling gradient as a producer of their fills (1), loader
    waves over a dC that stays a buffer (2)."""
    from descent_amd import workloads

    monkeypatch.setenv("DSC_CONV_BWD_LOADERS", loaders)
    genv, cenv = _envs(hip_backend_session)
    gw = workloads.convnet(genv, batch=batch, seed=31, side=side)
    cw = workloads.convnet(cenv, batch=batch, seed=31, side=side)
    for step in range(2):
        genv.run(gw.graph, 7 + step)
        cenv.run(cw.graph, 7 + step)
    listing = next(iter(gw.graph.__dict__["_schedules"].values())).describe()
    line = next(l for l in listing.splitlines() if "ConvBackward" in l)
    assert ("loader waves" in line) == (loaders != "0"), listing
    # (the pooling gradient becomes a producer of the fills only where the kernel is dC's one reader, which it is when
    # the bias gradient's column sums ride on it: batch 1000, tests/test_gpu_full_size.py)
    if loaders != "1":
        assert "fused producers>" not in line.split("[conv backward")[0], listing
    got, want = gw.snapshot(), cw.snapshot()
    for key in want:
        if key == "accuracy":
            assert np.array_equal(got[key], want[key]), key
        else:
            assert rel_l2(got[key], want[key]) <= TOL, (key, rel_l2(got[key], want[key]), listing)


@pytest.mark.parametrize("batch,side,loaders", [(1000, 28, "1"), (1000, 28, "0"), (1536, 20, "1")])
def test_pooling_gradients_read_off_window_words_are_bit_equal(hip_backend_session, monkeypatch, batch, side, loaders):
    """Two Adam steps of the ConvNet with the pooling gradients evaluated from the stored activations (DSC_POOL_WORDS=0)
    and read off the two bits per element the forward kernels write in their place: the comparisons are made on the
    same values, so every parameter, optimiser state and loss comes out bit for bit the same."""
    from descent_amd import Environment, workloads

    monkeypatch.setenv("DSC_CONV_BWD_LOADERS", loaders)
    results, listings = [], []
    for words in ("0", "1"):
        monkeypatch.setenv("DSC_POOL_WORDS", words)
        env = Environment(hip_backend_session)
        w = workloads.convnet(env, batch=batch, seed=17, side=side)
        for step in range(2):
            env.run(w.graph, 3 + step)
        results.append(w.snapshot())
        listings.append(next(iter(w.graph.__dict__["_schedules"].values())).describe())
    assert "pooling windows' words" not in listings[0] and "window words in place of its source" not in listings[0], listings[0]
    # the first convolution's filter gradient always reads the words; the second one's backward kernel where it took the
    # pooling gradient as a producer of its fills (loader waves)
    assert listings[1].count("dC read off the pooling windows' words") == (2 if loaders == "1" else 1), listings[1]
    assert listings[1].count("window words in place of its source") == (2 if loaders == "1" else 1), listings[1]
    for key in results[0]:
        assert np.array_equal(results[0][key], results[1][key]), (key, listings[1])


@pytest.mark.parametrize("side", [128, 100])
def test_masked_data_gradients_read_sign_bytes_bit_equal(hip_backend_session, monkeypatch, side):
    """Two Adam steps of the coordinate MLP (leaky_relu layers of 256) with the data gradients masked by the stored
    activations (DSC_SIGN_BYTES=0) and by the bytes of sign bits the forward products write beside them: "(a > 0)" is
    evaluated on the same values either way, so everything comes out bit for bit the same.  side 100: 10000 rows, the
    last tile reaches past them."""
    from descent_amd import Environment, workloads

    results, listings = [], []
    for on in ("0", "1"):
        monkeypatch.setenv("DSC_SIGN_BYTES", on)
        env = Environment(hip_backend_session)
        w = workloads.coordinate_mlp(env, side=side)
        for step in range(2):
            env.run(w.graph, 5 + step)
        results.append(w.snapshot())
        listings.append(next(iter(w.graph.__dict__["_schedules"].values())).describe())
    assert "sign bytes" not in listings[0], listings[0]
    assert listings[1].count("masks by sign bytes") == 3 and listings[1].count("writes its output's sign bytes") == 3, listings[1]
    for key in results[0]:
        assert np.array_equal(results[0][key], results[1][key]), (key, listings[1])


def _conv_grad_case(env, m, h, w, c_in, c_out, fh, fw, pad, groups, seed):
    """x -> conv2d -> 0.5 * sum(y^2): the gradients with respect to the image and the filter."""
    from descent_amd import Initializer

    rng = np.random.default_rng(seed)
    xp = env.trainable_parameter([m, h, w, c_in], "x", Initializer.zero())
    fp = env.trainable_parameter([groups, c_out // groups, fh, fw, c_in // groups], "f", Initializer.zero())
    env.write_parameter(xp, rng.standard_normal((m, h, w, c_in), dtype=np.float32))
    env.write_parameter(fp, rng.standard_normal((groups, c_out // groups, fh, fw, c_in // groups), dtype=np.float32) * 0.2)
    dx, df = env.static_parameter([m, h, w, c_in], "dx"), env.static_parameter(list(fp.shape), "df")
    y_out = env.static_parameter([m, h + 2 * pad - fh + 1, w + 2 * pad - fw + 1, c_out], "y")

    def build(s):
        x, f = s.parameter(xp), s.parameter(fp)
        y = x.conv2d(f, pad)
        s.write_parameter_value(y_out, y.value() * 1.0)
        (y.square() * 0.5).set_loss()
        s.write_parameter_value(dx, x.loss_grad())
        s.write_parameter_value(df, f.loss_grad())

    g = env.build_graph(build)
    env.run(g, 0)
    return g, env.read_parameter(y_out), env.read_parameter(dx), env.read_parameter(df)


CONV_GEOMETRIES = [
    # m, h, w, c_in, c_out, fh, fw, pad, groups
    (64, 14, 14, 16, 32, 3, 3, 1, 2),   # the ConvNet's second convolution
    (50, 12, 10, 4, 8, 3, 3, 1, 1),     # not square
    (40, 9, 9, 8, 8, 5, 5, 2, 2),       # 5x5 taps, pad 2
    (30, 20, 20, 4, 4, 3, 3, 1, 1),     # padded image larger than one pass of 256 pixels
    (60, 8, 8, 4, 8, 3, 3, 0, 1),       # no padding: no Unpads to fold
    (25, 7, 5, 16, 16, 3, 1, 0, 1),     # 3x1 taps
    (40, 10, 10, 6, 8, 3, 3, 1, 1),     # six channels: the data gradient stays on the vector units beside the filter gradient
    (3, 6, 6, 64, 64, 3, 3, 1, 1),      # many channels: stays on the generic path
    (20, 10, 10, 3, 6, 3, 3, 1, 1),     # three input channels, six outputs: no 16-byte pieces anywhere
    (16, 8, 8, 6, 20, 3, 3, 1, 2),      # the same per group, ten outputs
]
CONV_WITHOUT_DATA_GRAD_KERNEL = set(CONV_GEOMETRIES[-3:])
CONV_WITHOUT_FORWARD_KERNEL = {CONV_GEOMETRIES[-3]}


@pytest.mark.parametrize("geom", CONV_GEOMETRIES, ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("fused", [True, "split-conv-grads", "generic-conv", False])
def test_conv2d_gradients_over_geometries(hip_backend_session, geom, fused):
    genv, cenv = _envs(hip_backend_session, fused=fused)
    g, gy, gdx, gdf = _conv_grad_case(genv, *geom, seed=90)
    _, cy, cdx, cdf = _conv_grad_case(cenv, *geom, seed=90)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    if fused in (True, "split-conv-grads"):  # the dedicated kernels: image tile in LDS
        # (the data gradient alone, or together with the filter gradient where that one's k is long enough to be split)
        assert ("ConvDataGrad" in listing or "ConvBackward" in listing) == (geom not in CONV_WITHOUT_DATA_GRAD_KERNEL), listing
        assert ("ConvForward" in listing) == (geom not in CONV_WITHOUT_FORWARD_KERNEL), listing
    if fused == "split-conv-grads":
        assert "ConvBackward" not in listing, listing
    if fused == "generic-conv":
        assert "ConvDataGrad" not in listing and "ConvBackward" not in listing and "ConvForward" not in listing, listing
    assert rel_l2(gy, cy) <= TOL, listing
    assert rel_l2(gdx, cdx) <= TOL, (rel_l2(gdx, cdx), listing)
    assert rel_l2(gdf, cdf) <= TOL, (rel_l2(gdf, cdf), listing)


def _strided_conv_grad_case(env, m, h, w, c_in, c_out, fh, fw, pad, stride, groups, seed):
    """x -> conv2d with a stride -> 0.5 * sum(y^2): the product and the gradients with respect to the image and the filter."""
    from descent_amd import Initializer

    rng = np.random.default_rng(seed)
    xp = env.trainable_parameter([m, h, w, c_in], "x", Initializer.zero())
    fp = env.trainable_parameter([groups, c_out // groups, fh, fw, c_in // groups], "f", Initializer.zero())
    env.write_parameter(xp, rng.standard_normal((m, h, w, c_in), dtype=np.float32))
    env.write_parameter(fp, rng.standard_normal(tuple(fp.shape), dtype=np.float32) * 0.2)
    dx, df = env.static_parameter([m, h, w, c_in], "dx"), env.static_parameter(list(fp.shape), "df")
    oh, ow = (h + 2 * pad - fh) // stride[1] + 1, (w + 2 * pad - fw) // stride[0] + 1
    y_out = env.static_parameter([m, oh, ow, c_out], "y")

    def build(s):
        x, f = s.parameter(xp), s.parameter(fp)
        y = x.conv2d(f, pad, stride)
        s.write_parameter_value(y_out, y.value() * 1.0)
        (y.square() * 0.5).set_loss()
        s.write_parameter_value(dx, x.loss_grad())
        s.write_parameter_value(df, f.loss_grad())

    g = env.build_graph(build)
    env.run(g, 0)
    return g, env.read_parameter(y_out), env.read_parameter(dx), env.read_parameter(df)


@pytest.mark.parametrize("geom", [
    # m, h, w, c_in, c_out, fh, fw, pad, stride (w, h), groups
    (300, 27, 27, 16, 16, 3, 3, 1, (2, 2), 16),  # the blur of a MaxBlurPool2D: one group per channel, the chain one launch
    (200, 13, 13, 32, 32, 3, 3, 1, (2, 2), 32),
    (120, 12, 12, 8, 16, 2, 2, 0, (2, 2), 1),    # windows that tile the image: a copy, no sums
    (90, 11, 9, 4, 8, 3, 3, 0, (2, 2), 2),       # no padding: no Unpads
    (80, 11, 13, 6, 6, 4, 3, 1, (2, 3), 3),      # strides that differ, an even filter height
    (70, 16, 16, 8, 8, 5, 5, 2, (3, 3), 8),      # depthwise, stride 3, two replicated pixels per side
], ids=lambda g: "x".join(str(v) for v in g[:8]) + "s%dx%dg%d" % (g[8][0], g[8][1], g[9]))
def test_strided_conv2d_gradients_with_gathered_sums_on_demand(hip_backend_session, monkeypatch, geom):
    """Strided convolutions (src/array.rs:989-1031) take no dedicated kernel: the data gradient's WindowsToImage and
    Unpads, and the outer product in front of them where a group has one output channel, are evaluated on demand by
    the last of them.  Against the oracle within the tolerance, and bit for bit against the same kernels launched one
    by one (the sums are made in the standalone kernels' order)."""
    genv, cenv = _envs(hip_backend_session, fused=True)
    g, gy, gdx, gdf = _strided_conv_grad_case(genv, *geom, seed=41)
    _, cy, cdx, cdf = _strided_conv_grad_case(cenv, *geom, seed=41)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    assert rel_l2(gy, cy) <= TOL, listing
    assert rel_l2(gdx, cdx) <= TOL, (rel_l2(gdx, cdx), listing)
    assert rel_l2(gdf, cdf) <= TOL, (rel_l2(gdf, cdf), listing)
    monkeypatch.setenv("DSC_FUSE_GATHER_SUMS", "0")
    aenv, _ = _envs(hip_backend_session, fused=True)
    a, ay, adx, adf = _strided_conv_grad_case(aenv, *geom, seed=41)
    apart = next(iter(a.__dict__["_schedules"].values())).describe()
    assert int(apart.split()[0]) >= int(listing.split()[0]), (listing, apart)
    if geom[7] > 0:  # with padding there are Unpads, and the first of them is evaluated by the second
        assert apart.count("Unpad [") > listing.count("Unpad ["), (listing, apart)
    assert np.array_equal(gdx, adx) and np.array_equal(gy, ay) and np.array_equal(gdf, adf), (listing, apart)


def _first_layer_case(env, m, h, w, c_in, c_out, fh, fw, pad, pool, seed):
    """data -> conv2d + bias -> leaky_relu (-> 2x2 max-pool) -> 0.5 * sum(y^2), the data a plain parameter: only the
    filter and the bias have gradients, as for the first layer of a network."""
    from descent_amd import Initializer

    rng = np.random.default_rng(seed)
    xp = env.static_parameter_with_data([m, h, w, c_in], "x", rng.standard_normal((m, h, w, c_in), dtype=np.float32))
    fp = env.trainable_parameter([1, c_out, fh, fw, c_in], "f", Initializer.zero())
    bp = env.trainable_parameter([c_out], "b", Initializer.zero())
    env.write_parameter(fp, rng.standard_normal((1, c_out, fh, fw, c_in), dtype=np.float32) * 0.3)
    env.write_parameter(bp, rng.standard_normal(c_out, dtype=np.float32) * 0.1)
    df, db = env.static_parameter(list(fp.shape), "df"), env.static_parameter([c_out], "db")

    def build(s):
        f, b = s.parameter(fp), s.parameter(bp)
        y = (s.parameter(xp).conv2d(f, pad) + b).leaky_relu(0.01)
        if pool:
            y = y.max_pool2d((2, 2), (2, 2))
        (y.square() * 0.5).set_loss()
        s.write_parameter_value(df, f.loss_grad())
        s.write_parameter_value(db, b.loss_grad())

    g = env.build_graph(build)
    env.run(g, 0)
    return g, env.read_parameter(df), env.read_parameter(db)


@pytest.mark.parametrize("geom", [
    # m, h, w, c_in, c_out, fh, fw, pad, pool
    (600, 28, 28, 1, 16, 3, 3, 1, True),    # the ConvNet's first layer: four bands of seven rows
    (500, 20, 12, 1, 8, 3, 3, 1, True),     # not square, eight outputs
    (700, 10, 10, 3, 16, 3, 3, 1, True),    # three channels, two bands of five rows
    (900, 9, 9, 2, 12, 5, 5, 2, False),     # one band, 5x5 taps, no pooling: dC comes from the activation derivative alone
    (800, 16, 16, 4, 16, 3, 3, 0, True),    # no padding: 14 output rows, two bands
], ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("fused", [True, "split-conv-grads"])
def test_first_layer_filter_gradient(hip_backend_session, geom, fused):
    genv, cenv = _envs(hip_backend_session, fused=fused)
    g, gdf, gdb = _first_layer_case(genv, *geom, seed=77)
    _, cdf, cdb = _first_layer_case(cenv, *geom, seed=77)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    if fused is True:
        # the filter gradient (k = images x output pixels, long enough to be split) on the convolution backward kernel
        # without its data-gradient phase, dC evaluated where the kernel fills its tile
        assert "ConvFilterGrad" in listing and "no data gradient" in listing, listing
        if geom[-1]:
            assert "WindowsToImage" not in listing, listing
    else:
        assert "ConvFilterGrad" not in listing, listing
    assert rel_l2(gdf, cdf) <= TOL, (rel_l2(gdf, cdf), listing)
    assert rel_l2(gdb, cdb) <= TOL, (rel_l2(gdb, cdb), listing)


def _random_conv_geometry(rng):
    while True:
        groups = int(rng.choice([1, 1, 2, 3, 4]))
        c_in = groups * int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16]))
        c_out = groups * int(rng.choice([1, 2, 4, 6, 8, 10, 16, 20]))
        fh, fw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        pad = int(rng.integers(0, min(fh, fw) // 2 + 2))
        h, w = int(rng.integers(max(fh, 3), 24)), int(rng.integers(max(fw, 3), 24))
        if h + 2 * pad - fh + 1 >= 1 and w + 2 * pad - fw + 1 >= 1:
            return (int(rng.integers(1, 40)), h, w, c_in, c_out, fh, fw, pad, groups)


@pytest.mark.parametrize("seed", list(range(24)))
def test_conv2d_random_geometries(hip_backend_session, seed):
    """Seeded random convolutions (filters 1x1..5x5 not square, padding 0..3, 1-4 groups, channel counts with and without
    16-byte pieces, images down to the filter's size): forward, data gradient and filter gradient through whatever
    kernels the schedule picks (the dedicated forward / data-gradient kernels where they fit, the dot-product, row and
    MFMA kernels elsewhere) against the oracle."""
    geom = _random_conv_geometry(np.random.default_rng(4000 + seed))
    genv, cenv = _envs(hip_backend_session, fused=True)
    g, gy, gdx, gdf = _conv_grad_case(genv, *geom, seed=seed)
    _, cy, cdx, cdf = _conv_grad_case(cenv, *geom, seed=seed)
    listing = next(iter(g.__dict__["_schedules"].values())).describe()
    for name, got, want in (("y", gy, cy), ("dx", gdx, cdx), ("df", gdf, cdf)):
        assert rel_l2(got, want) <= TOL, (geom, name, rel_l2(got, want), listing)


@pytest.mark.parametrize("batch,fused", [(64, True), (1000, True), (64, "graph-replay")])
def test_overlapped_uploads_and_readbacks_match_the_serial_path(hip_backend_session, batch, fused):
    """Fourteen ConvNet steps (batch 64: steps shorter than an upload's latency; batch 1000: 3 MB uploads beside
    270 us steps), a new mini-batch uploaded before each: once through Environment.writer on
    the compute stream, once through the copy stream from alternating pinned arrays (uploads overlap the step before,
    the host never waits for a step), with a non-blocking read-back of the running loss after every step.  Same
    kernels, same data, no float atomics in this graph: every parameter and every loss must be bit-equal."""
    from descent_amd import Environment, workloads

    be = hip_backend_session
    steps = 14
    rng = np.random.default_rng(5)
    xs = [rng.random((batch, 28, 28, 1), dtype=np.float32) for _ in range(steps)]
    ys = [rng.integers(0, 10, (batch, 1)).astype(np.float32) for _ in range(steps)]

    env_a, env_b = Environment(be), Environment(be, fused=fused)  # with graph replay: copies join before the capture
    wa = workloads.convnet(env_a, batch=batch, seed=23)
    wb = workloads.convnet(env_b, batch=batch, seed=23)
    losses_a = []
    for i in range(steps):
        env_a.write_parameter(wa.inputs["x"], xs[i])
        env_a.write_parameter(wa.inputs["y"], ys[i])
        env_a.run(wa.graph, 900 + i)
        losses_a.append(env_a.read_parameter_scalar(wa.scalars["loss"]))

    px = [env_b.host_array(wb.inputs["x"]) for _ in range(2)]
    py = [env_b.host_array(wb.inputs["y"]) for _ in range(2)]
    loss_out = [be.host_array((1,), np.float32) for _ in range(steps)]
    upload_fence, read_fence = [0, 0], []
    for i in range(steps):
        s = i & 1
        if upload_fence[s]:
            be.fence_wait(upload_fence[s])  # the pinned pair is free again once its last upload has finished
        px[s][...] = xs[i]
        py[s][...] = ys[i]
        env_b.write_parameter_async(wb.inputs["x"], px[s])
        upload_fence[s] = env_b.write_parameter_async(wb.inputs["y"], py[s])
        env_b.run(wb.graph, 900 + i)
        read_fence.append(env_b.read_parameter_async(wb.scalars["loss"], loss_out[i]))
    for f in read_fence:
        be.fence_wait(f)
    losses_b = [float(v[0]) for v in loss_out]
    assert losses_a == losses_b
    got, want = wb.snapshot(), wa.snapshot()
    for key in want:
        assert np.array_equal(got[key], want[key]), key
    for arr in px + py + loss_out:
        be.host_release(arr)


def test_overlapped_io_argument_checks(hip_backend_session):
    from descent_amd.hip_backend import DescentHipError

    be = hip_backend_session
    buf = be.alloc_io(4096)
    pinned = be.host_array((1024,), np.float32)
    pinned[:] = np.arange(1024, dtype=np.float32)
    compute_fence = be.fence_record()
    copy_fence = be.write_async(buf, 0, pinned)
    be.fence_wait(copy_fence)
    # ids are shared between the streams, order is per stream: the older compute fence is still known and waitable
    be.fence_wait(compute_fence)
    assert be.fence_finished(copy_fence) and be.fence_finished(compute_fence)
    back = be.host_array((1024,), np.float32)
    be.fence_wait(be.read_async(buf, 0, back))
    assert np.array_equal(back, pinned)
    # pageable sources are staged (the array may be reused at once); pageable destinations are refused
    data = np.full(1024, 3.0, np.float32)
    be.write_async(buf, 0, data)
    data[:] = 0.0
    assert np.array_equal(np.frombuffer(be.read(buf, 0, 4096), np.float32), np.full(1024, 3.0, np.float32))
    with pytest.raises(DescentHipError):
        be.read_async(buf, 0, np.empty(1024, np.float32))
    with pytest.raises(DescentHipError):
        be.write_async(buf, 8, pinned)  # range outside the buffer
    be.host_release(pinned)
    be.host_release(back)
    be.free(buf)


def test_schedule_dot_export_and_launch_labels(hip_backend_session):
    """The fused schedule as graphviz text: every launch is a box, every buffer between launches an edge, and the
    parameter slots the graph writes appear as sinks; ROCTx ranges around launches switch on and off without
    changing results."""
    from descent_amd import Environment, workloads

    be = hip_backend_session
    env = Environment(be)
    w = workloads.convnet(env, batch=16, seed=2)
    env.run(w.graph, 1)
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    dot = sched.dot()
    launches, _ = sched.launch_count()
    assert dot.startswith("digraph schedule {") and dot.rstrip().endswith("}")
    assert dot.count("[shape=box,style=filled") == launches
    assert "ConvBackward" in dot and "RowFused" in dot
    assert dot.count("peripheries=2") == len(w.trainable) + len(w.state) + len(w.scalars)
    assert dot.count("{") == dot.count("}") and dot.count('"') % 2 == 0
    before = w.snapshot()
    be.markers(True)
    env.run(w.graph, 2)
    be.markers(False)
    env2 = Environment(be)
    w2 = workloads.convnet(env2, batch=16, seed=2)
    env2.run(w2.graph, 1)
    env2.run(w2.graph, 2)
    after, want = w.snapshot(), w2.snapshot()
    for key in want:
        assert np.array_equal(after[key], want[key]), key
    assert any(not np.array_equal(before[k], after[k]) for k in want)


def test_sin_cos_accuracy_over_argument_ranges(hip_backend_session):
    """The kernels carry their own sin/cos (three-piece pi/2 reduction + polynomial) below 65536 and the device
    library's above: against float64 the absolute error stays within 2.5e-7 (2 ulp at 1.0) at every magnitude a
    network produces, the switch-over point included; infinities and NaN give NaN as in the reference's GLSL."""
    from descent_amd import Environment

    env = Environment(hip_backend_session)
    rng = np.random.default_rng(11)
    parts = [rng.standard_normal(1 << 16).astype(np.float32) * s for s in (1e-3, 1.0, 30.0, 1e3, 6e4, 1e6, 1e9)]
    parts.append(np.array([0.0, -0.0, np.pi / 2, np.pi, 65536.0, -65536.0, 65536.004, 3.4e38, 1e-40], np.float32))
    k = np.arange(-2000, 2000, dtype=np.float64)
    parts.append((k * np.pi / 4).astype(np.float32))  # quadrant boundaries, where the reduced argument is +-pi/4
    x = np.concatenate(parts)
    xp = env.static_parameter_with_data([x.size], "x", x)
    sp, cp = env.static_parameter([x.size], "s"), env.static_parameter([x.size], "c")

    def build(s):
        v = s.parameter_value(xp)
        s.write_parameter_value(sp, v.sin())
        s.write_parameter_value(cp, v.cos())

    env.run(env.build_graph(build), 0)
    got_s, got_c = env.read_parameter(sp), env.read_parameter(cp)
    want_s, want_c = np.sin(x.astype(np.float64)), np.cos(x.astype(np.float64))
    assert np.abs(got_s - want_s).max() <= 2.5e-7
    assert np.abs(got_c - want_c).max() <= 2.5e-7
    bad = env.static_parameter_with_data([3], "bad", np.array([np.inf, -np.inf, np.nan], np.float32))
    out = env.static_parameter([3], "out")
    env.run(env.build_graph(lambda s: s.write_parameter_value(out, s.parameter_value(bad).sin() + s.parameter_value(bad).cos())), 0)
    assert np.all(np.isnan(env.read_parameter(out)))


def test_long_loop_keeps_device_and_host_memory_bounded(hip_backend_session):
    """4000 ConvNet steps (batch 16) with an overlapped upload before each and a read-back started after each, none
    of whose fences is ever waited for: the heap's live-buffer count and arena size, and the process's resident set,
    stay where they were after the first 500 steps (buffers recycle; marks, events and fences of finished work are
    pooled or retired, not accumulated)."""
    import psutil

    from descent_amd import Environment, workloads

    be = hip_backend_session
    env = Environment(be)
    w = workloads.convnet(env, batch=16, seed=4)
    px = [env.host_array(w.inputs["x"]) for _ in range(2)]
    out = be.host_array((1,), np.float32)
    for a in px:
        a[...] = 0.5

    def loop(n, base):
        for i in range(n):
            env.write_parameter_async(w.inputs["x"], px[i & 1])
            env.run(w.graph, base + i)
            env.read_parameter_async(w.scalars["loss"], out)
        be.sync()

    loop(500, 0)
    live0, _, arena0 = be.heap_stats()
    rss0 = psutil.Process().memory_info().rss
    loop(3500, 500)
    live1, _, arena1 = be.heap_stats()
    rss1 = psutil.Process().memory_info().rss
    assert (live1, arena1) == (live0, arena0)
    assert rss1 - rss0 < 64 << 20, f"resident set grew by {(rss1 - rss0) >> 20} MiB"
    assert np.isfinite(out[0])
    for a in px + [out]:
        be.host_release(a)


def test_a_run_that_cannot_be_put_together_changes_nothing(hip_backend_session):
    """One parameter's buffer handle is stale (freed behind the schedule's back), which the run only notices when it
    resolves the pointers of the launch that reads it, several launches and allocations into its bookkeeping.  The
    call must fail with every other handle untouched, every trainable value intact and no buffer leaked; the same
    schedule then runs normally once the parameter has a buffer again."""
    from descent_amd import Environment, workloads
    from descent_amd.hip_backend import DescentHipError

    be = hip_backend_session
    env = Environment(be)
    w = workloads.convnet(env, batch=16, seed=4)
    env.run(w.graph, 1)
    be.sync()
    sched = next(iter(w.graph.__dict__["_schedules"].values()))
    before = w.snapshot()
    y = w.inputs["y"]
    labels = env.read_parameter(y)
    handles = [p.buffer for p in sched.params]
    be.free(y.buffer)  # the handle in `handles` is now stale
    live = be.heap_stats()[0]
    with pytest.raises(DescentHipError):
        sched.run(list(handles), 2)
    assert be.heap_stats()[0] == live  # what the attempt allocated was given back
    assert [sched._slots[i] for i in range(len(handles))] == handles  # the parameter table the library was given
    y.buffer = None
    env.write_parameter(y, labels)
    after = w.snapshot()
    for key in before:
        assert np.array_equal(before[key].view(np.uint32), after[key].view(np.uint32)), key
    env.run(w.graph, 2)
    be.sync()
    assert np.all(np.isfinite(w.snapshot()["loss"]))
