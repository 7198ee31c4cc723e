"""The reference's own known-answer tests (src/lib.rs:19-232 and examples/array_api/main.rs:24), restated
against `descent_amd.Environment` so the same case runs on the CPU oracle and on the GPU backend.

Each case is a function(env) -> (actual, expected) with exact float32 expectations (all values are small
integers, as in the reference, which asserts with assert_eq!)."""
import numpy as np

TEST_RAND_SEED = 0x5EED5EED  # src/lib.rs:24


def parameters(env):  # src/lib.rs:27-34
    data = np.arange(10, dtype=np.float32)
    a = env.static_parameter_with_data([10], "a", data)
    return env.read_parameter_to_vec(a), data


def reduce(env):  # src/lib.rs:37-55
    a_data = np.arange(100, dtype=np.float32)
    a = env.static_parameter_with_data([10, 10], "a", a_data)
    b = env.static_parameter([10, 1], "b")
    g = env.build_graph(lambda s: s.write_parameter_value(b, s.parameter_value(a).reduce_sum(-1, True)))
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(b), a_data.reshape(10, 10).sum(axis=1)


def pad_image(env):  # src/lib.rs:58-73
    a = env.static_parameter_with_data([1, 8, 8, 1], "a", np.ones(64, np.float32))
    b = env.static_parameter([1, 10, 10, 1], "b")
    g = env.build_graph(lambda s: s.write_parameter_value(b, s.parameter_value(a).pad_image(1)))
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(b), np.ones(100, np.float32)


def unpad_image(env):  # src/lib.rs:76-98
    a = env.static_parameter_with_data([1, 10, 10, 1], "a", np.ones(100, np.float32))
    b = env.static_parameter([1, 8, 8, 1], "b")
    g = env.build_graph(lambda s: s.write_parameter_value(b, s.parameter_value(a).unpad_image(1)))
    env.run(g, TEST_RAND_SEED)
    edge = np.array([2.0 if i in (0, 7) else 1.0 for i in range(8)], np.float32)
    return env.read_parameter_to_vec(b), np.outer(edge, edge).ravel()


def conv2d(env):  # src/lib.rs:101-124
    a = env.static_parameter_with_data([1, 10, 10, 1], "a", np.ones(100, np.float32))
    b = env.static_parameter_with_data([1, 1, 3, 3, 1], "b", np.ones(9, np.float32))
    c = env.static_parameter([1, 8, 8, 1], "c")
    g = env.build_graph(lambda s: s.write_parameter_value(c, s.parameter(a).conv2d(b, 0, (1, 1)).value()))
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(c), np.full(64, 9.0, np.float32)


def max_pool2d(env):  # src/lib.rs:127-147
    a = env.static_parameter_with_data([1, 10, 10, 1], "a", np.arange(100, dtype=np.float32))
    b = env.static_parameter([1, 5, 5, 1], "b")
    g = env.build_graph(lambda s: s.write_parameter_value(b, s.parameter(a).max_pool2d((2, 2), (2, 2)).value()))
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(b), np.array([11 + 2 * (i % 5) + 20 * (i // 5) for i in range(25)], np.float32)


def gather(env):  # src/lib.rs:150-173
    a = env.static_parameter_with_data([1, 200, 1], "a", np.array([i * i for i in range(200)], np.float32))
    b = env.static_parameter_with_data([100], "b", np.array([99 - i for i in range(100)], np.float32))
    c = env.static_parameter([1, 100, 1], "c")
    g = env.build_graph(
        lambda s: s.write_parameter_value(c, s.parameter_value(a).gather(1, s.parameter_value(b).into_u32()) + 1.0)
    )
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(c), np.array([(99 - i) * (99 - i) + 1 for i in range(100)], np.float32)


def scatter_add(env):  # src/lib.rs:176-202
    a = env.static_parameter_with_data([1, 100, 1], "a", np.ones(100, np.float32))
    b = env.static_parameter_with_data([100], "b", np.array([i % 10 for i in range(100)], np.float32))
    c = env.static_parameter([1, 10, 1], "c")
    g = env.build_graph(
        lambda s: s.write_parameter_value(
            c, s.literal(0.0).value().broadcast([1, 10, 1]).scatter_add(a, -2, s.parameter_value(b).into_u32())
        )
    )
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(c), np.full(10, 10.0, np.float32)


def concat(env):  # src/lib.rs:205-231
    a_data = np.array([i for i in range(200) if ((i // 10) & 1) == 0], np.float32)
    b_data = np.array([i for i in range(200) if ((i // 10) & 1) == 1], np.float32)
    a = env.static_parameter_with_data([10, 10], "a", a_data)
    b = env.static_parameter_with_data([10, 10], "b", b_data)
    c = env.static_parameter([10, 20], "c")
    g = env.build_graph(lambda s: s.write_parameter_value(c, s.parameter_value(a).concat(b, -1)))
    env.run(g, TEST_RAND_SEED)
    return env.read_parameter_to_vec(c), np.arange(200, dtype=np.float32)


def array_api(env):  # examples/array_api/main.rs:9-24
    m = env.static_parameter_with_data([3, 3], "m", [1, 0, 0, 0, 1, 0, 0, 0, 1])
    x = env.static_parameter_with_data([3, 1], "x", [4, 5, 6])
    y = env.static_parameter_with_data([3, 1], "y", [1, 2, 3])
    z = env.static_parameter([3, 1], "z")

    def build(s):
        mv, xv, yv = s.parameter_value(m), s.parameter_value(x), s.parameter_value(y)
        s.write_parameter_value(z, 2.0 * mv.matmul(xv) + yv * yv + 1.0)

    env.run(env.build_graph(build), TEST_RAND_SEED)
    return env.read_parameter_to_vec(z), np.array([10.0, 15.0, 22.0], np.float32)


ALL = [parameters, reduce, pad_image, unpad_image, conv2d, max_pool2d, gather, scatter_add, concat, array_api]
