"""Pins the CPU oracle (oracle/oracle.cpp): every kernel kind is checked against the reference's own
known-answer tests and against independent mathematics (numpy / torch-CPU library routines, adjoint
identities, closed forms), chosen so that a wrong sign, index or transposition fails.

Nothing here uses a GPU."""
import numpy as np
import pytest

import reference_cases
from conftest import rel_l2
from descent_amd import Environment, Initializer, kernel as K, workloads
from descent_amd.shape import BATCHES, ROWS, Shape, View
from oracle import cpu_backend
from oracle.cpu_backend import CpuBackend


def _env():
    return Environment(CpuBackend())


@pytest.mark.parametrize("case", reference_cases.ALL, ids=lambda c: c.__name__)
def test_reference_known_answers(case):
    actual, expected = case(_env())
    assert np.array_equal(actual, np.asarray(expected, np.float32))


# ---- pcg / rand ----------------------------------------------------------------------------------------------
def _pcg_py(v):
    """PCG-RXS-M-XS-32 output function, written independently with Python integers."""
    state = (v * 747796405 + 2891336453) & 0xFFFFFFFF
    word = (((state >> ((state >> 28) + 4)) ^ state) * 277803737) & 0xFFFFFFFF
    return ((word >> 22) ^ word) & 0xFFFFFFFF


def test_pcg_matches_independent_integer_implementation():
    lib = cpu_backend.lib()
    rng = np.random.default_rng(0)
    for v in [0, 1, 2, 0xFFFFFFFF, 0x5EED5EED] + [int(x) for x in rng.integers(0, 2**32, 200)]:
        assert lib.orc_pcg(v) == _pcg_py(v)
    # hand-computed: state = 2891336453, shift = (state >> 28) + 4 = 14
    state = 2891336453
    assert _pcg_py(0) == (((((state >> 14) ^ state) * 277803737) & 0xFFFFFFFF) >> 22) ^ ((((state >> 14) ^ state) * 277803737) & 0xFFFFFFFF)


def test_rand_from_index_formula_and_range():
    lib = cpu_backend.lib()
    seed, uid = 0x5EED5EED, 3
    vals = []
    for index in range(2000):
        h = _pcg_py((_pcg_py(index) + seed + uid) & 0xFFFFFFFF)
        want = np.float32(np.float32(h) / np.float32(4294967296.0))
        got = lib.orc_rand_from_index(uid, index, seed)
        assert np.float32(got) == want
        vals.append(got)
    vals = np.array(vals)
    assert vals.min() >= 0.0 and vals.max() <= 1.0 and 0.45 < vals.mean() < 0.55


def test_dropout_mask_is_shared_by_forward_and_backward():
    """select_gt(rand, 0.5, 2a, 0): same rand stream in both directions, survivors scaled by 2."""
    env = _env()
    x = env.trainable_parameter([4, 64], "x", Initializer.zero())
    y = env.static_parameter([4, 64], "y")
    from descent_amd import Dropout, EvalContext

    def build(s):
        d = Dropout(0.5).eval(s.parameter(x), EvalContext(True))
        (d * 1.0).set_loss()
        s.write_parameter_value(y, d.value())
        s.write_parameter_value(x, s.parameter(x).loss_grad())

    env.write_parameter(x, np.full(256, 3.0, np.float32))
    env.run(env.build_graph(build), 42)
    fwd, grad = env.read_parameter(y), env.read_parameter(x)
    assert set(np.unique(fwd)) <= {0.0, 6.0}
    assert np.array_equal(fwd != 0, grad != 0)
    assert np.allclose(grad[grad != 0], 2.0 / 4.0)


# ---- views -------------------------------------------------------------------------------------------------
def _gather_through(view, data):
    out = np.empty(tuple(view.output_shape), np.float32)
    flat = data.ravel()
    for coord in np.ndindex(*view.output_shape):
        a, b = view.load_index(coord), cpu_backend.load_index(view, coord)
        assert a == b
        out[coord] = flat[a]
    return out


def test_view_addressing_against_numpy():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 5, 4)).astype(np.float32)
    sh = Shape(x.shape)
    # replicate padding == numpy edge padding
    v = View.padded(sh, 1, 2, 1)
    assert np.array_equal(_gather_through(v, x), np.pad(x, ((0, 0), (2, 1), (0, 0)), mode="edge"))
    # slicing
    assert np.array_equal(_gather_through(View.limited(sh, 2, 1, 3), x), x[:, :, 1:3])
    # transpose / permute
    assert np.array_equal(_gather_through(sh.identity_view().transposed(), x), x.transpose(0, 2, 1))
    assert np.array_equal(_gather_through(sh.identity_view().permute_axes([2, 0, 1]), x), x.transpose(2, 0, 1))
    # broadcast
    b = rng.standard_normal((1, 4)).astype(np.float32)
    assert np.array_equal(_gather_through(View.broadcast(Shape(b.shape), Shape((3, 5, 4))), b), np.broadcast_to(b, (3, 5, 4)))
    # composition: pad then slice then transpose equals doing it in numpy
    comp = View.padded(sh, 1, 1, 1).through(View.limited(Shape((3, 7, 4)), 1, 0, 6), False).transposed()
    assert np.array_equal(_gather_through(comp, x), np.pad(x, ((0, 0), (1, 1), (0, 0)), mode="edge")[:, :6].transpose(0, 2, 1))


def test_image_to_windows_view_against_sliding_windows():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 7, 9, 4)).astype(np.float32)
    env = _env()
    a = env.static_parameter_with_data(x.shape, "a", x)
    out = env.static_parameter([2, 3, 4, 2, 3, 3, 2], "w")
    g = env.build_graph(lambda s: s.write_parameter_value(out, s.parameter_value(a).image_to_windows((3, 3), (2, 2), 2)))
    env.run(g, 0)
    got = env.read_parameter(out)
    win = np.lib.stride_tricks.sliding_window_view(x, (3, 3), axis=(1, 2))[:, ::2, ::2]  # [m,oh,ow,c,fh,fw]
    want = win.reshape(2, 3, 4, 2, 2, 3, 3).transpose(0, 1, 2, 3, 5, 6, 4)  # -> [m,oh,ow,g,fh,fw,c/g]
    assert np.array_equal(got, want)


def test_try_from_reshape_cases():  # src/shape.rs:658-668
    ok = [((8,), (1, 1, 8)), ((8,), (1, 8, 1)), ((8,), (8, 1, 1)), ((1, 8, 1), (1, 1, 8)), ((1, 8, 1), (8, 1, 1))]
    for a, b in ok:
        assert View.try_from_reshape(Shape(a), Shape(b)) is not None
    assert View.try_from_reshape(Shape((8,)), Shape((1, 9, 1))) is None


# ---- matmul ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("b,m,n,k", [(1, 7, 5, 3), (2, 33, 17, 40), (1, 20, 12, 2500), (3, 16, 16, 1024)])
@pytest.mark.parametrize("mode", [BATCHES, ROWS])
def test_matmul_against_float64_and_split_k_invariant(b, m, n, k, mode):
    rng = np.random.default_rng(b * 1000 + m + n + k)
    A = rng.standard_normal((b, m, k)).astype(np.float32)
    B = rng.standard_normal((b, k, n)).astype(np.float32)
    shape = Shape((b, m, k)).batched_matmul(Shape((b, k, n)), mode)
    r = shape[0]
    assert r == -(-k // 1024)
    kern = K.MatMulKernel(shape, mode, Shape(A.shape).identity_view(), Shape(B.shape).identity_view())
    C = np.full(tuple(shape), np.nan, np.float32)
    cpu_backend.run_kernel(kern, [A, B, C])
    total = C.sum(axis=0, dtype=np.float64)
    if mode == ROWS:
        total = total.transpose(1, 0, 2)  # [m,b,n] -> [b,m,n]
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert rel_l2(total, want) < 2e-6
    # chunk c holds exactly k in [c*chunk, (c+1)*chunk): chunk = ceil(ceil(k/16)/r)*16 (src/kernel.rs:436)
    chunk = -(-(-(-k // 16)) // r) * 16
    for c in range(r):
        part = A[:, :, c * chunk:(c + 1) * chunk].astype(np.float64) @ B[:, c * chunk:(c + 1) * chunk].astype(np.float64)
        got = C[c].transpose(1, 0, 2) if mode == ROWS else C[c]
        assert rel_l2(got, part) < 2e-6


def test_matmul_transposed_views_detect_swapped_operands():
    rng = np.random.default_rng(3)
    A = rng.standard_normal((1, 6, 4)).astype(np.float32)   # read as A^T: [1,4,6]
    B = rng.standard_normal((1, 6, 5)).astype(np.float32)
    kern = K.MatMulKernel(Shape((1, 1, 4, 5)), BATCHES, Shape(A.shape).identity_view().transposed(), Shape(B.shape).identity_view())
    C = np.zeros((1, 1, 4, 5), np.float32)
    cpu_backend.run_kernel(kern, [A, B, C])
    assert rel_l2(C[0, 0], A[0].T.astype(np.float64) @ B[0]) < 1e-6


# ---- reduce ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["Sum", "Max"])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_reduce_against_numpy(op, axis):
    rng = np.random.default_rng(axis)
    x = rng.standard_normal((5, 9, 6)).astype(np.float32)
    out_shape = Shape(x.shape).reduce(axis)
    out = np.zeros(tuple(out_shape), np.float32)
    cpu_backend.run_kernel(K.ReduceKernel(out_shape, Shape(x.shape).identity_view(), op, axis), [x, out])
    want = x.sum(axis=axis, keepdims=True, dtype=np.float64) if op == "Sum" else x.max(axis=axis, keepdims=True)
    assert rel_l2(out, want) < 1e-6


# ---- adjoints ----------------------------------------------------------------------------------------------
def _run_single(env_fn_in, in_shape, out_shape, x):
    env = _env()
    a = env.static_parameter_with_data(in_shape, "a", x)
    o = env.static_parameter(out_shape, "o")
    env.run(env.build_graph(lambda s: s.write_parameter_value(o, env_fn_in(s.parameter_value(a)))), 0)
    return env.read_parameter(o).astype(np.float64)


@pytest.mark.parametrize("filt,stride,groups", [((3, 3), (1, 1), 1), ((2, 2), (2, 2), 1), ((3, 3), (2, 2), 2), ((3, 2), (1, 2), 1)])
def test_windows_to_image_is_the_adjoint_of_image_to_windows(filt, stride, groups):
    rng = np.random.default_rng(4)
    fw, fh = filt
    sw, sh = stride
    oh, ow, c = 3, 4, 4
    h, w = (oh - 1) * sh + fh, (ow - 1) * sw + fw
    x = rng.standard_normal((2, h, w, c)).astype(np.float32)
    wshape = tuple(Shape(x.shape).image_to_windows(filt, stride, groups))
    y = rng.standard_normal(wshape).astype(np.float32)
    Wx = _run_single(lambda a: a.image_to_windows(filt, stride, groups), x.shape, wshape, x)
    Wty = _run_single(lambda a: a.windows_to_image(stride), wshape, x.shape, y)
    assert abs((Wx * y).sum() - (x.astype(np.float64) * Wty).sum()) < 1e-4 * np.abs(Wx * y).sum()


def test_unpad_is_the_adjoint_of_replicate_padding():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 5, 6, 3)).astype(np.float32)
    y = rng.standard_normal((2, 9, 10, 3)).astype(np.float32)
    Px = _run_single(lambda a: a.pad_image(2), x.shape, y.shape, x)
    assert np.array_equal(Px, np.pad(x, ((0, 0), (2, 2), (2, 2), (0, 0)), mode="edge"))
    Pty = _run_single(lambda a: a.unpad_image(2), y.shape, x.shape, y)
    assert abs((Px * y).sum() - (x.astype(np.float64) * Pty).sum()) < 1e-5 * np.abs(Px * y).sum()


# ---- conv / pool against torch (CPU) -------------------------------------------------------------------------
def _torch():
    return pytest.importorskip("torch")


@pytest.mark.parametrize("groups,pad,stride", [(1, 0, 1), (1, 1, 1), (2, 1, 1), (4, 1, 2)])
def test_conv2d_forward_and_backward_against_torch(groups, pad, stride):
    torch = _torch()
    rng = np.random.default_rng(6)
    m, h, w, ic, oc = 2, 9, 9, 4, 8
    x = rng.standard_normal((m, h, w, ic)).astype(np.float32)
    f = rng.standard_normal((groups, oc // groups, 3, 3, ic // groups)).astype(np.float32)
    oh = (h + 2 * pad - 3) // stride + 1
    gy = rng.standard_normal((m, oh, oh, oc)).astype(np.float32)

    env = _env()
    xp = env.trainable_parameter(x.shape, "x", Initializer.zero())
    fp = env.trainable_parameter(f.shape, "f", Initializer.zero())
    gp = env.static_parameter_with_data(gy.shape, "gy", gy)
    yp = env.static_parameter(gy.shape, "y")
    env.write_parameter(xp, x)
    env.write_parameter(fp, f)

    def build(s):
        xd, fd = s.parameter(xp), s.parameter(fp)
        y = xd.conv2d(fd, pad, (stride, stride))
        s.write_parameter_value(yp, y.value())
        # loss = sum(y * gy) / m  (set_loss scales the root gradient by 1/m)
        (y * s.parameter(gp)).reduce_sum(-1, True).reduce_sum(-2, True).reduce_sum(-3, True).set_loss()
        s.write_parameter_value(xp, xd.loss_grad())
        s.write_parameter_value(fp, fd.loss_grad())

    env.run(env.build_graph(build), 0)
    y, dx, df = env.read_parameter(yp), env.read_parameter(xp), env.read_parameter(fp)

    xt = torch.tensor(x.transpose(0, 3, 1, 2), dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(f.reshape(oc, 3, 3, ic // groups).transpose(0, 3, 1, 2).copy(), dtype=torch.float64, requires_grad=True)
    xpad = torch.nn.functional.pad(xt, (pad, pad, pad, pad), mode="replicate") if pad else xt
    yt = torch.nn.functional.conv2d(xpad, wt, stride=stride, groups=groups)
    (yt * torch.tensor(gy.transpose(0, 3, 1, 2), dtype=torch.float64)).sum().div(m).backward()
    assert rel_l2(y, yt.detach().numpy().transpose(0, 2, 3, 1)) < 1e-5
    assert rel_l2(dx, xt.grad.numpy().transpose(0, 2, 3, 1)) < 1e-5
    assert rel_l2(df, wt.grad.numpy().transpose(0, 2, 3, 1).reshape(f.shape)) < 1e-5


def test_max_pool_forward_torch_and_backward_tie_rule():
    torch = _torch()
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 8, 8, 3)).astype(np.float32)
    env = _env()
    xp = env.trainable_parameter(x.shape, "x", Initializer.zero())
    yp = env.static_parameter([2, 4, 4, 3], "y")

    def build(s):
        xd = s.parameter(xp)
        y = xd.max_pool2d((2, 2), (2, 2))
        s.write_parameter_value(yp, y.value())
        y.reduce_sum(-1, True).reduce_sum(-2, True).reduce_sum(-3, True).set_loss()
        s.write_parameter_value(xp, xd.loss_grad())

    g = env.build_graph(build)
    env.write_parameter(xp, x)
    env.run(g, 0)
    y, dx = env.read_parameter(yp), env.read_parameter(xp)
    xt = torch.tensor(x.transpose(0, 3, 1, 2), requires_grad=True)
    yt = torch.nn.functional.max_pool2d(xt, 2)
    yt.sum().div(2).backward()
    assert np.array_equal(y, yt.detach().numpy().transpose(0, 2, 3, 1))
    assert np.allclose(dx, xt.grad.numpy().transpose(0, 2, 3, 1))  # no ties in random data
    # ties: every element equal to the window maximum receives the gradient (src/array.rs:1054)
    env.write_parameter(xp, np.ones(x.shape, np.float32))
    env.run(g, 0)
    assert np.allclose(env.read_parameter(xp), 0.5)


# ---- softmax cross entropy / argmax ----------------------------------------------------------------------------
def test_softmax_cross_entropy_against_scipy_and_closed_form_gradient():
    from scipy.special import log_softmax, softmax

    from descent_amd import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss

    rng = np.random.default_rng(8)
    m, n = 32, 10
    z = (rng.standard_normal((m, n)) * 3).astype(np.float32)
    z[5, 2] = z[5, 7] = z[5].max() + 1.0  # a tie: argmax must pick the larger index
    labels = rng.integers(0, n, m)
    labels[5] = 7
    env = _env()
    zp = env.trainable_parameter([m, n], "z", Initializer.zero())
    yp = env.static_parameter_with_data([m, 1], "y", labels.astype(np.float32))
    lp = env.static_parameter([m, 1], "loss")
    ap = env.static_parameter([m, 1], "acc")

    def build(s):
        zd = s.parameter(zp)
        loss = softmax_cross_entropy_loss(zd, yp)
        s.write_parameter_value(lp, loss.set_loss())
        s.write_parameter_value(ap, softmax_cross_entropy_accuracy(zd, yp))
        s.write_parameter_value(zp, zd.loss_grad())

    env.write_parameter(zp, z)
    env.run(env.build_graph(build), 0)
    want_loss = -log_softmax(z.astype(np.float64), axis=1)[np.arange(m), labels]
    assert rel_l2(env.read_parameter(lp).ravel(), want_loss) < 1e-5
    onehot = np.eye(n)[labels]
    assert rel_l2(env.read_parameter(zp), (softmax(z.astype(np.float64), axis=1) - onehot) / m) < 1e-5
    pred = np.array([np.flatnonzero(row == row.max()).max() for row in z])
    assert np.array_equal(env.read_parameter(ap).ravel(), (pred == labels).astype(np.float32))
    assert env.read_parameter(ap)[5, 0] == 1.0


# ---- gather / scatter / concat -------------------------------------------------------------------------------
def test_gather_and_scatter_add_against_numpy():
    rng = np.random.default_rng(9)
    table = rng.standard_normal((3, 50, 2)).astype(np.float32)
    idx = rng.integers(0, 50, 200)
    vals = rng.standard_normal((3, 200, 2)).astype(np.float32)
    env = _env()
    tp = env.static_parameter_with_data(table.shape, "t", table)
    ip = env.static_parameter_with_data([200], "i", idx.astype(np.float32))
    vp = env.static_parameter_with_data(vals.shape, "v", vals)
    gp = env.static_parameter([3, 200, 2], "g")
    sp = env.static_parameter([3, 50, 2], "s")

    def build(s):
        ind = s.parameter_value(ip).into_u32()
        s.write_parameter_value(gp, s.parameter_value(tp).gather(1, ind))
        s.write_parameter_value(sp, s.literal(0.5).value().broadcast([3, 50, 2]).scatter_add(vp, 1, ind))

    env.run(env.build_graph(build), 0)
    assert np.array_equal(env.read_parameter(gp), table[:, idx])
    want = np.full((3, 50, 2), 0.5, np.float64)
    np.add.at(want, (slice(None), idx), vals.astype(np.float64))
    assert rel_l2(env.read_parameter(sp), want) < 1e-6


def test_concat_along_each_axis():
    rng = np.random.default_rng(10)
    a = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for axis, bshape in ((0, (2, 4, 5)), (1, (3, 6, 5)), (2, (3, 4, 1))):
        b = rng.standard_normal(bshape).astype(np.float32)
        env = _env()
        ap = env.static_parameter_with_data(a.shape, "a", a)
        bp = env.static_parameter_with_data(b.shape, "b", b)
        want = np.concatenate([a, b], axis=axis)
        cp = env.static_parameter(want.shape, "c")
        env.run(env.build_graph(lambda s: s.write_parameter_value(cp, s.parameter_value(ap).concat(bp, axis))), 0)
        assert np.array_equal(env.read_parameter(cp), want)


# ---- u32 arithmetic, conversions, transcendentals (src/kernel.rs:470-520 per-element op table) ----------------
def _u32_param(env, name, bits):
    return env.static_parameter_with_data([bits.size], name, bits.astype(np.uint32).view(np.float32))


def test_u32_ops_wrap_and_are_unsigned():
    """UAdd / UMul / URem / UBitXor on bit-cast words: full-range operands, so a signed remainder, a missing
    wrap-around or swapped operands of `%` give different bits than numpy's uint32 arithmetic."""
    rng = np.random.default_rng(21)
    n = 4096
    a = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(1, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    b[: n // 2] = rng.integers(1, 1 << 20, n // 2)  # small moduli beside full-range ones
    a[:8] = [0, 1, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 0xFFFFFFFE, 0x80000001, 12345]
    env = _env()
    ap, bp = _u32_param(env, "a", a), _u32_param(env, "b", b)
    outs = {k: env.static_parameter([n], k) for k in ("add", "mul", "rem", "xor", "mixed")}

    def build(s):
        x, y = s.parameter_value(ap).to_u32_bits(), s.parameter_value(bp).to_u32_bits()
        s.write_parameter_value(outs["add"], (x + y).to_f32_bits())
        s.write_parameter_value(outs["mul"], (x * y).to_f32_bits())
        s.write_parameter_value(outs["rem"], (x % y).to_f32_bits())
        s.write_parameter_value(outs["xor"], (x ^ y).to_f32_bits())
        s.write_parameter_value(outs["mixed"], (((x + 1) ^ (y * 1526263 + 1526263)) % (1 << 19)).to_f32_bits())

    env.run(env.build_graph(build), 0)
    got = {k: env.read_parameter(v).view(np.uint32) for k, v in outs.items()}
    with np.errstate(over="ignore"):
        assert np.array_equal(got["add"], a + b)
        assert np.array_equal(got["mul"], a * b)
        assert np.array_equal(got["rem"], a % b)
        assert np.array_equal(got["xor"], a ^ b)
        assert np.array_equal(got["mixed"], ((a + np.uint32(1)) ^ (b * np.uint32(1526263) + np.uint32(1526263))) % np.uint32(1 << 19))
    assert not np.array_equal(a % b, (a.view(np.int32) % b.view(np.int32)).view(np.uint32))  # signedness is visible


def test_uint_float_conversions():
    """FloatToUint truncates toward zero; UintToFloat reads the word as unsigned (values above 2^31 stay
    positive) and rounds to nearest even above 2^24 -- both against numpy's conversions."""
    rng = np.random.default_rng(22)
    n = 2048
    bits = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    bits[:6] = [0, 1, (1 << 24) + 1, (1 << 24) + 3, 0x80000000, 0xFFFFFFFF]
    vals = (rng.random(n, dtype=np.float32) * np.float32(4.0e9)).astype(np.float32)
    vals[:5] = [0.0, 0.99999994, 1.0, 16777217.0, 2147483648.0]
    env = _env()
    bp = _u32_param(env, "b", bits)
    vp = env.static_parameter_with_data([n], "v", vals)
    as_float, as_uint = env.static_parameter([n], "f"), env.static_parameter([n], "u")

    def build(s):
        s.write_parameter_value(as_float, s.parameter_value(bp).to_u32_bits().into_f32())
        s.write_parameter_value(as_uint, s.parameter_value(vp).into_u32().to_f32_bits())

    env.run(env.build_graph(build), 0)
    assert np.array_equal(env.read_parameter(as_float), bits.astype(np.float32))
    assert np.array_equal(env.read_parameter(as_uint).view(np.uint32), vals.astype(np.uint32))


@pytest.mark.parametrize("grid_size,entry_count", [(16, 1 << 19), (80, 1 << 19), (111, 1 << 14), (2048, 1 << 19)])
def test_hash_grid_corner_indices_and_fractions_against_numpy(grid_size, entry_count):
    """The four corner indices and the fractional position of a hash-grid level
    (examples/image_fit/main.rs:132-170) for a dense level (stride = points per side) and for hashed ones
    (stride = 1526263), bit for bit against numpy uint32 / float32 arithmetic written from the formula."""
    rng = np.random.default_rng(grid_size)
    m = 5000
    x = (rng.random((m, 2), dtype=np.float32) * np.float32(2.0 * (1.0 - 1e-6)) - np.float32(1.0)).astype(np.float32)
    points = grid_size + 1
    dense = entry_count >= points * points
    entries = min(entry_count, points * points)
    stride = points if dense else workloads.HASH_PRIME
    assert workloads.HASH_PRIME == 1526263
    env = _env()
    xp = env.static_parameter_with_data([m, 2], "x", x)
    idx = [env.static_parameter([m], "i%d" % i) for i in range(4)]
    frac = env.static_parameter([m, 2], "f")

    def build(s):
        cf = (s.parameter_value(xp) * 0.5 + 0.5) * float(grid_size)
        c = cf.into_u32()
        s.write_parameter_value(frac, cf - c.into_f32())
        c0, c1 = c.lock_axis(-1, 0, False), c.lock_axis(-1, 1, False)
        corners = (((c0 + 0) ^ (c1 * stride + 0)), ((c0 + 1) ^ (c1 * stride + 0)),
                   ((c0 + 0) ^ (c1 * stride + stride)), ((c0 + 1) ^ (c1 * stride + stride)))
        for out, corner in zip(idx, corners):
            s.write_parameter_value(out, (corner % entries).to_f32_bits())

    env.run(env.build_graph(build), 0)
    cf = ((x * np.float32(0.5) + np.float32(0.5)) * np.float32(grid_size)).astype(np.float32)
    c = cf.astype(np.uint32)
    assert np.array_equal(env.read_parameter(frac), cf - c.astype(np.float32))
    c0, c1, st = c[:, 0], c[:, 1], np.uint32(stride)
    with np.errstate(over="ignore"):
        want = [(c0 + np.uint32(di)) ^ (c1 * st + np.uint32(dj) * st) for dj in (0, 1) for di in (0, 1)]
    for out, w in zip(idx, want):
        got = env.read_parameter(out).view(np.uint32).ravel()
        assert np.array_equal(got, w % np.uint32(entries))
    if dense:  # a dense level's index is the row-major grid point: y * points + x, never wrapped
        got = env.read_parameter(idx[3]).view(np.uint32).ravel()
        assert np.array_equal(got, (c0 + 1) ^ ((c1 + 1) * st)) and got.max() < entries + points


def test_hash_level_sizes_fixture():
    """The sixteen level resolutions are committed as data with the f32 evaluation of the reference's formula
    beside them (examples/image_fit/main.rs:222-228: b = exp((ln 2048 - ln 16) / 15), size = trunc(16 * b^i) with
    `powi` as repeated squaring).  The last product lands within one f32 step of 2048, so the top level is 2047
    or 2048 depending on the libm in use; the first fifteen are fixed."""
    import json
    import os

    fixture = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "hash_level_sizes.json")))
    assert tuple(fixture["sizes"]) == workloads.HASH_LEVEL_SIZES
    f = np.float32
    b = f(np.exp(f((np.log(f(2048)) - np.log(f(16))) / f(15))))

    def powi(a, n):
        r = f(1)
        while True:
            if n & 1:
                r = f(r * a)
            n //= 2
            if n == 0:
                return r
            a = f(a * a)

    products = [float(f(16) * powi(b, i)) for i in range(16)]
    assert [int(v) for v in products[:15]] == fixture["sizes"][:15]
    assert int(products[15]) in (2047, 2048) and fixture["sizes"][15] == 2048
    assert np.allclose(products, fixture["f32_products"], rtol=1e-6)


def test_positional_encoding_sin_and_pow_against_numpy():
    """sin(x * 2^i * pi + {0, pi/2}) (examples/image_fit/main.rs:259-275): `pow(2, i)` must be the exact power of
    two, the feature order [coordinate][phase][frequency], and Sin within an ulp or two of float64's sine of the
    same f32 argument."""
    rng = np.random.default_rng(23)
    m, freq_count = 300, 16
    x = rng.random((m, 2), dtype=np.float32)
    env = _env()
    xp = env.static_parameter_with_data([m, 2], "x", x)
    out = env.static_parameter([m, 4 * freq_count], "pe")
    powers = env.static_parameter([freq_count], "p")

    def build(s):
        s.write_parameter_value(out, workloads.positional_encoding(s.parameter(xp), freq_count).value())
        s.write_parameter_value(powers, s.literal(2.0).pow(s.coord(freq_count)).value())

    env.run(env.build_graph(build), 0)
    assert np.array_equal(env.read_parameter(powers), 2.0 ** np.arange(freq_count, dtype=np.float32))
    pi32 = np.float32(np.pi)
    freq = (np.float32(2.0) ** np.arange(freq_count, dtype=np.float32)) * pi32
    phase = (np.arange(2, dtype=np.float32) * np.float32(0.5) * pi32).astype(np.float32)
    arg = (x[:, :, None, None] * freq[None, None, None, :]).astype(np.float32) + phase[None, None, :, None]
    want = np.sin(arg.astype(np.float32).astype(np.float64)).reshape(m, 4 * freq_count)
    got = env.read_parameter(out).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2.5e-7
    # the phase-pi/2 half is the cosine of the same product: a dropped phase or swapped axes fails here
    cos_half = got.reshape(m, 2, 2, freq_count)[:, :, 1, :3]
    assert np.max(np.abs(cos_half - np.cos((x[:, :, None] * freq[None, None, :3]).astype(np.float64)))) <= 1e-5


def test_sin_cos_pow_ops_against_numpy():
    rng = np.random.default_rng(24)
    n = 4096
    x = (rng.standard_normal(n) * 40).astype(np.float32)
    base = (rng.random(n, dtype=np.float32) * 3 + np.float32(0.1)).astype(np.float32)
    expo = (rng.standard_normal(n) * 2).astype(np.float32)
    env = _env()
    xp, bp, ep = (env.static_parameter_with_data([n], k, v) for k, v in (("x", x), ("b", base), ("e", expo)))
    sp, cp, pp = (env.static_parameter([n], k) for k in ("s", "c", "p"))

    def build(s):
        s.write_parameter_value(sp, s.parameter_value(xp).sin())
        s.write_parameter_value(cp, s.parameter_value(xp).cos())
        s.write_parameter_value(pp, s.parameter_value(bp).pow(s.parameter_value(ep)))

    env.run(env.build_graph(build), 0)
    x64 = x.astype(np.float64)
    assert np.max(np.abs(env.read_parameter(sp) - np.sin(x64))) <= 1.5e-7
    assert np.max(np.abs(env.read_parameter(cp) - np.cos(x64))) <= 1.5e-7
    assert rel_l2(env.read_parameter(pp), base.astype(np.float64) ** expo.astype(np.float64)) <= 2e-7
    assert env.read_parameter(pp)[0] != np.float32(expo[0].astype(np.float64) ** base[0].astype(np.float64))  # base ^ exponent, not swapped


# ---- optimisers ------------------------------------------------------------------------------------------------
def _quadratic_problem(env, opt_factory, steps):
    """loss = sum((theta * x)^2) / m with fixed x; returns theta after `steps` updates."""
    rng = np.random.default_rng(11)
    theta0 = rng.standard_normal((4, 6)).astype(np.float32)
    x = rng.standard_normal((4, 6)).astype(np.float32)
    tp = env.trainable_parameter([4, 6], "theta", Initializer.zero())
    xp = env.static_parameter_with_data([4, 6], "x", x)
    scope = env.scope()
    t = scope.parameter(tp)
    (t * scope.parameter(xp)).square().reduce_sum(-1, True).set_loss()
    opt_factory(env, scope, [tp])
    g = scope.build_graph()
    env.write_parameter(tp, theta0)
    for i in range(steps):
        env.run(g, i)
    return theta0.astype(np.float64), x.astype(np.float64), env.read_parameter(tp)


def test_sgd_momentum_closed_form():
    from descent_amd import StochasticGradientDescent

    th, x, got = _quadratic_problem(_env(), lambda e, s, p: StochasticGradientDescent(e, s, p, 0.1, 0.9), 5)
    v = np.zeros_like(th)
    for _ in range(5):
        grad = 2 * th * x * x / 4
        v = 0.9 * v + grad
        th = th - 0.1 * v
    assert rel_l2(got, th) < 1e-5


def test_adam_closed_form_epsilon_outside_bias_correction():
    from descent_amd import Adam

    th, x, got = _quadratic_problem(_env(), lambda e, s, p: Adam(e, s, p, 1e-2, 0.9, 0.999, 1e-8), 6)
    mom, var = np.zeros_like(th), np.zeros_like(th)
    for t in range(1, 7):
        grad = 2 * th * x * x / 4
        alpha = 1e-2 * np.sqrt(1 - 0.999**t) / (1 - 0.9**t)
        mom = 0.9 * mom + 0.1 * grad
        var = 0.999 * var + 0.001 * grad * grad
        th = th - alpha * mom / (np.sqrt(var) + 1e-8)
    assert rel_l2(got, th) < 1e-4


# ---- whole configs stay finite and learn --------------------------------------------------------------------------
def test_convnet_loss_decreases_on_oracle():
    env = _env()
    w = workloads.convnet(env, batch=16, seed=1)
    losses = []
    for step in range(6):
        env.writer(w.scalars["loss"]).zero_fill()
        env.run(w.graph, step)
        losses.append(env.read_parameter_scalar(w.scalars["loss"]))
    assert all(np.isfinite(losses)) and losses[-1] < losses[0]
