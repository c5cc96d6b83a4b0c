"""Kernel-level parity on the GPU, through the C ABI (ctypes) on torch device memory.

Each kernel family is compared with the NumPy/SciPy library routine it replaces, on seeded
inputs, over every layout path of the planner (flat / rows / nd; row / column / middle / full
and two-stage reductions; GEMM operand layouts and ragged sizes).  Tolerances: elementwise
float ops 4 ulp-ish (rtol 1e-6 f32 / 1e-14 f64 of the element, they are single roundings plus
device libm); reductions and GEMM rtol 1e-5 (f32) / 1e-12 (f64) of |ref| + max|ref|; integer /
index / copy / scatter work bit-exact.
"""

import numpy as onp
import pytest
import scipy.special

pytestmark = pytest.mark.gpu

F32, F64 = onp.float32, onp.float64


@pytest.fixture(scope="module")
def dnp():
    import autograd_amd.numpy as dnp

    return dnp


def P(dnp, a):
    return dnp.asarray(a)


def close(got, want, rtol):
    got = onp.asarray(got)
    want = onp.asarray(want)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert got.dtype == want.dtype, (got.dtype, want.dtype)
    g, w = got.astype(F64), want.astype(F64)
    scale = onp.max(onp.abs(w)) if w.size else 0.0
    tol = rtol * onp.abs(w) + rtol * scale
    bad = ~((onp.abs(g - w) <= tol) | (onp.isnan(g) & onp.isnan(w)) | (g == w))
    assert not bad.any(), f"max err {onp.max(onp.abs(g - w)[bad])} at {onp.argwhere(bad)[:3].tolist()}"


RT = {F32: 1e-5, F64: 1e-12}
RT_EW = {F32: 2e-6, F64: 2e-15}


# ---- elementwise --------------------------------------------------------------------------------
UNARY = [
    ("negative", onp.negative, False), ("exp", onp.exp, False), ("log", onp.log, True), ("tanh", onp.tanh, False),
    ("sinh", onp.sinh, False), ("cosh", onp.cosh, False), ("sin", onp.sin, False), ("cos", onp.cos, False),
    ("sqrt", onp.sqrt, True), ("square", onp.square, False), ("abs", onp.abs, False), ("sign", onp.sign, False),
    ("reciprocal", onp.reciprocal, True), ("log1p", onp.log1p, True), ("expm1", onp.expm1, False),
    ("exp2", onp.exp2, False), ("log2", onp.log2, True), ("log10", onp.log10, True), ("tan", onp.tan, False),
    ("arctan", onp.arctan, False), ("arcsinh", onp.arcsinh, False), ("fabs", onp.fabs, False),
    ("rad2deg", onp.rad2deg, False), ("deg2rad", onp.deg2rad, False), ("degrees", onp.degrees, False),
]


@pytest.mark.parametrize("dtype", [F32, F64])
def test_unary_bounded_domains(dnp, dtype):
    rs = onp.random.RandomState(4)
    inside = (rs.rand(1031) * 1.9 - 0.95).astype(dtype)     # (-1, 1)
    above = (rs.rand(1031) * 5 + 1.01).astype(dtype)        # (1, 6)
    for name, x in (("arcsin", inside), ("arccos", inside), ("arctanh", inside), ("arccosh", above)):
        close(getattr(dnp, name)(P(dnp, x)).numpy(), getattr(onp, name)(x), RT_EW[dtype] * 8)
    edge = onp.array([0.0, -0.0, 1.0, -1.0, 2.0, onp.nan, onp.inf, -onp.inf], dtype)
    with onp.errstate(all="ignore"):
        for name in ("arcsin", "arccos", "arctanh", "arccosh", "log2", "exp2", "arctan", "tan"):
            close(getattr(dnp, name)(P(dnp, edge)).numpy(), getattr(onp, name)(edge), RT_EW[dtype] * 8)


@pytest.mark.parametrize("dtype", [F32, F64])
def test_fmax_fmin_clip_and_two_argument_functions(dnp, dtype):
    rs = onp.random.RandomState(5)
    a, b = rs.randn(37, 29).astype(dtype), rs.randn(29).astype(dtype)
    a[0, :3] = onp.nan
    b[2] = onp.nan
    A, B = P(dnp, a), P(dnp, b)
    for name in ("fmax", "fmin", "maximum", "minimum"):          # NaN handling differs between the pairs
        assert onp.array_equal(getattr(dnp, name)(A, B).numpy(), getattr(onp, name)(a, b), equal_nan=True), name
    assert onp.array_equal(dnp.clip(A, -0.5, 0.25).numpy(), onp.clip(a, -0.5, 0.25), equal_nan=True)
    lo = (rs.randn(29) - 1).astype(dtype)
    assert onp.array_equal(dnp.clip(A, P(dnp, lo), 0.25).numpy(), onp.clip(a, lo, 0.25), equal_nan=True)
    x, y = rs.randn(37, 29).astype(dtype), rs.randn(37, 1).astype(dtype)
    for name in ("arctan2", "hypot", "logaddexp"):
        close(getattr(dnp, name)(P(dnp, x), P(dnp, y)).numpy(), getattr(onp, name)(x, y), RT_EW[dtype] * 8)
    big = onp.array([1000.0, -1000.0, 5.0, onp.inf, -onp.inf, onp.nan], dtype)
    oth = onp.array([1000.0, 3.0, 5.0, 1.0, -onp.inf, 1.0], dtype)
    with onp.errstate(all="ignore"):
        close(dnp.logaddexp(P(dnp, big), P(dnp, oth)).numpy(), onp.logaddexp(big, oth), RT_EW[dtype] * 8)


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("name,ref,positive", UNARY)
def test_unary(dnp, dtype, name, ref, positive):
    rs = onp.random.RandomState(0)
    for shape in [(), (1,), (7,), (1031,), (33, 65)]:
        x = onp.asarray(rs.rand(*shape) * 3 + 0.1 if positive else rs.randn(*shape) * 2).astype(dtype)
        close(getattr(dnp, name)(P(dnp, x)).numpy(), ref(x), RT_EW[dtype] * 8)


BINARY = [("add", onp.add), ("subtract", onp.subtract), ("multiply", onp.multiply), ("true_divide", onp.true_divide),
          ("maximum", onp.maximum), ("minimum", onp.minimum), ("power", onp.power)]


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("name,ref", BINARY)
def test_binary_layouts(dnp, dtype, name, ref):
    rs = onp.random.RandomState(1)
    op = getattr(dnp, name)

    def mk(*shape):
        a = rs.rand(*shape) + 0.5 if name in ("power", "true_divide") else rs.randn(*shape)
        return onp.asarray(a).astype(dtype)

    cases = [
        (mk(1000), mk(1000)),             # flat
        (mk(37, 29), mk(29)),             # rows: broadcast along rows
        (mk(37, 29), mk(37, 1)),          # rows: per-row scalar
        (mk(37, 1), mk(1, 29)),           # both broadcast
        (mk(5, 6, 7), mk(6, 1)),          # nd
        (mk(8, 9), mk(9, 8).T),           # transposed operand: nd path
        (mk(3, 1, 5), mk(4, 1)),
        (mk(6), mk()),                    # 0-d operand
    ]
    for a, b in cases:
        close(op(P(dnp, a), P(dnp, b)).numpy(), ref(a, b), RT_EW[dtype] * 8)
    a = mk(50, 20)
    for s in (2.0, 0.5, 3, -1.25):
        close(op(P(dnp, a), s).numpy(), ref(a, dtype(s) if False else s).astype(dtype), RT_EW[dtype] * 8)
        close(op(s, P(dnp, a)).numpy(), ref(s, a).astype(dtype), RT_EW[dtype] * 8)


def test_power_shortcuts_are_exact(dnp):
    x = onp.random.RandomState(2).randn(4099)
    for e in (2, 1, 0, -1, 0.5, 2.0):
        xx = onp.abs(x) + 0.1 if e == 0.5 else x
        assert onp.array_equal(dnp.power(P(dnp, xx), e).numpy(), xx**e), e


def test_views_and_slices(dnp):
    rs = onp.random.RandomState(3)
    x = rs.randn(2**12 + 3)
    X = P(dnp, x)
    assert onp.array_equal((X[1:] - X[:-1] ** 2).numpy(), x[1:] - x[:-1] ** 2)  # misaligned 16-byte vectors
    assert onp.array_equal((X[3:-5:2] * 2.0).numpy(), x[3:-5:2] * 2.0)
    A = rs.randn(6, 8, 10).astype(F32)
    DA = P(dnp, A)
    assert onp.array_equal(dnp.transpose(DA, (2, 0, 1)).numpy(), A.transpose(2, 0, 1))
    assert onp.array_equal((dnp.swapaxes(DA, 0, 2) + 1.0).numpy(), A.swapaxes(0, 2) + F32(1.0))
    assert onp.array_equal(dnp.reshape(dnp.swapaxes(DA, 0, 1), (8, 60)).numpy(), A.swapaxes(0, 1).reshape(8, 60))
    assert onp.array_equal(DA[2, :, None, 3].numpy(), A[2, :, None, 3])
    assert onp.array_equal(dnp.repeat(DA[:, :1], 4, axis=1).numpy(), onp.repeat(A[:, :1], 4, axis=1))
    assert onp.array_equal(dnp.repeat(DA, 3, axis=2).numpy(), onp.repeat(A, 3, axis=2))
    assert onp.array_equal(dnp.concatenate((DA, DA[:, :2]), axis=1).numpy(), onp.concatenate((A, A[:, :2]), axis=1))
    assert onp.array_equal(dnp.hstack((DA[0], DA[1, :, :3])).numpy(), onp.hstack((A[0], A[1, :, :3])))
    assert onp.array_equal(dnp.astype(DA, F64).numpy(), A.astype(F64))
    assert onp.array_equal((DA > 0.3).numpy(), A > 0.3)
    assert onp.array_equal(dnp.where(DA > 0, DA, 0.0).numpy(), onp.where(A > 0, A, F32(0)))
    assert onp.array_equal(dnp.ones((3, 5), dtype=F32).numpy(), onp.ones((3, 5), F32))
    assert onp.array_equal(dnp.full((1027,), 2.5).numpy(), onp.full((1027,), 2.5))
    assert [r.shape for r in DA] == [(8, 10)] * 6


FUSED = [
    ("DIV_VJP1", 3, lambda g, x, y: -g * x / y**2),
    ("TANH_VJP", 2, lambda g, x: g / onp.cosh(x) ** 2),
    ("POW_VJP1", 3, lambda g, x, a: g * onp.log(onp.where(x, x, 1.0)) * a),
    ("LSE_VJP", 4, lambda g, b, x, a: g * b * onp.exp(x - a)),
    ("RECIPROCAL_VJP", 2, lambda g, x: -g / x**2),
    ("SQRT_VJP", 2, lambda g, x: g * 0.5 * x**-0.5),
    ("SIN_VJP", 2, lambda g, x: g * onp.cos(x)),
    ("COS_VJP", 2, lambda g, x: -g * onp.sin(x)),
    ("SINH_VJP", 2, lambda g, x: g * onp.cosh(x)),
    ("COSH_VJP", 2, lambda g, x: g * onp.sinh(x)),
    ("SQUARE_VJP", 2, lambda g, x: g * 2 * x),
    ("LOG1P_VJP", 2, lambda g, x: g / (x + 1)),
    ("EXPM1_VJP", 2, lambda g, a: (a + 1) * g),
    ("MUL_ADD", 3, lambda a, x, y: a * x + y),
]


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("opname,nin,ref", FUSED)
def test_fused_rule_kernels(dnp, dtype, opname, nin, ref):
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(4)
    xs = [(rs.rand(513, 40) + 0.5).astype(dtype) for _ in range(nin)]
    got = D.map_op(getattr(Op, opname), onp.dtype(dtype), *[P(dnp, x) for x in xs]).numpy()
    close(got, ref(*xs).astype(dtype), RT_EW[dtype] * 16)


def test_pow_vjp0_and_choose(dnp):
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(5)
    g, x = rs.randn(999), rs.rand(999) + 0.5
    for y in (2.0, 3.0, 0.0, 1.0, -1.5):
        want = g * y * x ** onp.where(y, y - 1, 1.0)
        close(D.map_op(Op.POW_VJP0, onp.dtype(F64), P(dnp, g), P(dnp, x), y).numpy(), want, 1e-14)
    a, b = rs.randint(0, 3, 999).astype(F64), rs.randint(0, 3, 999).astype(F64)
    ans = onp.maximum(a, b)
    want = g * ((a == ans) / (1.0 + (a == b)))
    assert onp.array_equal(D.map_op(Op.CHOOSE_VJP, onp.dtype(F64), P(dnp, g), P(dnp, a), P(dnp, ans), P(dnp, b)).numpy(), want)
    gy, gx = D.map_op(Op.DIV_VJP_BOTH, onp.dtype(F64), P(dnp, g), P(dnp, a), P(dnp, x), n_out=2)
    assert onp.array_equal(gy.numpy(), g / x) and onp.array_equal(gx.numpy(), -g * a / x**2)


# ---- reductions ---------------------------------------------------------------------------------
RED_SHAPES = [
    ((7,), None), ((5000,), None), ((300000,), None),             # full: group, block, two-stage
    ((33, 10), 1), ((33, 10), 0), ((1024, 10), 1), ((1024, 10), 0),
    ((64, 300), 1), ((64, 300), 0), ((20, 5000), 1), ((20, 5000), 0),
    ((3000, 260), 0), ((3000, 256), 0), ((2, 70000), 1),          # two-stage column / row
    ((6, 50, 8), 1), ((6, 50, 8), (0, 2)), ((6, 50, 8), (1, 2)), ((6, 50, 8), (0, 1)), ((6, 50, 8), None),
    ((4, 1, 9), 1), ((0, 5), 0), ((5, 0), 0),
    # few reduced elements per output (one thread walks them): pooling windows, short middle axes, vector tails
    ((64, 2, 24), 1), ((18, 3, 6, 2, 12, 2), 3), ((18, 3, 6, 2, 12, 2), 5), ((500, 16, 7), 1), ((500, 17, 8), 1),
    ((2, 300000), 0), ((5, 3), 0), ((16, 4099), 0),
]


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("shape,axis", RED_SHAPES)
def test_sum_max_min(dnp, dtype, shape, axis):
    rs = onp.random.RandomState(6)
    x = rs.randn(*shape).astype(dtype)
    X = P(dnp, x)
    for keepdims in (False, True):
        close(dnp.sum(X, axis=axis, keepdims=keepdims).numpy(), onp.sum(x, axis=axis, keepdims=keepdims), RT[dtype])
        if x.size and all(s for s in shape):
            assert onp.array_equal(dnp.max(X, axis=axis, keepdims=keepdims).numpy(), onp.max(x, axis=axis, keepdims=keepdims))
            assert onp.array_equal(dnp.min(X, axis=axis, keepdims=keepdims).numpy(), onp.min(x, axis=axis, keepdims=keepdims))
            close(dnp.mean(X, axis=axis, keepdims=keepdims).numpy(), onp.mean(x, axis=axis, keepdims=keepdims), RT[dtype])


def test_sum_of_small_integers_is_exact_in_any_order(dnp):
    # integer-valued floats: every partial sum is exact, so any summation tree must agree bit for bit
    rs = onp.random.RandomState(7)
    x = rs.randint(-8, 9, (777, 513)).astype(F32)
    X = P(dnp, x)
    for axis in (None, 0, 1):
        assert onp.array_equal(dnp.sum(X, axis=axis).numpy(), onp.sum(x, axis=axis, dtype=F64).astype(F32))
    assert onp.array_equal(dnp.sum(dnp.transpose(X), axis=0).numpy(), onp.sum(x.T, axis=0, dtype=F64).astype(F32))


def test_reductions_are_deterministic(dnp):
    x = P(dnp, onp.random.RandomState(8).randn(4096, 600).astype(F32))
    for axis in (None, 0, 1):
        a = dnp.sum(x, axis=axis).numpy()
        for _ in range(3):
            assert onp.array_equal(a, dnp.sum(x, axis=axis).numpy())


@pytest.mark.parametrize("dtype", [F32, F64])
def test_fused_map_reduce_is_unbroadcast(dnp, dtype):
    from autograd_amd._lib import Op, Red
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(9)
    x, g = rs.randn(300, 170).astype(dtype), rs.randn(300, 170).astype(dtype)
    dt = onp.dtype(dtype)
    close(D.map_reduce(Op.MUL, Red.SUM, dt, (P(dnp, x), P(dnp, g)), (0,), True).numpy(),
          onp.sum(x * g, axis=0, keepdims=True), RT[dtype])
    close(D.map_reduce(Op.MUL, Red.SUM, dt, (P(dnp, x), P(dnp, g)), (1,), True).numpy(),
          onp.sum(x * g, axis=1, keepdims=True), RT[dtype])
    b = rs.rand(170).astype(dtype) + 0.5
    close(D.map_reduce(Op.DIV_VJP1, Red.SUM, dt, (P(dnp, g), P(dnp, x), P(dnp, b)), (0,), True, shape=(300, 170)).numpy(),
          onp.sum(-g * x / b**2, axis=0, keepdims=True), RT[dtype])
    close(D.map_reduce(Op.NEG, Red.SUM, dt, (P(dnp, g),), (0, 1), False).numpy(), onp.sum(-g), RT[dtype])


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("shape,axis", [((1024, 10), 1), ((256, 128), 1), ((37, 4096), 1), ((37, 4096), 0),
                                        ((5, 4), None), ((6, 50, 8), 1), ((3, 70000), 1), ((4, 5), (0, 1)), ((9, 700), 0), ((6, 12, 8), 1)])
def test_logsumexp_forward(dnp, dtype, shape, axis):
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(10)
    x = (rs.randn(*shape) * 5).astype(dtype)
    for keepdims in (False, True):
        want = scipy.special.logsumexp(x, axis=axis, keepdims=keepdims)
        close(logsumexp(P(dnp, x), axis=axis, keepdims=keepdims).numpy(), onp.asarray(want, dtype=dtype), RT[dtype])


def test_logsumexp_special_values(dnp):
    from autograd_amd.scipy.special import logsumexp

    x = onp.array([[-onp.inf, -onp.inf, -onp.inf], [0.0, -onp.inf, 0.0], [1000.0, 1000.0, 999.0],
                   [onp.inf, 1.0, 2.0], [-1000.0, -1001.0, -1002.0], [onp.nan, 1.0, 2.0]])
    with onp.errstate(all="ignore"):
        want = scipy.special.logsumexp(x, axis=1)
    got = logsumexp(P(dnp, x), axis=1).numpy()
    assert onp.allclose(got, want, rtol=1e-13, equal_nan=True), (got, want)


def test_weighted_logsumexp_follows_scipy(dnp):
    """The ``b=`` form (reference tests/test_scipy.py:237-255: positive weights of shapes (4,), (3, 4), (2, 3, 4)
    over axis None/0/1, keepdims both ways) and weights of either sign, which scipy sums before the logarithm."""
    from autograd_amd.scipy.special import logsumexp
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(21)
    for shape in ((4,), (3, 4), (2, 3, 4)):
        x, w = rs.randn(*shape), onp.exp(rs.randn(*shape))
        signed = w.copy()
        signed.flat[1::5] *= -0.02  # a few negative weights, every total still positive
        for axis in (None, 0, 1)[: 2 + (len(shape) > 1)]:
            for keepdims in (True, False):
                for b in (w, signed, 2.5):
                    want = scipy.special.logsumexp(x, axis=axis, b=b, keepdims=keepdims)
                    assert onp.all(onp.isfinite(want))
                    B = b if isinstance(b, float) else dnp.asarray(b)
                    got = logsumexp(dnp.asarray(x), axis=axis, b=B, keepdims=keepdims)
                    assert got.shape == onp.shape(want)
                    close(got.numpy(), want, 1e-13)
                    check_grads(lambda a: logsumexp(a, axis=axis, b=B, keepdims=keepdims), modes=["fwd", "rev"])(dnp.asarray(x))  # noqa: B023
    # weights broadcast against x, a total below zero (NaN, as in scipy), float32
    x, w = rs.randn(3, 4), onp.exp(rs.randn(4))
    close(logsumexp(dnp.asarray(x), axis=1, b=dnp.asarray(w)).numpy(), scipy.special.logsumexp(x, axis=1, b=w), 1e-13)
    with onp.errstate(all="ignore"):
        want = scipy.special.logsumexp(x, axis=1, b=onp.array([1.0, -50.0, 1.0, 1.0]))
    got = logsumexp(dnp.asarray(x), axis=1, b=dnp.asarray(onp.array([1.0, -50.0, 1.0, 1.0]))).numpy()
    assert onp.isnan(want).any() and onp.array_equal(onp.isnan(got), onp.isnan(want))
    x32, w32 = x.astype(onp.float32), onp.exp(rs.randn(3, 4)).astype(onp.float32)
    got = logsumexp(dnp.asarray(x32), axis=0, b=dnp.asarray(w32))
    assert got.dtype == onp.float32
    close(got.numpy(), scipy.special.logsumexp(x32, axis=0, b=w32), 1e-5)
    # an infinite element with weights (no shift is applied then: exp(+inf) must come out inf, not NaN), both precisions
    for dt in (onp.float32, onp.float64):
        xi = onp.array([[0.5, onp.inf, -1.0], [0.25, -onp.inf, 2.0]], dt)
        wi = onp.array([1.5, 0.5, 2.0], dt)
        with onp.errstate(all="ignore"):
            want = scipy.special.logsumexp(xi, axis=1, b=wi)
        got = logsumexp(dnp.asarray(xi), axis=1, b=dnp.asarray(wi)).numpy()
        assert want[0] == onp.inf and got[0] == onp.inf and got.dtype == dt
        close(got[1:], want[1:], 1e-6 if dt == onp.float32 else 1e-13)


# ---- contractions -------------------------------------------------------------------------------
GEMM_SHAPES = [(1, 1, 1), (5, 7, 3), (64, 64, 16), (65, 63, 17), (130, 70, 33), (256, 128, 641), (1024, 10, 1024),
               (10, 1024, 300), (300, 300, 1), (129, 257, 100), (512, 512, 512),
               # few output tiles and a long K (the K split inside one block): whole and partial chunks, ragged tiles
               (256, 512, 641), (641, 512, 256), (33, 31, 257), (96, 40, 288), (64, 64, 5000), (200, 130, 4100),
               # the shortest K that is cut (four waves), around it, and K just short of a whole chunk
               (256, 512, 128), (100, 70, 130), (33, 257, 200), (64, 64, 127), (70, 30, 159)]


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_dot_all_operand_layouts(dnp, dtype, M, N, K):
    rs = onp.random.RandomState(11)
    a, b = rs.randn(M, K).astype(dtype), rs.randn(K, N).astype(dtype)
    want = (a.astype(F64) @ b.astype(F64)).astype(dtype)
    rt = RT[dtype] * max(1.0, onp.sqrt(K) / 8)
    A, B = P(dnp, a), P(dnp, b)
    close(dnp.dot(A, B).numpy(), want, rt)                                                  # NN
    At, Bt = P(dnp, onp.ascontiguousarray(a.T)), P(dnp, onp.ascontiguousarray(b.T))
    close(dnp.dot(dnp.transpose(At), B).numpy(), want, rt)                                  # TN  (A^T . G)
    close(dnp.dot(A, dnp.transpose(Bt)).numpy(), want, rt)                                  # NT  (G . B^T)
    close(dnp.dot(dnp.transpose(At), dnp.transpose(Bt)).numpy(), want, rt)                  # TT
    if M > 4 and K > 4:
        close(dnp.dot(A[1:-1, 2:], B[2:]).numpy(), (a[1:-1, 2:].astype(F64) @ b[2:].astype(F64)).astype(dtype), rt)
    if M >= 8 and N >= 8 and K >= 8:
        close(dnp.dot(A[::2, ::2], B[::2, ::2]).numpy(),
              (a[::2, ::2].astype(F64) @ b[::2, ::2].astype(F64)).astype(dtype), rt)        # generic strides


@pytest.mark.parametrize("K", [1, 2, 3, 5, 30, 33, 127, 641])
def test_dot_rows_that_end_inside_a_vector_do_not_see_their_neighbours(dnp, K):
    """An operand contiguous along k whose K is not a multiple of 4: the 16 bytes fetched at the end of a row run
    into the next row.  Whatever lies there, an infinity included, must not reach the product (inf * 0 is NaN)."""
    rs = onp.random.RandomState(K)
    M, N = 70, 45
    a, b = rs.randn(M, K).astype(F32), rs.randn(K, N).astype(F32)
    bt = onp.ascontiguousarray(b.T)
    a[5, 0] = a[33, min(1, K - 1)] = onp.inf      # the elements right after rows 4 and 32
    bt[7, 0] = bt[20, min(2, K - 1)] = -onp.inf
    with onp.errstate(invalid="ignore"):
        want_nn = a.astype(F64) @ b.astype(F64)
        want_nt = a.astype(F64) @ bt.T.astype(F64)
    A, B, Bt = P(dnp, a), P(dnp, b), P(dnp, bt)
    for got, want in ((dnp.dot(A, B).numpy(), want_nn), (dnp.dot(A, dnp.transpose(Bt)).numpy(), want_nt),
                      (dnp.dot(Bt, dnp.transpose(A)).numpy(), want_nt.T)):
        assert onp.array_equal(onp.isfinite(got), onp.isfinite(want))
        assert onp.array_equal(onp.isnan(got), onp.isnan(want)) and onp.array_equal(onp.isposinf(got), onp.isposinf(want))
        fin = onp.isfinite(want)
        close(got[fin], want[fin].astype(F32), RT[F32] * max(1.0, onp.sqrt(K) / 8))


@pytest.mark.parametrize("dtype", [F32, F64])
def test_concatenate_in_one_launch_is_a_copy(dnp, dtype):
    """Pieces that are strided views (slices, transposes, broadcasts, launch-free constants) are joined by one kernel;
    anything else (pending maps, other dtypes, more pieces than one launch takes) goes piece by piece.  Either way the result
    is NumPy's, bit for bit."""
    from autograd_amd import _lib

    rs = onp.random.RandomState(71)
    a, b, c = rs.randn(6, 5, 4).astype(dtype), rs.randn(6, 3, 4).astype(dtype), rs.randn(6, 1, 4).astype(dtype)
    A, B, C = P(dnp, a), P(dnp, b), P(dnp, c)
    calls = []
    real = _lib.concat
    _lib.concat = lambda *args: (calls.append(len(args[3])), real(*args))[1]
    try:
        for axis in (0, 1, 2, -1):
            if axis in (1,):
                got, want = dnp.concatenate((A, B, C), axis=axis), onp.concatenate((a, b, c), axis=axis)
            else:
                got, want = dnp.concatenate((A, A[::-1][::-1], A * 1.0), axis=axis), onp.concatenate((a, a, a), axis=axis)
            assert got.dtype == want.dtype and onp.array_equal(got.numpy(), want), axis
        assert len(calls) == 4
        x, h = rs.randn(7, 13).astype(dtype), rs.randn(7, 30).astype(dtype)
        X, H = P(dnp, x), P(dnp, h)
        got = dnp.hstack((X, H, dnp.ones((7, 1), dtype=dtype)))  # the recurrent net's state
        assert onp.array_equal(got.numpy(), onp.hstack((x, h, onp.ones((7, 1), dtype)))) and calls[-1] == 3
        got = dnp.hstack((X[:, ::2], dnp.transpose(P(dnp, onp.ascontiguousarray(h.T)))[:, 3:9], dnp.broadcast_to(X[:, :1], (7, 4))))
        assert onp.array_equal(got.numpy(), onp.hstack((x[:, ::2], h[:, 3:9], onp.broadcast_to(x[:, :1], (7, 4)))))
        assert onp.array_equal(dnp.vstack((X[1:3], X[5:], X[:0])).numpy(), onp.vstack((x[1:3], x[5:], x[:0])))
        assert onp.array_equal(dnp.concatenate((X[:, 0], H[:, 1])).numpy(), onp.concatenate((x[:, 0], h[:, 1])))
        assert onp.array_equal(dnp.stack((X, X * 2.0), axis=1).numpy(), onp.stack((x, x * dtype(2.0)), axis=1))
        n = len(calls)
        # ten pieces are still one launch
        assert onp.array_equal(dnp.hstack((X,) * 10).numpy(), onp.hstack((x,) * 10)) and calls[-1] == 10
        n = len(calls)
        # not one launch: a pending map that is no constant, more pieces than the kernel's table holds, mixed precision
        assert onp.array_equal(dnp.hstack((X, -H)).numpy(), onp.hstack((x, -h)))
        assert onp.array_equal(dnp.hstack((X,) * (_lib.MAX_CONCAT + 1)).numpy(), onp.hstack((x,) * (_lib.MAX_CONCAT + 1)))
        other = F64 if dtype == F32 else F32
        mixed = dnp.hstack((X, P(dnp, h.astype(other))))
        assert mixed.dtype == F64 and onp.array_equal(mixed.numpy(), onp.hstack((x, h.astype(other))))
        assert len(calls) == n
    finally:
        _lib.concat = real
    from autograd_amd.test_util import check_grads

    check_grads(lambda u, v: dnp.hstack((u, v * v, dnp.ones((7, 1)))) ** 2, modes=["fwd", "rev"], order=2)(
        dnp.asarray(rs.randn(7, 3)), dnp.asarray(rs.randn(7, 2)))


def test_dot_small_integers_exact(dnp):
    rs = onp.random.RandomState(12)
    a = rs.randint(-4, 5, (200, 333)).astype(F32)
    b = rs.randint(-4, 5, (333, 150)).astype(F32)
    assert onp.array_equal(dnp.dot(P(dnp, a), P(dnp, b)).numpy(), a @ b)
    assert onp.array_equal(dnp.dot(P(dnp, a.astype(F64)), P(dnp, b.astype(F64))).numpy(), a.astype(F64) @ b.astype(F64))


@pytest.mark.parametrize("dtype", [F32, F64])
def test_dot_vector_forms_matmul_tensordot(dnp, dtype):
    rs = onp.random.RandomState(13)
    rt = RT[dtype] * 4
    A, v, u = rs.randn(30, 40).astype(dtype), rs.randn(40).astype(dtype), rs.randn(30).astype(dtype)
    close(dnp.dot(P(dnp, A), P(dnp, v)).numpy(), A @ v, rt)
    close(dnp.dot(P(dnp, u), P(dnp, A)).numpy(), u @ A, rt)
    close(dnp.dot(P(dnp, v), P(dnp, v)).numpy(), onp.asarray(v @ v), rt)
    close(dnp.dot(P(dnp, A), 2.0).numpy(), A * dtype(2.0), rt)
    B3, C3 = rs.randn(4, 30, 40).astype(dtype), rs.randn(4, 40, 20).astype(dtype)
    close(dnp.matmul(P(dnp, B3), P(dnp, C3)).numpy(), onp.matmul(B3, C3), rt)
    close(dnp.matmul(P(dnp, B3), P(dnp, C3[0])).numpy(), onp.matmul(B3, C3[0]), rt)
    close(dnp.matmul(P(dnp, A), P(dnp, C3)).numpy(), onp.matmul(A, C3), rt)
    close(dnp.matmul(P(dnp, B3), P(dnp, v)).numpy(), onp.matmul(B3, v), rt)
    # batches of small outputs with a long K (float32: the K split inside one block, one block row of the grid per matrix)
    B4, C4 = rs.randn(3, 40, 300).astype(dtype), rs.randn(3, 300, 50).astype(dtype)
    long_k = rt * onp.sqrt(300) / 8
    close(dnp.matmul(P(dnp, B4), P(dnp, C4)).numpy(), onp.matmul(B4, C4), long_k)
    close(dnp.matmul(P(dnp, B4), P(dnp, C4[1])).numpy(), onp.matmul(B4, C4[1]), long_k)
    close(dnp.matmul(dnp.swapaxes(P(dnp, onp.ascontiguousarray(B4.transpose(0, 2, 1))), 1, 2), P(dnp, C4)).numpy(),
          onp.matmul(B4, C4), long_k)
    T1, T2 = rs.randn(2, 3, 5, 4).astype(dtype), rs.randn(5, 4, 2, 3).astype(dtype)
    close(dnp.tensordot(P(dnp, T1), P(dnp, T2), 2).numpy(), onp.tensordot(T1, T2, 2), rt)
    close(dnp.tensordot(P(dnp, T1), P(dnp, T2), [[0, 1], [2, 3]]).numpy(), onp.tensordot(T1, T2, [[0, 1], [2, 3]]), rt)
    close(dnp.tensordot(P(dnp, T1), P(dnp, T2), [[3, 0], [1, 2]]).numpy(), onp.tensordot(T1, T2, [[3, 0], [1, 2]]), rt)
    close(dnp.tensordot(P(dnp, A), P(dnp, v), 0).numpy(), onp.tensordot(A, v, 0), rt)
    close(dnp.dot(P(dnp, B3), P(dnp, C3[0])).numpy(), onp.dot(B3, C3[0]), rt)
    close(dnp.outer(P(dnp, u), P(dnp, v)).numpy(), onp.outer(u, v), rt)


# ---- index / scatter: bit exact -----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, F64])
def test_take_and_ordered_scatter_add(dnp, dtype):
    from autograd_amd.numpy import wrapper as W

    rs = onp.random.RandomState(14)
    A = rs.randn(50, 7).astype(dtype)
    for idx in ([0, 0], [0, 1, 0], [3, -1, 3, 3, 49, -50], list(rs.randint(-50, 50, 500)), []):
        got = P(dnp, A)[idx].numpy()
        assert onp.array_equal(got, A[onp.array(idx, dtype="int64")])
        x = (rs.randn(len(idx), 7) * 1e3).astype(dtype)
        dst = rs.randn(50, 7).astype(dtype)
        want = dst.copy()
        onp.add.at(want, onp.array(idx, dtype="int64"), x)
        got = W.scatter_add(dnp.asarray(dst) + 0.0, idx, P(dnp, x)).numpy()
        assert onp.array_equal(got, want), idx[:6]
    v = rs.randn(1000).astype(dtype)
    idx = list(rs.randint(0, 10, 4000))           # long runs: sequential order matters in floating point
    x = (rs.randn(4000) * onp.exp(rs.randn(4000) * 5)).astype(dtype)
    want = v[:10].copy()
    onp.add.at(want, onp.array(idx), x)
    assert onp.array_equal(W.scatter_add(dnp.asarray(v[:10]) + 0.0, idx, P(dnp, x)).numpy(), want)
    for sl in (slice(1, None), slice(None, -1), slice(2, 9, 3), 4, (slice(None), 2), (Ellipsis, slice(1, 3))):
        dst = rs.randn(12, 5).astype(dtype)
        x = rs.randn(*onp.shape(dst[sl])).astype(dtype)
        want = dst.copy()
        onp.add.at(want, sl, x)
        assert onp.array_equal(W.scatter_add(dnp.asarray(dst) + 0.0, sl, P(dnp, x)).numpy(), want)


def test_vspace_axioms(dnp):
    # tests/test_vspaces.py:10-159 of the reference, for the device vspace
    from autograd_amd.extend import vspace

    x = P(dnp, onp.random.RandomState(15).randn(4, 3))
    vs = vspace(x)
    assert vs.shape == (4, 3) and vs.dtype == onp.float64 and vs.size == 12 and vs.ndim == 2
    assert vs == vspace(vs.zeros()) and vs == vspace(vs.ones()) and vs == vspace(vs.randn())
    a, b = vs.randn(), vs.randn()
    assert onp.array_equal(vs.add(a, b).numpy(), a.numpy() + b.numpy())
    assert onp.array_equal(vs.add(a, vs.zeros()).numpy(), a.numpy())
    assert onp.array_equal(vs.scalar_mul(a, 2.5).numpy(), a.numpy() * 2.5)
    assert abs(float(vs.inner_prod(a, b)) - onp.sum(a.numpy() * b.numpy())) < 1e-12
    basis = list(vs.standard_basis())
    assert len(basis) == 12 and onp.array_equal(onp.sum([e.numpy() for e in basis], axis=0), onp.ones((4, 3)))
    from autograd_amd.numpy import fusion

    for fused in (False, True):
        was, fusion.ENABLED = fusion.ENABLED, fused
        try:
            acc = vs.mut_add(None, a)          # 0 + a: borrows a's memory, never writes it
            acc2 = vs.mut_add(acc, b)          # first real accumulation goes to fresh memory (or stays an expression)
            acc3 = vs.mut_add(acc2, b)         # from then on in place when the sums are launched one by one
        finally:
            fusion.ENABLED = was
        assert acc2 is not acc and (fused or acc3 is acc2)
        assert onp.array_equal(acc.numpy(), a.numpy())
        assert onp.array_equal(acc3.numpy(), ((0.0 + a.numpy()) + b.numpy()) + b.numpy())
    assert vspace(dnp.ones((2,), dtype=F32)).dtype == onp.float32


# ---- edge cases: empty, single-element and ragged extents, special values ------------------------
def test_empty_and_degenerate_shapes(dnp):
    for shape in [(0,), (0, 5), (5, 0), (3, 0, 2)]:
        x = onp.zeros(shape, F32)
        X = P(dnp, x)
        assert (X + 1.0).shape == shape and dnp.exp(X).shape == shape
        assert onp.array_equal(dnp.sum(X).numpy(), onp.sum(x))
        assert dnp.sum(X, axis=0).shape == onp.sum(x, axis=0).shape
        assert onp.array_equal(dnp.sum(X, axis=-1).numpy(), onp.sum(x, axis=-1))
        assert dnp.reshape(X, (-1,)).shape == (0,)
    a, b = onp.ones((0, 4), F32), onp.ones((4, 3), F32)
    assert onp.array_equal(dnp.dot(P(dnp, a), P(dnp, b)).numpy(), a @ b)
    a, b = onp.ones((2, 0), F32), onp.ones((0, 3), F32)
    assert onp.array_equal(dnp.dot(P(dnp, a), P(dnp, b)).numpy(), a @ b)  # K = 0: zeros
    assert onp.array_equal(dnp.concatenate((P(dnp, onp.ones((0, 3))), P(dnp, onp.ones((2, 3)))), axis=0).numpy(), onp.ones((2, 3)))
    s = P(dnp, onp.float64(3.0))
    assert (s * s).shape == () and float(s * s) == 9.0 and float(dnp.sum(s)) == 3.0


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 256, 257, 1023, 1025, 4099])
def test_ragged_lengths_every_vector_tail(dnp, n):
    rs = onp.random.RandomState(n)
    for dtype in (F32, F64):
        x, y = rs.randn(n).astype(dtype), rs.randn(n).astype(dtype)
        assert onp.array_equal((P(dnp, x) * P(dnp, y)).numpy(), x * y)
        assert onp.array_equal((P(dnp, x)[1:] + 2.0).numpy(), x[1:] + dtype(2.0))
        close(dnp.sum(P(dnp, x)).numpy(), onp.sum(x), RT[dtype])
        m = rs.randn(7, n).astype(dtype)
        assert onp.array_equal((P(dnp, m) - P(dnp, y)).numpy(), m - y)
        close(dnp.sum(P(dnp, m), axis=0).numpy(), m.sum(axis=0), RT[dtype])
        close(dnp.sum(P(dnp, m), axis=1).numpy(), m.sum(axis=1), RT[dtype])
        assert onp.array_equal(dnp.max(P(dnp, m), axis=1).numpy(), m.max(axis=1))


def test_special_values_propagate_like_numpy(dnp):
    x = onp.array([0.0, -0.0, onp.inf, -onp.inf, onp.nan, 1.0, -1.0])
    X = P(dnp, x)
    with onp.errstate(all="ignore"):
        for name in ("exp", "tanh", "negative", "abs", "square", "sign"):
            got, want = getattr(dnp, name)(X).numpy(), getattr(onp, name)(x)
            assert onp.array_equal(got, want, equal_nan=True), name
        assert onp.array_equal(dnp.maximum(X, 0.5).numpy(), onp.maximum(x, 0.5), equal_nan=True)
        assert onp.array_equal(dnp.minimum(X, X[::1] * 0.0).numpy(), onp.minimum(x, x * 0.0), equal_nan=True)
        assert onp.isnan(dnp.max(X).numpy()) and onp.isnan(dnp.sum(X).numpy())
        assert dnp.max(X[:4]).numpy() == onp.inf and dnp.min(X[:4]).numpy() == -onp.inf
        assert onp.array_equal((X / 0.0).numpy(), x / 0.0, equal_nan=True)
    assert onp.array_equal(dnp.logical_and(X[5:] > 0, X[5:] < 2).numpy(), [True, False])
    assert onp.array_equal(dnp.logical_or(X[5:] > 0, X[5:] < 0).numpy(), [True, True])
    assert onp.array_equal(dnp.logical_not(X[5:] > 0).numpy(), [False, True])


def test_rank_limits_are_reported(dnp):
    from autograd_amd._lib import AgmiError

    x = P(dnp, onp.zeros((2,) * 8, F32))
    assert dnp.exp(x).shape == (2,) * 8                      # rank 8 merges to one axis
    y = dnp.transpose(x)                                    # fully reversed: 8 unmergeable axes
    with pytest.raises(AgmiError, match="axes remain after merging"):
        y + x
    with pytest.raises(AgmiError):
        dnp.exp(P(dnp, onp.zeros((1,) * 9, F32)))


# ---- pending affine maps (negation / scalar factor / scalar offset folded into the consumer) -----
def _lazy_cases(dnp, x):
    """(device expression, NumPy expression) pairs whose device side is a pending map."""
    X = P(dnp, x)
    one = x.dtype.type(1)
    return [
        (-X, -x), (X * 3.0, x * one * x.dtype.type(3.0)), (0.1 * X, x.dtype.type(0.1) * x), (X + 1.5, x + x.dtype.type(1.5)),
        (1.0 - X, one - x), (1.0 - 2.0 * X, one - x.dtype.type(2) * x), (-(X * 0.3), -(x * x.dtype.type(0.3))),
        ((X + 0.7) * 4.0, (x + x.dtype.type(0.7)) * x.dtype.type(4)), (X + 0.0, x + x.dtype.type(0)),
        ((X * 3.0) * 0.5, (x * x.dtype.type(3)) * x.dtype.type(0.5)),
    ]


@pytest.mark.parametrize("dtype", [F32, F64])
def test_pending_maps_are_bit_exact_on_every_kernel_path(dnp, dtype):
    from autograd_amd.numpy.devarray import LazyDevArray

    rng = onp.random.RandomState(11)
    x = rng.randn(67, 130).astype(dtype)
    x[0, :4] = [0.0, -0.0, onp.inf, onp.nan]
    y = rng.randn(67, 130).astype(dtype)
    Y = P(dnp, y)
    for k, (L, ref) in enumerate(_lazy_cases(dnp, x)):
        assert type(L) is LazyDevArray, k
        assert ref.dtype == dtype
        # written out by the copy kernel (flat path), bit for bit incl. signed zeros
        got = L.numpy()
        nan = onp.isnan(ref)  # (the sign of a NaN is not specified: compare bits everywhere else)
        assert got.dtype == dtype and onp.array_equal(onp.isnan(got), nan), k
        assert onp.array_equal(got[~nan].view(onp.uint8), ref[~nan].view(onp.uint8)), k
        # as an operand: flat, row-broadcast, strided (nd) and transposed consumers
        assert onp.array_equal((L * Y).numpy(), ref * y, equal_nan=True), k
        assert onp.array_equal((Y[:, :1] + L).numpy(), y[:, :1] + ref, equal_nan=True), k
        assert onp.array_equal((L[::2, 1::3] - Y[::2, 1::3]).numpy(), ref[::2, 1::3] - y[::2, 1::3], equal_nan=True), k
        assert onp.array_equal((L.T * Y.T).numpy(), ref.T * y.T, equal_nan=True), k
        assert onp.array_equal((L[3] * Y).numpy(), ref[3] * y, equal_nan=True), k  # row operand pending
        # two pending operands in one launch
        assert onp.array_equal((L * (1.0 - Y)).numpy(), ref * (dtype(1) - y), equal_nan=True), k
        # compare / cast / gather / contraction consumers see the written-out value
        assert onp.array_equal((L > Y).numpy(), ref > y), k
        assert onp.array_equal(dnp.take(L, onp.array([5, 1, 5])).numpy(), ref[[5, 1, 5]], equal_nan=True), k
    # reductions: row / column / full, fused map, logsumexp (finite rows)
    xf, yf = x[1:], y[1:]
    for k, (L, ref) in enumerate(_lazy_cases(dnp, xf)):
        close(dnp.sum(L, axis=1).numpy(), ref.sum(axis=1), RT[dtype])
        close(dnp.sum(L, axis=0).numpy(), ref.sum(axis=0), RT[dtype])
        close(dnp.sum(L).numpy(), ref.sum(), RT[dtype])
        close(dnp.max(L, axis=1).numpy(), ref.max(axis=1), 0.0)
        close(dnp.sum(L * Y[1:], axis=0).numpy(), (ref * yf).sum(axis=0), RT[dtype])
        from autograd_amd.scipy.special import logsumexp

        close(logsumexp(L, axis=1).numpy(), scipy.special.logsumexp(ref, axis=1), RT[dtype])
        close(logsumexp(L, axis=0).numpy(), scipy.special.logsumexp(ref, axis=0), RT[dtype])
        A, B = rng.randn(5, 66).astype(dtype), rng.randn(130, 3).astype(dtype)
        close(dnp.dot(P(dnp, A), L).numpy(), A @ ref, RT[dtype])
        close(dnp.dot(L, P(dnp, B)).numpy(), ref @ B, RT[dtype])


def test_pending_maps_through_grad_match_eager_numpy(dnp):
    """Differentiating through folded operations gives what NumPy gives op by op."""
    from autograd_amd import elementwise_grad, grad

    x = onp.linspace(-1.5, 1.5, 4099)
    X = P(dnp, x)

    def f(np):
        return lambda v: np.sum((1.0 - np.exp(-2.0 * v)) / (1.0 + np.exp(-(2 * v))) * 0.5 - (3.0 - v) ** 2)

    g = grad(f(dnp))(X)
    e = onp.exp(-2.0 * x)
    want = 0.5 * (2.0 * e / (1.0 + e) + (1.0 - e) * 2.0 * e / (1.0 + e) ** 2) + 2.0 * (3.0 - x)
    close(g.numpy(), want, 1e-13)
    h = elementwise_grad(elementwise_grad(lambda v: -dnp.tanh(-v) * 2.0))(X)
    t = onp.tanh(x)
    close(h.numpy(), 2.0 * (-2.0 * t * (1.0 - t * t)), 1e-13)
    # accumulation over a fan-out whose contributions are pending maps of one array
    k = grad(lambda v: dnp.sum(-v) + dnp.sum(2.0 * v) + dnp.sum(v + 1.0) + dnp.sum(v * v))(X)
    close(k.numpy(), 2.0 + 2.0 * x, 1e-15)


@pytest.mark.parametrize("dtype", [F32, F64])
def test_einsum_matches_numpy(dnp, dtype):
    rs = onp.random.RandomState(9)
    shapes = dict(a=(33, 20), b=(20, 17), c=(17, 5), t=(3, 33, 20), u=(3, 20, 17), w=(1, 20, 17), v=(9, 20), x=(20,))
    H = {k: rs.randn(*s).astype(dtype) for k, s in shapes.items()}
    Dv = {k: P(dnp, h) for k, h in H.items()}
    specs = [("ij,jk->ik", "ab"), ("ij,jk", "ab"), ("ij,jk->ki", "ab"), ("bij,bjk->bik", "tu"), ("bij,bjk->kbi", "tu"),
             ("ij,kj->i", "av"), ("ij,kj->ik", "av"), ("ij,jk,kl->il", "abc"), ("ij->ji", "a"), ("ij->", "a"), ("ij->j", "a"),
             ("ij,j->i", "ax"), ("i,i->", "xx"), ("i,j->ij", "xx"), ("...ij,...jk->...ik", "tw"), ("bij,bij->b", "tt"),
             ("bij,ij->b", "ta"), ("ij,kl->", "ac")]
    for spec, ops in specs:
        got = dnp.einsum(spec, *[Dv[o] for o in ops]).numpy()
        want = onp.einsum(spec, *[H[o] for o in ops])
        close(got, onp.asarray(want, dtype), RT[dtype] * 4)
    close(dnp.einsum("ij,jk->ik", Dv["a"].T.T, Dv["b"][:, ::2]).numpy(), H["a"] @ H["b"][:, ::2], RT[dtype] * 4)
    # repeated subscripts (diagonals) and the operand/sublist convention
    H["q"], H["s"] = rs.randn(6, 6).astype(dtype), rs.randn(3, 5, 5).astype(dtype)
    Dv["q"], Dv["s"] = P(dnp, H["q"]), P(dnp, H["s"])
    for spec, ops in [("ii->i", "q"), ("ii->", "q"), ("ii", "q"), ("bii->bi", "s"), ("bjj->b", "s"), ("ii,ij->j", "qq"), ("ij,jj->i", "qq")]:
        close(dnp.einsum(spec, *[Dv[o] for o in ops]).numpy(), onp.asarray(onp.einsum(spec, *[H[o] for o in ops]), dtype), RT[dtype] * 4)
    close(dnp.einsum(Dv["a"], [0, 1], Dv["b"], [1, 2], [0, 2]).numpy(), H["a"] @ H["b"], RT[dtype] * 4)
    close(dnp.einsum(Dv["a"], [0, 1], Dv["b"], [1, 2]).numpy(), H["a"] @ H["b"], RT[dtype] * 4)
    close(dnp.einsum(Dv["t"], [Ellipsis, 0, 1], Dv["b"], [1, 2], [Ellipsis, 2, 0]).numpy(),
          onp.einsum("...ij,jk->...ki", H["t"], H["b"]), RT[dtype] * 4)
    with pytest.raises(ValueError):
        dnp.einsum("ij->ii", Dv["q"])


def test_einsum_rules_beyond_the_reference_agree_with_finite_differences(dnp):
    """The reference's einsum cotangent (numpy_vjps.py:790-854) raises for an operand that carries a repeated
    subscript, and for the operand/sublist form without an output sublist, so no reference vector exists for
    these: they are checked against numerical differentiation."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(12)
    Q, W, T = (dnp.asarray(rs.randn(*s)) for s in ((4, 4), (4, 4), (2, 3, 3)))
    for fun, x in [(lambda q: dnp.einsum("ii->", q) ** 2, Q), (lambda q: dnp.einsum("ii->i", q) ** 2, Q),
                   (lambda q: dnp.einsum("ii,ij->j", q, W) ** 2, Q), (lambda q: dnp.einsum("ij,jj->i", W, q) ** 2, Q),
                   (lambda t: dnp.einsum("bii->bi", t) ** 2, T), (lambda t: dnp.einsum("bii->", t) ** 2, T),
                   (lambda q: dnp.einsum(q, [0, 0], W, [0, 1], [1]) ** 2, Q), (lambda q: dnp.einsum(q, [0, 1], W, [1, 2]) ** 2, Q),
                   (lambda q: dnp.einsum(W, [1, 0], q, [0, 2]) ** 2, Q)]:
        check_grads(fun, modes=["fwd", "rev"], order=2)(x)


def test_gradient_and_linspace_follow_numpy_and_differentiate(dnp):
    """Values are NumPy's bit for bit (the same subtractions, halvings and affine steps).  The reference's
    gradient cotangent needs four samples along the axis and its linspace rules take no ``endpoint``; the
    shorter axes and ``endpoint=False`` are checked against numerical differentiation."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(13)
    for shp, ax in [((6,), None), ((4, 5), None), ((2, 5), 0), ((3, 5), 0), ((4, 5), -1), ((3, 4, 5), (0, 2))]:
        x = rs.randn(*shp)
        want, got = onp.gradient(x, axis=ax), dnp.gradient(dnp.asarray(x), axis=ax)
        if isinstance(want, (tuple, list)):
            assert len(want) == len(got) and all(onp.array_equal(w, g.numpy()) for w, g in zip(want, got))
            check_grads(lambda a: sum(dnp.sum(dnp.sin(p)) for p in dnp.gradient(a, axis=ax)), modes=["fwd", "rev"], order=2)(dnp.asarray(x))  # noqa: B023
        else:
            assert onp.array_equal(want, got.numpy()), (shp, ax)
            check_grads(lambda a: dnp.gradient(a, axis=ax), modes=["fwd", "rev"], order=2)(dnp.asarray(x))  # noqa: B023
    with pytest.raises(ValueError):
        dnp.gradient(dnp.asarray(rs.randn(1, 4)), axis=0)
    with pytest.raises(NotImplementedError):
        dnp.gradient(dnp.asarray(rs.randn(5)), 2.0)
    for num in (1, 2, 5, 50):
        for endpoint in (True, False):
            want = onp.linspace(1.3, -0.7, num, endpoint=endpoint)
            got = dnp.linspace(dnp.asarray(1.3), dnp.asarray(-0.7), num, endpoint=endpoint)
            assert onp.array_equal(want, got.numpy()), (num, endpoint)
            check_grads(lambda s, t: dnp.linspace(s, t, num, endpoint=endpoint), modes=["fwd", "rev"], order=2)(  # noqa: B023
                dnp.asarray(1.3), dnp.asarray(-0.7))
    assert dnp.linspace(dnp.asarray(onp.float32(0.5)), 2.0, 4).dtype == onp.float32
    assert onp.array_equal(dnp.linspace(0.0, 1.0, 5).numpy(), onp.linspace(0.0, 1.0, 5))


def test_sort_and_partition_differentiate_along_any_axis(dnp):
    """The reference's rules stop at vectors (numpy_vjps.py:773-795 raise for anything else), so there is no
    reference vector: each line's cotangent must come back through the inverse of that line's permutation,
    checked against ``take_along_axis`` on the host and numerical differentiation."""
    from autograd_amd import grad
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(15)
    for shape, axis in (((5, 7), -1), ((5, 7), 0), ((3, 4, 6), 1), ((3, 4, 6), None), ((6,), 0)):
        x, w = rs.randn(*shape), rs.randn(*(shape if axis is not None else (int(onp.prod(shape)),)))
        X, W = dnp.asarray(x), dnp.asarray(w)
        got = grad(lambda a: dnp.sum(dnp.sort(a, axis=axis) * W))(X).numpy()  # noqa: B023
        if axis is None:
            want = onp.empty(x.size)
            want[onp.argsort(x, axis=None, kind="stable")] = w
            want = want.reshape(shape)
        else:
            want = onp.take_along_axis(w, onp.argsort(onp.argsort(x, axis=axis, kind="stable"), axis=axis, kind="stable"), axis)
        assert onp.array_equal(got, want), (shape, axis)
        check_grads(lambda a: dnp.sort(a, axis=axis) * W, modes=["fwd", "rev"], order=2)(X)  # noqa: B023
        if axis is not None:
            check_grads(lambda a: dnp.sort(a, axis=axis)[(slice(None),) * (axis % len(shape)) + (slice(0, 2),)] ** 2,  # noqa: B023
                        modes=["fwd", "rev"])(X)


def test_astype_tangent_is_the_cast_of_the_tangent(dnp):
    """The reference defines no forward-mode rule for ``astype`` (numpy_jvps.py has none); this one does, so
    it is checked against numerical differentiation instead of a reference vector."""
    from autograd_amd.test_util import check_grads

    x = dnp.asarray(onp.random.RandomState(14).randn(3, 4))
    check_grads(lambda a: dnp.sin(a).astype(onp.float64) ** 2, modes=["fwd", "rev"], order=2)(x)
    check_grads(lambda a: dnp.astype(a * a, onp.float64), modes=["fwd"], order=1)(x)


@pytest.mark.parametrize("dtype", [F32, F64])
def test_pending_maps_with_broadcast_operands_are_bit_exact(dnp, dtype):
    """``A * b[None, :] + c[:, None]`` and friends launch nothing; every consumer kernel applies the
    steps on load and must round exactly like the NumPy passes."""
    from autograd_amd.numpy.devarray import LazyDevArray
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(21)
    a = rs.randn(67, 130).astype(dtype)
    b = rs.uniform(0.5, 1.5, 130).astype(dtype)
    c = rs.randn(67).astype(dtype)
    y = rs.randn(67, 130).astype(dtype)
    a[0, :3] = [0.0, -0.0, onp.inf]
    A, B, C, Y = P(dnp, a), P(dnp, b), P(dnp, c), P(dnp, y)
    one = dtype(1)
    cases = [
        (A * B[None, :], a * b[None, :]),
        (A + C[:, None], a + c[:, None]),
        (A * B[None, :] + C[:, None], a * b[None, :] + c[:, None]),
        (C[:, None] + B * A, c[:, None] + b * a),
        (-(A * B), -(a * b)),
        ((A * B) * 2.0 + 1.0, (a * b) * dtype(2) + one),
        (C[:, None] - A, c[:, None] - a),
        (2.0 * A * C[:, None], dtype(2) * a * c[:, None]),
        (A * B[0], a * b[0]),                                     # 0-d array operand
    ]
    for k, (L, ref) in enumerate(cases):
        assert type(L) is LazyDevArray, k
        nan = onp.isnan(ref)
        got = L.numpy()
        assert got.dtype == dtype and onp.array_equal(onp.isnan(got), nan), k
        assert onp.array_equal(got[~nan].view(onp.uint8), ref[~nan].view(onp.uint8)), k
        with onp.errstate(all="ignore"):
            assert onp.array_equal((L * Y).numpy(), ref * y, equal_nan=True), k                 # flat / rows consumer
            assert onp.array_equal((L.T + Y.T).numpy(), ref.T + y.T, equal_nan=True), k         # transposed view keeps the steps
            assert onp.array_equal((L[1::2, 3:99] - Y[1::2, 3:99]).numpy(), ref[1::2, 3:99] - y[1::2, 3:99], equal_nan=True), k
            assert onp.array_equal(dnp.reshape(L, (67, 10, 13)).numpy(), ref.reshape(67, 10, 13), equal_nan=True), k
            assert onp.array_equal(dnp.exp(L[5]).numpy()[:0], onp.exp(ref[5])[:0]), k
            close(dnp.exp(L[5] * 0.01).numpy(), onp.exp(ref[5] * dtype(0.01)), RT_EW[dtype] * 8)
        # more array-valued steps than one launch takes: operands are written out as needed
        M = (A * B[None, :] + C[:, None]) * (Y * B + C[:, None])
        with onp.errstate(all="ignore"):
            assert onp.array_equal(M.numpy(), (a * b[None, :] + c[:, None]) * (y * b + c[:, None]), equal_nan=True)
    # reductions over finite data: row / column / full sums, fused map, logsumexp in every form
    af = a[1:]
    Af, Cf, Yf = P(dnp, af), P(dnp, c[1:]), P(dnp, y[1:])
    forms = [
        (Af * B[None, :] + Cf[:, None], af * b[None, :] + c[1:, None]),   # row-varying factor, row-constant offset
        (Af * Cf[:, None] + B[None, :], af * c[1:, None] + b[None, :]),   # the other way round
        (Af * B[None, :], af * b[None, :]),
        (Af + Cf[:, None], af + c[1:, None]),
        (Af * 0.5 + B, af * dtype(0.5) + b),
    ]
    for L, ref in forms:
        assert type(L) is LazyDevArray
        close(dnp.sum(L, axis=1).numpy(), ref.sum(axis=1), RT[dtype])
        close(dnp.sum(L, axis=0).numpy(), ref.sum(axis=0), RT[dtype])
        close(dnp.sum(L).numpy(), ref.sum(), RT[dtype])
        close(dnp.max(L, axis=0).numpy(), ref.max(axis=0), 0.0)
        close(dnp.sum(L * Yf, axis=0).numpy(), (ref * y[1:]).sum(axis=0), RT[dtype])
        close(logsumexp(L, axis=1).numpy(), scipy.special.logsumexp(ref, axis=1), RT[dtype])
        close(logsumexp(L, axis=0).numpy(), scipy.special.logsumexp(ref, axis=0), RT[dtype])
        close(logsumexp(L[:, :37], axis=1).numpy(), scipy.special.logsumexp(ref[:, :37], axis=1), RT[dtype])
        close(logsumexp(L).numpy(), scipy.special.logsumexp(ref), RT[dtype])
    wide = rs.randn(9, 5000).astype(dtype)  # rows longer than one block pass: chunked logsumexp
    wb = rs.uniform(0.5, 1.5, 5000).astype(dtype)
    close(logsumexp(P(dnp, wide) * P(dnp, wb) + 0.25, axis=1).numpy(),
          scipy.special.logsumexp(wide * wb + dtype(0.25), axis=1), RT[dtype])


@pytest.mark.parametrize("dtype", [F32, F64])
def test_max_min_reduction_rules_share_the_cotangent_between_ties(dnp, dtype):
    """numpy_vjps.py:515-530: g * (x == ans) / count, here one fused count and one fused product;
    the arithmetic is the reference's, so the result is compared bit for bit with the oracle."""
    import autograd_amd as ag
    import oracle.anp as anp

    rs = onp.random.RandomState(21)
    x = rs.randint(-3, 4, (6, 5, 8)).astype(dtype)  # many ties
    x[0] += rs.randn(5, 8).astype(dtype)            # and a slab without
    X = P(dnp, x)
    for fname in ("max", "min"):
        for axis in (None, 0, 1, 2, (0, 2), (1, 2)):
            for keepdims in (False, True):
                w = onp.asarray(rs.randn(*onp.shape(getattr(onp, fname)(x, axis=axis, keepdims=keepdims)))).astype(dtype)
                got = ag.grad(lambda z: dnp.sum(getattr(dnp, fname)(z, axis=axis, keepdims=keepdims) * P(dnp, w)))(X)
                want = ag.grad(lambda z: anp.sum(getattr(anp, fname)(z, axis=axis, keepdims=keepdims) * w))(x)
                assert got.dtype == want.dtype and onp.array_equal(got.numpy(), want), (fname, axis, keepdims)
    # second order goes through the traced form of the rule
    v = P(dnp, rs.randn(7).astype(dtype))
    h = ag.grad(lambda z: dnp.sum(ag.grad(lambda t: dnp.max(t * t) * dnp.sum(t))(z)))(v)
    vo = v.numpy()
    ho = ag.grad(lambda z: anp.sum(ag.grad(lambda t: anp.max(t * t) * anp.sum(t))(z)))(vo)
    close(h.numpy(), ho, RT[dtype])


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("rows,inner,cols", [(256, 641, 512), (1024, 784, 1024), (64, 33, 10), (7, 5, 3)])
def test_matrix_cotangents_accumulate_inside_the_contraction(dnp, dtype, rows, inner, cols):
    """A weight used by several products: from the second contribution on, the cotangent's contraction
    runs with beta = 1 into the accumulator.  Bit for bit the same as contracting and adding separately,
    for both operands, whether the contraction is split over K or not."""
    import autograd_amd as ag

    rs = onp.random.RandomState(31)
    X1, X2, X3 = (P(dnp, rs.randn(rows, inner).astype(dtype)) for _ in range(3))
    C1, C2, C3 = (P(dnp, rs.randn(rows, cols).astype(dtype)) for _ in range(3))
    W = P(dnp, rs.randn(inner, cols).astype(dtype))
    f = lambda w: dnp.sum(dnp.dot(X1, w) * C1) + dnp.sum(dnp.dot(X2, w) * C2)  # noqa: E731
    got = ag.grad(f)(W).numpy()
    want = (dnp.dot(X1.T, C1) + dnp.dot(X2.T, C2)).numpy()
    assert onp.array_equal(got, want)
    # three uses, and the left operand of the product this time
    V1, V2, V3 = (P(dnp, rs.randn(inner, cols).astype(dtype)) for _ in range(3))
    h = lambda x: dnp.sum(dnp.dot(x, V1) * C1) + dnp.sum(dnp.dot(x, V2) * C2) + dnp.sum(dnp.dot(x, V3) * C3)  # noqa: E731
    got = ag.grad(h)(X1).numpy()
    parts = [dnp.dot(C, V.T).numpy().astype(onp.float64) for C, V in ((C1, V1), (C2, V2), (C3, V3))]
    ref = parts[0] + parts[1] + parts[2]
    close(got, ref.astype(dtype), RT[dtype])
    # against NumPy as well
    close(ag.grad(f)(W).numpy(), X1.numpy().T @ C1.numpy() + X2.numpy().T @ C2.numpy(), RT[dtype] * 10)
    # the @ operator takes the same route
    fm = lambda w: dnp.sum((X1 @ w) * C1) + dnp.sum(dnp.matmul(X2, w) * C2)  # noqa: E731
    assert onp.array_equal(ag.grad(fm)(W).numpy(), want)
    hm = lambda x: dnp.sum((x @ V1) * C1) + dnp.sum((x @ V2) * C2)  # noqa: E731
    assert onp.array_equal(ag.grad(hm)(X1).numpy(), (dnp.dot(C1, V1.T) + dnp.dot(C2, V2.T)).numpy())


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("steps,rows,inner,cols", [(4, 16, 33, 10), (11, 64, 129, 48), (65, 256, 641, 128), (9, 7, 5, 3)])
def test_many_products_into_one_weight_are_one_contraction(dnp, dtype, steps, rows, inner, cols):
    """A weight used once per step of a loop (numpy_vjps.py:615-638 through core.py:185-205): from four
    products on, the cotangent is ONE contraction over the stacked operands (one launch instead of one
    per step, joined by a few copies).  The order of the additions is not the loop's, so the bound is the
    floating-point one; the result does not change from run to run."""
    import autograd_amd as ag
    from autograd_amd import _lib

    rs = onp.random.RandomState(steps)
    xs = [rs.randn(rows + (t % 3), inner).astype(dtype) for t in range(steps)]  # (the steps need not be equally long)
    cs = [rs.randn(rows + (t % 3), cols).astype(dtype) for t in range(steps)]
    Xs, Cs = [P(dnp, x) for x in xs], [P(dnp, c) for c in cs]
    W = P(dnp, rs.randn(inner, cols).astype(dtype))

    def f(w):
        total = 0.0
        for X, C in zip(Xs, Cs):
            total = total + dnp.sum(dnp.dot(X, w) * C)
        return total

    launches = []
    was = _lib.gemm

    def counting(*a, **k):
        launches.append(a[2:5])
        return was(*a, **k)

    _lib.gemm = counting
    try:
        got = ag.grad(f)(W).numpy()
    finally:
        _lib.gemm = was
    want = sum(x.astype(F64).T @ c.astype(F64) for x, c in zip(xs, cs))
    close(got, want.astype(dtype), RT[dtype] * max(1.0, onp.sqrt(steps * rows) / 8))
    backward = [l for l in launches if l[:2] == (inner, cols)]
    assert len(backward) == 1 and backward[0][2] == sum(x.shape[0] for x in xs), launches
    assert onp.array_equal(ag.grad(f)(W).numpy(), got)


# ---- remainder, nan_to_num and the array functions built on views and copy kernels: bit-exact ---------------
@pytest.mark.parametrize("dtype", [F32, F64])
def test_remainder_and_nan_to_num_are_bit_exact(dnp, dtype):
    rs = onp.random.RandomState(31)
    a = (rs.randn(257, 33) * 7).astype(dtype)
    b = (rs.uniform(0.2, 3.0, (257, 33)) * rs.choice([-1.0, 1.0], (257, 33))).astype(dtype)
    # exact multiples (signed zero results), zero dividends and divisors, infinities and NaN
    a[0, :8] = onp.array([6.0, -6.0, 0.0, -0.0, 5.0, -5.0, onp.inf, onp.nan], dtype)
    b[0, :8] = onp.array([3.0, 3.0, -2.0, 2.0, 0.0, onp.inf, 2.0, 2.0], dtype)
    b[1, :4] = onp.array([-3.0, -3.0, onp.inf, -onp.inf], dtype)
    a[1, :4] = onp.array([6.0, -6.0, -5.0, 5.0], dtype)
    with onp.errstate(all="ignore"):
        want = onp.remainder(a, b)
        got = dnp.remainder(P(dnp, a), P(dnp, b)).numpy()
        assert got.dtype == want.dtype and onp.array_equal(got, want, equal_nan=True)
        ok = ~onp.isnan(want)  # the sign of a zero result is the divisor's; a NaN's sign means nothing
        assert onp.array_equal(onp.signbit(got[ok]), onp.signbit(want[ok]))
        assert onp.array_equal(dnp.mod(P(dnp, a), 0.75).numpy(), onp.mod(a, dtype(0.75)), equal_nan=True)
        assert onp.array_equal((P(dnp, a) % P(dnp, b)).numpy(), want, equal_nan=True)
        assert onp.array_equal((2.5 % P(dnp, b)).numpy(), 2.5 % b, equal_nan=True)
    x = a.copy()
    x[2, :3] = [onp.nan, onp.inf, -onp.inf]
    got = dnp.nan_to_num(P(dnp, x)).numpy()
    assert got.dtype == dtype and onp.array_equal(got, onp.nan_to_num(x))


@pytest.mark.parametrize("dtype", [F32, F64])
def test_array_functions_on_views_and_copies_are_bit_exact(dnp, dtype):
    rs = onp.random.RandomState(32)
    a, q, v, t = (rs.randn(*s).astype(dtype) for s in ((5, 7), (6, 6), (7,), (3, 5, 7)))
    A, Q, V, T = (P(dnp, h) for h in (a, q, v, t))

    def same(got, want):
        got = got.numpy()
        assert got.shape == want.shape and got.dtype == want.dtype, (got.shape, want.shape, got.dtype, want.dtype)
        assert onp.array_equal(got, want, equal_nan=True)

    for shift, axis in ((1, 0), (-2, 1), (9, -1), (0, 0), (5, None), (-3, None)):
        same(dnp.roll(A, shift, axis=axis), onp.roll(a, shift, axis=axis))
    same(dnp.roll(T[:, ::2], 2, axis=1), onp.roll(t[:, ::2], 2, axis=1))
    for k in (-2, 0, 1, 3):
        same(dnp.diag(Q, k), onp.diag(q, k))
        same(dnp.diag(A, k), onp.diag(a, k))
        same(dnp.diag(V, k), onp.diag(v, k))
        same(dnp.tril(A, k), onp.tril(a, k))
        same(dnp.triu(A, k), onp.triu(a, k))
        same(dnp.triu(T, k), onp.triu(t, k))
        same(dnp.diagonal(T, k, 1, 2), onp.diagonal(t, k, 1, 2))
        same(dnp.diagonal(T, k, -1, 0), onp.diagonal(t, k, -1, 0))
    same(Q.diagonal(), q.diagonal())
    same(dnp.tril(dnp.asarray(onp.array([[onp.nan, onp.inf], [1.0, -onp.inf]], dtype))),
         onp.tril(onp.array([[onp.nan, onp.inf], [1.0, -onp.inf]], dtype)))  # masked entries are zeros, not NaN
    for reps in (3, (2,), (2, 3), (2, 1, 2), (1, 1), (0, 2)):
        same(dnp.tile(A, reps), onp.tile(a, reps))
    same(dnp.tile(V, 4), onp.tile(v, 4))
    same(dnp.tile(T.T, (2, 1, 3)), onp.tile(t.T, (2, 1, 3)))
    for x, y, hx, hy in ((A, Q, a, q), (V, V, v, v), (A, V, a, v), (V, A, v, a), (T, A, t, a), (A.T, Q[:2], a.T, q[:2])):
        same(dnp.kron(x, y), onp.kron(hx, hy))
    wide = onp.zeros(a.shape + (a.shape[-1],))
    for i in range(a.shape[0]):
        wide[i] = onp.diag(a[i].astype(F64))
    same(dnp.make_diagonal(A, 0, -1, -2), wide)  # float64 zeros whatever the operand, as the reference builds them
    with pytest.raises(NotImplementedError):
        dnp.make_diagonal(A)
    same(dnp.real(A), a)
    same(dnp.conj(A), a)
    # traces and inner products accumulate: tolerance of the reductions / contractions
    for k in (-1, 0, 2):
        close(dnp.trace(Q, k).numpy(), onp.asarray(onp.trace(q, k)), RT[dtype])
        close(dnp.trace(T, k).numpy(), onp.trace(t, k), RT[dtype])
    close(Q.trace().numpy(), onp.asarray(q.trace()), RT[dtype])
    close(dnp.inner(A, T).numpy(), onp.inner(a, t), RT[dtype])
    close(dnp.inner(V, V).numpy(), onp.asarray(onp.inner(v, v)), RT[dtype])
    close(dnp.inner(T, V).numpy(), onp.inner(t, v), RT[dtype])
    same(dnp.inner(A, 2.0), onp.inner(a, dtype(2.0)))


@pytest.mark.parametrize("dtype", [F32, F64])
def test_reversals_running_sums_and_pieces_are_bit_exact(dnp, dtype):
    import autograd_amd as ag

    rs = onp.random.RandomState(33)
    a, q, t = (rs.randn(*s).astype(dtype) for s in ((5, 7), (6, 6), (3, 5, 7)))
    A, Q, T = (P(dnp, h) for h in (a, q, t))

    def same(got, want):
        got = got.numpy()
        assert got.shape == want.shape and got.dtype == want.dtype, (got.shape, want.shape, got.dtype, want.dtype)
        assert onp.array_equal(got, want)

    # slices that step backwards: one gather per reversed axis on top of the forward-stepping view
    for idx in ((slice(None, None, -1),), (slice(None), slice(None, None, -2)), (slice(3, 0, -1), slice(None, None, -1)),
                (Ellipsis, slice(None, None, -1)), (1, None, slice(None, None, -1)), (slice(-2, None, -1),),
                (slice(0, 3, -1),), (slice(None, None, -3), 2), (slice(10, -10, -1), slice(5, 1, -2))):
        same(T[idx], t[idx])
        same(A[idx[:2]] if Ellipsis not in idx and None not in idx else A[idx], a[idx[:2]] if Ellipsis not in idx and None not in idx else a[idx])
    w = rs.randn(3, 5, 7).astype(dtype)
    got = ag.grad(lambda x: dnp.sum(x[::-1, 1:4, ::-2] * P(dnp, w[:, 1:4, ::2])))(T).numpy()
    want = onp.zeros_like(t)
    want[::-1, 1:4, ::-2] = w[:, 1:4, ::2]
    assert onp.array_equal(got, want)
    same(dnp.flipud(A), onp.flipud(a))
    same(dnp.fliplr(T), onp.fliplr(t))
    same(dnp.flip(T), onp.flip(t))
    same(dnp.flip(T, (0, 2)), onp.flip(t, (0, 2)))
    same(dnp.flip(A.T, 1), onp.flip(a.T, 1))
    for k in range(-3, 5):
        same(dnp.rot90(A, k), onp.rot90(a, k))
        same(dnp.rot90(T, k, axes=(2, 0)), onp.rot90(t, k, axes=(2, 0)))
    # running sums: every layout path of both kernels, ragged against the 64-wide tiles
    for shape, axis in (((1000,), 0), ((130, 4100), 1), ((130, 4100), 0), ((7, 300, 65), 1), ((7, 300, 65), 2),
                        ((7, 300, 65), None), ((5, 7), -1), ((1, 1), 0), ((64, 64), 1), ((65, 129), -1), ((3, 0, 4), 1)):
        x = rs.randn(*shape).astype(dtype)
        if x.size:
            x.flat[0] = -0.0
        same(dnp.cumsum(P(dnp, x), axis=axis), onp.cumsum(x, axis=axis))
    same(dnp.cumsum(Q.T, axis=1), onp.cumsum(q.T, axis=1))  # a transposed view: summed in its memory order
    big = (rs.randn(300, 5000) * 1e3).astype(dtype)
    same(dnp.cumsum(P(dnp, big), axis=1), onp.cumsum(big, axis=1))
    # pieces are views of the operand
    for fn, args in (("split", (2, 0)), ("split", ([1, 4], 1)), ("array_split", (4, 1)), ("array_split", ([2, 2, 9], 1)),
                     ("vsplit", (3,)), ("hsplit", ([1, 2],)), ("split", ([-2], 1))):
        got, want = getattr(dnp, fn)(Q, *args), getattr(onp, fn)(q, *args)
        assert len(got) == len(want)
        for g_, w_ in zip(got, want):
            same(g_, w_)
    for g_, w_ in zip(dnp.dsplit(T, [3]), onp.dsplit(t, [3])):
        same(g_, w_)
    with pytest.raises(ValueError):
        dnp.split(A, 2, axis=1)
    for n_, axis in ((1, -1), (2, 0), (3, 1), (0, 0), (7, 1)):
        same(dnp.diff(A, n_, axis), onp.diff(a, n_, axis))
    for axis, start in ((2, 0), (0, 3), (1, 1), (-1, 1), (0, -1)):
        same(dnp.rollaxis(T, axis, start), onp.rollaxis(t, axis, start))
    u, v = rs.randn(4, 3).astype(dtype), rs.randn(4, 3).astype(dtype)
    same(dnp.cross(P(dnp, u), P(dnp, v)), onp.cross(u, v))
    same(dnp.cross(P(dnp, u.T), P(dnp, v[0]), axisa=0), onp.cross(u.T, v[0], axisa=0))
    same(dnp.cross(P(dnp, u.T), P(dnp, v.T), axis=0), onp.cross(u.T, v.T, axis=0))
    z = a.copy()
    z[0, 0] = 0.0
    close(dnp.sinc(P(dnp, z)).numpy(), onp.sinc(z), RT_EW[dtype] * 8)
    assert dnp.sinc(P(dnp, z)).numpy()[0, 0] == 1.0
    b = rs.randn(5, 7).astype(dtype)
    b[0, :3] = a[0, :3]
    a2 = a.copy()
    a2[1, :3], b[1, :3] = [onp.inf, -onp.inf, onp.nan], [onp.inf, 1.0, 1.0]
    with onp.errstate(all="ignore"):
        for x in (a2, a2 * 50):
            got, want = dnp.logaddexp2(P(dnp, x), P(dnp, b)).numpy(), onp.logaddexp2(x, b)
            special = ~onp.isfinite(want)
            assert onp.array_equal(got[special], want[special], equal_nan=True)
            close(got[~special], want[~special], RT_EW[dtype] * 8)


def test_identity_matrices_are_made_on_the_device(dnp):
    for args in ((3,), (3, 5), (4, 2, 1), (4, 4, -2), (2, 3, 5), (1, 1), (5, 3, -1)):
        got = dnp.eye(*args).numpy()
        assert got.dtype == onp.float64 and onp.array_equal(got, onp.eye(*args)), args
    assert onp.array_equal(dnp.eye(4, 6, 1, dtype=F32).numpy(), onp.eye(4, 6, 1, dtype=F32))
    assert dnp.eye(3, dtype=F32).numpy().dtype == F32


@pytest.mark.parametrize("dtype", [F32, F64])
def test_sort_is_stable_and_puts_nans_last(dnp, dtype):
    import autograd_amd as ag

    rs = onp.random.RandomState(51)
    for n in (1, 2, 7, 255, 256, 257, 1000, 5003):
        x = rs.randn(n).astype(dtype)
        if n > 6:
            x[rs.randint(0, n, n // 5)] = x[0]          # ties
            x[rs.randint(0, n, 3)] = onp.nan            # NaNs sort last, in their original order
            x[rs.randint(0, n, 2)] = onp.inf
            x[rs.randint(0, n, 2)] = -onp.inf
        want_order = onp.argsort(x, kind="stable")
        assert onp.array_equal(dnp.sort(P(dnp, x)).numpy(), x[want_order], equal_nan=True)
        order = dnp.argsort(P(dnp, x)).numpy()
        assert order.dtype == onp.int64 and onp.array_equal(order, want_order)
        part = dnp.partition(P(dnp, x), n // 2).numpy()
        assert onp.array_equal(part, onp.sort(x), equal_nan=True)
    a = rs.randn(5, 33, 7).astype(dtype)
    for axis in (0, 1, 2, -1, None):
        got = dnp.sort(P(dnp, a), axis=axis).numpy()
        assert got.dtype == dtype and onp.array_equal(got, onp.sort(a, axis=axis))
        if axis is not None:
            assert onp.array_equal(dnp.argsort(P(dnp, a), axis=axis).numpy(), onp.argsort(a, axis=axis, kind="stable"))
    assert onp.array_equal(dnp.sort(P(dnp, a).T[::2], axis=1).numpy(), onp.sort(a.T[::2], axis=1))
    assert dnp.sort(P(dnp, onp.zeros((0, 4), dtype))).shape == (0, 4)
    with pytest.raises(NotImplementedError):
        dnp.sort(P(dnp, onp.zeros(70000, dtype)))
    # cotangents go back to where the sorted elements came from; second order exists
    x = rs.randn(300).astype(dtype)
    w = rs.randn(300).astype(dtype)
    g = ag.grad(lambda v: dnp.sum(dnp.sort(v) * P(dnp, w)))(P(dnp, x)).numpy()
    want = onp.empty_like(x)
    want[onp.argsort(x, kind="stable")] = w
    assert onp.array_equal(g, want)
    # along an axis of a stack too (the reference's rule raises there): every cotangent of ones comes back as ones
    assert onp.array_equal(ag.grad(lambda v: dnp.sum(dnp.sort(v, axis=0)))(P(dnp, a)).numpy(), onp.ones_like(a))
    h = ag.grad(lambda v: dnp.sum(ag.grad(lambda u: dnp.sum(dnp.sort(u * u) * P(dnp, w)))(v) * P(dnp, w)))(P(dnp, x)).numpy()
    want2 = onp.empty_like(x)
    want2[onp.argsort(x * x, kind="stable")] = w
    close(h, (dtype(2.0) * want2 * w).astype(dtype), RT_EW[dtype] * 4)


def test_real_array_trivia_and_data_dependent_shapes(dnp):
    """The last names of the reference's rule table (numpy_vjps.py:13-68, 220-224): what is trivial for real
    arrays (imag, angle, isreal, iscomplex), floor_divide, array_equiv, and the functions whose result shape
    depends on the data (answered by NumPy on the host, indices uploaded)."""
    import autograd_amd as ag

    rs = onp.random.RandomState(62)
    x = rs.randn(4, 5)
    y = rs.uniform(0.3, 2.0, (4, 5)) * rs.choice([-1, 1], (4, 5))
    X, Y = dnp.asarray(x), dnp.asarray(y)
    assert onp.array_equal(dnp.imag(X).numpy(), onp.imag(x)) and onp.array_equal(dnp.angle(X).numpy(), onp.angle(x))
    assert onp.array_equal(dnp.isreal(X).numpy(), onp.isreal(x)) and onp.array_equal(dnp.iscomplex(X).numpy(), onp.iscomplex(x))
    assert onp.array_equal(dnp.floor_divide(X * 7, Y).numpy(), onp.floor_divide(x * 7, y))
    assert onp.array_equal(dnp.floor_divide(X * 7, 0.7).numpy(), onp.floor_divide(x * 7, 0.7))
    with onp.errstate(all="ignore"):
        z = y.copy()
        z[0, 0] = z[1, 1] = 0.0
        assert onp.array_equal(dnp.floor_divide(X, dnp.asarray(z)).numpy(), onp.floor_divide(x, z), equal_nan=True)
    assert dnp.array_equiv(X, X[:1] * 0 + X) and not dnp.array_equiv(X, Y)
    assert dnp.array_equiv(dnp.asarray(onp.ones((3, 1))), dnp.asarray(onp.ones((1, 4)))) and not dnp.array_equiv(X, X[:, :3])
    m = x > 0.3
    assert all(onp.array_equal(a.numpy(), b) for a, b in zip(dnp.nonzero(X > 0.3), onp.nonzero(m)))
    assert onp.array_equal(dnp.flatnonzero(X > 0.3).numpy(), onp.flatnonzero(m))
    assert onp.array_equal(dnp.argwhere(X > 0.3).numpy(), onp.argwhere(m))
    v = onp.sort(rs.randn(9))
    assert onp.array_equal(dnp.searchsorted(dnp.asarray(v), X).numpy(), onp.searchsorted(v, x))
    assert onp.array_equal(X[dnp.nonzero(X > 0.3)].numpy(), x[onp.nonzero(m)])
    g = ag.grad(lambda a: dnp.sum(dnp.imag(a) + dnp.angle(a) * 3.0 + a))(X)
    assert onp.array_equal(g.numpy(), onp.ones_like(x))
    t = ag.make_jvp(lambda a: dnp.angle(a) + dnp.imag(a) + 2.0 * a)(X)(dnp.asarray(onp.ones_like(x)))[1]
    assert onp.array_equal(t.numpy(), 2 * onp.ones_like(x))
    g = ag.grad(lambda a: dnp.sum(a[dnp.nonzero(a > 0.3)] ** 2))(X)
    assert onp.array_equal(g.numpy(), onp.where(m, 2 * x, 0.0))


def test_truth_tests_and_closeness(dnp):
    rs = onp.random.RandomState(61)
    a = rs.randn(6, 9)
    a[a < -0.5] = 0.0
    A = P(dnp, a)
    for axis in (None, 0, 1, (0, 1)):
        for keepdims in (False, True):
            for mine, ref in ((dnp.all, onp.all), (dnp.any, onp.any), (dnp.count_nonzero, onp.count_nonzero)):
                got, want = mine(A, axis=axis, keepdims=keepdims).numpy(), onp.asarray(ref(a, axis=axis, keepdims=keepdims))
                assert got.dtype == want.dtype and got.shape == want.shape and onp.array_equal(got, want), (ref.__name__, axis)
    assert bool(dnp.all(A * 0.0 + 1.0)) and not bool(dnp.any(A * 0.0)) and bool(dnp.any(A > 1.0))
    x = onp.array([1.0, 1.0 + 1e-9, 1.1, onp.inf, onp.inf, -onp.inf, onp.nan, onp.nan, 0.0, 1e-9])
    y = onp.array([1.0, 1.0, 1.0, onp.inf, -onp.inf, -onp.inf, onp.nan, 1.0, 1e-9, 0.0])
    for kw in ({}, {"equal_nan": True}, {"rtol": 0.2}, {"atol": 0.0, "rtol": 0.0}):
        assert onp.array_equal(dnp.isclose(P(dnp, x), P(dnp, y), **kw).numpy(), onp.isclose(x, y, **kw)), kw
    assert onp.array_equal(dnp.isclose(P(dnp, x.astype(F32)), 1.0).numpy(), onp.isclose(x.astype(F32), 1.0))
    assert dnp.array_equal(A, P(dnp, a.copy())) and not dnp.array_equal(A, A + 1.0) and not dnp.array_equal(A, A[:, :3])
    assert not dnp.array_equal(P(dnp, x), P(dnp, x)) and dnp.array_equal(P(dnp, x), P(dnp, x), equal_nan=True)
    assert onp.array_equal(dnp.isposinf(P(dnp, x)).numpy(), onp.isposinf(x))
    assert onp.array_equal(dnp.isneginf(P(dnp, x)).numpy(), onp.isneginf(x))
    f = dnp.full_like(A, 2.5)
    assert f.shape == (6, 9) and f.dtype == onp.float64 and onp.all(f.numpy() == 2.5)
    assert dnp.full_like(P(dnp, a.astype(F32)), 1.5).numpy().dtype == F32 and dnp.empty_like(A).shape == (6, 9)


@pytest.mark.parametrize("dtype", [F32, F64])
def test_reversal_and_triangle_vector_paths(dnp, dtype):
    """Extents that are multiples of the 16-byte vector length take the vector kernels; offset views whose start is not
    16-byte aligned fall back to the element kernels.  All are copies: bit-exact."""
    rs = onp.random.RandomState(71)
    for shape in ((8, 12), (4, 6, 8), (16, 4), (3, 8, 4), (2, 2, 2, 8), (260, 516)):
        a = rs.randn(*shape).astype(dtype)
        a.flat[::7] = onp.nan
        A = P(dnp, a)
        for axis in range(len(shape)):
            assert onp.array_equal(dnp.flip(A, axis).numpy(), onp.flip(a, axis), equal_nan=True), (shape, axis)
        assert onp.array_equal(dnp.flip(A).numpy(), onp.flip(a), equal_nan=True)
        assert onp.array_equal(dnp.flip(A[1:], 0).numpy(), onp.flip(a[1:], 0), equal_nan=True)       # offset start
        assert onp.array_equal(dnp.flip(A[..., 1:], -1).numpy(), onp.flip(a[..., 1:], -1), equal_nan=True)
        for k in (-3, -1, 0, 1, 2, 5):
            assert onp.array_equal(dnp.tril(A, k).numpy(), onp.where(onp.tri(*shape[-2:], k, dtype=bool), a, 0),
                                   equal_nan=True), (shape, k)
            assert onp.array_equal(dnp.triu(A, k).numpy(), onp.where(~onp.tri(*shape[-2:], k - 1, dtype=bool), a, 0),
                                   equal_nan=True), (shape, k)
            assert onp.array_equal(dnp.tril(A[1:], k).numpy(), onp.where(onp.tri(*a[1:].shape[-2:], k, dtype=bool), a[1:], 0),
                                   equal_nan=True)


# ---- logsumexp cotangent with its consumers fused (agmi_lse_cotangent_fused) ---------------------------
def _lse_cotangent_reference(mem, scale, svec, shift, hvec, g):
    x = mem.astype(F64)
    if scale is not None:
        x = x * scale
    if svec is not None:
        x = x * svec
    if shift is not None:
        x = x + shift
    if hvec is not None:
        x = x + hvec
    ans = scipy.special.logsumexp(x, axis=1, keepdims=True)
    return ans, g * onp.exp(x - ans)


def test_the_probe_times_the_first_kernel_of_a_call_that_launches_two(dnp):
    """``agmi_probe_arm``: the logsumexp-cotangent entry point launches its tile kernel and then a kernel that adds up
    partial sums; events around the call bracket both, the library's own pair the first alone."""
    import ctypes

    import autograd_amd as ag
    from autograd_amd import _lib
    from autograd_amd.scipy.special import logsumexp

    L = _lib.lib()
    rs = onp.random.RandomState(2)
    A, b, c = (P(dnp, rs.randn(*shape).astype(F32)) for shape in ((2048, 4096), (4096,), (2048,)))
    g = ag.grad(lambda A, b, c: dnp.sum(logsumexp(A * b[None, :] + c[:, None], axis=1)), (0, 1, 2))
    g(A, b, c)
    with _lib.KernelTimer() as kt:
        for _ in range(3):
            g(A, b, c)
    rows = {k: v for k, v in kt.summary().items() if k.startswith("lse_cotangent_tile")}
    assert len(rows) == 1
    (row,) = rows.values()
    assert row["launches"] == 3 and 0.0 < row["avg_ms"] < row["avg_call_ms"]   # the tile kernel alone < tile + finish
    took = ctypes.c_float()
    never = L.agmi_probe_arm()                              # armed, but nothing runs before it is read
    assert L.agmi_probe_elapsed(never, ctypes.byref(took)) == -1 and b"never filled" in L.agmi_last_error()
    g(A, b, c)                                               # (fills the pair that is still armed)
    assert L.agmi_probe_elapsed(never, ctypes.byref(took)) == 0 and took.value > 0.0
    assert L.agmi_probe_elapsed(-5, ctypes.byref(took)) == -1


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("rows,cols", [(37, 8), (300, 64), (129, 1028), (1000, 4096), (64, 2), (1, 4), (15, 1024), (16, 1020),
                                       (17, 2052), (50, 9000)])
def test_lse_cotangent_fused_entry_point(dnp, dtype, rows, cols):
    import torch

    from autograd_amd import _lib

    if cols % (16 // onp.dtype(dtype).itemsize):
        pytest.skip("not a whole number of 16-byte vectors")
    rs = onp.random.RandomState(rows + cols)
    dev = _lib.device()
    code = _lib.DTYPE_CODE[onp.dtype(dtype)]
    mem = rs.randn(rows, cols).astype(dtype)
    by_col = rs.uniform(0.5, 1.5, (1, cols)).astype(dtype)
    by_row = rs.randn(rows, 1).astype(dtype)
    put = lambda a: torch.from_numpy(onp.ascontiguousarray(a)).to(dev)
    t_mem, t_col, t_row = put(mem), put(by_col), put(by_row)
    g_rows = rs.randn(rows, 1).astype(dtype)
    layouts = [
        ("plain", t_mem, (None, None, None, None)),
        ("A*b+c", _lib.Affine(t_mem, 1.0, t_row.expand(rows, cols), t_col.expand(rows, cols)), (None, by_col, None, by_row)),
        ("2A*c+b", _lib.Affine(t_mem, 2.0, t_col.expand(rows, cols), t_row.expand(rows, cols)), (2.0, by_row, None, by_col)),
        ("-A+0.5", _lib.Affine(t_mem, -1.0, 0.5, None), (-1.0, None, 0.5, None)),
    ]
    for name, operand, (scale, svec, shift, hvec) in layouts:
        for g in (g_rows, onp.full((1, 1), 0.75, dtype)):
            ans, S = _lse_cotangent_reference(mem, scale, svec, shift, hvec, g.astype(F64))
            t_ans = put(ans.astype(dtype))
            t_g = put(g).expand(rows, 1)
            for want in range(1, 8):
                row_sums = torch.full((rows, 1), float("nan"), dtype=t_mem.dtype, device=dev) if want & 2 else None
                scaled = torch.full((rows, cols), float("nan"), dtype=t_mem.dtype, device=dev) if want & 1 else None
                col_sums = torch.full((1, cols), float("nan"), dtype=t_mem.dtype, device=dev) if want & 4 else None
                assert _lib.lse_cotangent(code, operand, t_ans, t_g, row_sums=row_sums,
                                          col_factor=t_col.reshape(cols) if want & 1 else None, scaled=scaled, col_sums=col_sums)
                label = f"{name} want={want}"
                if want & 1:
                    close(scaled.cpu().numpy(), (by_col * S).astype(dtype), RT[dtype])
                if want & 2:
                    close(row_sums.cpu().numpy(), onp.sum(S, axis=1, keepdims=True).astype(dtype), RT[dtype])
                if want & 4:
                    close(col_sums.cpu().numpy(), onp.sum(mem.astype(F64) * S, axis=0, keepdims=True).astype(dtype), RT[dtype]), label


def test_lse_cotangent_tiles_grow_with_a_small_workspace(dnp):
    """Partial column sums take one row per band of 16 rows; when the workspace cannot hold that many the bands get
    taller (32, 48, 64 rows), and when even 64 do not fit the call reports the layout as unsupported."""
    import torch

    from autograd_amd import _lib

    rs = onp.random.RandomState(5)
    rows, cols = 200, 1028
    dev = _lib.device()
    code = _lib.DTYPE_CODE[onp.dtype(F32)]
    mem = rs.randn(rows, cols).astype(F32)
    by_col = rs.uniform(0.5, 1.5, (1, cols)).astype(F32)
    g = rs.randn(rows, 1).astype(F32)
    ans, S = _lse_cotangent_reference(mem, None, None, None, None, g.astype(F64))
    put = lambda a: torch.from_numpy(onp.ascontiguousarray(a)).to(dev)
    t_mem, t_col, t_ans, t_g = put(mem), put(by_col), put(ans.astype(F32)), put(g)
    real = _lib._WORKSPACE_BYTES
    try:
        for limit in (real, 40 << 10, 26 << 10, 20 << 10):  # bands of 16, 32, 48 and 64 rows
            _lib._WORKSPACE_BYTES = limit
            row_sums = torch.full((rows, 1), float("nan"), device=dev)
            scaled = torch.full((rows, cols), float("nan"), device=dev)
            col_sums = torch.full((1, cols), float("nan"), device=dev)
            assert _lib.lse_cotangent(code, t_mem, t_ans, t_g, row_sums=row_sums, col_factor=t_col.reshape(cols), scaled=scaled,
                                      col_sums=col_sums), limit
            close(scaled.cpu().numpy(), (by_col * S).astype(F32), RT[F32])
            close(row_sums.cpu().numpy(), onp.sum(S, axis=1, keepdims=True).astype(F32), RT[F32])
            close(col_sums.cpu().numpy(), onp.sum(mem.astype(F64) * S, axis=0, keepdims=True).astype(F32), RT[F32])
        _lib._WORKSPACE_BYTES = 8 << 10
        assert not _lib.lse_cotangent(code, t_mem, t_ans, t_g, row_sums=torch.zeros((rows, 1), device=dev),
                                      col_sums=torch.zeros((1, cols), device=dev))
    finally:
        _lib._WORKSPACE_BYTES = real


def test_lse_cotangent_layouts_outside_the_kernel_are_reported(dnp):
    import torch

    from autograd_amd import _lib

    dev = _lib.device()
    code = _lib.DTYPE_CODE[onp.dtype(F32)]
    ans, g = torch.zeros((6, 1), device=dev), torch.ones((6, 1), device=dev)
    out = torch.zeros((6, 1), device=dev)
    assert not _lib.lse_cotangent(code, torch.zeros((6, 10), device=dev), ans, g, row_sums=out)        # 10 % 4 != 0
    assert not _lib.lse_cotangent(code, torch.zeros((16, 6), device=dev).t(), ans, g, row_sums=out)    # column stride != 1
    diag = _lib.Affine(torch.zeros((6, 8), device=dev), 1.0, None, torch.zeros((6, 8), device=dev))    # factor varies both ways
    assert not _lib.lse_cotangent(code, diag, ans, g, row_sums=out)


@pytest.mark.parametrize("dtype", [F32, F64])
def test_deferred_logsumexp_cotangent_serves_any_subset_of_consumers(dnp, dtype):
    """The rules after a row-wise logsumexp ask its cotangent for row sums, a rescaled copy and column sums of a
    product; whichever subset a program needs, values and dtypes must be what the stored-cotangent path gives."""
    import autograd_amd as ag
    import oracle.anp as anp
    from autograd_amd.numpy import devarray as D
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(5)
    rows, cols = 260, 72
    A = rs.randn(rows, cols).astype(dtype)
    b = rs.uniform(0.5, 1.5, cols).astype(dtype)
    c = rs.randn(rows).astype(dtype)
    w = rs.randn(rows).astype(dtype)

    def programs(np_, lse):
        return {
            "A*b+c": (lambda A, b, c: np_.sum(lse(A * b[None, :] + c[:, None], axis=1) * w), (0, 1, 2)),
            "A*b+c wrt b": (lambda A, b, c: np_.sum(lse(A * b[None, :] + c[:, None], axis=1)), (1,)),
            "A*b+c wrt c,A": (lambda A, b, c: np_.sum(lse(A * b[None, :] + c[:, None], axis=1)), (2, 0)),
            "A+c": (lambda A, b, c: np_.sum(lse(A + c[:, None], axis=1, keepdims=True)), (0, 2)),
            "A*b": (lambda A, b, c: np_.sum(lse(A * b, axis=-1)), (0, 1)),
            "plain": (lambda A, b, c: np_.sum(lse(A, axis=1) * w), (0,)),
            "twice": (lambda A, b, c: np_.sum(lse(A * b[None, :] + c[:, None], axis=1)) + np_.sum(lse(A * b[None, :], axis=1) ** 2), (0, 1, 2)),
            "axis0": (lambda A, b, c: np_.sum(lse(A * b[None, :] + c[:, None], axis=0)), (0, 1, 2)),
            "used twice": (lambda A, b, c: np_.sum(np_.exp(lse(A * b[None, :], axis=1)[:, None] - A * b[None, :])), (0, 1)),
        }

    dev_args = (dnp.asarray(A), dnp.asarray(b), dnp.asarray(c))
    w_host = w
    for name in programs(anp, anp.logsumexp):
        w = w_host
        f_ref, argnums = programs(anp, anp.logsumexp)[name]
        want = ag.grad(f_ref, argnums)(A, b, c)
        w = dnp.asarray(w_host)
        f_dev, _ = programs(dnp, logsumexp)[name]
        got = ag.grad(f_dev, argnums)(*dev_args)
        for gd, wr in zip(got, want):
            assert type(gd) is D.DevArray, (name, type(gd))  # settled: no pending object leaves grad
            close(gd.numpy(), wr, RT[dtype])


def test_deferred_logsumexp_cotangent_survives_accumulation_and_second_order(dnp):
    import autograd_amd as ag
    import oracle.anp as anp
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(9)
    A = rs.randn(48, 16)
    b = rs.uniform(0.5, 1.5, 16)

    def make(np_, lse):
        # b reaches the loss twice (fan-in on its cotangent), and the outer derivative traces the inner backward pass
        f = lambda A, b: np_.sum(lse(A * b[None, :], axis=1)) + np_.sum(b * b)
        return ag.grad(lambda A, b: np_.sum(ag.grad(f, 1)(A, b) ** 2), (0, 1))

    want = make(anp, anp.logsumexp)(A, b)
    got = make(dnp, logsumexp)(dnp.asarray(A), dnp.asarray(b))
    for gd, wr in zip(got, want):
        close(gd.numpy(), wr, 1e-10)


# ---- every NumPy index form: one gather forward, the ordered scatter backward --------------------------
def _index_forms(rs):
    return [
        [0, 1, 2], ([0, 1, 2], slice(None), slice(None)), (3, slice(2, None), [1, 3]),       # tests/test_numpy.py:304-321
        (slice(None), [0, 5, 0]), (slice(None, None, -1), [1, 1], slice(1, 3)), ([[0, 1], [2, 3]], [[1], [2]]),
        (Ellipsis, [3, 0, 3]), (None, [4, 0], None, 2), ([0, 4, 0], slice(None), [1, 2, 1]), (onp.array([4, -1, 0, -1]),),
        rs.rand(5, 6, 4) > 0.5, (onp.array([True, False, True, False, True]),), (slice(1, 4), rs.rand(6, 4) > 0.3),
        (onp.array([1, 2, 0]), onp.array([True] * 3 + [False] * 3)), onp.zeros((0, 2), dtype=onp.int64),
    ]


@pytest.mark.parametrize("dtype", [F32, F64])
def test_advanced_indexing_matches_numpy_bit_for_bit(dnp, dtype):
    import autograd_amd as ag
    from autograd_amd.numpy import wrapper as W

    rs = onp.random.RandomState(21)
    x = rs.randn(5, 6, 4).astype(dtype)
    dx = dnp.asarray(x)
    for idx in _index_forms(rs):
        want = x[idx]
        got = dx[idx].numpy()
        assert got.shape == want.shape and onp.array_equal(got, want), idx
        # cotangent: numpy.add.at order, duplicates included (numpy_vjps.py:941-950)
        w = (rs.randn(*want.shape) * onp.exp(3 * rs.randn(*want.shape))).astype(dtype)
        dst = onp.zeros_like(x)
        onp.add.at(dst, idx, w)
        g = ag.grad(lambda a: dnp.sum(a[idx] * dnp.asarray(w)))(dx).numpy()
        assert g.dtype == dst.dtype and onp.array_equal(g, dst), idx
        # accumulation into an array that already holds values
        base = rs.randn(*x.shape).astype(dtype)
        ref = base.copy()
        onp.add.at(ref, idx, w)
        assert onp.array_equal(W.scatter_add(dnp.asarray(base) + 0.0, idx, dnp.asarray(w)).numpy(), ref), idx
    v = rs.randn(3).astype(dtype)
    for idx in ([0, 0], [0, 1, 0]):                                                        # tests/test_numpy.py:881-890
        g = ag.grad(lambda a: dnp.sum(a[idx]))(dnp.asarray(v)).numpy()
        dst = onp.zeros_like(v)
        onp.add.at(dst, idx, 1.0)
        assert onp.array_equal(g, dst)
    with pytest.raises(IndexError):
        dx[[5]]
    with pytest.raises(IndexError):
        dx[onp.array([True, False])]


def test_boolean_masks_select_elements_like_numpy(dnp):
    import autograd_amd as ag

    rs = onp.random.RandomState(2)
    A = rs.randn(7, 5)
    dA = dnp.asarray(A)
    mask = A > 0.1
    assert onp.array_equal(dA[mask].numpy(), A[mask])                     # N-d mask: the selected elements, 1-d
    assert onp.array_equal(dA[dA > 0.1].numpy(), A[A > 0.1])               # a mask computed on the device
    rows = onp.array([True, False, True, True, False, False, True])
    assert onp.array_equal(dA[rows].numpy(), A[rows])
    g = ag.grad(lambda a: dnp.sum(a[a > 0.1] ** 2))(dA).numpy()
    assert onp.array_equal(g, onp.where(mask, 2 * A, 0.0))
    with pytest.raises(IndexError):
        dA[onp.array([True, False, True])]                                   # wrong length, as NumPy


def test_reference_index_cases_pass_check_grads(dnp):
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(0)
    A = dnp.asarray(rs.randn(5, 6, 4))
    for fun in (lambda x: x[3, 0, 1], lambda x: x[::-1, 2:4, :], lambda x: x[[0, 1, 2], :, :], lambda x: x[3, 2:, [1, 3]],
                lambda x: x[::-1, 2:4, :] + x[::-1, 3:5, :]):
        check_grads(fun)(A)
    v = dnp.asarray(rs.randn(7))
    check_grads(lambda x: x[2:6][1:3])(v)
    check_grads(lambda x: dnp.sum(x[[0, 1, 0]]))(dnp.asarray(rs.randn(3)))


@pytest.mark.parametrize("dtype", [F32, F64])
def test_device_resident_row_index_gathers_and_scatters_in_order(dnp, dtype):
    from autograd_amd.numpy import wrapper as W

    rs = onp.random.RandomState(8)
    A = rs.randn(40, 6).astype(dtype)
    for n in (1, 7, 300, 5000):
        idx = rs.randint(-40, 40, n)
        d_idx = dnp.asarray(idx)                                             # int64 on the device
        assert onp.array_equal(dnp.asarray(A)[d_idx].numpy(), A[idx])
        x = (rs.randn(n, 6) * onp.exp(3 * rs.randn(n, 6))).astype(dtype)
        want = A.copy()
        onp.add.at(want, idx, x)
        assert onp.array_equal(W.scatter_add(dnp.asarray(A) + 0.0, d_idx, dnp.asarray(x)).numpy(), want), n


# ---- dense-layer epilogues of the contraction ------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(64, 64, 32), (200, 130, 70), (256, 512, 641), (1024, 1024, 784), (7, 3, 5), (70, 45, 300),
                                   (256, 512, 128), (90, 33, 150)])
def test_gemm_epilogues_equal_the_separate_kernels(dnp, M, N, K):
    """``agmi_gemm_fused``: tanh(A.B + bias) and (G.W^T) / cosh(x + bias)**2 formed inside the contraction are, bit for
    bit, what the product followed by the elementwise kernels gives (examples/neural_net.py:33-35,
    autograd/numpy/numpy_vjps.py:178)."""
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(M + N + K)
    A = P(dnp, rs.randn(M, K).astype(F32))
    B = P(dnp, (0.1 * rs.randn(K, N)).astype(F32))
    bias = P(dnp, rs.randn(N).astype(F32))
    x = P(dnp, rs.randn(M, N).astype(F32))
    code = _lib.DTYPE_CODE[onp.dtype(F32)]
    for operands in ((A._t, B._t), (P(dnp, rs.randn(K, M).astype(F32))._t.t(), B._t), (A._t, P(dnp, rs.randn(N, K).astype(F32))._t.t())):
        a, b = operands
        plain = DevArray_from(D.gemm2d(a, b, onp.dtype(F32)))
        for with_bias in (True, False):
            vec = bias._t if with_bias else None
            z = D.map_op(Op.ADD, onp.dtype(F32), plain, bias) if with_bias else plain
            want_act = D.plain(D.map_op(Op.TANH, onp.dtype(F32), z)).numpy()
            C = _lib.empty((M, N), onp.dtype(F32))
            act = _lib.empty((M, N), onp.dtype(F32))
            assert _lib.gemm_fused(code, a, b, C, _lib.EPILOGUE_BIAS_TANH, bias=vec, out=act)
            assert onp.array_equal(C.cpu().numpy(), plain.numpy())
            assert onp.array_equal(act.cpu().numpy(), want_act)
            zx = D.map_op(Op.ADD, onp.dtype(F32), x, bias) if with_bias else x
            want_vjp = D.plain(D.map_op(Op.TANH_VJP, onp.dtype(F32), plain, zx)).numpy()
            out = _lib.empty((M, N), onp.dtype(F32))
            assert _lib.gemm_fused(code, a, b, out, _lib.EPILOGUE_TANH_VJP, bias=vec, x=x._t)
            assert onp.array_equal(out.cpu().numpy(), want_vjp)
            # beta = 1: the product joins what the output holds (an earlier product) before the rule is applied
            first = rs.randn(M, N).astype(F32)
            summed = DevArray_from(D.gemm2d(a, b, onp.dtype(F32), out=P(dnp, first)._t.clone(), beta=1.0))
            want_sum = D.plain(D.map_op(Op.TANH_VJP, onp.dtype(F32), summed, zx)).numpy()
            out = P(dnp, first)._t.clone()
            assert _lib.gemm_fused(code, a, b, out, _lib.EPILOGUE_TANH_VJP, bias=vec, x=x._t, beta=1.0)
            assert onp.array_equal(out.cpu().numpy(), want_sum)


@pytest.mark.parametrize("M,N,K1,K2,layout", [(256, 512, 512, 128, "kk"), (256, 512, 641, 128, "kx"), (64, 96, 130, 257, "xk"),
                                             (33, 70, 128, 4000, "xx"), (256, 512, 128, 128, "kk")])
def test_two_products_under_one_tanh_rule_in_one_launch_equal_the_two_launches(dnp, M, N, K1, K2, layout):
    """``agmi_gemm_fused`` with a second product: ``(A1.B1 + A2.B2) / cosh(x + bias)**2`` from ONE launch is, bit for bit,
    ``A1.B1`` written out followed by ``A2.B2`` added to it (beta = 1) under the rule (the cotangent of a recurrent net's
    state, examples/rnn.py:37-50: two ``G . W^T`` products, core.py:185-205, then numpy_vjps.py:178); pairs the kernel
    does not take are refused and nothing runs."""
    from autograd_amd import _lib

    rs = onp.random.RandomState(M + K1 + K2)
    f32 = onp.dtype(F32)
    code = _lib.DTYPE_CODE[f32]

    def operand(rows, cols, contiguous_k_is_cols):
        if contiguous_k_is_cols:
            return P(dnp, rs.randn(rows, cols).astype(F32))._t
        return P(dnp, rs.randn(cols, rows).astype(F32))._t.t()

    ka, kb = layout[0] == "k", layout[1] == "k"
    A1, A2 = operand(M, K1, ka), operand(M, K2, ka)          # K along the columns of A: contiguous when `ka`
    B1, B2 = operand(K1, N, not kb), operand(K2, N, not kb)  # K along the rows of B: contiguous when `kb`
    x = P(dnp, rs.randn(M, N).astype(F32))._t
    bias = P(dnp, rs.randn(N).astype(F32))._t
    one = _lib.empty((M, N), f32)
    assert _lib.gemm_fused(code, A1, B1, one, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x, second=(A2, B2))
    two = _lib.empty((M, N), f32)
    _lib.gemm(code, 1, M, N, K1, 1.0, A1, A1.stride(0), A1.stride(1), 0, B1, B1.stride(0), B1.stride(1), 0, 0.0, two, N, 0)
    assert _lib.gemm_fused(code, A2, B2, two, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x, beta=1.0)
    assert onp.array_equal(one.cpu().numpy(), two.cpu().numpy())
    want = (A1.cpu().numpy().astype(F64) @ B1.cpu().numpy() + A2.cpu().numpy().astype(F64) @ B2.cpu().numpy()) \
        / onp.cosh(x.cpu().numpy().astype(F64) + bias.cpu().numpy()) ** 2
    close(one.cpu().numpy(), want.astype(F32), RT[F32] * max(1.0, onp.sqrt(K1 + K2) / 8))
    # refused: a product too short to be cut, operands that differ in which one is contiguous along k, a large output
    short = operand(M, 64, ka)
    assert not _lib.gemm_fused(code, A1, B1, one, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x, second=(short, operand(64, N, not kb)))
    assert not _lib.gemm_fused(code, A1, B1, one, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x, second=(operand(M, K2, not ka), B2))
    big = P(dnp, rs.randn(1024, 256).astype(F32))._t
    assert not _lib.gemm_fused(code, big, P(dnp, rs.randn(256, 1024).astype(F32))._t, _lib.empty((1024, 1024), f32),
                               _lib.EPILOGUE_TANH_VJP, x=P(dnp, rs.randn(1024, 1024).astype(F32))._t, second=(big, P(dnp, rs.randn(256, 1024).astype(F32))._t))


def test_an_independent_product_rides_in_a_dense_layers_launch(dnp):
    """``agmi_gemm_fused`` with an accompanying problem: the tiles of a second, independent product are computed by
    further blocks of a dense layer's launch, each result bit for bit that of its own launch (the output head of a
    recurrent net's previous step beside this step's recurrence, examples/rnn.py:37-50); and the host side: a forward
    product left pending is taken along by the next dense layer, once, and read back as computed."""
    from autograd_amd import _lib
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(41)
    f32 = onp.dtype(F32)
    code = _lib.DTYPE_CODE[f32]
    for (M, N, K), (M2, N2, K2) in (((256, 512, 641), (256, 128, 513)), ((64, 96, 300), (200, 33, 130)), ((33, 40, 128), (70, 257, 4000))):
        A, B = P(dnp, rs.randn(M, K).astype(F32))._t, P(dnp, (0.1 * rs.randn(K, N)).astype(F32))._t
        A2, B2 = P(dnp, rs.randn(M2, K2).astype(F32))._t, P(dnp, (0.1 * rs.randn(K2, N2)).astype(F32))._t
        bias = P(dnp, rs.randn(N).astype(F32))._t
        c1, t1, c2 = _lib.empty((M, N), f32), _lib.empty((M, N), f32), _lib.empty((M2, N2), f32)
        assert _lib.gemm_fused(code, A, B, c1, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=t1, beside=(A2, B2, c2))
        d1, u1, d2 = _lib.empty((M, N), f32), _lib.empty((M, N), f32), _lib.empty((M2, N2), f32)
        assert _lib.gemm_fused(code, A, B, d1, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=u1)
        _lib.gemm(code, 1, M2, N2, K2, 1.0, A2, A2.stride(0), A2.stride(1), 0, B2, B2.stride(0), B2.stride(1), 0, 0.0, d2, N2, 0)
        for got, want in ((c1, d1), (t1, u1), (c2, d2)):
            assert onp.array_equal(got.cpu().numpy(), want.cpu().numpy())
        close(c2.cpu().numpy(), (A2.cpu().numpy().astype(F64) @ B2.cpu().numpy()).astype(F32), RT[F32] * max(1.0, onp.sqrt(K2) / 8))
    # refused (nothing runs): a companion that is not the kernel's (a large output), or contiguous the other way round
    big_a, big_b = P(dnp, rs.randn(1024, 256).astype(F32))._t, P(dnp, rs.randn(256, 1024).astype(F32))._t
    assert not _lib.gemm_fused(code, A, B, c1, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=t1, beside=(big_a, big_b, _lib.empty((1024, 1024), f32)))
    At = P(dnp, rs.randn(K2, M2).astype(F32))._t.t()
    assert not _lib.gemm_fused(code, A, B, c1, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=t1, beside=(At, B2, c2))
    # through the namespace: head = dot(h, Wp) stays pending and is computed by the launch of the next tanh(dot(...))
    H, Wp = P(dnp, rs.randn(256, 513).astype(F32)), P(dnp, (0.1 * rs.randn(513, 128)).astype(F32))
    X, Wc = P(dnp, rs.randn(256, 641).astype(F32)), P(dnp, (0.1 * rs.randn(641, 512)).astype(F32))
    calls = []
    real = _lib.gemm_fused
    _lib.gemm_fused = lambda *a, **k: (calls.append(k.get("beside") is not None), real(*a, **k))[1]
    try:
        del D._FORWARD_PRODUCTS[:]  # (nothing another test left pending takes part)
        head = dnp.dot(H, Wp)
        assert type(head) is D.PendingProduct and not head.computed()
        state = dnp.tanh(dnp.dot(X, Wc)).numpy()
        assert calls == [True] and head.computed()
        got_head = head.numpy()
        again = dnp.tanh(dnp.dot(X, Wc)).numpy()                   # nothing pending now: a launch of its own
        assert calls == [True, False]
    finally:
        _lib.gemm_fused = real
    assert onp.array_equal(again, state)
    assert onp.array_equal(got_head, D.gemm2d(H._t, Wp._t, f32).cpu().numpy())


def test_the_tanh_rule_over_a_sum_of_sliced_products_is_one_chain_of_contractions(dnp):
    """The state of a recurrent net is read by the next step and by the output head (examples/rnn.py:37-50): its cotangent is
    the sum of two `G . W^T` products, of each of which only the state's columns are wanted (the `hstack` rule slices
    them out), and the tanh rule follows.  The slices stay products of the factors' columns, the sum stays a sum of
    products, and the rule runs in the second contraction's epilogue: same bits as product, slice, add and rule one
    by one."""
    import autograd_amd as ag
    from autograd_amd import _lib
    from autograd_amd.numpy import devarray as D
    from autograd_amd.numpy import fusion, wrapper

    rs = onp.random.RandomState(12)
    B_, I, H, O = 64, 24, 96, 20
    Wc, Wp = P(dnp, (0.2 * rs.randn(I + H + 1, H)).astype(F32)), P(dnp, (0.2 * rs.randn(H + 1, O)).astype(F32))
    x0, h0 = P(dnp, rs.randn(B_, I).astype(F32)), P(dnp, rs.randn(B_, H).astype(F32))
    t1, t2 = P(dnp, rs.randn(B_, O).astype(F32)), P(dnp, rs.randn(B_, H).astype(F32))
    ones = dnp.ones((B_, 1), dtype=F32)

    def f(h):
        h1 = dnp.tanh(dnp.dot(dnp.hstack((x0, h, ones)), Wc))
        head = dnp.dot(dnp.hstack((h1, ones)), Wp)
        h2 = dnp.tanh(dnp.dot(dnp.hstack((x0, h1, ones)), Wc))
        return dnp.sum(head * t1) + dnp.sum(h2 * t2)

    names = []
    real_fused, real_gemm = _lib.gemm_fused, _lib.gemm
    _lib.gemm_fused = lambda *a, **k: (names.append(("fused", 1.0 if k.get("second") is not None else k.get("beta", 0.0))),
                                       real_fused(*a, **k))[1]
    _lib.gemm = lambda *a, **k: (names.append(("gemm", a[2:5])), real_gemm(*a, **k))[1]
    try:
        got = ag.grad(f)(h0).numpy()
    finally:
        _lib.gemm_fused, _lib.gemm = real_fused, real_gemm
    assert ("fused", 1.0) in names                                   # the rule of h1 ran on a sum of two products (one launch, or two with beta = 1)
    assert ("gemm", (B_, H, H)) in names and ("gemm", (B_, I + H + 1, H)) not in names   # only the state's columns were contracted
    was, fusion.ENABLED = fusion.ENABLED, False
    try:
        want = ag.grad(f)(h0).numpy()
    finally:
        fusion.ENABLED = was
    assert onp.array_equal(got, want)
    # a slice of less than half of an axis is a view of the whole product
    Pd = D.PendingProduct(x0._t, P(dnp, rs.randn(I, 50).astype(F32))._t, onp.dtype(F32))
    small = wrapper.take(Pd, (slice(None), slice(0, 10)))
    assert type(small) is not D.PendingProduct and Pd.computed()
    Pd = D.PendingProduct(x0._t, P(dnp, rs.randn(I, 50).astype(F32))._t, onp.dtype(F32))
    big = wrapper.take(Pd, (slice(8, None), slice(0, 40)))
    assert type(big) is D.PendingProduct and not Pd.computed() and big.shape == (B_ - 8, 40)
    assert onp.array_equal(big.numpy(), D.plain(Pd).numpy()[8:, :40])


def DevArray_from(t):
    from autograd_amd.numpy.devarray import DevArray

    return DevArray(t)


def test_device_resident_row_index_out_of_range_reads_nothing(dnp):
    """A row number held on the device is not known to the host, so NumPy's IndexError cannot be raised for it: the
    gather gives NaN rows for indices outside [-n, n), the scatter of the cotangent drops them, and neither touches
    memory outside the array."""
    import autograd_amd as ag

    x = onp.arange(12.0).reshape(4, 3)
    rows = onp.array([0, 7, -1, -9, 3])
    X, R = P(dnp, x), dnp.asarray(rows)
    got = X[R].numpy()
    assert onp.array_equal(got[[0, 2, 4]], x[[0, -1, 3]]) and onp.isnan(got[[1, 3]]).all()
    g = ag.grad(lambda a: dnp.sum(dnp.nan_to_num(a[R]) * 2.0))(X).numpy()
    want = onp.zeros_like(x)
    onp.add.at(want, [0, -1, 3], 2.0)
    assert onp.array_equal(g, want)
    # host indices keep NumPy's error
    with pytest.raises(IndexError):
        X[onp.array([0, 7])]


def test_row_gather_keeps_rows_and_the_plan_cache_is_bounded(dnp):
    """``X[batch_rows]`` with host row numbers: n entries and rows of `inner` elements (not a position per element);
    the plans kept on the device are bounded in bytes, least recently used first out."""
    import autograd_amd as ag
    from autograd_amd.numpy import wrapper

    rs = onp.random.RandomState(0)
    x = rs.randn(50, 7, 3)
    X = P(dnp, x)
    idx = rs.randint(-50, 50, 20)
    plan = wrapper._index_plan(X.shape, idx)
    assert plan.n == 20 and plan.inner == 21 and plan.n_rows == 50 and plan.shape == (20, 7, 3)
    assert onp.array_equal(X[idx].numpy(), x[idx])
    g = ag.grad(lambda a: dnp.sum(a[idx] * a[idx]))(X).numpy()
    want = onp.zeros_like(x)
    onp.add.at(want, idx, 2 * x[idx])
    assert onp.array_equal(g, want)
    for k in range(wrapper._INDEX_PLAN_LIMIT + 10):
        wrapper._index_plan((1000,), onp.array([k % 1000, (k * 7) % 1000]))
    assert len(wrapper._INDEX_PLANS) <= wrapper._INDEX_PLAN_LIMIT
    assert 0 < wrapper._INDEX_PLAN_BYTES[0] <= wrapper._INDEX_PLAN_BUDGET
    huge = onp.arange(300000) % 50
    assert wrapper._index_plan(X.shape, huge) is not wrapper._index_plan(X.shape, huge)  # too large to keep
