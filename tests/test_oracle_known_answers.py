"""Pin the CPU oracle with answers that do not depend on it.

Sources: known answers held by the reference's own tests and README (cited per
test), closed forms / brute force from ``oracle.closed_forms``, and central
finite differences (the reference's ``check_grads`` construction,
autograd/test_util.py:60-78) over the shape lists of the reference's binary-op
and systematic tests.  A dropped term, wrong sign, wrong axis or transposed
operand in a rule fails at least one of these.
"""

import warnings

import numpy as onp
import pytest

import oracle.anp as np
from autograd_amd import (
    configs,
    deriv,
    elementwise_grad,
    grad,
    hessian,
    jacobian,
    make_hvp,
    make_jvp,
    make_vjp,
    value_and_grad,
)
from autograd_amd.test_util import check_grads
from conftest import oracle_backend
from oracle import closed_forms as cf

f64 = onp.float64


# ---- known answers from the reference ------------------------------------------------
def test_readme_tanh_known_answer():
    # README.md:27-34
    def tanh(x):
        y = np.exp(-2.0 * x)
        return (1.0 - y) / (1.0 + y)

    assert abs(grad(tanh)(f64(1.0)) - 0.419974341614026) < 1e-15
    assert abs((tanh(1.0001) - tanh(0.9999)) / 0.0002 - 0.41997434264973155) < 1e-10


def test_direct_known_answer():
    # tests/test_direct.py:13-24
    fun = lambda x: (x + np.sin(x**2)) * x
    assert abs(grad(fun)(f64(1.3)) - 3.190948746871) < 1e-6
    assert abs(deriv(fun)(f64(1.3)) - 3.190948746871) < 1e-6


def test_grad_identity_and_constant():
    # tests/test_graphs.py:28-33
    fun = lambda x: x
    assert onp.allclose(grad(fun)(f64(1.3)), 1.0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        assert onp.allclose(grad(grad(fun))(f64(1.3)), 0.0)


def test_power_zero_exponent():
    # tests/test_scalar_ops.py:134-143
    assert grad(lambda x: x**0)(f64(0.0)) == 0.0
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        assert grad(grad(lambda x: x**0))(f64(0.0)) == 0.0


@pytest.mark.parametrize("kind", ["tuple", "list", "dict"])
def test_container_exact_answers(kind):
    # tests/test_tuple.py:11-24, test_list.py:11-24, test_dict.py:13-26
    A, B, C = onp.random.randn(5, 6), onp.random.randn(4, 3), onp.random.randn(2, 4)
    if kind == "dict":
        arg = {"first": A, "second": B, "third": C}
        k0, k1, k2 = "first", "second", "third"
    else:
        arg = (A, B, C) if kind == "tuple" else [A, B, C]
        k0, k1, k2 = 0, 1, 2

    def fun(c):
        return np.sum(c[k0]) + 2.0 * np.sum(c[k1])

    res = grad(fun)(arg)
    assert type(res) is type(arg)
    assert onp.array_equal(res[k0], onp.ones_like(A))
    assert onp.array_equal(res[k1], 2 * onp.ones_like(B))
    assert onp.array_equal(res[k2], onp.zeros_like(C))
    check_grads(lambda c: np.sum(np.sin(c[k0])) + np.sum(np.cos(c[k1])))(arg)


def test_hessian_closed_form():
    # tests/test_wrappers.py:54-64: hessian of x^T H x is H + H^T
    D = 5
    H = onp.random.randn(D, D)
    fun = lambda x: np.dot(np.dot(x, H), x)
    assert onp.allclose(hessian(fun)(onp.random.randn(D)), H + H.T)


def test_hvp_equals_hessian_times_v():
    # tests/test_wrappers.py:147-153
    fun = lambda a: np.sum(np.sin(a))
    a, v = onp.random.randn(7), onp.random.randn(7)
    assert onp.allclose(make_hvp(fun)(a)[0](v), onp.dot(hessian(fun)(a), v))


def test_elementwise_grad_is_per_element_grad():
    # tests/test_wrappers.py:115-123
    def simple_fun(a):
        return a + np.sin(a) + np.cosh(a)

    A = onp.random.randn(10)
    exact = elementwise_grad(simple_fun)(A)
    assert onp.allclose(exact, [grad(simple_fun)(f64(a)) for a in A])


@pytest.mark.parametrize("dtype", [onp.float16, onp.float32, onp.float64])
def test_dtype_preserved(dtype):
    # tests/test_wrappers.py:268-283
    x = onp.arange(4, dtype=dtype) + 1
    assert grad(lambda x: np.sum(np.sin(x) * 3.0))(x).dtype == dtype
    assert grad(lambda x: np.sum(x[0] ** 2))(x).dtype == dtype


def test_astype_grad_dtype():
    # tests/test_numpy.py:1032-1038
    x = onp.arange(3, dtype="float32")
    f = lambda x: np.sum(np.sin(x.astype("float64")))
    assert grad(f)(x).dtype == onp.dtype("float32")


def test_comparison_grads_are_zero():
    # tests/test_binary_ops.py:76-91
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for op in (np.greater, np.less, np.equal, np.greater_equal, np.less_equal, np.not_equal):
            for argnum in (0, 1):
                assert grad(lambda x, y: 1.0 * op(x, y), argnum)(f64(1.0), f64(2.0)) == 0.0


def test_mean_std_var_of_pair():
    # tests/test_numpy.py:272-285: d/dx of stats of [x, x + 2]
    assert onp.allclose(grad(lambda x: np.mean(np.array([x, x + 2.0])))(f64(0.3)), 1.0)
    assert onp.allclose(grad(lambda x: np.std(np.array([x, x + 2.0])))(f64(0.3)), 0.0)
    assert onp.allclose(grad(lambda x: np.var(np.array([x, x + 2.0])))(f64(0.3)), 0.0)


# ---- scatter rules: bit-exact against numpy.add.at -----------------------------------
@pytest.mark.parametrize("idx", [[0, 0], [0, 1, 0], [2, 2, 2, 1], slice(1, 4), 3, (slice(None, -1),)])
def test_getitem_vjp_is_add_at(idx):
    # tests/test_numpy.py:881-890 (repeated indices) and 288-352 (slices, ints)
    x = onp.random.randn(6)
    w = onp.random.randn(*onp.shape(x[idx]))
    got = grad(lambda x: np.sum(x[idx] * w))(x)
    want = onp.zeros_like(x)
    onp.add.at(want, onp.array(idx, dtype="int64") if isinstance(idx, list) else idx, w)
    assert onp.array_equal(got, want)


def test_mixed_index():
    # tests/test_numpy.py:315-321
    A = onp.random.randn(5, 6, 4)
    check_grads(lambda A: np.sum(np.sin(A[3, 2:, [1, 3]])))(A)


# ---- graphs: fan-out, dense+sparse accumulation, higher order -----------------------
def test_fanout_and_mutating_outgrads():
    # tests/test_graphs.py:13-17, 71-92
    check_grads(lambda x: np.sum(np.sin(x) + np.sin(x) * x))(onp.random.randn(4))

    def fun(a):
        b = a + 1.0
        c = b + 1.5
        d = a + b
        e = d + c
        return np.sum(e * e)

    check_grads(fun)(onp.random.randn(3))

    def fun2(a):
        b = a + 1.0
        c = b[0] + 1.5
        d = a + b
        e = d + c
        return np.sum(e * a)

    check_grads(fun2)(onp.random.randn(3))


def test_third_derivative():
    # tests/test_graphs.py:121-151
    fun = lambda x: np.sin(np.sin(x) + np.sin(x))
    d3 = grad(grad(grad(fun)))(f64(0.7))
    num = (grad(grad(fun))(f64(0.7 + 1e-5)) - grad(grad(fun))(f64(0.7 - 1e-5))) / 2e-5
    assert abs(d3 - num) < 1e-5 * max(1.0, abs(num))


def test_assignment_raises():
    # tests/test_graphs.py:184-191
    def fun(A, b):
        A[1] = b
        return A

    with pytest.raises(TypeError):
        grad(lambda A, b: np.sum(fun(A, b)), 0)(onp.random.randn(5), 3.0)


def test_error_conventions():
    with pytest.raises(TypeError):  # differential_operators.py:31-35
        grad(lambda x: x * 2.0)(onp.ones(3))
    with pytest.raises(TypeError):  # tracer.py:190
        grad(lambda x: x)("abc")
    from autograd_amd.extend import primitive

    @primitive
    def no_rule(x):
        return x * 2.0

    with pytest.raises(NotImplementedError):  # core.py:43-45
        grad(lambda x: np.sum(no_rule(x)))(onp.ones(3))
    with pytest.raises(NotImplementedError):  # core.py:133-135
        make_jvp(lambda x: no_rule(x))(onp.ones(3))(onp.ones(3))
    with warnings.catch_warnings(record=True) as w:  # tracer.py:21, core.py:14-17
        warnings.simplefilter("always")
        g = grad(lambda x: f64(3.0))(onp.ones(3))
    assert onp.array_equal(g, onp.zeros(3)) and any("independent" in str(m.message) for m in w)


# ---- finite differences over the reference's shape lists ---------------------------
SHAPES = [(), (4,), (3, 4), (1, 4)]  # tests/test_binary_ops.py:12-18


def _arg(shape, positive=False):
    a = onp.random.randn(*shape) if shape else f64(onp.random.randn())
    return onp.abs(a) + 1.1 if positive else a


@pytest.mark.parametrize("opname", ["add", "subtract", "multiply", "true_divide", "maximum", "minimum", "power"])
def test_binary_rules_all_broadcast_patterns(opname):
    op = getattr(np, opname)
    for sa in SHAPES:
        for sb in SHAPES:
            a = _arg(sa, positive=opname == "power")
            b = _arg(sb, positive=opname == "true_divide")
            check_grads(lambda a, b: op(a, b), (0, 1))(a, b)


@pytest.mark.parametrize(
    "opname,positive",
    [("negative", False), ("exp", False), ("tanh", False), ("sinh", False), ("cosh", False), ("sin", False),
     ("cos", False), ("log", True), ("sqrt", True), ("square", False), ("abs", True), ("reciprocal", True),
     ("log1p", True), ("expm1", False)],
)
def test_unary_rules(opname, positive):
    check_grads(getattr(np, opname))(_arg((3, 4), positive))


@pytest.mark.parametrize("axis", [None, 0, 1])
@pytest.mark.parametrize("keepdims", [False, True])
def test_reduction_rules(axis, keepdims):
    # tests/test_systematic.py:14-45 (stat_check)
    x = onp.random.randn(3, 4)
    for red in (np.sum, np.mean, np.max, np.min, np.var, np.std, np.prod):
        check_grads(lambda x: red(x, axis=axis, keepdims=keepdims))(x)
    check_grads(lambda x: np.logsumexp(x, axis=axis, keepdims=keepdims))(x)  # tests/test_scipy.py:227-264


def test_contraction_rules():
    # tests/test_systematic.py:294-349 (dot order 3, matmul, tensordot)
    rs = onp.random.RandomState(0)
    shapes = [((), ()), ((4,), (4,)), ((3, 4), (4,)), ((4,), (4, 5)), ((3, 4), (4, 5)), ((2, 3, 4), (4, 5))]
    for sa, sb in shapes:
        a = rs.randn(*sa) if sa else f64(rs.randn())
        b = rs.randn(*sb) if sb else f64(rs.randn())
        check_grads(np.dot, (0, 1), order=3 if len(sa) < 3 else 2)(a, b)
    for sa, sb in [((4,), (4,)), ((3, 4), (4,)), ((4,), (4, 5)), ((3, 4), (4, 5)), ((2, 3, 4), (4, 5)), ((2, 3, 4), (2, 4, 5))]:
        check_grads(np.matmul, (0, 1))(rs.randn(*sa), rs.randn(*sb))
    A, B = rs.randn(2, 3, 4), rs.randn(4, 3, 5)
    check_grads(lambda A, B: np.tensordot(A, B, axes=[[1, 2], [1, 0]]), (0, 1), order=3)(A, B)
    check_grads(lambda A, B: np.tensordot(A, B, axes=1), (0, 1))(A, rs.randn(4, 6))
    check_grads(lambda A, B: np.tensordot(A, B, axes=2), (0, 1))(A, rs.randn(3, 4, 2))
    check_grads(lambda A, B: np.tensordot(A, B, axes=0), (0, 1))(rs.randn(2, 2), rs.randn(3))
    check_grads(lambda A, B: np.tensordot(A, B, axes=[2, 0]), (0, 1))(A, B)


def test_shape_rules():
    x = onp.random.randn(2, 3, 4)
    check_grads(lambda x: np.reshape(x, (6, 4)))(x)
    check_grads(lambda x: np.ravel(x))(x)
    check_grads(lambda x: np.transpose(x, (2, 0, 1)))(x)
    check_grads(lambda x: np.swapaxes(x, 0, 2))(x)
    check_grads(lambda x: np.expand_dims(x, 1))(x)
    check_grads(lambda x: np.squeeze(np.expand_dims(x, 1)))(x)
    check_grads(lambda x: np.repeat(x, 3, axis=1))(x)
    check_grads(lambda x: np.repeat(x[:, :1], 5, axis=1))(x)
    check_grads(lambda x, y: np.concatenate((x, y), axis=1), (0, 1))(x, onp.random.randn(2, 2, 4))
    check_grads(lambda x: np.hstack((x[0], x[1])))(x)
    check_grads(lambda x: np.broadcast_to(x[:, :1], (2, 3, 4)))(x)


# ---- the five workloads against closed forms ----------------------------------------
def _close(got, want, rtol):
    got, want = onp.asarray(got, onp.float64), onp.asarray(want, onp.float64)
    assert got.shape == want.shape
    tol = rtol * onp.abs(want) + rtol * onp.max(onp.abs(want))
    assert onp.all(onp.abs(got - want) <= tol), onp.max(onp.abs(got - want) / (tol + 1e-300))


def test_workload_tanh_closed_form():
    inp = configs.tanh_inputs(n=1001)
    out = configs.run_config("tanh", oracle_backend(), inp)
    want = cf.tanh_derivatives(inp["x"])
    for k in ("d1", "d2", "d3"):
        _close(out[k], want[k], 1e-12)


def test_workload_bcast_closed_form():
    inp = configs.bcast_inputs(rows=64, cols=48)
    out = configs.run_config("bcast", oracle_backend(), inp)
    want = cf.bcast_grads(**inp)
    for k in ("dA", "db", "dc"):
        assert out[k].dtype == onp.float32
        _close(out[k], want[k], 1e-5)


def test_workload_mlp_closed_form():
    inp = configs.mlp_inputs(batch=32, layer_sizes=(20, 16, 12, 10))
    out = configs.run_config("mlp", oracle_backend(), inp)["grad"]
    want = cf.mlp_grads(inp["params"], inp["X"], inp["T"])
    for (gW, gb), (wW, wb) in zip(out, want):
        assert gW.dtype == onp.float32 and gb.dtype == onp.float32
        _close(gW, wW, 1e-5)
        _close(gb, wb, 1e-5)


def test_workload_rnn_closed_form():
    inp = configs.rnn_inputs(seq_len=6, batch=8, input_size=9, state_size=10, output_size=9)
    out = configs.run_config("rnn", oracle_backend(), inp)["grad"]
    want = cf.rnn_grads(inp["params"], inp["inputs"], inp["targets"])
    for k in want:
        assert out[k].dtype == onp.float32
        _close(out[k], want[k], 1e-5)


def test_workload_rosen_closed_form():
    inp = configs.rosen_inputs(n=257)
    out = configs.run_config("rosen", oracle_backend(), inp)
    _close(out["grad"], cf.rosen_grad(inp["x"]), 1e-12)
    want = cf.rosen_hvp(inp["x"], inp["v"])
    _close(out["hvp_rev"], want, 1e-12)
    _close(out["hvp_fwd"], want, 1e-12)
    # and the closed forms themselves against brute force
    f = lambda x: onp.sum(100 * (x[1:] - x[:-1] ** 2) ** 2 + (1 - x[:-1]) ** 2)
    x = inp["x"][:9]
    assert onp.allclose(cf.rosen_grad(x), cf.numerical_grad(f, x), rtol=1e-6, atol=1e-5)
    H = onp.stack([cf.rosen_hvp(x, e) for e in onp.eye(9)])
    assert onp.allclose(H, H.T)
    Hnum = onp.stack([cf.numerical_grad(lambda y: cf.rosen_grad(y)[i], x) for i in range(9)])
    assert onp.allclose(H, Hnum, rtol=1e-5, atol=1e-4)


def test_jacobian_and_value_and_grad():
    x = onp.random.randn(4)
    J = jacobian(lambda x: np.sin(x) * x[0])(x)
    Jn = onp.stack([cf.numerical_grad(lambda y: (onp.sin(y) * y[0])[i], x) for i in range(4)])
    assert onp.allclose(J, Jn, atol=1e-6)
    val, g = value_and_grad(lambda x: np.sum(x**3))(x)
    assert onp.allclose(val, onp.sum(x**3)) and onp.allclose(g, 3 * x**2)
    vjp, ans = make_vjp(lambda x: x * 2.0)(x)
    assert onp.array_equal(vjp(onp.ones(4)), 2 * onp.ones(4))
