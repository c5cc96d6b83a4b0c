"""Names and calling conventions a program written for the reference expects to find: the cases are the ones the
reference's own tests exercise (tests/test_numpy.py, test_wrappers.py, test_tuple.py, test_misc.py, test_scipy.py),
checked against NumPy on the host for values and against finite differences (``check_grads``) for derivatives.
"""

import warnings

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ag():
    import autograd_amd

    return autograd_amd


@pytest.fixture(scope="module")
def np(ag):
    import autograd_amd.numpy as np

    return np


def _host(x):
    return x.numpy() if hasattr(x, "numpy") else onp.asarray(x)


def test_version_and_dtype_names(np):
    assert np.__version__ == onp.__version__
    assert np.dtype("float32") == onp.float32
    x = np.arange(3, dtype="float32")
    assert x.astype("float64").dtype == onp.float64
    assert onp.dtype(np.int64) == onp.int64 and onp.dtype(np.int32) == onp.int32
    assert np.int64(3.7) == 3 and type(np.int64(3.7)) is onp.int64
    assert np.zeros(2, dtype=np.int64).dtype == onp.int64


def test_integer_cast_of_a_traced_column_indexes(ag, np):
    """tests/test_numpy.py:920-935: a column of the traced matrix, cast to integers, indexes its rows."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(0)
    W = rs.randn(5, 10)
    W[:, -1] = [0.5, 3.5, 1.5, 4.5, 2.5]  # (truncated to 0, 3, 1, 4, 2; away from the steps, for the finite differences)

    def fun(W):
        picked = np.int64(W[:, -1])
        assert picked.dtype == np.int64
        return W[:, :-1][picked].sum()

    check_grads(fun)(np.array(W))
    expected = onp.zeros_like(W)
    expected[:, :-1] = 1.0
    onp.testing.assert_array_equal(_host(ag.grad(fun)(np.array(W))), expected)


@pytest.mark.parametrize("pieces", ["x", "xx", "xc", "xcx", "c"])
def test_row_joiner(np, pieces):
    """tests/test_numpy.py:668-736."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(1)
    c, A = rs.randn(3, 2), rs.randn(3, 2)
    dc = np.array(c)

    def fun(x):
        return np.r_[tuple(x if p == "x" else dc for p in pieces)]

    out = fun(np.array(A))
    onp.testing.assert_array_equal(_host(out), onp.r_[tuple(A if p == "x" else c for p in pieces)])
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")  # "c": the output does not depend on the input
        check_grads(fun)(np.array(A))


def test_row_joiner_takes_ranges_and_scalars(np):
    """tests/test_numpy.py:739-748."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(2)
    c, A = rs.randn(10), rs.randn(10)
    dc = np.array(c)
    out = np.r_[np.array(A), dc, 1:10, 2.5]
    onp.testing.assert_array_equal(_host(out), onp.r_[A, c, 1:10, 2.5])
    check_grads(lambda x: np.r_[x, dc, 1:10])(np.array(A))
    with pytest.raises(NotImplementedError):
        np.r_["0,2", np.array(A)]


def test_column_joiner_and_column_stack(np):
    """tests/test_numpy.py:751-772, tests/test_systematic.py column_stack cases."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(3)
    c, A, v = rs.randn(3, 2), rs.randn(3, 2), rs.randn(3)
    dc, dv = np.array(c), np.array(v)
    onp.testing.assert_array_equal(_host(np.c_[np.array(A), dc, np.array(A)]), onp.c_[A, c, A])
    onp.testing.assert_array_equal(_host(np.c_[dv, dv]), onp.c_[v, v])
    onp.testing.assert_array_equal(_host(np.column_stack((dv, dc, dv))), onp.column_stack((v, c, v)))
    check_grads(lambda x: np.c_[x, dc, x])(np.array(A))
    check_grads(lambda x: np.column_stack((x, dc)))(dv)


def test_append(np):
    """tests/test_numpy.py:405-427: flattened without an axis; nested lists with an axis."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(4)
    A, B = rs.randn(2, 3), rs.randn(1, 3)
    onp.testing.assert_array_equal(_host(np.append(np.array(A), np.array(B))), onp.append(A, B))
    onp.testing.assert_array_equal(_host(np.append(np.array(A), np.array(B), axis=0)), onp.append(A, B, axis=0))
    check_grads(np.append, argnum=(0, 1))(np.array(A), np.array(B), axis=0)
    check_grads(np.append, argnum=(0, 1))([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], [[7.0, 8.0, 9.0]], axis=0)
    check_grads(np.append, argnum=(0, 1))(np.array([1.0, 2.0]), 3.0)


def test_select(np):
    """tests/test_systematic.py test_select: the first condition that holds wins, the default fills the rest."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(5)
    conds = [rs.randn(3, 4, 5) > 0, rs.randn(1, 5) > 0]
    choices = [rs.randn(3, 4, 5), rs.randn(3, 4, 1)]
    got = np.select([np.array(c) for c in conds], [np.array(c) for c in choices], default=0.5)
    onp.testing.assert_array_equal(_host(got), onp.select(conds, choices, default=0.5))
    dconds = [np.array(c) for c in conds]
    check_grads(lambda a, b: np.select(dconds, [a, b], default=0.0), argnum=(0, 1))(*[np.array(c) for c in choices])
    with pytest.raises(ValueError):
        np.select(dconds, [np.array(choices[0])])


def test_where_calling_conventions(np):
    """tests/test_wrappers.py:307-330: host masks, keywords, and the one-argument form."""
    x, y = np.array([1.0, 2.0, 3.0]), np.array([4.0, 5.0, 6.0])
    condition = [True, False, True]
    for got in (np.where(condition, x, y), np.where(condition=condition, x=x, y=y), np.where(condition, x, y=y),
                np.where(onp.array(condition), x, y)):
        onp.testing.assert_array_equal(_host(got), [1.0, 5.0, 3.0])
    (positions,) = np.where(condition)
    onp.testing.assert_array_equal(_host(positions), [0, 2])
    with pytest.raises(ValueError):
        np.where(condition, x)
    assert np.where([True, False], 1.0, 2.0) == [1.0, 2.0]
    assert np.where(False, 1.0, 2.0) == 2.0 and type(np.where(True, 1.0, 2.0)) is float


def test_array_of_a_traced_tuple(ag, np):
    """tests/test_tuple.py nested higher order: ``np.array`` of a boxed tuple sees the traced elements."""

    def outer(params):
        return np.sum(np.array(params) ** 2)

    got = ag.grad(outer)((1.0, 2.0, 3.0))
    assert [float(_host(g)) for g in got] == [2.0, 4.0, 6.0]

    def through_a_list(x):
        return np.sum(np.array([x, 2.0 * x, x * x]))

    assert float(_host(ag.grad(through_a_list)(3.0))) == 1.0 + 2.0 + 6.0


def test_gradient_over_several_axes_is_traced(ag, np):
    """tests/test_numpy.py:1041-1047: with several axes the derivatives come back in a tuple and stay traced."""
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(6)
    x = rs.randn(6, 5, 4)
    for axis in (None, (0, 1), (0, -1)):
        got = np.gradient(np.array(x), axis=axis)
        want = onp.gradient(x, axis=axis)
        assert type(got) is tuple and len(got) == len(want)
        for g, w in zip(got, want):
            onp.testing.assert_allclose(_host(g), w, rtol=1e-12, atol=1e-15)
        check_grads(np.gradient, 0)(np.array(x), axis=axis)
    total = lambda x: sum(np.sum(g * g) for g in np.gradient(x))  # noqa: E731
    assert float(onp.abs(_host(ag.grad(total)(np.array(x)))).max()) > 0.0


def test_plain_numpy_reductions_on_a_box(ag, np):
    """tests/test_numpy.py:157-180: NumPy's own ``sum`` / ``prod`` / ``max`` / ``min`` called on a box forward an
    ``out=None`` keyword to the box's method."""
    base = np.array(onp.abs(onp.random.RandomState(7).randn(5)) + 0.5)
    for plain, ours in ((onp.sum, np.sum), (onp.prod, np.prod), (onp.max, np.max), (onp.min, np.min)):
        a = float(_host(ag.grad(lambda t: plain(np.exp(t) * base))(0.7)))
        b = float(_host(ag.grad(lambda t: ours(np.exp(t) * base))(0.7)))
        assert a == b and a != 0.0


def test_legacy_rule_registration(ag, np):
    """autograd/core.py:347-415: the pre-1.2 spellings of rule registration still attach a rule, with a warning."""
    from autograd_amd import primitive
    from autograd_amd.util import quick_grad_check

    @primitive
    def cube(x):
        return x * x * x

    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        cube.defvjp(lambda g, ans, vs, gvs, x: 3.0 * x * x * g)
        assert seen
    assert float(_host(ag.grad(lambda x: np.sum(cube(x)))(np.array([2.0])))[0]) == 12.0

    @primitive
    def count(x):
        return float(onp.floor(x))

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        count.defvjp_is_zero()
        quick_grad_check(lambda x: np.sum(np.sin(x) * x), np.array([0.3, 0.4]))
    assert float(_host(ag.grad(lambda x: x * count(x))(2.5))) == 2.0


def test_const_graph_replays_only_what_depends_on_the_arguments(ag, np):
    """tests/test_misc.py:9-51."""
    from autograd_amd import primitive
    from autograd_amd.misc import const_graph

    seen = []

    @primitive
    def tagged(value, tag):
        seen.append(tag)
        return value

    def fun(x, y, z):
        return np.sum(tagged(x, "x") + 2 * tagged(y, "y") + 3 * tagged(z, "z"))

    x, y, z = np.array([1.0, 1.5]), np.array([2.0, -1.0]), np.array([3.0, 0.5])
    want = float(_host(fun(x, y, z)))
    seen.clear()
    replaying = const_graph(fun, x, z=z)
    assert seen == []
    assert float(_host(replaying(y))) == want and seen == ["x", "y", "z"]
    seen.clear()
    doubled = float(_host(fun(x, 2 * y, z)))
    seen.clear()
    assert float(_host(replaying(2 * y))) == doubled and seen == ["y"]
    seen.clear()
    assert float(_host(replaying(y))) == want and seen == ["y"]
    inner = const_graph(lambda a, b: ag.grad(lambda t: np.sum(np.sin(t) + t * 2))(a * b))
    for a, b in ((0.0, 0.0), (1.0, 0.5), (np.array([1.0, 2.0]), np.array([0.5, 0.25]))):
        onp.testing.assert_allclose(_host(inner(a, b)), onp.cos(_host(a) * _host(b)) + 2.0, rtol=1e-12)
    with pytest.raises(ValueError):
        const_graph(lambda a: 1.0)(2.0)


def test_full_graph_keeps_values_and_recipes(np):
    from autograd_amd.misc.tracers import full_graph

    x = np.array([0.5, 1.0])
    last = full_graph(lambda a, b: np.sin(a) * b, x, 2.0)
    fun, args, kwargs, parents = last.recipe
    assert fun is np.multiply and kwargs == {} and [argnum for argnum, _ in parents] == [0, 1]
    onp.testing.assert_allclose(_host(last.value), onp.sin([0.5, 1.0]) * 2.0, rtol=1e-12)
    assert parents[0][1].recipe[0] is np.sin
    assert parents[1][1].value == 2.0  # (the second argument, taken out of the traced tuple of arguments)


def test_fixed_point_differentiates_without_unrolling(ag, np):
    """examples/fixed_points.py: Newton's iteration for the square root; d sqrt(a)/da = 1/(2 sqrt(a)) and the second
    derivative -1/4 a^(-3/2) come out of the adjoint iteration of autograd/misc/fixed_points.py:15-23."""
    from autograd_amd.misc.fixed_points import fixed_point

    newton = lambda a: lambda x: 0.5 * (x + a / x)  # noqa: E731
    distance = lambda x, y: float(_host(np.max(np.abs(x - y))))  # noqa: E731
    root_sum = lambda a: np.sum(fixed_point(newton, a, np.ones(3), distance, 1e-13))  # noqa: E731
    a = onp.array([2.0, 3.0, 5.0])
    onp.testing.assert_allclose(float(_host(root_sum(np.array(a)))), onp.sqrt(a).sum(), rtol=1e-12)
    onp.testing.assert_allclose(_host(ag.grad(root_sum)(np.array(a))), 0.5 / onp.sqrt(a), rtol=1e-10)
    second = ag.grad(lambda a: np.sum(ag.grad(root_sum)(a)))(np.array(a))
    onp.testing.assert_allclose(_host(second), -0.25 * a**-1.5, rtol=1e-8)


def test_convolve_with_nothing_sliding_is_a_contraction(np):
    """tests/test_scipy.py:279-284: no convolved axes leaves the contraction over ``dot_axes``."""
    from autograd_amd.scipy.signal import convolve
    from autograd_amd.test_util import check_grads

    rs = onp.random.RandomState(8)
    A, B = rs.randn(3, 5), rs.randn(3, 4)
    for mode in ("valid", "full"):
        got = convolve(np.array(A), np.array(B), axes=([], []), dot_axes=([0], [0]), mode=mode)
        onp.testing.assert_allclose(_host(got), onp.tensordot(A, B, axes=([0], [0])), rtol=1e-12)
    check_grads(lambda a, b: convolve(a, b, axes=([], []), dot_axes=([0], [0])), argnum=(0, 1), modes=["rev"])(
        np.array(A), np.array(B))


def test_item_assignment_outside_a_trace(ag, np):
    """examples/rnn.py:86 fills its one-hot batches with ``seqs[:, ix, :] = ...``: plain device arrays take basic
    indices and whole-array masks; arithmetic that was pending on the old contents keeps the old contents; a view
    taken before the assignment sees it; traced values stay out."""
    h = onp.arange(24.0).reshape(2, 3, 4)
    d = np.array(h)
    cases = [((slice(None), 1, slice(None)), onp.ones((2, 4))), (0, 7.0), ((1, slice(0, 3, 2)), onp.arange(4.0)),
             ((Ellipsis, 2), -1.0), ((slice(None), None, 1), 5.0), ((1, 2, 3), 9.5), ((slice(0, 0),), 3.0)]
    for idx, value in cases:
        h[idx] = value
        d[idx] = np.array(value) if isinstance(value, onp.ndarray) else value
        onp.testing.assert_array_equal(_host(d), h)
    mask = h > 10
    h[mask] = 0.0
    d[np.array(mask)] = 0.0
    onp.testing.assert_array_equal(_host(d), h)

    filled = np.zeros((3, 4))  # (a lazy fill until first written)
    for row in range(3):
        filled[row, row:] = float(row + 1)
    onp.testing.assert_array_equal(_host(filled), onp.triu(onp.ones((3, 4))) * onp.arange(1.0, 4.0)[:, None])
    counts = np.zeros(3, dtype=np.int64)
    counts[1:] = np.array([4, 5])
    onp.testing.assert_array_equal(_host(counts), [0, 4, 5])

    x = np.ones(3)
    doubled, negated = x * 2.0 + 1.0, -x
    x[0] = 5.0
    onp.testing.assert_array_equal(_host(doubled), [3.0, 3.0, 3.0])
    onp.testing.assert_array_equal(_host(negated), [-1.0, -1.0, -1.0])
    onp.testing.assert_array_equal(_host(x), [5.0, 1.0, 1.0])

    z = np.zeros((2, 2))
    first_row = z[0]
    first_row[:] = 1.0
    z.T[0, 1] = 4.0
    onp.testing.assert_array_equal(_host(z), [[1.0, 1.0], [4.0, 0.0]])

    # a view of an array whose arithmetic is still pending: the write could not reach that array, so it is refused
    y = 1.0 - np.array(onp.arange(4.0))
    v = y[1:]
    with pytest.raises(ValueError, match="still pending"):
        v[:] = 0.0
    y[1:] = 0.0  # assigning into the array itself is fine
    onp.testing.assert_array_equal(_host(y), [1.0, 0.0, 0.0, 0.0])

    with pytest.raises(NotImplementedError):
        d[::-1] = 1.0
    with pytest.raises(NotImplementedError):
        d[[0, 1]] = 1.0
    with pytest.raises(ValueError):
        d[0] = onp.ones(5)
    with pytest.raises(TypeError):
        ag.grad(lambda v: (d.__setitem__(0, v), np.sum(d))[1])(np.ones(4))
    with pytest.raises(TypeError):
        ag.grad(lambda v: (v.__setitem__(0, 1.0), np.sum(v))[1])(np.ones(4))


def test_integer_scalars_index_python_sequences(np):
    """examples/rnn.py:74: ``chr(np.argmax(c))``."""
    best = np.argmax(np.array([0.0, 70.0, 3.0]))
    assert chr(best) == "\x01" and [10, 20, 30][best] == 20 and "abc"[best] == "b"
    with pytest.raises(TypeError):
        [10, 20][np.array(1.0)]


def test_meshgrid(ag, np):
    a, b, c = onp.arange(3.0), onp.arange(4.0) + 10, onp.arange(2.0) + 100
    for kw in ({}, {"indexing": "ij"}, {"sparse": True}, {"indexing": "ij", "sparse": True}):
        for args in ((a,), (a, b), (a, b, c)):
            got = np.meshgrid(*[np.array(x) for x in args], **kw)
            want = onp.meshgrid(*args, **kw)
            assert len(got) == len(want)
            for g, w in zip(got, want):
                onp.testing.assert_array_equal(_host(g), w)
    through = ag.grad(lambda x: np.sum(np.meshgrid(x, np.array(b))[0] ** 2))(np.array(a))
    onp.testing.assert_array_equal(_host(through), 2 * a * 4)


HOST_ARRAY_PROGRAM = r"""
import numpy as onp
import autograd_amd as ag, autograd_amd.numpy as np
from scipy.optimize import minimize

def rosenbrock(x):
    return 100 * (x[1] - x[0] ** 2) ** 2 + (1 - x[0]) ** 2

x0 = onp.array([0.5, -0.3])
g = ag.grad(rosenbrock)(x0)
assert isinstance(g, np.DevArray)
want = [-400 * x0[0] * (x0[1] - x0[0] ** 2) - 2 * (1 - x0[0]), 200 * (x0[1] - x0[0] ** 2)]
onp.testing.assert_allclose(g.numpy(), want, rtol=1e-12)
found = minimize(ag.value_and_grad(rosenbrock), onp.array([0.0, 0.0]), jac=True, method="CG")
onp.testing.assert_allclose(found.x, [1.0, 1.0], atol=1e-4)
d = ag.grad(lambda t: np.sin(t) * t)(onp.float64(0.5))
assert abs(float(d) - (onp.sin(0.5) + 0.5 * onp.cos(0.5))) < 1e-15
assert ag.grad(lambda t: np.sum(t * t))(onp.ones(3, dtype=onp.float32)).dtype == onp.float32
J = ag.jacobian(lambda t: np.tanh(t) * 2.0)(onp.array([0.1, 0.2]))
onp.testing.assert_allclose(J.numpy(), onp.diag(2.0 / onp.cosh([0.1, 0.2]) ** 2), rtol=1e-12)
print("host arrays ok")
"""


def test_host_arrays_enter_at_the_differential_operator():
    """examples/rosenbrock.py: ``scipy.optimize.minimize(value_and_grad(f), x0, jac=True)`` hands host arrays in and
    reads the value and the gradient back through ``float()`` / ``numpy.asarray``.  Host arrays are the device
    namespace's only while no other array library on the tracer claims them (the CPU oracle of these tests does), so
    the check runs in a process of its own."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    env.pop("AUTOGRAD_AMD_HOST", None)
    done = subprocess.run([sys.executable, "-c", HOST_ARRAY_PROGRAM], env=env, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0 and "host arrays ok" in done.stdout, done.stdout + done.stderr


def test_host_arrays_stay_with_an_array_library_that_claims_them(ag, np):
    """The CPU oracle registers ``numpy.ndarray`` as its own value type: whichever is imported first, its programs
    keep running on the host (a parity test that compared the device with itself would prove nothing)."""
    import oracle.anp as anp
    from autograd_amd.extend import Box, vspace

    assert Box.type_mappings[onp.ndarray].__name__ == "ArrayBox"
    got = ag.grad(lambda t: anp.sum(anp.sin(t)))(onp.array([0.1, 0.2]))
    assert type(got) is onp.ndarray and type(vspace(onp.ones(2))).__name__ == "ArrayVSpace"


def test_names_that_take_no_array_data(np):
    assert np.random.RandomState(0).randn(2).shape == (2,)
    with np.errstate(divide="ignore"):
        old = np.seterr(over="ignore")
    np.seterr(**old)
    assert np.finfo(np.float32).eps == onp.finfo(onp.float32).eps and np.uint8 is onp.uint8
    assert np.issubdtype(np.float64, np.floating) and np.broadcast_shapes((3, 1), (4,)) == (3, 4)
    onp.testing.assert_array_equal(_host(np.identity(3)), onp.identity(3))
    onp.testing.assert_array_equal(_host(np.arange(10.0)[np.s_[2:5]]), [2.0, 3.0, 4.0])


def test_numpy_ufuncs_called_on_device_arrays_and_boxes(ag, np):
    """``numpy.abs(x)``, ``host * x``, ``numpy.float64(2) * x`` and ``numpy.sin(box)`` run the namespace's function of
    the same name (tests/test_numpy.py:157-180 feeds ``npr.randn`` results to plain NumPy functions); forms the
    namespace has no counterpart for are declined, which NumPy reports as a TypeError."""
    h, g = onp.array([1.0, -2.0, 3.0]), onp.array([2.0, 2.0, 2.0])
    x = np.array(h)
    onp.testing.assert_array_equal(_host(onp.abs(x)), onp.abs(h))
    onp.testing.assert_allclose(_host(onp.exp(x)), onp.exp(h), rtol=1e-15)
    onp.testing.assert_array_equal(_host(g * x), g * h)
    onp.testing.assert_array_equal(_host(g < x), g < h)
    onp.testing.assert_array_equal(_host(onp.maximum(g, x)), onp.maximum(g, h))
    x32 = np.array(h.astype(onp.float32))
    assert (onp.float64(2.0) * x32).dtype == onp.float64 and (2.0 * x32).dtype == onp.float32
    assert (g.astype(onp.float32) * x32).dtype == onp.float32
    got = ag.grad(lambda v: np.sum(onp.sin(v) * g))(x)
    onp.testing.assert_allclose(_host(got), onp.cos(h) * g, rtol=1e-15)
    with pytest.raises(TypeError):
        onp.add(x, x, out=onp.zeros(3))
    with pytest.raises(TypeError):
        onp.add.reduce(x)
