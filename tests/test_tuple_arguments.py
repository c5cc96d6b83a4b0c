"""``make_vjp`` traces a tuple argument element by element (``core._make_vjp_by_element``) instead of boxing the tuple
as the reference does (autograd/builtins.py:37-96).  The reference's observable effects of the boxed form must
survive: checked here on the CPU oracle against what the reference's mechanism implies (and, for whole workloads and
container cases, by the reference vectors of ``test_oracle_golden.py`` / ``test_oracle_next.py``, which go through
the same path)."""

import warnings

import numpy as onp
import pytest

import autograd_amd as ag
import oracle.anp as np


def test_cotangents_take_the_dtype_of_their_argument():
    """The rule of ``where`` (numpy_vjps.py:226-230) makes a float32 cotangent float64.  With one ``argnum`` that is
    what comes back; with several, each cotangent is added into zeros of its argument's vector space
    (core.py:185-215 via builtins.py:24-34) and comes back float32."""
    x = onp.array([1.0, -2.0, 3.0], dtype=onp.float32)
    y = onp.array([0.5, 0.25, 2.0], dtype=onp.float32)
    f = lambda a, b: np.sum(np.where(a > 0, a * b, b))  # noqa: E731
    assert ag.grad(f, 0)(x, y).dtype == onp.float64
    both = ag.grad(f, (0, 1))(x, y)
    assert [g.dtype for g in both] == [onp.float32, onp.float32]
    onp.testing.assert_array_equal(both[0], [0.5, 0.0, 2.0])
    onp.testing.assert_array_equal(both[1], [1.0, 1.0, 3.0])
    packed = ag.grad(lambda p: f(p[0], p[1]))((x, y))
    assert [g.dtype for g in packed] == [onp.float32, onp.float32]


def test_negative_zero_is_added_to_zero():
    x = onp.array([1.0, 2.0])
    f = lambda a, b: np.sum(a * -0.0) + np.sum(b)  # noqa: E731
    assert onp.signbit(ag.grad(f, 0)(x, x)).all()  # one argnum: the cotangent as the rule made it
    assert not onp.signbit(ag.grad(f, (0, 1))(x, x)[0]).any()  # several: 0.0 + -0.0


def test_unused_repeated_and_nested_elements():
    x, y = onp.array([1.0, 2.0, 3.0]), onp.array([[1.0, 2.0]], dtype=onp.float32)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        gx, gy = ag.grad(lambda a, b: np.sum(a * a), (0, 1))(x, y)
    onp.testing.assert_array_equal(gx, 2 * x)
    assert gy.shape == (1, 2) and gy.dtype == onp.float32 and not gy.any()
    g0, g1 = ag.grad(lambda a, b: np.sum(a * b * b), (0, 1))(x, x)  # the same array twice: two arguments
    onp.testing.assert_array_equal(g0, x * x)
    onp.testing.assert_array_equal(g1, 2 * x * x)
    params = (onp.array([[1.0, 2.0], [3.0, 4.0]]), {"b": onp.array([0.5, -0.5]), "scale": onp.array(2.0)})
    loss = lambda p: np.sum(np.tanh(np.dot(p[0], p[1]["b"]) * p[1]["scale"]))  # noqa: E731
    got = ag.grad(loss)(params)
    listed = ag.grad(loss)(list(params))  # a list argument keeps the boxed-container path
    assert isinstance(got, tuple) and isinstance(got[1], dict) and isinstance(listed, list)
    onp.testing.assert_array_equal(got[0], listed[0])
    for key in ("b", "scale"):
        onp.testing.assert_array_equal(got[1][key], listed[1][key])
    one, zero = ag.grad(lambda a, b: a, (0, 1))(onp.float64(2.0), onp.float64(3.0))  # the output IS an input
    assert one == 1.0 and zero == 0.0


def test_higher_order_and_untraced_outputs():
    x, y = onp.array([0.3, -0.7]), onp.array([1.5, 0.5])
    f = lambda a, b: np.sum(np.sin(a) * b * b)  # noqa: E731
    second = ag.grad(lambda a, b: np.sum(ag.grad(f, (0, 1))(a, b)[0] ** 2) + np.sum(ag.grad(f, (0, 1))(a, b)[1]), (0, 1))(x, y)
    d0 = onp.cos(x) * y * y  # df/da;  df/db = 2 sin(a) b
    want_a = 2 * d0 * (-onp.sin(x) * y * y) + 2 * onp.cos(x) * y
    want_b = 2 * d0 * (2 * onp.cos(x) * y) + 2 * onp.sin(x)
    onp.testing.assert_allclose(second[0], want_a, rtol=1e-12)
    onp.testing.assert_allclose(second[1], want_b, rtol=1e-12)
    with pytest.warns(UserWarning, match="independent of input"):
        zeros = ag.grad(lambda a, b: onp.float64(3.0), (0, 1))(x, y)
    assert all(not z.any() and z.shape == (2,) for z in zeros)
    value, (ga, gb) = ag.value_and_grad(f, (0, 1))(x, y)
    assert value == onp.sum(onp.sin(x) * y * y) and ga.shape == gb.shape == (2,)
    pull_back, out = ag.make_vjp(lambda a, b: np.sin(a) * b, (0, 1))(x, y)
    ga, gb = pull_back(onp.ones(2))
    onp.testing.assert_allclose(ga, onp.cos(x) * y, rtol=1e-15)
    onp.testing.assert_allclose(gb, onp.sin(x), rtol=1e-15)


def test_repeated_item_access_shares_one_tape_node():
    """``params["W"]`` read at every step of a loop (examples/rnn.py:38-44) hands out the box of the first read: the
    gradient is, bit for bit, that of the program which keeps the item in a variable; slices are taken anew."""
    rs = onp.random.RandomState(0)
    params = {"W": rs.randn(4, 4), "b": rs.randn(4)}
    x = rs.randn(3, 4)

    def reads_every_step(p):
        h = x
        for _ in range(5):
            h = np.tanh(np.dot(h, p["W"]) + p["b"])
        return np.sum(h)

    def reads_once(p):
        W, b = p["W"], p["b"]
        h = x
        for _ in range(5):
            h = np.tanh(np.dot(h, W) + b)
        return np.sum(h)

    a, b = ag.grad(reads_every_step)(params), ag.grad(reads_once)(params)
    for key in params:
        onp.testing.assert_array_equal(a[key], b[key])
    seen = []
    ag.grad(lambda t: (seen.append((t[0] is t[0], t[0:1] is t[0:1])) or np.sum(t[0])))([params["W"], params["b"]])
    assert seen[-1] == (True, False)


def test_a_tuple_passed_as_one_argument_stays_a_boxed_container():
    """Only the tuple that several ``argnum`` s build is traced element by element; a caller's own tuple may be
    sliced and returned, or handed to a primitive, which needs the box (autograd/builtins.py:37-96)."""
    from autograd_amd.extend import defvjp, primitive

    x, y, z = onp.array([1.0, 2.0]), onp.array([3.0]), onp.array([4.0, 5.0, 6.0])
    pull_back, out = ag.make_vjp(lambda p: p[1:])((x, y, z))
    assert isinstance(out, tuple) and len(out) == 2
    got = pull_back((onp.array([7.0]), onp.array([1.0, 1.0, 1.0])))
    assert not got[0].any() and got[1][0] == 7.0 and got[2].sum() == 3.0

    @primitive
    def total(parts):
        return onp.float64(sum(float(onp.sum(part)) for part in parts))

    defvjp(total, lambda ans, parts: lambda g: tuple(g * onp.ones_like(part) for part in parts))
    grads = ag.grad(lambda p: total(p) * 2.0)((x, y, z))
    assert [g.tolist() for g in grads] == [[2.0, 2.0], [2.0], [2.0, 2.0, 2.0]]
