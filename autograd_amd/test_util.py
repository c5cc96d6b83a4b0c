"""Derivative checker used by the tests and offered to authors of new primitives.

Same checks and names as the reference's autograd/test_util.py:6-91.  A VJP is checked through the
identity <x_v, vjp(y_v)> == <y_v, J x_v>, with J x_v taken by central differences; a JVP by
projecting it and the same numerical J x_v on one random direction; higher orders by recursing on
(x, v) -> vjp(v) / jvp(v).  Everything goes through the value's ``VSpace``, so any registered value
type (device arrays, containers of them, floats) can be checked.
"""

from itertools import product

from .core import make_jvp, make_vjp, vspace
from .wrap_util import get_name, unary_to_nary

TOL = 1e-6
RTOL = 1e-6
EPS = 1e-6


def scalar_close(a, b):
    """Absolute OR relative agreement of two scalars (device scalars are read back)."""
    gap = abs(float(a) - float(b))
    return gap < TOL or gap / abs(float(a) + float(b)) < RTOL


def make_numerical_jvp(f, x):
    """``v -> (f(x + EPS/2 v) - f(x - EPS/2 v)) / EPS`` with the arithmetic of the values' vector spaces."""
    x_vs, y_vs = vspace(x), vspace(f(x))

    def moved(v, step):
        return f(x_vs.add(x, x_vs.scalar_mul(v, step)))

    def jvp(v):
        rise = y_vs.add(moved(v, EPS / 2), y_vs.scalar_mul(moved(v, -EPS / 2), -1.0))
        return y_vs.scalar_mul(rise, 1.0 / EPS)

    return jvp


def check_vjp(f, x):
    vjp, y = make_vjp(f, x)
    x_vs, y_vs = vspace(x), vspace(y)
    x_v, y_v = x_vs.randn(), y_vs.randn()
    pulled_back = x_vs.covector(vjp(y_vs.covector(y_v)))
    assert vspace(pulled_back) == x_vs, f"VSpace mismatch:\nvjp: {vspace(pulled_back)}\nx:   {x_vs}"
    analytic = x_vs.inner_prod(x_v, pulled_back)
    numeric = y_vs.inner_prod(y_v, make_numerical_jvp(f, x)(x_v))
    assert scalar_close(numeric, analytic), (
        f"Derivative (VJP) check of {get_name(f)} failed with arg {x}:\nanalytic: {analytic}\nnumeric:  {numeric}"
    )


def check_jvp(f, x):
    direction = vspace(x).randn()
    check_equivalent(make_jvp(f, x)(direction)[1], make_numerical_jvp(f, x)(direction))


def check_equivalent(x, y):
    """Same vector space, and the same projection on one random vector of it."""
    x_vs, y_vs = vspace(x), vspace(y)
    assert x_vs == y_vs, f"VSpace mismatch:\nx: {x_vs}\ny: {y_vs}"
    probe = x_vs.randn()
    assert scalar_close(x_vs.inner_prod(x, probe), x_vs.inner_prod(y, probe)), f"Value mismatch:\nx: {x}\ny: {y}"


def _next_order(f, mode):
    """(x, v) -> the derivative of ``f`` at ``x`` applied to ``v``: what the next order differentiates."""
    if mode == "fwd":
        derived = lambda x, v: make_jvp(f, x)(v)[1]  # noqa: E731
    else:
        derived = lambda x, v: make_vjp(f, x)[0](v)  # noqa: E731
    derived.__name__ = ("jvp_" if mode == "fwd" else "vjp_") + get_name(f)
    return derived


@unary_to_nary
def check_grads(f, x, modes=None, order=2):
    modes = ["fwd", "rev"] if modes is None else modes
    assert all(m in ["fwd", "rev"] for m in modes)
    for mode, check in (("fwd", check_jvp), ("rev", check_vjp)):
        if mode not in modes:
            continue
        check(f, x)
        if order > 1:
            # forward mode is seeded from the input's space, reverse mode from the output's
            seed = vspace(x if mode == "fwd" else f(x)).randn()
            check_grads(_next_order(f, mode), (0, 1), modes, order=order - 1)(x, seed)


def combo_check(fun, *args, **kwargs):
    """``check_grads(fun, *args, **kwargs)`` over every combination of the given argument / keyword choices."""

    def run(*arg_choices, **kwarg_choices):
        keys = list(kwarg_choices)
        for chosen in product(*arg_choices):
            for values in product(*(kwarg_choices[k] for k in keys)):
                check_grads(fun, *args, **kwargs)(*chosen, **dict(zip(keys, values)))

    return run
