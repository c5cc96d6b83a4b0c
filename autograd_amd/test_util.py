"""Derivative checker used by the tests and offered to authors of new primitives.

The construction is the reference's (autograd/test_util.py:6-91): a VJP is
checked through the identity <x_v, vjp(y_v)> == <y_v, J x_v> with J x_v taken by
central differences, a JVP by a random projection of the same numerical JVP,
and higher orders by recursing on (x, v) -> vjp(v) / jvp(v).  Everything goes
through the value's ``VSpace`` so it works for any registered value type.
"""

from itertools import product

from .core import make_jvp, make_vjp, vspace
from .wrap_util import get_name, unary_to_nary

TOL = 1e-6
RTOL = 1e-6
EPS = 1e-6


def scalar_close(a, b):
    a, b = float(a), float(b)
    return abs(a - b) < TOL or abs(a - b) / abs(a + b) < RTOL


def make_numerical_jvp(f, x):
    y = f(x)
    x_vs, y_vs = vspace(x), vspace(y)

    def jvp(v):
        hi = f(x_vs.add(x, x_vs.scalar_mul(v, EPS / 2)))
        lo = f(x_vs.add(x, x_vs.scalar_mul(v, -EPS / 2)))
        diff = y_vs.add(hi, y_vs.scalar_mul(lo, -1.0))
        return y_vs.scalar_mul(diff, 1.0 / EPS)

    return jvp


def check_vjp(f, x):
    vjp, y = make_vjp(f, x)
    jvp = make_numerical_jvp(f, x)
    x_vs, y_vs = vspace(x), vspace(y)
    x_v, y_v = x_vs.randn(), y_vs.randn()

    vjp_y = x_vs.covector(vjp(y_vs.covector(y_v)))
    assert vspace(vjp_y) == x_vs, f"VSpace mismatch:\nvjp: {vspace(vjp_y)}\nx:   {x_vs}"
    vjv_exact = x_vs.inner_prod(x_v, vjp_y)
    vjv_numeric = y_vs.inner_prod(y_v, jvp(x_v))
    assert scalar_close(vjv_numeric, vjv_exact), (
        f"Derivative (VJP) check of {get_name(f)} failed with arg {x}:\n"
        f"analytic: {vjv_exact}\nnumeric:  {vjv_numeric}"
    )


def check_jvp(f, x):
    jvp = make_jvp(f, x)
    jvp_numeric = make_numerical_jvp(f, x)
    x_v = vspace(x).randn()
    check_equivalent(jvp(x_v)[1], jvp_numeric(x_v))


def check_equivalent(x, y):
    x_vs, y_vs = vspace(x), vspace(y)
    assert x_vs == y_vs, f"VSpace mismatch:\nx: {x_vs}\ny: {y_vs}"
    v = x_vs.randn()
    assert scalar_close(x_vs.inner_prod(x, v), x_vs.inner_prod(y, v)), f"Value mismatch:\nx: {x}\ny: {y}"


@unary_to_nary
def check_grads(f, x, modes=None, order=2):
    if modes is None:
        modes = ["fwd", "rev"]
    assert all(m in ["fwd", "rev"] for m in modes)
    if "fwd" in modes:
        check_jvp(f, x)
        if order > 1:

            def grad_f(x, v):
                return make_jvp(f, x)(v)[1]

            grad_f.__name__ = f"jvp_{get_name(f)}"
            v = vspace(x).randn()
            check_grads(grad_f, (0, 1), modes, order=order - 1)(x, v)
    if "rev" in modes:
        check_vjp(f, x)
        if order > 1:

            def grad_f(x, v):
                return make_vjp(f, x)[0](v)

            grad_f.__name__ = f"vjp_{get_name(f)}"
            v = vspace(f(x)).randn()
            check_grads(grad_f, (0, 1), modes, order=order - 1)(x, v)


def combo_check(fun, *args, **kwargs):
    """Run ``check_grads`` over the product of the given argument/kwarg choices."""

    def _combo_check(*arg_choices, **kwarg_choices):
        kw_lists = [[(k, v) for v in vs] for k, vs in kwarg_choices.items()]
        for chosen_args in product(*arg_choices):
            for chosen_kw in product(*kw_lists):
                check_grads(fun, *args, **kwargs)(*chosen_args, **dict(chosen_kw))

    return _combo_check
