"""Differentiable fixed-point iteration (reference autograd/misc/fixed_points.py:6-26).

``fixed_point(f, a, x0, distance, tol)`` iterates ``x <- f(a)(x)`` from ``x0`` until two successive iterates are
closer than ``tol`` under ``distance``.  Its derivative with respect to ``a`` does not unroll the loop: at the
fixed point x* = f(a)(x*), the cotangent is  vjp_a( w )  where  w = g + J_x^T w  is itself found by the same
iteration (J_x is the Jacobian of f(a) at x*).  With device arrays, every step of both loops is kernel launches.
"""

from .. import make_vjp
from ..builtins import tuple as traced_tuple
from ..extend import defvjp, primitive, vspace


@primitive
def fixed_point(f, a, x0, distance, tol):
    step = f(a)
    before, x = x0, step(x0)
    while distance(x, before) > tol:
        before, x = x, step(x)
    return x


def _fixed_point_cotangent(ans, f, a, x0, distance, tol):
    pull_back_a, _ = make_vjp(lambda p, x: f(p)(x))(a, ans)

    def iteration(packed):
        p, at, g = packed
        pull_back_x, _ = make_vjp(f(p))(at)
        space = vspace(at)
        return lambda w: space.add(pull_back_x(w), g)

    return lambda g: pull_back_a(fixed_point(iteration, traced_tuple((a, ans, g)), vspace(x0).zeros(), distance, tol))


defvjp(fixed_point, None, _fixed_point_cotangent, None)
