"""User-facing differential operators: closures over ``make_vjp`` / ``make_jvp``.

Same surface and semantics as the reference's autograd/differential_operators.py:19-242 (names,
argument meaning, error messages).  Nothing here touches array data directly: seeds come from the
value's ``VSpace`` and every array operation goes through the value type's array namespace, by
default the device namespace ``autograd_amd.numpy``.

Operators decorated with ``unary_to_nary`` are written for a function of one argument and a point;
the decorator makes them ``op(fun, argnum=0)(*args, **kwargs)`` for any argument position(s).
"""

import inspect
import warnings
from collections import OrderedDict

from . import core
from .builtins import tuple as atuple
from .extend import defvjp_argnum, primitive, vspace
from .wrap_util import unary_to_nary

make_vjp = unary_to_nary(core.make_vjp)
make_jvp = unary_to_nary(core.make_jvp)


def _anp(*values):
    """Array namespace to use for ``values``.

    A box class may name the namespace its value type lives in through a ``_namespace`` attribute
    (a callable returning the module); the default is the device namespace ``autograd_amd.numpy``.
    """
    from .tracer import Box, getval

    for v in values:
        box_cls = Box.type_mappings.get(type(getval(v)))
        ns = getattr(box_cls, "_namespace", None)
        if ns is not None:
            return ns()
    from . import numpy as anp  # deferred: the device namespace imports this package

    return anp


def _seeded_with_ones(fun, x, who=None):
    """``(fun(x), cotangent of x for a cotangent of ones on fun(x))``.  With ``who`` given the output
    has to be a single real number, and ``who`` is named in the error otherwise."""
    pull_back, ans = core.make_vjp(fun, x)
    out_space = vspace(ans)
    if who is not None and out_space.size != 1:
        raise TypeError(
            f"{who} only applies to real scalar-output functions. "
            "Try jacobian, elementwise_grad or holomorphic_grad."
        )
    return ans, pull_back(out_space.ones())


@unary_to_nary
def grad(fun, x):
    """Gradient of a scalar-valued ``fun`` with respect to its argument number ``argnum``: a function
    of the same arguments as ``fun`` whose result has the type and structure of that argument."""
    return _seeded_with_ones(fun, x, "Grad")[1]


@unary_to_nary
def value_and_grad(fun, x):
    """Like ``grad``, returning ``(fun's value, gradient)`` from the one forward pass."""
    value, gradient = _seeded_with_ones(fun, x, "value_and_grad")
    settle = getattr(core, "settle", None)  # (a hosting package's core has none: values then stay as they are)
    return (settle(value) if settle is not None else value), gradient  # deferred arithmetic is completed here, as the gradient's is


@unary_to_nary
def elementwise_grad(fun, x):
    """Column sums of the Jacobian of ``fun`` in one backward pass (the cotangent seed is all ones);
    for a function acting element by element this is its derivative at every element."""
    pull_back, ans = core.make_vjp(fun, x)
    out_space = vspace(ans)
    if out_space.iscomplex:
        raise TypeError("Elementwise_grad only applies to real-output functions.")
    return pull_back(out_space.ones())


@unary_to_nary
def deriv(fun, x):
    """Forward-mode derivative along the all-ones direction of the input."""
    return core.make_jvp(fun, x)(vspace(x).ones())[1]


JACOBIAN_BLOCK_BYTES = 4 << 30  # what the stacked cotangents of one replay of `jacobian` may hold (estimate, see there)


@unary_to_nary
def jacobian(fun, x):
    """Jacobian of an array-valued ``fun`` of an array (or scalar): output axes first, input axes
    last.  The reference runs one backward pass per output element, each seeded with a standard basis
    vector of the output space (differential_operators.py:57-73); here the basis vectors go through the
    tape together, stacked along a leading axis (``core.batched_backward_pass``), when the value type
    offers ``stacked_standard_basis``; the per-element loop remains for value types that do not."""
    pull_back, pull_back_all, ans = core.make_vjp_and_batched(fun, x)
    np = _anp(ans, x)
    out_space, in_space = vspace(ans), vspace(x)
    stacked_basis = getattr(out_space, "stacked_standard_basis", None)
    if pull_back_all is not None and stacked_basis is not None and out_space.size > 0 and type(in_space) is type(out_space):
        # all basis cotangents in ONE replay of the tape, stacked along a leading axis; every cotangent on the tape then
        # carries that axis, so a large output space goes through in blocks of basis vectors that keep the stacked
        # values within a byte budget (a tape is taken to hold a few values of about its larger end's size per vector)
        n = out_space.size
        per_vector = 16 * max(in_space.size, n, 1) * getattr(getattr(out_space, "dtype", None), "itemsize", 8)
        block = max(1, min(n, JACOBIAN_BLOCK_BYTES // per_vector))
        try:
            basis = stacked_basis()
            if block >= n:
                rows = pull_back_all(basis, n, lambda value, i: value[i], np.stack)
            else:
                rows = np.concatenate([pull_back_all(basis[k:k + block], min(block, n - k), lambda value, i: value[i], np.stack)
                                       for k in range(0, n, block)], axis=0)
            return np.reshape(rows, out_space.shape + in_space.shape)
        except core.NotBatchable:
            pass
    rows = [pull_back(unit) for unit in out_space.standard_basis()]
    return np.reshape(np.stack(rows), out_space.shape + in_space.shape)


@unary_to_nary
def hessian(fun, x):
    """Exact Hessian: the Jacobian of the Jacobian (for scalar ``fun``, of the gradient)."""
    return jacobian(jacobian(fun))(x)


@unary_to_nary
def holomorphic_grad(fun, x):
    if not vspace(x).iscomplex:
        warnings.warn("Input to holomorphic_grad is not complex")
    np = _anp(x)
    return grad(lambda z: np.real(fun(z)))(x)


def grad_named(fun, argname):
    """Gradient with respect to the positional argument called ``argname``."""
    position = inspect.getfullargspec(fun).args.index(argname)
    return grad(fun, position)


@unary_to_nary
def make_hvp(fun, x):
    """``(hvp, gradient at x)`` where ``hvp(v)`` is the Hessian of ``fun`` at ``x`` times ``v``:
    the VJP of ``grad(fun)`` (reverse over reverse), so one forward pass serves many products."""
    return core.make_vjp(grad(fun), x)


def _split_last(args):
    return args[:-1], args[-1]


def hessian_tensor_product(fun, argnum=0):
    """Function of ``(*args, tensor, **kwargs)``: the Hessian of ``fun`` contracted with ``tensor``,
    as the gradient of <grad fun, tensor> (no Hessian is formed)."""
    first_derivative = grad(fun, argnum)

    def contracted_gradient(*args, **kwargs):
        point, tensor = _split_last(args)
        np = _anp(tensor)
        return np.tensordot(first_derivative(*point, **kwargs), tensor, np.ndim(tensor))

    return grad(contracted_gradient, argnum)


def tensor_jacobian_product(fun, argnum=0):
    """Function of ``(*args, tensor, **kwargs)``: ``tensor`` contracted with the output axes of the
    Jacobian of ``fun``."""

    def contracted_output(*args, **kwargs):
        point, tensor = _split_last(args)
        np = _anp(tensor)
        return np.tensordot(tensor, fun(*point, **kwargs), axes=np.ndim(tensor))

    return jacobian(contracted_output, argnum)


hessian_vector_product = hessian_tensor_product
vector_jacobian_product = tensor_jacobian_product


def _transpose_of(linear_map, like):
    """The VJP of a linear map (linear maps are their own derivative), seeded at zero."""
    return core.make_vjp(linear_map, vspace(like).zeros())[0]


@unary_to_nary
def make_jvp_reversemode(fun, x):
    """Jacobian-vector products from reverse mode only: the VJP is linear in its cotangent, so its
    own VJP is multiplication by the Jacobian.  Pays off when many products are taken at one point."""
    pull_back, y = core.make_vjp(fun, x)
    return _transpose_of(pull_back, y)


def make_ggnvp(f, g=None, f_argnum=0):
    """Generalized Gauss-Newton vector products of ``g(f(x))`` at a point: ``v -> J' H_g J v``.
    ``g`` defaults to half the squared norm along the last axis."""
    if g is None:

        def g(y):
            return 1.0 / 2 * _anp(y).sum(y**2, axis=-1)

    @unary_to_nary
    def at_point(f, x):
        j_transposed, y = core.make_vjp(f, x)
        hessian_of_g, dg = core.make_vjp(grad(g), y)
        j = _transpose_of(j_transposed, dg)
        return lambda v: j_transposed(hessian_of_g(j(v)))

    return at_point(f, f_argnum)


@unary_to_nary
def grad_and_aux(fun, x):
    """For ``fun`` returning ``(value, aux)``: the gradient of ``value`` and ``aux`` as it is."""
    pull_back, (ans, aux) = core.make_vjp(lambda arg: atuple(fun(arg)), x)
    seed = (vspace(ans).ones(), vspace(aux).zeros())
    return pull_back(seed), aux


def multigrad_dict(fun):
    """Gradients with respect to all arguments at once, as an ordered ``{argument name: gradient}``;
    ``*args`` / ``**kwargs`` of ``fun`` appear under their own names as a tuple / dict of gradients."""
    signature = inspect.signature(fun)
    kinds = {name: p.kind for name, p in signature.parameters.items()}
    star = [n for n, k in kinds.items() if k == inspect.Parameter.VAR_POSITIONAL]
    double_star = [n for n, k in kinds.items() if k == inspect.Parameter.VAR_KEYWORD]
    named = [n for n in kinds if n not in star + double_star]

    def call_with(values):
        positional = tuple(values[n] for n in named)
        if star:
            positional += tuple(values[star[0]])
        keywords = {k: values[double_star[0]][k] for k in values[double_star[0]]} if double_star else {}
        return fun(*positional, **keywords)

    def gradfun(*args, **kwargs):
        given = signature.bind(*args, **kwargs).arguments
        values = OrderedDict()
        for name, p in signature.parameters.items():
            if name in given:
                values[name] = given[name]
            elif p.default is not p.empty:
                values[name] = p.default
        gradients = grad(call_with)(dict(values))
        return OrderedDict((name, gradients[name]) for name in values)

    return gradfun


def checkpoint(fun):
    """``fun`` as a primitive that keeps no intermediate values: its VJP traces ``fun`` again when
    the backward pass gets there (memory for recomputation)."""
    as_primitive = primitive(fun)
    defvjp_argnum(as_primitive, lambda argnum, ans, args, kwargs: make_vjp(fun, argnum)(*args, **kwargs)[0])
    return as_primitive
