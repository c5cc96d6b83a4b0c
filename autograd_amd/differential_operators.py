"""User-facing differential operators, all thin closures over ``make_vjp`` / ``make_jvp``.

Same surface and semantics as the reference's
autograd/differential_operators.py:19-242.  Nothing here touches array data
directly: seeds come from the value's ``VSpace`` and every array operation goes
through the device namespace (``autograd_amd.numpy``).
"""

import warnings
from inspect import getfullargspec as _getargspec

from .builtins import tuple as atuple
from .core import make_jvp as _make_jvp
from .core import make_vjp as _make_vjp
from .extend import defvjp_argnum, primitive, vspace
from .wrap_util import unary_to_nary

make_vjp = unary_to_nary(_make_vjp)
make_jvp = unary_to_nary(_make_jvp)


def _anp(*values):
    """Array namespace to use for ``values``.

    A box class may name the namespace its value type lives in through a
    ``_namespace`` attribute (a callable returning the module); the default is
    the device namespace ``autograd_amd.numpy``.
    """
    from .tracer import Box, getval

    for v in values:
        box_cls = Box.type_mappings.get(type(getval(v)))
        ns = getattr(box_cls, "_namespace", None)
        if ns is not None:
            return ns()
    from . import numpy as anp  # deferred: the device namespace imports this package

    return anp


_SCALAR_ONLY = (
    "{name} only applies to real scalar-output functions. "
    "Try jacobian, elementwise_grad or holomorphic_grad."
)


@unary_to_nary
def grad(fun, x):
    """
    Returns a function which computes the gradient of `fun` with respect to
    positional argument number `argnum`. The returned function takes the same
    arguments as `fun`, but returns the gradient instead. The function `fun`
    should be scalar-valued. The gradient has the same type as the argument."""
    vjp, ans = _make_vjp(fun, x)
    if not vspace(ans).size == 1:
        raise TypeError(_SCALAR_ONLY.format(name="Grad"))
    return vjp(vspace(ans).ones())


@unary_to_nary
def elementwise_grad(fun, x):
    """
    Returns a function that computes the sum of each column of the Jacobian of
    `fun`, in one pass. If the Jacobian is diagonal, then this is the diagonal
    of the Jacobian.
    """
    vjp, ans = _make_vjp(fun, x)
    if vspace(ans).iscomplex:
        raise TypeError("Elementwise_grad only applies to real-output functions.")
    return vjp(vspace(ans).ones())


@unary_to_nary
def deriv(fun, x):
    return _make_jvp(fun, x)(vspace(x).ones())[1]


@unary_to_nary
def jacobian(fun, x):
    """
    Returns a function which computes the Jacobian of `fun` with respect to
    positional argument number `argnum`, which must be a scalar or array. If the
    input has shape (in1, in2, ...) and the output (out1, out2, ...), the
    Jacobian has shape (out1, out2, ..., in1, in2, ...).  One VJP per output
    element (reference differential_operators.py:57-73).
    """
    vjp, ans = _make_vjp(fun, x)
    np = _anp(ans, x)
    ans_vspace = vspace(ans)
    jacobian_shape = ans_vspace.shape + vspace(x).shape
    grads = map(vjp, ans_vspace.standard_basis())
    return np.reshape(np.stack(grads), jacobian_shape)


@unary_to_nary
def holomorphic_grad(fun, x):
    if not vspace(x).iscomplex:
        warnings.warn("Input to holomorphic_grad is not complex")
    np = _anp(x)
    return grad(lambda x: np.real(fun(x)))(x)


def grad_named(fun, argname):
    """Gradient with respect to a named argument (not *args / **kwargs)."""
    return grad(fun, _getargspec(fun).args.index(argname))


@unary_to_nary
def hessian(fun, x):
    "Returns a function that computes the exact Hessian."
    return jacobian(jacobian(fun))(x)


@unary_to_nary
def make_hvp(fun, x):
    """Builds a function for evaluating the Hessian-vector product at a point:
    the VJP of ``grad(fun)`` (reverse-over-reverse), so the forward pass is
    shared between many products at the same point."""
    return _make_vjp(grad(fun), x)


def hessian_tensor_product(fun, argnum=0):
    """Returns a function of (*args, tensor, **kwargs) giving the exact
    Hessian-tensor product."""
    fun_grad = grad(fun, argnum)

    def vector_dot_grad(*args, **kwargs):
        args, vector = args[:-1], args[-1]
        np = _anp(vector)
        return np.tensordot(fun_grad(*args, **kwargs), vector, np.ndim(vector))

    return grad(vector_dot_grad, argnum)


hessian_vector_product = hessian_tensor_product


def tensor_jacobian_product(fun, argnum=0):
    """Returns a function of (*args, tensor, **kwargs) giving the Jacobian
    left-multiplied by tensor."""

    def vector_dot_fun(*args, **kwargs):
        args, vector = args[:-1], args[-1]
        np = _anp(vector)
        return np.tensordot(vector, fun(*args, **kwargs), axes=np.ndim(vector))

    return jacobian(vector_dot_fun, argnum)


vector_jacobian_product = tensor_jacobian_product


@unary_to_nary
def make_jvp_reversemode(fun, x):
    """Jacobian-vector product built from two reverse passes (the VJP is linear
    in its argument, so the VJP of the VJP is the JVP)."""
    vjp, y = _make_vjp(fun, x)
    vjp_vjp, _ = _make_vjp(vjp, vspace(y).zeros())
    return vjp_vjp


def make_ggnvp(f, g=None, f_argnum=0):
    """Generalized-Gauss-Newton-vector products at a point."""
    if g is None:

        def g(x):
            np = _anp(x)
            return 1.0 / 2 * np.sum(x**2, axis=-1)

    @unary_to_nary
    def _make_ggnvp(f, x):
        f_vjp, f_x = _make_vjp(f, x)
        g_hvp, grad_g_x = _make_vjp(grad(g), f_x)
        f_jvp, _ = _make_vjp(f_vjp, vspace(grad_g_x).zeros())

        def ggnvp(v):
            return f_vjp(g_hvp(f_jvp(v)))

        return ggnvp

    return _make_ggnvp(f, f_argnum)


@unary_to_nary
def value_and_grad(fun, x):
    """Returns a function that returns both value and gradient."""
    vjp, ans = _make_vjp(fun, x)
    if not vspace(ans).size == 1:
        raise TypeError(_SCALAR_ONLY.format(name="value_and_grad"))
    return ans, vjp(vspace(ans).ones())


@unary_to_nary
def grad_and_aux(fun, x):
    """Gradient of the first output of a two-output function, plus the
    (unmodified) second output."""
    vjp, (ans, aux) = _make_vjp(lambda x: atuple(fun(x)), x)
    return vjp((vspace(ans).ones(), vspace(aux).zeros())), aux


def multigrad_dict(fun):
    "Takes gradients wrt all arguments simultaneously; returns {argname: grad}."
    import inspect
    from collections import OrderedDict

    sig = inspect.signature(fun)
    params = sig.parameters
    var_pos = [n for n, p in params.items() if p.kind == p.VAR_POSITIONAL]
    var_kwd = [n for n, p in params.items() if p.kind == p.VAR_KEYWORD]
    plain = [n for n in params if n not in var_pos + var_kwd]

    def gradfun(*args, **kwargs):
        bound = sig.bind(*args, **kwargs)
        argdict = OrderedDict()
        for name, p in params.items():
            if name in bound.arguments:
                argdict[name] = bound.arguments[name]
            elif p.default is not p.empty:
                argdict[name] = p.default

        def newfun(dct):
            pos = tuple(dct[n] for n in plain) + (tuple(dct[var_pos[0]]) if var_pos else ())
            kw = {k: dct[var_kwd[0]][k] for k in dct[var_kwd[0]]} if var_kwd else {}
            return fun(*pos, **kw)

        grad_dict = grad(newfun)(dict(argdict))
        return OrderedDict((name, grad_dict[name]) for name in argdict)

    return gradfun


def checkpoint(fun):
    """Gradient checkpointing: intermediate values of ``fun`` are dropped after
    the forward pass and recomputed when its VJP is needed."""

    def wrapped_grad(argnum, ans, args, kwargs):
        return make_vjp(fun, argnum)(*args, **kwargs)[0]

    wrapped = primitive(fun)
    defvjp_argnum(wrapped, wrapped_grad)
    return wrapped
