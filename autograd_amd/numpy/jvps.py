"""Forward-mode rules of the device namespace.

The part of the reference's autograd/numpy/numpy_jvps.py that the hot path touches (line
numbers in the comments).  Linear functions use ``"same"`` / ``def_linear`` (the primitive
applied to the tangent, i.e. the same kernels); non-linear ufuncs reuse the fused
single-kernel forms of the reverse rules when their operands are concrete.
"""

import numpy as onp

from .._lib import Op
from ..extend import JVPNode, def_linear, defjvp, defjvp_argnum, register_notrace, vspace
from ..tracer import isbox
from ..util import func
from . import devarray as D
from . import wrapper as anp
from .boxes import DevArrayBox
from .vjps import (
    _float64_zeros,
    _strong_scalar,
    balanced_eq,
    dot_adjoint_0,
    dot_adjoint_1,
    nograd_functions,
    replace_zero,
    tensordot_adjoint_0,
    tensordot_adjoint_1,
    untake,
)

for _f in nograd_functions:
    register_notrace(JVPNode, _f)


def _concrete(*xs):
    for x in xs:
        if isbox(x):
            return False
    return True


def broadcast(x, target):
    """Tangent of a broadcast operand brought to the result's shape (numpy_jvps.py:291-300):
    a stride-0 view instead of the reference's ``repeat`` copies."""
    target_shape, target_ndim, _dtype, _c = anp.metadata(target)
    while anp.ndim(x) < target_ndim:
        x = anp.expand_dims(x, 0)
    if anp.shape(x) != target_shape:
        x = anp.broadcast_to(x, target_shape)
    return x


def _fused_or(op, operands, traced):
    if _concrete(*operands):
        return D.float_map(op, *operands)
    return traced()


# indexing and array construction (23-32)
defjvp(func(DevArrayBox.__getitem__), "same")
defjvp(untake, "same")
defjvp_argnum(anp.array_from_args, lambda argnum, g, ans, args, kwargs: untake(g, argnum - 2, vspace(ans)))
defjvp(
    anp._array_from_scalar_or_array,
    None,
    None,
    lambda g, ans, args, kwargs, _: anp._array_from_scalar_or_array(args, kwargs, g),
)

defjvp(anp.full, "same", argnums=(1,))  # numpy_jvps.py:33
for _flat in (anp.imag, anp.angle):  # numpy_jvps.py:142-146 for a real argument: a zero tangent
    defjvp(_flat, lambda g, ans, x: anp.zeros_like(ans))
defjvp(  # numpy_jvps.py:169-173
    anp.linspace,
    lambda g, ans, start, stop, *args, **kwargs: anp.linspace(g, 0, *args, **kwargs),
    lambda g, ans, start, stop, *args, **kwargs: anp.linspace(0, g, *args, **kwargs),
)

# binary ufuncs (38-74)
def_linear(anp.multiply)
defjvp(anp.add, lambda g, ans, x, y: broadcast(g, ans), lambda g, ans, x, y: broadcast(g, ans))
defjvp(anp.subtract, lambda g, ans, x, y: broadcast(g, ans), lambda g, ans, x, y: broadcast(-g, ans))
defjvp(
    anp.true_divide,
    "same",
    lambda g, ans, x, y: _fused_or(Op.DIV_VJP1, (g, x, y), lambda: -g * x / y**2),
)
defjvp(
    anp.power,
    lambda g, ans, x, y: _fused_or(Op.POW_VJP0, (g, x, y), lambda: g * y * x ** anp.where(y, y - 1, 1.0)),
    lambda g, ans, x, y: _fused_or(Op.POW_VJP1, (g, _strong_scalar(x), ans),
                                   lambda: g * anp.log(replace_zero(x, 1.0)) * ans),
)
defjvp(  # numpy_jvps.py:67-68 (numpy.mod is the same function)
    anp.remainder,
    lambda g, ans, x, y: broadcast(g, ans),
    lambda g, ans, x, y: -g * anp.floor(x / y),
)
defjvp(anp.nan_to_num, lambda g, ans, x: anp.where(anp.isfinite(x), g, 0.0))  # numpy_jvps.py:35
defjvp(anp.kron, "same", "same")  # numpy_jvps.py:155


def _sort_tangent(g, x, axis):  # numpy_jvps.py:256-271 (sort and partition alike): the tangent in sorted order
    if axis is None:
        order_, rank = anp.sort_permutations(anp.ravel(x), 0)
        return anp._reorder(anp.ravel(g), order_, rank, 0)
    order_, rank = anp.sort_permutations(x, axis)
    return anp._reorder(g, order_, rank, axis)


defjvp(anp.sort, lambda g, ans, x, axis=-1, kind=None, order=None: _sort_tangent(g, x, axis))
defjvp(anp.partition, lambda g, ans, x, kth, axis=-1, kind="introselect", order=None: _sort_tangent(g, x, axis))
defjvp(anp._reorder, "same")
def_linear(anp.cross)  # numpy_jvps.py:106
defjvp(anp.logaddexp2, lambda g, ans, x, y: g * 2 ** (x - ans), lambda g, ans, x, y: g * 2 ** (y - ans))  # 65
defjvp(  # numpy_jvps.py:135-138
    anp.sinc,
    lambda g, ans, x: g * (anp.cos(anp.pi * x) * anp.pi * x - anp.sin(anp.pi * x)) / (anp.pi * x**2),
)
for _chooser in (anp.maximum, anp.minimum, anp.fmax, anp.fmin):
    defjvp(
        _chooser,
        lambda g, ans, x, y: g * balanced_eq(x, ans, y),
        lambda g, ans, x, y: g * balanced_eq(y, ans, x),
    )

def_linear(anp.einsum)  # numpy_jvps.py:287
defjvp(anp.pad, lambda g, ans, array, width, mode, **kwargs: anp.pad(g, width, mode))  # numpy_jvps.py:303

# linear one-argument functions (77-105, 150-162)
for _name in (
    "negative reshape ravel expand_dims squeeze swapaxes moveaxis broadcast_to repeat transpose sum "
    "_primitive_mean roll diag diagonal make_diagonal trace triu tril tile real real_if_close conjugate flipud fliplr flip rot90 "
    "array_split split vsplit hsplit dsplit rollaxis diff cumsum"
).split():
    defjvp(getattr(anp, _name), "same")

# unary ufuncs (108-134)
defjvp(anp.exp, lambda g, ans, x: ans * g)
defjvp(anp.log, lambda g, ans, x: g / x)
defjvp(anp.tanh, lambda g, ans, x: _fused_or(Op.TANH_VJP, (g, x), lambda: g / anp.cosh(x) ** 2))
defjvp(anp.sinh, lambda g, ans, x: _fused_or(Op.SINH_VJP, (g, x), lambda: g * anp.cosh(x)))
defjvp(anp.cosh, lambda g, ans, x: _fused_or(Op.COSH_VJP, (g, x), lambda: g * anp.sinh(x)))
defjvp(anp.sin, lambda g, ans, x: _fused_or(Op.SIN_VJP, (g, x), lambda: g * anp.cos(x)))
defjvp(anp.cos, lambda g, ans, x: _fused_or(Op.COS_VJP, (g, x), lambda: -g * anp.sin(x)))
defjvp(anp.sqrt, lambda g, ans, x: _fused_or(Op.SQRT_VJP, (g, x), lambda: g * 0.5 * x**-0.5))
defjvp(anp.square, lambda g, ans, x: _fused_or(Op.SQUARE_VJP, (g, x), lambda: g * 2 * x))
defjvp(anp.reciprocal, lambda g, ans, x: _fused_or(Op.RECIPROCAL_VJP, (g, x), lambda: -g / x**2))
defjvp(anp.log1p, lambda g, ans, x: _fused_or(Op.LOG1P_VJP, (g, x), lambda: g / (x + 1)))
defjvp(anp.expm1, lambda g, ans, x: _fused_or(Op.EXPM1_VJP, (g, ans), lambda: (ans + 1) * g))
defjvp(
    anp.abs,
    lambda g, ans, x: _fused_or(
        Op.ABS_VJP, (g, x, ans), lambda: g * replace_zero(x, 0.0) / replace_zero(ans, 1.0)
    ),
)
# the rest of the table (numpy_jvps.py:63-73, 108-147)
defjvp(anp.logaddexp, lambda g, ans, x, y: g * anp.exp(x - ans), lambda g, ans, x, y: g * anp.exp(y - ans))
defjvp(anp.arctan2, lambda g, ans, x, y: g * y / (x**2 + y**2), lambda g, ans, x, y: g * -x / (x**2 + y**2))
defjvp(anp.hypot, lambda g, ans, x, y: g * x / ans, lambda g, ans, x, y: g * y / ans)
defjvp(anp.fabs, lambda g, ans, x: anp.sign(x) * g)
defjvp(anp.exp2, lambda g, ans, x: ans * anp.log(2) * g)
defjvp(anp.log2, lambda g, ans, x: g / x / anp.log(2))
defjvp(anp.log10, lambda g, ans, x: g / x / anp.log(10))
defjvp(anp.tan, lambda g, ans, x: g / anp.cos(x) ** 2)
defjvp(anp.arcsin, lambda g, ans, x: g / anp.sqrt(1 - x**2))
defjvp(anp.arccos, lambda g, ans, x: -g / anp.sqrt(1 - x**2))
defjvp(anp.arctan, lambda g, ans, x: g / (1 + x**2))
defjvp(anp.arcsinh, lambda g, ans, x: g / anp.sqrt(x**2 + 1))
defjvp(anp.arccosh, lambda g, ans, x: g / anp.sqrt(x**2 - 1))
defjvp(anp.arctanh, lambda g, ans, x: g / (1 - x**2))
defjvp(anp.rad2deg, "same")  # numpy_jvps.py:78-81: the function itself applied to the tangent
defjvp(anp.deg2rad, "same")
defjvp(anp.clip, lambda g, ans, x, a_min, a_max: g * anp.logical_and(ans != a_min, ans != a_max))

def _like_result(ans, tangent):
    """A tangent of ``where`` in the result's shape, also when the other choice is what made the result larger."""
    return tangent if anp.shape(tangent) == anp.shape(ans) else anp.broadcast_to(tangent, anp.shape(ans))


defjvp(
    anp._where3,
    None,
    # numpy_jvps.py:150-151: float64 zeros, so a float32 tangent comes out float64
    lambda g, ans, c, x, y: _like_result(ans, anp.where(c, g, _float64_zeros(anp.shape(g)))),
    lambda g, ans, c, x, y: _like_result(ans, anp.where(c, _float64_zeros(anp.shape(g)), g)),
)
defjvp(anp.astype, lambda g, ans, A, dtype, *a, **k: anp.astype(g, dtype))
defjvp(
    anp.prod,
    lambda g, ans, x, axis=None, keepdims=False, **kwargs: ans * anp.sum(g / x, axis=axis, keepdims=keepdims),
)


def _count(shape, axis):
    n = 1
    for d in D.normalize_axes(axis, len(shape)):
        n *= shape[d]
    return n


def _fwd_var(g, ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_jvps.py:165-177
    x_minus_mean = x - anp.mean(x, axis=axis, keepdims=True)
    return 2.0 * anp.sum(g * x_minus_mean, axis=axis, keepdims=keepdims) / (_count(anp.shape(g), axis) - ddof)


def _fwd_std(g, ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_jvps.py:180-193
    num_reps = _count(anp.shape(g), axis)
    if num_reps <= 1:
        return anp.zeros_like(ans)
    x_minus_mean = x - anp.mean(x, axis=axis, keepdims=True)
    return anp.sum(g * x_minus_mean, axis=axis, keepdims=keepdims) / ((num_reps - ddof) * ans)


defjvp(anp._primitive_var, _fwd_var)
defjvp(anp._primitive_std, _fwd_std)


def _fwd_chooser(g, ans, x, axis=None, keepdims=False, **kwargs):
    # numpy_jvps.py:196-215
    if anp.isscalar(x):
        return g
    if not keepdims:
        if isinstance(axis, int):
            ans = anp.expand_dims(ans, axis)
        elif isinstance(axis, tuple):
            for ax in sorted(axis):
                ans = anp.expand_dims(ans, ax)
        elif axis is None:
            ans = anp.reshape(ans, (1,) * anp.ndim(x))
    # the reference multiplies by the boolean mask and divides by its integer sum: float64 results
    chosen = anp.astype(x == ans, onp.float64)
    return anp.sum(g * chosen, axis=axis, keepdims=keepdims) / anp.sum(chosen, axis=axis, keepdims=keepdims)


defjvp(anp.max, _fwd_chooser)
defjvp(anp.min, _fwd_chooser)

# contractions (230-240)
for _f in (anp.matmul, anp.dot, anp.tensordot, anp.outer, anp.inner):
    def_linear(_f)
for _f in (dot_adjoint_0, dot_adjoint_1, tensordot_adjoint_0, tensordot_adjoint_1):
    def_linear(_f)


def _fwd_concatenate_args(argnum, g, ans, axis_args, kwargs):
    parts = [g if i == argnum else anp.zeros_like(axis_args[i]) for i in range(1, len(axis_args))]
    return anp.concatenate_args(axis_args[0], *parts)


defjvp_argnum(anp.concatenate_args, _fwd_concatenate_args)


def _atleast_jvp(fun):
    def jvp(g, ans, *arys):
        if len(arys) > 1:
            raise NotImplementedError("Can't handle multiple arguments yet.")
        return fun(g)

    return jvp


for _f in (anp.atleast_1d, anp.atleast_2d, anp.atleast_3d):
    defjvp(_f, _atleast_jvp(_f))
