"""Forward-mode rules of the oracle's NumPy value type.

Restates the part of the reference's autograd/numpy/numpy_jvps.py that the hot
path touches (line numbers in the comments).  TEST INFRASTRUCTURE: see
``oracle/__init__.py``.
"""

from autograd_amd.extend import JVPNode, def_linear, defjvp, defjvp_argnum, register_notrace, vspace
from autograd_amd.util import func

from . import np_namespace as anp
from .np_boxes import ArrayBox
from .np_vjps import (
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


def broadcast(x, target):
    """Repeat size-1 axes of ``x`` until it has ``target``'s shape (numpy_jvps.py:291-300)."""
    target_shape, target_ndim, _dtype, target_iscomplex = anp.metadata(target)
    while anp.ndim(x) < target_ndim:
        x = anp.expand_dims(x, 0)
    for axis, size in enumerate(anp.shape(x)):
        if size == 1:
            x = anp.repeat(x, target_shape[axis], axis=axis)
    if target_iscomplex and not anp.iscomplexobj(x):
        x = x + 0j
    return x


# contractions (230-240)
for _f in (anp.inner, anp.matmul, anp.dot, anp.tensordot, anp.outer, anp.einsum, anp.cross):
    def_linear(_f)
for _f in (dot_adjoint_0, dot_adjoint_1, tensordot_adjoint_0, tensordot_adjoint_1):
    def_linear(_f)


def _num_reps(g, axis):
    if axis is None:
        return anp.size(g)
    if isinstance(axis, int):
        return anp.shape(g)[axis]
    return anp.prod(anp.array(anp.shape(g))[list(axis)])


def _fwd_var(g, ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_jvps.py:165-177
    num_reps = _num_reps(g, axis)
    x_minus_mean = anp.conj(x - anp.mean(x, axis=axis, keepdims=True))
    return 2.0 * anp.sum(anp.real(g * x_minus_mean), axis=axis, keepdims=keepdims) / (num_reps - ddof)


def _fwd_std(g, ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_jvps.py:180-193
    num_reps = _num_reps(g, axis)
    if num_reps <= 1:
        return anp.zeros_like(ans)
    x_minus_mean = anp.conj(x - anp.mean(x, axis=axis, keepdims=True))
    return anp.sum(anp.real(g * x_minus_mean), axis=axis, keepdims=keepdims) / ((num_reps - ddof) * ans)


defjvp(anp._primitive_var, _fwd_var)
defjvp(anp._primitive_std, _fwd_std)


def _fwd_chooser(g, ans, x, axis=None, keepdims=False, **kwargs):
    if anp.isscalar(x):
        return g
    if not keepdims:
        if isinstance(axis, int):
            ans = anp.expand_dims(ans, axis)
        elif isinstance(axis, tuple):
            for ax in sorted(axis):
                ans = anp.expand_dims(ans, ax)
    chosen = x == ans
    return anp.sum(g * chosen, axis=axis, keepdims=keepdims) / anp.sum(chosen, axis=axis, keepdims=keepdims)


for _f in (anp.max, anp.min, anp.amax, anp.amin):
    defjvp(_f, _fwd_chooser)

# linear one-argument functions (77-105, 150-162)
for _name in (
    "negative reshape ravel expand_dims squeeze swapaxes moveaxis roll flipud fliplr diag diagonal "
    "trace triu tril broadcast_to repeat tile transpose sum _primitive_mean cumsum "
    "array_split split vsplit hsplit dsplit rollaxis rot90 diff"
).split():
    defjvp(getattr(anp, _name), "same")
defjvp(anp.full, "same", argnums=(1,))
defjvp(anp.make_diagonal, "same")  # numpy_jvps.py:94
defjvp(anp.kron, "same", "same")  # numpy_jvps.py:155


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

defjvp(anp.pad, lambda g, ans, array, width, mode, **kwargs: anp.pad(g, width, mode))  # numpy_jvps.py:303
defjvp(anp.gradient, "same")  # numpy_jvps.py:157
defjvp(  # numpy_jvps.py:169-173
    anp.linspace,
    lambda g, ans, start, stop, *args, **kwargs: anp.linspace(g, 0, *args, **kwargs),
    lambda g, ans, start, stop, *args, **kwargs: anp.linspace(0, g, *args, **kwargs),
)
# numpy_jvps.py:256-271: the tangent taken in sorted (partitioned) order
defjvp(anp.sort, lambda g, ans, x, axis=-1, kind="quicksort", order=None: g[anp.argsort(x, axis, kind, order)])
defjvp(
    anp.partition,
    lambda g, ans, x, kth, axis=-1, kind="introselect", order=None: g[anp.argpartition(x, kth, axis, kind, order)],
)

# unary ufuncs (108-134)
_unary = {
    "abs": lambda g, ans, x: anp.real(g * replace_zero(anp.conj(x), 0.0)) / replace_zero(ans, 1.0),
    "arccos": lambda g, ans, x: -g / anp.sqrt(1 - x**2),
    "arccosh": lambda g, ans, x: g / anp.sqrt(x**2 - 1),
    "arcsin": lambda g, ans, x: g / anp.sqrt(1 - x**2),
    "arcsinh": lambda g, ans, x: g / anp.sqrt(x**2 + 1),
    "arctan": lambda g, ans, x: g / (1 + x**2),
    "arctanh": lambda g, ans, x: g / (1 - x**2),
    "conj": lambda g, ans, x: anp.conj(g),
    "cos": lambda g, ans, x: -g * anp.sin(x),
    "cosh": lambda g, ans, x: g * anp.sinh(x),
    "exp": lambda g, ans, x: ans * g,
    "exp2": lambda g, ans, x: ans * anp.log(2) * g,
    "expm1": lambda g, ans, x: (ans + 1) * g,
    "fabs": lambda g, ans, x: anp.sign(x) * g,
    "log": lambda g, ans, x: g / x,
    "log10": lambda g, ans, x: g / x / anp.log(10),
    "log1p": lambda g, ans, x: g / (x + 1),
    "log2": lambda g, ans, x: g / x / anp.log(2),
    "nan_to_num": lambda g, ans, x: anp.where(anp.isfinite(x), g, 0.0),
    "real": lambda g, ans, x: anp.real(g),
    "reciprocal": lambda g, ans, x: -g / x**2,
    "sin": lambda g, ans, x: g * anp.cos(x),
    "sinc": lambda g, ans, x: g * (anp.cos(anp.pi * x) * anp.pi * x - anp.sin(anp.pi * x)) / (anp.pi * x**2),
    "sinh": lambda g, ans, x: g * anp.cosh(x),
    "sqrt": lambda g, ans, x: g * 0.5 * x**-0.5,
    "square": lambda g, ans, x: g * 2 * x,
    "tan": lambda g, ans, x: g / anp.cos(x) ** 2,
    "tanh": lambda g, ans, x: g / anp.cosh(x) ** 2,
}
for _name, _rule in _unary.items():
    defjvp(getattr(anp, _name), _rule)

for _f in (anp.rad2deg, anp.degrees, anp.deg2rad, anp.radians):  # numpy_jvps.py:78-81: the ufunc itself on the tangent
    defjvp(_f, "same")
defjvp(anp.clip, lambda g, ans, x, a_min, a_max: g * anp.logical_and(ans != a_min, ans != a_max))
defjvp(
    anp._raw_where,
    None,
    lambda g, ans, c, x=None, y=None: anp.where(c, g, anp.zeros(anp.shape(g))),
    lambda g, ans, c, x=None, y=None: anp.where(c, anp.zeros(g.shape), g),
)
defjvp(
    anp.prod,
    lambda g, ans, x, axis=None, keepdims=False, **kwargs: ans * anp.sum(g / x, axis=axis, keepdims=keepdims),
)

# binary ufuncs (38-74)
def_linear(anp.multiply)
defjvp(anp.add, lambda g, ans, x, y: broadcast(g, ans), lambda g, ans, x, y: broadcast(g, ans))
defjvp(anp.subtract, lambda g, ans, x, y: broadcast(g, ans), lambda g, ans, x, y: broadcast(-g, ans))
defjvp(anp.true_divide, "same", lambda g, ans, x, y: -g * x / y**2)
for _chooser in (anp.maximum, anp.minimum, anp.fmax, anp.fmin):
    defjvp(
        _chooser,
        lambda g, ans, x, y: g * balanced_eq(x, ans, y),
        lambda g, ans, x, y: g * balanced_eq(y, ans, x),
    )
defjvp(anp.logaddexp, lambda g, ans, x, y: g * anp.exp(x - ans), lambda g, ans, x, y: g * anp.exp(y - ans))
defjvp(anp.mod, lambda g, ans, x, y: broadcast(g, ans), lambda g, ans, x, y: -g * anp.floor(x / y))
defjvp(anp.logaddexp2, lambda g, ans, x, y: g * 2 ** (x - ans), lambda g, ans, x, y: g * 2 ** (y - ans))  # 65
defjvp(
    anp.power,
    lambda g, ans, x, y: g * y * x ** anp.where(y, y - 1, 1.0),
    lambda g, ans, x, y: g * anp.log(replace_zero(x, 1.0)) * ans,
)
defjvp(anp.arctan2, lambda g, ans, x, y: g * y / (x**2 + y**2), lambda g, ans, x, y: g * -x / (x**2 + y**2))

# indexing and array construction (23-32)
defjvp(func(ArrayBox.__getitem__), "same")
defjvp(untake, "same")
defjvp_argnum(anp.array_from_args, lambda argnum, g, ans, args, kwargs: untake(g, argnum - 2, vspace(ans)))
defjvp(
    anp._array_from_scalar_or_array,
    None,
    None,
    lambda g, ans, args, kwargs, _: anp._array_from_scalar_or_array(args, kwargs, g),
)
