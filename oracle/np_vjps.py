"""Reverse-mode rules of the oracle's NumPy value type.

Each rule restates the formula AND the operation order of the cited line of
the reference's autograd/numpy/numpy_vjps.py, so that on NumPy the results are
the reference's to the last bit (checked against fixtures written by the real
reference).  Rules are written with the wrapped namespace ``anp`` wherever the
reference does so, which keeps them differentiable for higher orders.
TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

from functools import partial

import numpy as onp

from autograd_amd.extend import SparseObject, VJPNode, defvjp, defvjp_argnum, primitive, register_notrace, vspace
from autograd_amd.util import func

from . import np_namespace as anp
from .np_boxes import ArrayBox

# ---- functions with no derivative (numpy_vjps.py:13-68) ---------------------------
nograd_functions = [
    getattr(anp, n)
    for n in (
        "floor ceil round rint around fix trunc all any argmax argmin argsort argpartition nonzero "
        "count_nonzero searchsorted sign ndim shape floor_divide logical_and logical_or "
        "logical_not logical_xor isfinite isinf isnan allclose isclose array_equal greater "
        "greater_equal less less_equal equal not_equal iscomplexobj iscomplex size isscalar "
        "isreal zeros_like ones_like empty_like full_like result_type"
    ).split()
]
for _f in nograd_functions:
    register_notrace(VJPNode, _f)


# ---- helpers (numpy_vjps.py:872-916) ----------------------------------------------
def match_complex(target, x):
    target_c, x_c = anp.iscomplexobj(target), anp.iscomplexobj(x)
    if x_c and not target_c:
        return anp.real(x)
    if target_c and not x_c:
        return x + 0j
    return x


def unbroadcast(x, target_meta, broadcast_idx=0):
    """Sum ``x`` down to the shape it was broadcast from (numpy_vjps.py:883-892):
    leading extra axes one ``sum(axis=0)`` at a time, then every size-1 target
    axis with ``keepdims``."""
    target_shape, target_ndim, _dtype, target_iscomplex = target_meta
    while anp.ndim(x) > target_ndim:
        x = anp.sum(x, axis=broadcast_idx)
    for axis, size in enumerate(target_shape):
        if size == 1:
            x = anp.sum(x, axis=axis, keepdims=True)
    if anp.iscomplexobj(x) and not target_iscomplex:
        x = anp.real(x)
    return x


def unbroadcast_f(target, f):
    target_meta = anp.metadata(target)
    return lambda g: unbroadcast(f(g), target_meta)


def balanced_eq(x, z, y):
    return (x == z) / (1.0 + (x == y))


def replace_zero(x, val):
    return anp.where(x, x, val)


def _binary(fun, wrt_x, wrt_y):
    """Register a two-argument ufunc rule; both cotangents are unbroadcast."""
    defvjp(
        fun,
        lambda ans, x, y: unbroadcast_f(x, wrt_x(ans, x, y)),
        lambda ans, x, y: unbroadcast_f(y, wrt_y(ans, x, y)),
    )


# ---- binary ufuncs (numpy_vjps.py:76-153) -----------------------------------------
_binary(anp.add, lambda ans, x, y: lambda g: g, lambda ans, x, y: lambda g: g)
_binary(anp.multiply, lambda ans, x, y: lambda g: y * g, lambda ans, x, y: lambda g: x * g)
_binary(anp.subtract, lambda ans, x, y: lambda g: g, lambda ans, x, y: lambda g: -g)
_binary(anp.true_divide, lambda ans, x, y: lambda g: g / y, lambda ans, x, y: lambda g: -g * x / y**2)
for _chooser in (anp.maximum, anp.minimum, anp.fmax, anp.fmin):
    _binary(
        _chooser,
        lambda ans, x, y: lambda g: g * balanced_eq(x, ans, y),
        lambda ans, x, y: lambda g: g * balanced_eq(y, ans, x),
    )
_binary(
    anp.logaddexp,
    lambda ans, x, y: lambda g: g * anp.exp(x - ans),
    lambda ans, x, y: lambda g: g * anp.exp(y - ans),
)
_binary(anp.mod, lambda ans, x, y: lambda g: g, lambda ans, x, y: lambda g: -g * anp.floor(x / y))
_binary(  # numpy_vjps.py:119-123
    anp.logaddexp2,
    lambda ans, x, y: lambda g: g * 2 ** (x - ans),
    lambda ans, x, y: lambda g: g * 2 ** (y - ans),
)
_binary(
    anp.power,
    lambda ans, x, y: lambda g: g * y * x ** anp.where(y, y - 1, 1.0),
    lambda ans, x, y: lambda g: g * anp.log(replace_zero(x, 1.0)) * ans,
)
_binary(
    anp.arctan2,
    lambda ans, x, y: lambda g: g * y / (x**2 + y**2),
    lambda ans, x, y: lambda g: g * -x / (x**2 + y**2),
)
_binary(anp.hypot, lambda ans, x, y: lambda g: g * x / ans, lambda ans, x, y: lambda g: g * y / ans)

# ---- unary ufuncs (numpy_vjps.py:157-191) -----------------------------------------
_unary = {
    "negative": lambda ans, x: lambda g: -g,
    "reciprocal": lambda ans, x: lambda g: -g / x**2,
    "exp": lambda ans, x: lambda g: ans * g,
    "exp2": lambda ans, x: lambda g: ans * anp.log(2) * g,
    "expm1": lambda ans, x: lambda g: (ans + 1) * g,
    "log": lambda ans, x: lambda g: g / x,
    "log2": lambda ans, x: lambda g: g / x / anp.log(2),
    "log10": lambda ans, x: lambda g: g / x / anp.log(10),
    "log1p": lambda ans, x: lambda g: g / (x + 1),
    "sin": lambda ans, x: lambda g: g * anp.cos(x),
    "cos": lambda ans, x: lambda g: -g * anp.sin(x),
    "tan": lambda ans, x: lambda g: g / anp.cos(x) ** 2,
    "arcsin": lambda ans, x: lambda g: g / anp.sqrt(1 - x**2),
    "arccos": lambda ans, x: lambda g: -g / anp.sqrt(1 - x**2),
    "arctan": lambda ans, x: lambda g: g / (1 + x**2),
    "sinh": lambda ans, x: lambda g: g * anp.cosh(x),
    "cosh": lambda ans, x: lambda g: g * anp.sinh(x),
    "tanh": lambda ans, x: lambda g: g / anp.cosh(x) ** 2,
    "arcsinh": lambda ans, x: lambda g: g / anp.sqrt(x**2 + 1),
    "arccosh": lambda ans, x: lambda g: g / anp.sqrt(x**2 - 1),
    "arctanh": lambda ans, x: lambda g: g / (1 - x**2),
    "square": lambda ans, x: lambda g: g * 2 * x,
    "sqrt": lambda ans, x: lambda g: g * 0.5 * x**-0.5,
    "fabs": lambda ans, x: lambda g: anp.sign(x) * g,
    "abs": lambda ans, x: lambda g: g * replace_zero(anp.conj(x), 0.0) / replace_zero(ans, 1.0),
    "real": lambda ans, x: lambda g: match_complex(x, g),
    "conj": lambda ans, x: lambda g: anp.conj(g),
    "nan_to_num": lambda ans, x: lambda g: anp.where(anp.isfinite(x), g, 0.0),
    "sinc": lambda ans, x: lambda g: g * (anp.cos(anp.pi * x) * anp.pi * x - anp.sin(anp.pi * x)) / (anp.pi * x**2),
}
for _name, _maker in _unary.items():
    defvjp(getattr(anp, _name), _maker)
# numpy_vjps.py:182-185
defvjp(anp.rad2deg, lambda ans, x: lambda g: g / anp.pi * 180.0)
defvjp(anp.degrees, lambda ans, x: lambda g: g / anp.pi * 180.0)
defvjp(anp.deg2rad, lambda ans, x: lambda g: g * anp.pi / 180.0)
defvjp(anp.radians, lambda ans, x: lambda g: g * anp.pi / 180.0)

# ---- shape-only functions (numpy_vjps.py:192-217, 407-413, 804-812) ---------------
defvjp(anp.reshape, lambda ans, x, shape, order=None: lambda g: anp.reshape(g, anp.shape(x), order=order))
defvjp(anp.ravel, lambda ans, x, order=None: lambda g: anp.reshape(g, anp.shape(x), order=order))
defvjp(anp.expand_dims, lambda ans, x, axis: lambda g: anp.reshape(g, anp.shape(x)))
defvjp(anp.squeeze, lambda ans, x, axis=None: lambda g: anp.reshape(g, anp.shape(x)))
defvjp(anp.swapaxes, lambda ans, x, axis1, axis2: lambda g: anp.swapaxes(g, axis2, axis1))
defvjp(anp.moveaxis, lambda ans, a, source, destination: lambda g: anp.moveaxis(g, destination, source))
defvjp(anp.roll, lambda ans, x, shift, axis=None: lambda g: anp.roll(g, -shift, axis=axis))
defvjp(anp.flipud, lambda ans, x: lambda g: anp.flipud(g))
defvjp(anp.fliplr, lambda ans, x: lambda g: anp.fliplr(g))
defvjp(anp.diag, lambda ans, x, k=0: lambda g: anp.diag(g, k))
defvjp(anp.triu, lambda ans, x, k=0: lambda g: anp.triu(g, k=k))
defvjp(anp.tril, lambda ans, x, k=0: lambda g: anp.tril(g, k=k))
defvjp(anp.clip, lambda ans, x, a_min, a_max: lambda g: g * anp.logical_and(ans != a_min, ans != a_max))
defvjp(
    anp._raw_where,
    None,
    lambda ans, c, x=None, y=None: lambda g: anp.where(c, g, anp.zeros(g.shape)),
    lambda ans, c, x=None, y=None: lambda g: anp.where(c, anp.zeros(g.shape), g),
)
defvjp(anp.full, lambda ans, shape, fill_value, dtype=None: lambda g: anp.sum(g), argnums=(1,))
defvjp(
    anp._astype,
    lambda ans, A, dtype, order="K", casting="unsafe", subok=True, copy=True: lambda g: anp._astype(g, A.dtype),
)


def _grad_transpose(ans, x, axes=None):
    if axes is not None:
        axes = anp.argsort(axes)
    return lambda g: anp.transpose(g, axes)


defvjp(anp.transpose, _grad_transpose)


def _grad_atleast(ans, *arys):
    if len(arys) > 1:
        raise NotImplementedError("Can't handle multiple arguments yet.")
    return lambda g: anp.reshape(g, anp.shape(arys[0]))


for _f in (anp.atleast_1d, anp.atleast_2d, anp.atleast_3d):
    defvjp(_f, _grad_atleast)


# ---- reductions (numpy_vjps.py:416-530) -------------------------------------------
def repeat_to_match_shape(g, shape, dtype, axis, keepdims):
    """Broadcast a reduction's cotangent back over the reduced axes.

    Returns ``(array, num_reps)``.  The broadcast is materialised by adding a
    zeros array of the full shape, and ``num_reps`` is a NumPy integer scalar,
    which under NumPy 2 promotion makes ``f32_array / num_reps`` float64
    (numpy_vjps.py:416-427)."""
    if shape == ():
        return g, 1
    axis = list(axis) if isinstance(axis, tuple) else axis
    new_shape = onp.array(shape)
    new_shape[axis] = 1
    num_reps = onp.prod(onp.array(shape)[axis])
    return anp.reshape(g, new_shape) + onp.zeros(shape, dtype=dtype), num_reps


def _grad_sum(ans, x, axis=None, keepdims=False, dtype=None, **kwargs):
    shape, dtype = anp.shape(x), anp.result_type(x)
    return lambda g: repeat_to_match_shape(g, shape, dtype, axis, keepdims)[0]


defvjp(anp.sum, _grad_sum)


def _grad_mean(ans, x, axis=None, keepdims=False, **kwargs):
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, num_reps = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        return g_repeated / num_reps

    return vjp


defvjp(anp._primitive_mean, _grad_mean)


def _grad_prod(ans, x, axis=None, keepdims=False, **kwargs):
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, _ = repeat_to_match_shape(g * ans, shape, dtype, axis, keepdims)
        return g_repeated / x

    return vjp


defvjp(anp.prod, _grad_prod)


def _grad_var(ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    shape, _, dtype, iscomplex = anp.metadata(x)

    def vjp(g):
        if iscomplex:
            g = g + 0j
        g_repeated, num_reps = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        x_minus_mean = anp.conj(x - anp.mean(x, axis=axis, keepdims=True))
        return 2.0 * g_repeated * x_minus_mean / (num_reps - ddof)

    return vjp


defvjp(anp._primitive_var, _grad_var)


def _grad_std(ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    shape, _, dtype, iscomplex = anp.metadata(x)

    def vjp(g):
        if iscomplex:
            g = g + 0j
        g_repeated, num_reps = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        if num_reps <= 1:
            return g_repeated * 0.0
        g_repeated, num_reps = repeat_to_match_shape(g / ans, shape, dtype, axis, keepdims)
        x_minus_mean = anp.conj(x - anp.mean(x, axis=axis, keepdims=True))
        return g_repeated * x_minus_mean / (num_reps - ddof)

    return vjp


defvjp(anp._primitive_std, _grad_std)


def _grad_chooser(ans, x, axis=None, keepdims=None, **kwargs):
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, _ = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        argmax_locations = x == repeat_to_match_shape(ans, shape, dtype, axis, keepdims)[0]
        return g_repeated * argmax_locations / onp.sum(argmax_locations, axis=axis, keepdims=True)

    return vjp


for _f in (anp.max, anp.min, anp.amax, anp.amin):
    defvjp(_f, _grad_chooser)


def _grad_broadcast_to(ans, x, new_shape):
    old_shape = anp.shape(x)
    assert anp.shape(ans) == new_shape
    assert len(old_shape) == len(new_shape), "Can't handle extra leading dims"
    axes = tuple(onp.where(onp.logical_and(onp.array(old_shape) == 1, onp.array(new_shape) > 1))[0])
    return lambda g: anp.sum(g, axis=axes, keepdims=True)


defvjp(anp.broadcast_to, _grad_broadcast_to)


def _grad_repeat(ans, x, repeats, axis=None):
    shape = anp.shape(x)

    def vjp(g):
        if axis is None:
            expanded = anp.reshape(g, (anp.prod(shape),) + (repeats,))
            return anp.reshape(anp.sum(expanded, axis=1, keepdims=False), shape)
        if shape[axis] == 1:
            return anp.sum(g, axis=axis, keepdims=True)
        expanded = anp.reshape(g, shape[0 : axis + 1] + (repeats,) + shape[axis + 1 :])
        return anp.sum(expanded, axis=axis + 1, keepdims=False)

    return vjp


defvjp(anp.repeat, _grad_repeat)
# numpy_vjps.py:194-198, 204
defvjp(anp.array_split, lambda ans, ary, idxs, axis=0: lambda g: anp.concatenate(g, axis=axis))
defvjp(anp.split, lambda ans, ary, idxs, axis=0: lambda g: anp.concatenate(g, axis=axis))
defvjp(anp.vsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=0))
defvjp(anp.hsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=1))
defvjp(anp.dsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=2))
defvjp(anp.rot90, lambda ans, x, k=1: lambda g: anp.rot90(g, -k))
defvjp(  # numpy_vjps.py:231-239
    anp.cross,
    lambda ans, a, b, axisa=-1, axisb=-1, axisc=-1, axis=None: lambda g: anp.cross(b, g, axisb, axisc, axisa, axis),
    lambda ans, a, b, axisa=-1, axisb=-1, axisc=-1, axis=None: lambda g: anp.cross(g, a, axisc, axisa, axisb, axis),
)


def _grad_rollaxis(ans, a, axis, start=0):  # numpy_vjps.py:255-267
    if axis < 0:
        raise NotImplementedError("Gradient of rollaxis not implemented for axis < 0. Please use moveaxis instead.")
    elif start < 0:
        raise NotImplementedError("Gradient of rollaxis not implemented for start < 0. Please use moveaxis instead.")
    return lambda g: anp.rollaxis(g, start - 1, axis) if start > axis else anp.rollaxis(g, start, axis + 1)


defvjp(anp.rollaxis, _grad_rollaxis)


def _grad_diff(ans, a, n=1, axis=-1):  # numpy_vjps.py:270-294
    nd = anp.ndim(a)
    ans_shape = anp.shape(ans)
    sl1 = [slice(None)] * nd
    sl1[axis] = slice(None, 1)
    sl2 = [slice(None)] * nd
    sl2[axis] = slice(-1, None)

    def undiff(g):
        if g.shape[axis] > 0:
            return anp.concatenate((-g[tuple(sl1)], -anp.diff(g, axis=axis), g[tuple(sl2)]), axis=axis)
        shape = list(ans_shape)
        shape[axis] = 1
        return anp.zeros(shape)

    def helper(g, n):
        return g if n == 0 else helper(undiff(g), n - 1)

    return lambda g: helper(g, n)


defvjp(anp.diff, _grad_diff)


def _unpermuter(g, permutation):  # numpy_vjps.py:798-801
    unsort = anp.zeros(len(permutation), dtype=int)
    unsort[permutation] = list(range(len(permutation)))
    return g[unsort]


def _grad_sort(ans, x, axis=-1, kind="quicksort", order=None):  # numpy_vjps.py:773-779
    if len(x.shape) > 1:
        raise NotImplementedError("Gradient of sort not implemented for multi-dimensional arrays.")
    sort_perm = anp.argsort(x, axis, kind, order)
    return lambda g: _unpermuter(g, sort_perm)


def _grad_partition(ans, x, kth, axis=-1, kind="introselect", order=None):  # numpy_vjps.py:787-792
    if len(x.shape) > 1:
        raise NotImplementedError("Gradient of partition not implemented for multi-dimensional arrays.")
    partition_perm = anp.argpartition(x, kth, axis, kind, order)
    return lambda g: _unpermuter(g, partition_perm)


defvjp(anp.sort, _grad_sort)
defvjp(anp.partition, _grad_partition)


def _grad_tile(ans, x, reps):  # numpy_vjps.py:352-364
    reps = [reps] if anp.isscalar(reps) else reps
    x_shape = anp.shape(x)

    def vjp(g):
        for axis, rep in enumerate(reps):
            g = sum(anp.split(g, rep, axis))
        return anp.reshape(g, x_shape)

    return vjp


defvjp(anp.tile, _grad_tile)


def _grad_kron(argnum, ans, orig_A, orig_B):  # numpy_vjps.py:367-392
    orig_A_shape, orig_B_shape = anp.shape(orig_A), anp.shape(orig_B)

    def vjp(G):
        A, B = anp.atleast_2d(orig_A), anp.atleast_2d(orig_B)
        shape = list(A.shape + B.shape)
        n = anp.ndim(A)
        shape[n - 1], shape[n] = shape[n], shape[n - 1]
        reshaped_G = anp.swapaxes(anp.reshape(G, shape), n - 1, n)
        if argnum == 0:
            return match_complex(orig_A, anp.reshape(anp.tensordot(reshaped_G, B, axes=anp.ndim(B)), orig_A_shape))
        return match_complex(orig_B, anp.reshape(anp.tensordot(A, reshaped_G, axes=anp.ndim(A)), orig_B_shape))

    return vjp


defvjp(anp.kron, partial(_grad_kron, 0), partial(_grad_kron, 1))
defvjp(  # numpy_vjps.py:205-210
    anp.trace,
    lambda ans, x, offset=0: lambda g: anp.einsum("ij,...->ij...", anp.eye(x.shape[0], x.shape[1], k=offset), g),
)
defvjp(  # numpy_vjps.py:863-870
    anp.diagonal,
    lambda ans, A, offset=0, axis1=0, axis2=1: lambda g: anp.make_diagonal(g, offset, axis1, axis2),
)
defvjp(
    anp.make_diagonal,
    lambda ans, D, offset=0, axis1=0, axis2=1: lambda g: anp.diagonal(g, offset, axis1, axis2),
)


def _reverse_axis(x, axis):
    x = x.swapaxes(axis, 0)
    x = x[::-1, ...]
    return x.swapaxes(0, axis)


def _grad_cumsum(ans, x, axis=None):
    def vjp(g):
        if axis:
            return _reverse_axis(anp.cumsum(_reverse_axis(g, axis), axis), axis)
        return anp.reshape(anp.cumsum(g[::-1], axis)[::-1], x.shape)

    return vjp


defvjp(anp.cumsum, _grad_cumsum)


# ---- dense contractions (numpy_vjps.py:552-747) -----------------------------------
@primitive
def dot_adjoint_0(B, G, A_meta, B_meta):
    """Cotangent of ``dot(A, B)`` with respect to ``A`` (numpy_vjps.py:615-624)."""
    _, A_ndim, A_dtype, _ = A_meta
    _, B_ndim, _, _ = B_meta
    if B_ndim == 0 or B_ndim == 1 or A_ndim == 0:
        contract_num = max(0, B_ndim - (A_ndim != 0))
        out = onp.tensordot(G, B, contract_num)
    else:
        out = onp.tensordot(G, onp.swapaxes(B, -1, -2), B_ndim - 1)
    return onp.asarray(out, dtype=A_dtype)


@primitive
def dot_adjoint_1(A, G, A_meta, B_meta):
    """Cotangent of ``dot(A, B)`` with respect to ``B`` (numpy_vjps.py:627-638);
    for matrices the result is the transposed view of ``G^T A``."""
    _, A_ndim, _, _ = A_meta
    _, B_ndim, B_dtype, _ = B_meta
    needs_transpose = B_ndim > 1 and A_ndim != 0
    swap = (lambda x: onp.swapaxes(x, -1, -2)) if needs_transpose else (lambda x: x)
    if A_ndim == 0 or A_ndim == 1 or B_ndim == 0:
        contract_num = max(0, A_ndim - (B_ndim != 0))
        out = swap(onp.tensordot(G, A, contract_num))
    else:
        out = swap(onp.tensordot(G, A, [range(-A_ndim - B_ndim + 2, -B_ndim + 1), range(A_ndim - 1)]))
    return onp.asarray(out, dtype=B_dtype)


def _dot_vjp_0(ans, A, B):
    A_meta, B_meta = anp.metadata(A), anp.metadata(B)
    return lambda g: match_complex(A, dot_adjoint_0(B, g, A_meta, B_meta))


def _dot_vjp_1(ans, A, B):
    A_meta, B_meta = anp.metadata(A), anp.metadata(B)
    return lambda g: match_complex(B, dot_adjoint_1(A, g, A_meta, B_meta))


defvjp(anp.dot, _dot_vjp_0, _dot_vjp_1)
defvjp(
    dot_adjoint_0,
    lambda ans, B, g, An, Bn: lambda A: match_complex(B, dot_adjoint_1(A, g, An, Bn)),
    lambda ans, B, g, An, Bn: lambda A: match_complex(g, anp.dot(A, B)),
)
defvjp(
    dot_adjoint_1,
    lambda ans, A, g, An, Bn: lambda B: match_complex(A, dot_adjoint_0(B, g, An, Bn)),
    lambda ans, A, g, An, Bn: lambda B: match_complex(g, anp.dot(A, B)),
)


def _matmul_adjoint_0(B, G, A_meta, B_ndim):
    if anp.ndim(G) == 0:
        return unbroadcast(G * B, A_meta)
    _, A_ndim, _, _ = A_meta
    if A_ndim == 1:
        G = anp.expand_dims(G, anp.ndim(G) - 1)
    if B_ndim == 1:
        B = anp.expand_dims(B, 0)
        G = anp.expand_dims(G, anp.ndim(G))
    else:
        B = anp.swapaxes(B, B_ndim - 2, B_ndim - 1)
    return unbroadcast(anp.matmul(G, B), A_meta)


def _matmul_adjoint_1(A, G, A_ndim, B_meta):
    if anp.ndim(G) == 0:
        return unbroadcast(G * A, B_meta)
    _, B_ndim, _, _ = B_meta
    B_is_vec = B_ndim == 1
    if B_is_vec:
        G = anp.expand_dims(G, anp.ndim(G))
    if A_ndim == 1:
        A = anp.expand_dims(A, 1)
        G = anp.expand_dims(G, anp.ndim(G) - 1)
    else:
        A = anp.swapaxes(A, A_ndim - 2, A_ndim - 1)
    result = anp.matmul(A, G)
    if B_is_vec:
        result = anp.squeeze(result, anp.ndim(G) - 1)
    return unbroadcast(result, B_meta)


def _matmul_vjp_0(ans, A, B):
    A_meta, B_ndim = anp.metadata(A), anp.ndim(B)
    return lambda g: _matmul_adjoint_0(B, g, A_meta, B_ndim)


def _matmul_vjp_1(ans, A, B):
    A_ndim, B_meta = anp.ndim(A), anp.metadata(B)
    return lambda g: _matmul_adjoint_1(A, g, A_ndim, B_meta)


defvjp(anp.matmul, _matmul_vjp_0, _matmul_vjp_1)


def _split_axes(axes, A_ndim, B_ndim):
    axes0 = [axes[0]] if type(axes[0]) is int else axes[0]
    axes1 = [axes[1]] if type(axes[1]) is int else axes[1]
    summed = [onp.asarray(axes0, dtype="int64") % A_ndim, onp.asarray(axes1, dtype="int64") % B_ndim]
    other = [onp.delete(onp.arange(A_ndim), summed[0]), onp.delete(onp.arange(B_ndim), summed[1])]
    return summed, other


@primitive
def tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim):
    """Adjoint of ``A -> tensordot(A, B, axes)`` (numpy_vjps.py:666-691)."""
    if B_ndim == 0:
        return G * B
    G_axes = onp.arange(onp.ndim(G))
    if type(axes) is int:
        axes = max(axes, 0)
        B_axes = onp.arange(B_ndim)
        return onp.tensordot(G, B, [G_axes[A_ndim - axes :], B_axes[axes:]])
    summed, other = _split_axes(axes, A_ndim, B_ndim)
    out = onp.tensordot(G, B, [G_axes[len(other[0]) :], other[1]])
    perm = onp.argsort(onp.concatenate((other[0], summed[0][onp.argsort(summed[1])])))
    return onp.transpose(out, perm)


@primitive
def tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim):
    """Adjoint of ``B -> tensordot(A, B, axes)`` (numpy_vjps.py:694-719)."""
    if A_ndim == 0:
        return G * A
    G_axes = onp.arange(onp.ndim(G))
    if type(axes) is int:
        axes = max(axes, 0)
        A_axes = onp.arange(A_ndim)
        return onp.tensordot(A, G, [A_axes[: A_ndim - axes], G_axes[: A_ndim - axes]])
    summed, other = _split_axes(axes, A_ndim, B_ndim)
    out = onp.tensordot(A, G, [other[0], G_axes[: len(other[0])]])
    perm = onp.argsort(onp.concatenate((summed[1][onp.argsort(summed[0])], other[1])))
    return onp.transpose(out, perm)


def _tensordot_vjp_0(ans, A, B, axes=2):
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    return lambda G: match_complex(A, tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim))


def _tensordot_vjp_1(ans, A, B, axes=2):
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    return lambda G: match_complex(B, tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim))


defvjp(anp.tensordot, _tensordot_vjp_0, _tensordot_vjp_1)
defvjp(
    tensordot_adjoint_0,
    lambda ans, B, G, axes, An, Bn: lambda A: match_complex(B, tensordot_adjoint_1(A, G, axes, An, Bn)),
    lambda ans, B, G, axes, An, Bn: lambda A: match_complex(G, anp.tensordot(A, B, axes)),
)
defvjp(
    tensordot_adjoint_1,
    lambda ans, A, G, axes, An, Bn: lambda B: match_complex(A, tensordot_adjoint_0(B, G, axes, An, Bn)),
    lambda ans, A, G, axes, An, Bn: lambda B: match_complex(G, anp.tensordot(A, B, axes)),
)


def _grad_inner(argnum, ans, A, B):
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    axes = ([], []) if A_ndim == 0 or B_ndim == 0 else ([A_ndim - 1], [B_ndim - 1])
    if argnum == 0:
        return lambda G: tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim)
    return lambda G: tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim)


defvjp(anp.inner, partial(_grad_inner, 0), partial(_grad_inner, 1))
defvjp(
    anp.outer,
    lambda ans, a, b: lambda g: match_complex(a, anp.dot(g, b.T)),
    lambda ans, a, b: lambda g: match_complex(b, anp.dot(a.T, g)),
)


# ---- einsum, both calling conventions (numpy_vjps.py:815-857, 900-908) -------------------------
def _unbroadcast_einsum(x, target_meta, subscript):
    if Ellipsis not in subscript:
        return x
    if subscript[0] == Ellipsis:
        return unbroadcast(x, target_meta, 0)
    if subscript[-1] == Ellipsis:
        return unbroadcast(x, target_meta, -1)
    return unbroadcast(x, target_meta, subscript.index(Ellipsis))


def _grad_einsum(argnum, ans, operands_, kwargs):
    result_meta = anp.metadata(operands_[argnum])

    def vjp(g):
        operands = operands_
        if not isinstance(operands[0], str):
            # (op0, sublist0, op1, sublist1, ..., sublistout) convention, numpy_vjps.py:848-857
            if len(operands) % 2 == 0:
                raise NotImplementedError("Need sublistout argument")
            operands = list(operands)
            rest_of_ops = [operands[-1]] + operands[:argnum] + operands[(argnum + 2) : -1] + [operands[argnum + 1]]
            return _unbroadcast_einsum(anp.einsum(g, *rest_of_ops), result_meta, operands[argnum + 1])
        in_subs, out_subs, _ = anp.parse_einsum_input(*operands)
        string, operands = operands[0], operands[1:]
        in_subs_list = in_subs.split(",")
        op_num = argnum - 1
        subs_wrt = in_subs_list[op_num]
        rest_of_ops = operands[:op_num] + operands[op_num + 1 :]
        rest_of_subs = in_subs_list[:op_num] + in_subs_list[op_num + 1 :]
        other_named_subs = set("".join([out_subs] + rest_of_subs))
        naked_summed = [(i, sub) for i, sub in enumerate(subs_wrt) if sub not in other_named_subs]
        if naked_summed:
            naked_summed_dims, ones_subs = zip(*naked_summed)
            ones_subs = "".join(ones_subs)
            ones = onp.ones(onp.array(operands[op_num].shape)[list(naked_summed_dims)])
            new_input_subs = ",".join([out_subs, ones_subs] + rest_of_subs)
            new_operands = (g, ones) + rest_of_ops
        else:
            new_input_subs = ",".join([out_subs] + rest_of_subs)
            new_operands = (g,) + rest_of_ops
        new_subscripts = new_input_subs + "->" + subs_wrt
        return unbroadcast(anp.einsum(new_subscripts, *new_operands), result_meta)

    return vjp


defvjp_argnum(anp.einsum, _grad_einsum)


# ---- concatenate / array construction (numpy_vjps.py:750-759, 922-938) ------------
def _grad_concatenate_args(argnum, ans, axis_args, kwargs):
    axis, args = axis_args[0], axis_args[1:]
    sizes = [anp.shape(a)[axis] for a in args[:argnum]]
    start = sum(sizes[:-1])
    idxs = [slice(None)] * ans.ndim
    idxs[axis] = slice(start, start + sizes[-1])
    return lambda g: g[tuple(idxs)]


defvjp_argnum(anp.concatenate_args, _grad_concatenate_args)
defvjp_argnum(anp.array_from_args, lambda argnum, ans, args, kwargs: lambda g: g[argnum - 2])


def _grad_array_from_scalar_or_array(ans, array_args, array_kwargs, scarray):
    ndmin = array_kwargs.get("ndmin", 0)
    scarray_ndim = anp.ndim(scarray)
    if ndmin > scarray_ndim:
        return lambda g: anp.squeeze(g, axis=tuple(range(ndmin - scarray_ndim)))
    return lambda g: g


defvjp(anp._array_from_scalar_or_array, _grad_array_from_scalar_or_array, argnums=(2, 3))


# ---- indexing (numpy_vjps.py:941-954) ---------------------------------------------
@primitive
def untake(x, idx, vs):
    """Cotangent of ``A[idx]``: a sparse object that scatters ``x`` into a dense
    buffer with ``numpy.add.at`` (sequential accumulation for repeated indices)."""
    if isinstance(idx, list) and (len(idx) == 0 or not isinstance(idx[0], slice)):
        idx = onp.array(idx, dtype="int64")

    def mut_add(A):
        onp.add.at(A, idx, x)
        return A

    return SparseObject(vs, mut_add)


defvjp(func(ArrayBox.__getitem__), lambda ans, A, idx: lambda g: untake(g, idx, vspace(A)))
defvjp(untake, lambda ans, x, idx, _: lambda g: g[idx])


# ---- zero padding (numpy_vjps.py:957-975) ------------------------------------------------------
def _unpad(array, width):
    if anp.isscalar(width):
        width = [[width, width]]
    elif anp.shape(width) == (1,):
        width = [anp.concatenate((width, width))]
    elif anp.shape(width) == (2,):
        width = [width]
    if anp.shape(width)[0] == 1:
        width = anp.repeat(width, anp.ndim(array), 0)
    return array[tuple(slice(lo, -hi or None) for lo, hi in width)]


def _pad_vjp(ans, array, pad_width, mode, **kwargs):
    assert mode == "constant", "Only constant mode padding is supported."
    return lambda g: _unpad(g, pad_width)


defvjp(anp.pad, _pad_vjp)


# ---- linspace (numpy_vjps.py:240-244) and gradient (297-342) ------------------------------------------
defvjp(
    anp.linspace,
    lambda ans, start, stop, num: lambda g: anp.dot(anp.linspace(1.0, 0.0, num), g),
    lambda ans, start, stop, num: lambda g: anp.dot(anp.linspace(0.0, 1.0, num), g),
)


def _grad_gradient(ans, x, *vargs, **kwargs):
    axis = kwargs.pop("axis", None)
    if vargs or kwargs:
        raise NotImplementedError("The only optional argument currently supported for np.gradient is axis.")
    if axis is None:
        axis = range(x.ndim)
    elif type(axis) is int:
        axis = [axis]
    else:
        axis = list(axis)
    x_dtype, x_shape, nd = x.dtype, x.shape, x.ndim

    def vjp(g):
        if anp.ndim(g) == nd:
            g = g[anp.newaxis]  # a single axis: numpy returned one array, not a list
        out = anp.zeros(x_shape, dtype=x_dtype)
        for i, a in enumerate(axis):
            g_swap = anp.swapaxes(g[i], 0, a)[:, anp.newaxis]
            out_axis = anp.concatenate(
                (
                    -g_swap[0] - 0.5 * g_swap[1],
                    g_swap[0] - 0.5 * g_swap[2],
                    (-1.0) * anp.gradient(g_swap, axis=0)[2:-2, 0],
                    0.5 * g_swap[-3] - g_swap[-1],
                    0.5 * g_swap[-2] + g_swap[-1],
                ),
                axis=0,
            )
            out = out + anp.swapaxes(out_axis, 0, a)
        return out

    return vjp


defvjp(anp.gradient, _grad_gradient)
