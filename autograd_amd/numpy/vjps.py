"""Reverse-mode rules of the device namespace.

Every rule computes what the cited rule of the reference's autograd/numpy/numpy_vjps.py
computes.  Each has two forms:

* concrete - when the cotangent and the saved values are plain ``DevArray`` s (the outermost
  backward pass, which is where the time goes), the whole rule, including the ``unbroadcast``
  sum that follows a broadcasting ufunc, is ONE fused kernel launch;
* traced - when any of them is a box (an outer differentiation is recording this backward
  pass), the rule is written with namespace primitives exactly like the reference's, so that
  it can itself be differentiated to any order.
"""

from functools import partial

import numpy as onp

from .._lib import REDUCE_FUSABLE, Op, Red
from ..core import BatchMode, NotBatchable, batch_safe
from ..extend import SparseObject, VJPNode, defvjp, defvjp_argnum, primitive, register_notrace, vspace
from ..tracer import isbox
from ..util import func
from . import devarray as D
from . import wrapper as anp
from .boxes import DevArrayBox
from .devarray import DevArray

# ---- functions with no derivative (numpy_vjps.py:13-68) -------------------------------------
nograd_functions = [
    anp.floor,
    anp.ceil,
    anp.rint,
    anp.round,
    anp.trunc,
    anp.sign,
    anp.equal,
    anp.not_equal,
    anp.less,
    anp.less_equal,
    anp.greater,
    anp.greater_equal,
]
for _f in nograd_functions:
    register_notrace(VJPNode, _f)


_F64 = onp.dtype("float64")


def _concrete(*xs):
    """True when no argument is a box: the fused kernels may be used."""
    for x in xs:
        if isbox(x):
            return False
    return True


def _shape_of(x):
    return x.shape if isinstance(x, DevArray) else onp.shape(x)


# ---- unbroadcast (numpy_vjps.py:883-897) -----------------------------------------------------
def unbroadcast(x, target_meta, broadcast_idx=0):
    """Traced form: sum ``x`` down to the shape it was broadcast from."""
    target_shape, target_ndim, _dtype, target_iscomplex = target_meta
    lead = BatchMode.active  # 1 while cotangents carry a leading batch axis, which is never summed away
    while anp.ndim(x) > target_ndim + lead:
        x = anp.sum(x, axis=broadcast_idx + lead)
    for axis, size in enumerate(target_shape):
        if size == 1:
            x = anp.sum(x, axis=axis + lead, keepdims=True)
    return x


def _fused_unbroadcast(op, target_meta, *operands):
    """Concrete form: ``unbroadcast(op(*operands), target_meta)`` in one launch.

    When the operands' broadcast shape equals the target shape this is a plain elementwise
    kernel; otherwise the sum over the broadcast axes runs in the same pass (map-reduce), so
    the full-size intermediate is never written.
    """
    target_shape, target_ndim, _dt, _c = target_meta
    target_shape = tuple(target_shape)
    batch = BatchMode.active  # the cotangent (and so the broadcast of the operands) has a leading batch axis
    if op == Op.COPY and _shape_of(operands[0])[batch:] == target_shape:
        return operands[0]  # add/subtract without broadcasting: the cotangent is `g` itself, no copy
    if not batch and type(operands[-1]) is D.LseCotangent and not operands[-1].computed():
        out = _consume_lse_cotangent(op, target_shape, operands)
        if out is not None:
            return out
    dt = D._float_dtype(D.result_dtype(*operands))
    shape = ()
    for x in operands:
        s = _shape_of(x)
        if s != shape:
            shape = D.broadcast_shapes(shape, s)
    if shape[batch:] == target_shape:
        return D.map_op(op, dt, *operands)
    lead = len(shape) - target_ndim - batch
    axes = [batch + i for i in range(lead)] + [batch + lead + a for a, size in enumerate(target_shape) if size == 1]
    if op not in REDUCE_FUSABLE:
        full = D.map_op(op, dt, *operands)
        out = D.map_reduce(Op.COPY, Red.SUM, dt, (full,), axes, True)
    else:
        out = D.map_reduce(op, Red.SUM, dt, operands, axes, True, shape=shape)
    return DevArray(out._t.reshape(shape[:batch] + target_shape), dt) if lead else out


def _consume_lse_cotangent(op, target_shape, operands):
    """``unbroadcast(op(*operands))`` when the cotangent (last operand) is an unwritten logsumexp cotangent
    and the request is one its fused pass serves; None otherwise."""
    s = operands[-1]
    rows, cols = s.shape
    if op == Op.COPY and target_shape in ((rows, 1), (rows,)):
        out = s.row_sums()
        return out if target_shape == (rows, 1) else out._view(lambda t: t.reshape(rows))
    if op == Op.MUL and len(operands) == 2 and isinstance(operands[0], DevArray) and operands[0].dtype == s.dtype:
        y = D.in_memory(operands[0])
        if target_shape == (rows, cols) and type(y) is DevArray and y.shape in ((1, cols), (cols,)):
            return s.scaled_by(y._t.reshape(1, cols).expand(rows, cols))
        if target_shape in ((1, cols), (cols,)) and y.shape == (rows, cols):
            out = s.col_sums_with(y)
            if out is not None and target_shape == (cols,):
                out = out._view(lambda t: t.reshape(cols))
            return out
    return None


def unbroadcast_f(target, f):
    target_meta = anp.metadata(target)
    return lambda g: unbroadcast(f(g), target_meta)


def _strong_scalar(x):
    """A scalar base of ``power`` as NumPy sees it inside the exponent's rule: ``anp.log(2.0)`` is a
    numpy.float64, which (unlike the Python float it came from) promotes a float32 array."""
    return onp.float64(x) if isinstance(x, (int, float)) and not isinstance(x, bool) else x


def _binary_rule(fun, traced0, traced1, fused0, fused1):
    """Register both cotangents of a broadcasting ufunc.

    ``traced*(ans, x, y)`` return ``g -> cotangent`` written with primitives (reference form);
    ``fused*(g, ans, x, y)`` return ``(op, operands)`` for the single-kernel form.
    """

    def maker(traced, fused, which):
        def make(ans, x, y):
            target = (x, y)[which]
            meta = anp.metadata(target)
            slow = traced(ans, x, y)

            def vjp(g):
                if _concrete(g, ans, x, y):
                    op, operands, *promote = fused(g, ans, x, y)
                    out = _fused_unbroadcast(op, meta, *operands)
                    if promote and out.dtype != promote[0]:
                        # the reference's expression has a float64 factor (see the rule): same
                        # values, NumPy's result dtype
                        out = D.astype(out, promote[0])
                    return out
                return unbroadcast(slow(g), meta)

            return vjp

        return make

    defvjp(fun, maker(traced0, fused0, 0), maker(traced1, fused1, 1))


# ---- binary ufuncs (numpy_vjps.py:76-143) ----------------------------------------------------
_binary_rule(
    anp.add,
    lambda ans, x, y: lambda g: g,
    lambda ans, x, y: lambda g: g,
    lambda g, ans, x, y: (Op.COPY, (g,)),
    lambda g, ans, x, y: (Op.COPY, (g,)),
)
_binary_rule(
    anp.subtract,
    lambda ans, x, y: lambda g: g,
    lambda ans, x, y: lambda g: -g,
    lambda g, ans, x, y: (Op.COPY, (g,)),
    lambda g, ans, x, y: (Op.NEG, (g,)),
)
_binary_rule(
    anp.multiply,
    lambda ans, x, y: lambda g: y * g,
    lambda ans, x, y: lambda g: x * g,
    lambda g, ans, x, y: (Op.MUL, (y, g)),
    lambda g, ans, x, y: (Op.MUL, (x, g)),
)
_binary_rule(
    anp.true_divide,
    lambda ans, x, y: lambda g: g / y,
    lambda ans, x, y: lambda g: -g * x / y**2,
    lambda g, ans, x, y: (Op.DIV, (g, y)),
    lambda g, ans, x, y: (Op.DIV_VJP1, (g, x, y)),
)
_binary_rule(
    anp.power,
    lambda ans, x, y: lambda g: g * y * x ** anp.where(y, y - 1, 1.0),
    lambda ans, x, y: lambda g: g * anp.log(replace_zero(x, 1.0)) * ans,
    lambda g, ans, x, y: (Op.POW_VJP0, (g, x, y)),
    lambda g, ans, x, y: (Op.POW_VJP1, (g, _strong_scalar(x), ans)),
)
for _chooser in (anp.maximum, anp.minimum, anp.fmax, anp.fmin):
    _binary_rule(
        _chooser,
        lambda ans, x, y: lambda g: g * balanced_eq(x, ans, y),
        lambda ans, x, y: lambda g: g * balanced_eq(y, ans, x),
        # balanced_eq divides a bool array by a float64 one, so `g * balanced_eq(...)` is float64
        # whatever g is; its factors 0, 1/2, 1 are exact in any precision
        lambda g, ans, x, y: (Op.CHOOSE_VJP, (g, x, ans, y), _F64),
        lambda g, ans, x, y: (Op.CHOOSE_VJP, (g, y, ans, x), _F64),
    )

def balanced_eq(x, z, y):
    return (x == z) / (1.0 + (x == y))


def replace_zero(x, val):
    return anp.where(x, x, val)


# ---- unary ufuncs (numpy_vjps.py:157-191) ----------------------------------------------------
def _unary_rule(fun, traced, fused):
    """``traced(ans, x)`` -> ``g -> cotangent`` with primitives; ``fused(g, ans, x)`` -> (op, operands)."""

    def make(ans, x):
        slow = traced(ans, x)

        def vjp(g):
            if _concrete(g, ans, x):
                op, operands = fused(g, ans, x)
                return D.float_map(op, *operands)
            return slow(g)

        return vjp

    defvjp(fun, make)


_unary_rule(anp.negative, lambda ans, x: lambda g: -g, lambda g, ans, x: (Op.NEG, (g,)))
_unary_rule(anp.exp, lambda ans, x: lambda g: ans * g, lambda g, ans, x: (Op.MUL, (ans, g)))
_unary_rule(anp.log, lambda ans, x: lambda g: g / x, lambda g, ans, x: (Op.DIV, (g, x)))
_unary_rule(anp.tanh, lambda ans, x: lambda g: g / anp.cosh(x) ** 2, lambda g, ans, x: (Op.TANH_VJP, (g, x)))
_unary_rule(anp.sinh, lambda ans, x: lambda g: g * anp.cosh(x), lambda g, ans, x: (Op.SINH_VJP, (g, x)))
_unary_rule(anp.cosh, lambda ans, x: lambda g: g * anp.sinh(x), lambda g, ans, x: (Op.COSH_VJP, (g, x)))
_unary_rule(anp.sin, lambda ans, x: lambda g: g * anp.cos(x), lambda g, ans, x: (Op.SIN_VJP, (g, x)))
_unary_rule(anp.cos, lambda ans, x: lambda g: -g * anp.sin(x), lambda g, ans, x: (Op.COS_VJP, (g, x)))
_unary_rule(anp.sqrt, lambda ans, x: lambda g: g * 0.5 * x**-0.5, lambda g, ans, x: (Op.SQRT_VJP, (g, x)))
_unary_rule(anp.square, lambda ans, x: lambda g: g * 2 * x, lambda g, ans, x: (Op.SQUARE_VJP, (g, x)))
_unary_rule(anp.reciprocal, lambda ans, x: lambda g: -g / x**2, lambda g, ans, x: (Op.RECIPROCAL_VJP, (g, x)))
_unary_rule(anp.log1p, lambda ans, x: lambda g: g / (x + 1), lambda g, ans, x: (Op.LOG1P_VJP, (g, x)))
_unary_rule(anp.expm1, lambda ans, x: lambda g: (ans + 1) * g, lambda g, ans, x: (Op.EXPM1_VJP, (g, ans)))
_unary_rule(
    anp.abs,
    lambda ans, x: lambda g: g * replace_zero(x, 0.0) / replace_zero(ans, 1.0),
    lambda g, ans, x: (Op.ABS_VJP, (g, x, ans)),
)

# the rest of the table (numpy_vjps.py:114-135, 160-185, 215): reference compositions, one launch per primitive
defvjp(
    anp.logaddexp,
    lambda ans, x, y: unbroadcast_f(x, lambda g: g * anp.exp(x - ans)),
    lambda ans, x, y: unbroadcast_f(y, lambda g: g * anp.exp(y - ans)),
)
defvjp(
    anp.logaddexp2,  # numpy_vjps.py:119-123
    lambda ans, x, y: unbroadcast_f(x, lambda g: g * 2 ** (x - ans)),
    lambda ans, x, y: unbroadcast_f(y, lambda g: g * 2 ** (y - ans)),
)
defvjp(
    anp.sinc,  # numpy_vjps.py:188-191
    lambda ans, x: lambda g: g * (anp.cos(anp.pi * x) * anp.pi * x - anp.sin(anp.pi * x)) / (anp.pi * x**2),
)
defvjp(
    anp.cross,  # numpy_vjps.py:231-239
    lambda ans, a, b, axisa=-1, axisb=-1, axisc=-1, axis=None: lambda g: anp.cross(b, g, axisb, axisc, axisa, axis),
    lambda ans, a, b, axisa=-1, axisb=-1, axisc=-1, axis=None: lambda g: anp.cross(g, a, axisc, axisa, axisb, axis),
)
defvjp(
    anp.remainder,  # numpy.mod is the same function (numpy_vjps.py:128-137)
    lambda ans, x, y: unbroadcast_f(x, lambda g: g),
    lambda ans, x, y: unbroadcast_f(y, lambda g: -g * anp.floor(x / y)),
)
defvjp(anp.nan_to_num, lambda ans, x: lambda g: anp.where(anp.isfinite(x), g, 0.0))  # 216
defvjp(
    anp.arctan2,
    lambda ans, x, y: unbroadcast_f(x, lambda g: g * y / (x**2 + y**2)),
    lambda ans, x, y: unbroadcast_f(y, lambda g: g * -x / (x**2 + y**2)),
)
defvjp(
    anp.hypot,
    lambda ans, x, y: unbroadcast_f(x, lambda g: g * x / ans),
    lambda ans, x, y: unbroadcast_f(y, lambda g: g * y / ans),
)
defvjp(anp.fabs, lambda ans, x: lambda g: anp.sign(x) * g)
defvjp(anp.exp2, lambda ans, x: lambda g: ans * anp.log(2) * g)
defvjp(anp.log2, lambda ans, x: lambda g: g / x / anp.log(2))
defvjp(anp.log10, lambda ans, x: lambda g: g / x / anp.log(10))
defvjp(anp.tan, lambda ans, x: lambda g: g / anp.cos(x) ** 2)
defvjp(anp.arcsin, lambda ans, x: lambda g: g / anp.sqrt(1 - x**2))
defvjp(anp.arccos, lambda ans, x: lambda g: -g / anp.sqrt(1 - x**2))
defvjp(anp.arctan, lambda ans, x: lambda g: g / (1 + x**2))
defvjp(anp.arcsinh, lambda ans, x: lambda g: g / anp.sqrt(x**2 + 1))
defvjp(anp.arccosh, lambda ans, x: lambda g: g / anp.sqrt(x**2 - 1))
defvjp(anp.arctanh, lambda ans, x: lambda g: g / (1 - x**2))
defvjp(anp.rad2deg, lambda ans, x: lambda g: g / anp.pi * 180.0)
defvjp(anp.deg2rad, lambda ans, x: lambda g: g * anp.pi / 180.0)
defvjp(anp.clip, lambda ans, x, a_min, a_max: lambda g: g * anp.logical_and(ans != a_min, ans != a_max))

def _float64_zeros(shape):
    """``numpy.zeros(shape)`` without the fill: a stride-0 view of the shared float64 zero."""
    from .vspaces import _shared_zero

    return DevArray(_shared_zero(_F64)._t.expand(tuple(shape)), _F64) if all(shape) else D.zeros(shape, _F64)


def _as_broadcast_from(operand, picked):
    """``picked`` summed down to the shape of ``operand`` when the choice was broadcast (numpy_vjps.py:228-229 leaves the
    cotangent in the shape of the result, which only fits an operand of that shape)."""
    if anp.shape(picked)[BatchMode.active:] == anp.shape(operand):
        return picked
    return unbroadcast(picked, anp.metadata(operand))


defvjp(
    anp._where3,
    None,
    # numpy_vjps.py:228-229: the zeros are float64 (anp.zeros(g.shape)), so a float32 cotangent comes out float64
    lambda ans, c, x, y: lambda g: _as_broadcast_from(x, anp.where(c, g, _float64_zeros(anp.shape(g)))),
    lambda ans, c, x, y: lambda g: _as_broadcast_from(y, anp.where(c, _float64_zeros(anp.shape(g)), g)),
)
defvjp(
    anp.astype,
    lambda ans, A, dtype, order="K", casting="unsafe", subok=True, copy=True: lambda g: anp.astype(g, anp.result_type(A)),
)

# ---- shape-only functions (numpy_vjps.py:192-217, 407-413, 804-812) --------------------------
def _shaped_like(g, shape, order=None):
    """The cotangent ``g`` of a reshaping function, given the operand's shape again (a leading batch axis stays)."""
    if BatchMode.active:
        shape = (anp.shape(g)[0],) + tuple(shape)
    return anp.reshape(g, shape, order=order)


defvjp(anp.reshape, lambda ans, x, shape, order=None: lambda g: _shaped_like(g, anp.shape(x), order))
defvjp(anp.ravel, lambda ans, x, order=None: lambda g: _shaped_like(g, anp.shape(x), order))
defvjp(anp.expand_dims, lambda ans, x, axis: lambda g: _shaped_like(g, anp.shape(x)))
defvjp(anp.squeeze, lambda ans, x, axis=None: lambda g: _shaped_like(g, anp.shape(x)))
def _behind_batch(axis, ndim):
    """Axis number(s) of an ``ndim``-d operand as they are in a cotangent that has a leading batch axis."""
    if isinstance(axis, (tuple, list)):
        return tuple(_behind_batch(a, ndim) for a in axis)
    return int(axis) % ndim + BatchMode.active


defvjp(anp.swapaxes, lambda ans, x, axis1, axis2: lambda g: anp.swapaxes(
    g, _behind_batch(axis2, anp.ndim(x)), _behind_batch(axis1, anp.ndim(x))))
defvjp(anp.moveaxis, lambda ans, a, source, destination: lambda g: anp.moveaxis(
    g, _behind_batch(destination, anp.ndim(a)), _behind_batch(source, anp.ndim(a))))


def _grad_transpose(ans, x, axes=None):
    nd = anp.ndim(x)
    back = tuple(int(i) for i in onp.argsort(axes)) if axes is not None else tuple(reversed(range(nd)))

    def vjp(g):
        if BatchMode.active:
            return anp.transpose(g, (0,) + tuple(i + 1 for i in back))
        return anp.transpose(g, back if axes is not None else None)

    return vjp


defvjp(anp.transpose, _grad_transpose)


def _grad_atleast(ans, *arys):
    if len(arys) > 1:
        raise NotImplementedError("Can't handle multiple arguments yet.")
    return lambda g: _shaped_like(g, anp.shape(arys[0]))


for _f in (anp.atleast_1d, anp.atleast_2d, anp.atleast_3d):
    defvjp(_f, _grad_atleast)


def _grad_broadcast_to(ans, x, new_shape):
    old_shape = anp.shape(x)
    assert len(old_shape) == len(new_shape), "Can't handle extra leading dims"
    axes = tuple(i for i, (o, n) in enumerate(zip(old_shape, new_shape)) if o == 1 and n > 1)
    return lambda g: anp.sum(g, axis=tuple(a + BatchMode.active for a in axes), keepdims=True) if axes else g


defvjp(anp.broadcast_to, _grad_broadcast_to)


# ---- reductions (numpy_vjps.py:416-461) ------------------------------------------------------
def repeat_to_match_shape(g, shape, dtype, axis, keepdims):
    """Broadcast a reduction's cotangent back over the reduced axes; returns ``(array, num_reps)``.

    The reference materialises the broadcast by adding a zeros array (numpy_vjps.py:416-427).
    Here it is a stride-0 view (``broadcast_to`` is a primitive with its own rules), so nothing
    is written; consumers read the small array through broadcast strides.  ``num_reps`` is a
    NumPy integer scalar as in the reference, which keeps its promotion behaviour: a float32
    cotangent divided by it becomes float64.
    """
    if shape == ():
        return g, 1
    axes = D.normalize_axes(axis, len(shape))
    new_shape = tuple(1 if d in axes else s for d, s in enumerate(shape))
    reps = 1
    for d in axes:
        reps *= shape[d]
    num_reps = onp.int64(reps)  # (what onp.prod(onp.array(shape)[axes]) gives, without three NumPy calls)
    if BatchMode.active:  # cotangents stacked along a leading axis: it is carried along
        n = anp.shape(g)[0]
        new_shape, shape = (n,) + new_shape, (n,) + shape
    elif type(g) is DevArray and (g.dtype == dtype or g.dtype == _F64):
        # the seed of `grad` (a shared one) or any other shared constant: the constant seen through the operand's
        # shape is a kept view (no tensor views are made for the commonest cotangent of a loss's final sum)
        t = g._t
        if t.numel() == 1:
            c = D.KNOWN_SCALARS.get(t.data_ptr())
            if c is not None:
                return D.constant(shape, c, g.dtype), num_reps
    if isinstance(g, DevArray) and (g.dtype == dtype or g.dtype == _F64):
        # a concrete cotangent that needs no promotion: the view itself, without the two primitive calls
        return g._view(lambda t: t.reshape(new_shape).expand(shape)), num_reps
    out = anp.broadcast_to(anp.reshape(g, new_shape), shape)
    if anp.result_type(g) != onp.result_type(anp.result_type(g), dtype):
        out = anp.astype(out, onp.result_type(anp.result_type(g), dtype))
    return out, num_reps


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


def _grad_var(ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_vjps.py:477-490
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, num_reps = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        x_minus_mean = x - anp.mean(x, axis=axis, keepdims=True)
        return 2.0 * g_repeated * x_minus_mean / (num_reps - ddof)

    return vjp


defvjp(anp._primitive_var, _grad_var)


def _grad_std(ans, x, axis=None, ddof=0, keepdims=False, **kwargs):
    # numpy_vjps.py:493-512
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, num_reps = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        if num_reps <= 1:
            return g_repeated * 0.0
        g_repeated, num_reps = repeat_to_match_shape(g / ans, shape, dtype, axis, keepdims)
        x_minus_mean = x - anp.mean(x, axis=axis, keepdims=True)
        return g_repeated * x_minus_mean / (num_reps - ddof)

    return vjp


defvjp(anp._primitive_std, _grad_std)


def _grad_prod(ans, x, axis=None, keepdims=False, **kwargs):
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        g_repeated, _ = repeat_to_match_shape(g * ans, shape, dtype, axis, keepdims)
        return g_repeated / x

    return vjp


defvjp(anp.prod, _grad_prod)


def _grad_chooser(ans, x, axis=None, keepdims=None, **kwargs):
    """max/min: the cotangent is shared equally by the positions that attain the extremum
    (numpy_vjps.py:515-530).  The reference multiplies by the boolean hit mask and divides by its
    integer sum, so the result is float64 whatever the operand's precision; the mask is taken as
    float64 here (0 and 1 are exact), which promotes the same way."""
    shape, dtype = anp.shape(x), anp.result_type(x)

    def vjp(g):
        if (_concrete(g, ans, x) and isinstance(x, DevArray) and isinstance(g, DevArray) and isinstance(ans, DevArray)
                and x.dtype == _F64 and g.dtype == _F64 and ans.dtype == _F64 and x.size and shape):
            # the same arithmetic in two launches: the number of hits per group (a comparison fused
            # into a sum), then (g * hit) / hits with g, ans and the count read through broadcast strides
            axes = D.normalize_axes(axis, len(shape))
            kept = D.reduce_shape(shape, axes, True)
            g_kept, ans_kept = (a._view(lambda t: t.reshape(kept)) for a in (g, ans))
            n_hits = D.map_reduce(Op.EQUAL_AS_FLOAT, Red.SUM, _F64, (x, ans_kept), axes, True, shape=shape)
            return D.map_op(Op.EXTREMUM_VJP, _F64, g_kept, x, ans_kept, n_hits)
        g_repeated, _ = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        ans_repeated, _ = repeat_to_match_shape(ans, shape, dtype, axis, keepdims)
        hits = anp.astype(x == ans_repeated, _F64)
        return g_repeated * hits / anp.sum(hits, axis=axis, keepdims=True)

    return vjp


defvjp(anp.max, _grad_chooser)
defvjp(anp.min, _grad_chooser)


def _grad_repeat(ans, x, repeats, axis=None):
    shape = anp.shape(x)

    def vjp(g):
        if axis is None:
            expanded = anp.reshape(g, (int(onp.prod(shape)),) + (repeats,))
            return anp.reshape(anp.sum(expanded, axis=1, keepdims=False), shape)
        ax = axis % len(shape)
        if shape[ax] == 1:
            return anp.sum(g, axis=ax, keepdims=True)
        expanded = anp.reshape(g, shape[0 : ax + 1] + (repeats,) + shape[ax + 1 :])
        return anp.sum(expanded, axis=ax + 1, keepdims=False)

    return vjp


defvjp(anp.repeat, _grad_repeat)


def _grad_tile(ans, x, reps):
    """numpy_vjps.py:352-362: the copies along every axis are added up, first axis first."""
    reps = (reps,) if anp.isscalar(reps) else tuple(reps)
    x_shape = anp.shape(x)

    def vjp(g):
        reps_full = (1,) * (anp.ndim(g) - len(reps)) + reps
        for axis, rep in enumerate(reps_full):
            shp = anp.shape(g)
            g = anp.sum(anp.reshape(g, shp[:axis] + (rep, shp[axis] // rep) + shp[axis + 1 :]), axis=axis)
        return anp.reshape(g, x_shape)

    return vjp


defvjp(anp.tile, _grad_tile)


def _grad_kron(argnum, ans, orig_A, orig_B):
    """numpy_vjps.py:368-392: G viewed with the two operands' axes side by side, then contracted
    with the other operand over all of its axes."""
    orig_A_shape, orig_B_shape = anp.shape(orig_A), anp.shape(orig_B)

    def vjp(G):
        A, B = anp.atleast_2d(orig_A), anp.atleast_2d(orig_B)
        shape = list(anp.shape(A) + anp.shape(B))
        n = anp.ndim(A)
        shape[n - 1], shape[n] = shape[n], shape[n - 1]
        paired = anp.swapaxes(anp.reshape(G, shape), n - 1, n)
        if argnum == 0:
            return anp.reshape(anp.tensordot(paired, B, axes=anp.ndim(B)), orig_A_shape)
        return anp.reshape(anp.tensordot(A, paired, axes=anp.ndim(A)), orig_B_shape)

    return vjp


defvjp(anp.kron, partial(_grad_kron, 0), partial(_grad_kron, 1))

# diagonals and triangles (numpy_vjps.py:193, 201, 205-213, 863-870)
defvjp(anp.roll, lambda ans, x, shift, axis=None: lambda g: anp.roll(g, -shift, axis=axis))
defvjp(anp.diag, lambda ans, x, k=0: lambda g: anp.diag(g, k))
# pieces of an array (numpy_vjps.py:194-198): the cotangent is the list of the pieces' cotangents, joined again
defvjp(anp.array_split, lambda ans, ary, idxs, axis=0: lambda g: anp.concatenate(g, axis=axis))
defvjp(anp.split, lambda ans, ary, idxs, axis=0: lambda g: anp.concatenate(g, axis=axis))
defvjp(anp.vsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=0))
defvjp(anp.hsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=1))
defvjp(anp.dsplit, lambda ans, ary, idxs: lambda g: anp.concatenate(g, axis=2))


def _grad_rollaxis(ans, a, axis, start=0):  # numpy_vjps.py:255-267
    if axis < 0:
        raise NotImplementedError("Gradient of rollaxis not implemented for axis < 0. Please use moveaxis instead.")
    if start < 0:
        raise NotImplementedError("Gradient of rollaxis not implemented for start < 0. Please use moveaxis instead.")
    return lambda g: anp.rollaxis(g, start - 1, axis) if start > axis else anp.rollaxis(g, start, axis + 1)


defvjp(anp.rollaxis, _grad_rollaxis)


def _grad_diff(ans, a, n=1, axis=-1):
    """numpy_vjps.py:270-294: each differencing is undone by joining minus the first cotangent, minus the
    differences of the cotangents, and the last cotangent."""
    nd = anp.ndim(a)
    ans_shape = anp.shape(ans)
    first, last = [slice(None)] * nd, [slice(None)] * nd
    first[axis], last[axis] = slice(None, 1), slice(-1, None)

    def undiff(g):
        if anp.shape(g)[axis] > 0:
            return anp.concatenate((-g[tuple(first)], -anp.diff(g, axis=axis), g[tuple(last)]), axis=axis)
        shape = list(ans_shape)
        shape[axis] = 1
        return anp.zeros(shape)

    def vjp(g):
        for _ in range(n):
            g = undiff(g)
        return g

    return vjp


defvjp(anp.diff, _grad_diff)


def _reverse_axis(x, axis):  # numpy_vjps.py:533-536
    x = anp.swapaxes(x, axis, 0)
    x = x[::-1, ...]
    return anp.swapaxes(x, 0, axis)


def _grad_cumsum(ans, x, axis=None):  # numpy_vjps.py:539-549
    def vjp(g):
        if axis:
            return _reverse_axis(anp.cumsum(_reverse_axis(g, axis), axis), axis)
        return anp.reshape(anp.cumsum(g[::-1], axis)[::-1], anp.shape(x))

    return vjp


defvjp(anp.cumsum, _grad_cumsum)


def _grad_sort(ans, x, axis=-1, kind="quicksort", order=None, *_):
    """numpy_vjps.py:773-795 (sort and partition alike): the cotangent goes back through the inverse of the
    sorting permutation.  The reference does this for vectors only and raises for anything else; here every
    line along ``axis`` is un-permuted (``axis=None`` sorts the flattened array)."""
    if axis is None:
        order_, rank = anp.sort_permutations(anp.ravel(x), 0)
        return lambda g: anp.reshape(anp._reorder(g, rank, order_, 0), anp.shape(x))
    order_, rank = anp.sort_permutations(x, axis)
    return lambda g: anp._reorder(g, rank, order_, axis)


defvjp(anp.sort, _grad_sort)
defvjp(anp.partition, lambda ans, x, kth, axis=-1, kind="introselect", order=None: _grad_sort(ans, x, axis))
defvjp(anp._reorder, lambda ans, x, index, inverse, axis=0: lambda g: anp._reorder(g, inverse, index, axis))
defvjp(anp.flipud, lambda ans, x: lambda g: anp.flipud(g))
defvjp(anp.fliplr, lambda ans, x: lambda g: anp.fliplr(g))
defvjp(anp.flip, lambda ans, x, axis=None: lambda g: anp.flip(g, axis))  # not in the reference's table: its own inverse
defvjp(anp.rot90, lambda ans, x, k=1: lambda g: anp.rot90(g, -k))
defvjp(anp.triu, lambda ans, x, k=0: lambda g: anp.triu(g, k=k))
defvjp(anp.tril, lambda ans, x, k=0: lambda g: anp.tril(g, k=k))
defvjp(
    anp.trace,  # the reference's einsum("ij,...->ij...", eye, g) has no summed index: a broadcast product
    lambda ans, x, offset=0: lambda g: anp.reshape(
        anp.eye(anp.shape(x)[0], anp.shape(x)[1], k=offset), anp.shape(x)[:2] + (1,) * anp.ndim(g)
    )
    * g,
)
defvjp(
    anp.diagonal,
    lambda ans, A, offset=0, axis1=0, axis2=1: lambda g: anp.make_diagonal(g, offset, axis1, axis2),
)
defvjp(
    anp.make_diagonal,
    lambda ans, D_, offset=0, axis1=0, axis2=1: lambda g: anp.diagonal(g, offset, axis1, axis2),
)
for _identity in (anp.real, anp.real_if_close, anp.conjugate):
    defvjp(_identity, lambda ans, x: lambda g: g)
for _flat in (anp.imag, anp.angle):  # numpy_vjps.py:220-224 evaluated for a real argument: nothing comes back
    defvjp(_flat, lambda ans, x: lambda g: anp.zeros_like(x))


# ---- dense contractions (numpy_vjps.py:552-747) ----------------------------------------------
def _as_dtype(x, dtype):
    return x if x.dtype == dtype else D.astype(x, dtype)


@primitive
def dot_adjoint_0(B, G, A_meta, B_meta):
    """Cotangent of ``dot(A, B)`` with respect to ``A`` (numpy_vjps.py:615-624): for matrices
    ``G . B^T``, read through swapped strides - B is never transposed in memory."""
    _, A_ndim, A_dtype, _ = A_meta
    _, B_ndim, _, _ = B_meta
    if A_ndim == 2 and B_ndim == 2:
        B, G = D.asarray(B), D.asarray(G)
        dt = D._float_dtype(D.result_dtype(B, G))
        out = DevArray(D.gemm2d(_as_dtype(G, dt)._t, _as_dtype(B, dt)._t.t(), dt), dt)
        return _as_dtype(out, onp.dtype(A_dtype))
    if B_ndim == 0 or B_ndim == 1 or A_ndim == 0:
        contract_num = max(0, B_ndim - (A_ndim != 0))
        out = anp.tensordot.fun(G, B, contract_num)
    else:
        out = anp.tensordot.fun(G, anp.swapaxes.fun(D.asarray(B), -1, -2), B_ndim - 1)
    return _as_dtype(out, onp.dtype(A_dtype))


@primitive
def dot_adjoint_1(A, G, A_meta, B_meta):
    """Cotangent of ``dot(A, B)`` with respect to ``B`` (numpy_vjps.py:627-638): for matrices
    ``A^T . G`` computed directly (the reference forms ``(G^T A)^T`` and returns a transposed
    view; the values are the same, the result here is contiguous)."""
    _, A_ndim, _, _ = A_meta
    _, B_ndim, B_dtype, _ = B_meta
    A, G = D.asarray(A), D.asarray(G)
    if A_ndim == 2 and B_ndim == 2:
        dt = D._float_dtype(D.result_dtype(A, G))
        out = DevArray(D.gemm2d(_as_dtype(A, dt)._t.t(), _as_dtype(G, dt)._t, dt), dt)
        return _as_dtype(out, onp.dtype(B_dtype))
    needs_transpose = B_ndim > 1 and A_ndim != 0
    swap = (lambda x: anp.swapaxes.fun(x, -1, -2)) if needs_transpose else (lambda x: x)
    if A_ndim == 0 or A_ndim == 1 or B_ndim == 0:
        contract_num = max(0, A_ndim - (B_ndim != 0))
        out = swap(anp.tensordot.fun(G, A, contract_num))
    else:
        out = swap(
            anp.tensordot.fun(G, A, [list(range(-A_ndim - B_ndim + 2, -B_ndim + 1)), list(range(A_ndim - 1))])
        )
    return _as_dtype(out, onp.dtype(B_dtype))


def _matrix_operands(dtype_wanted, *xs):
    """The operands as plain tensors when all are concrete 2-d float device arrays of one dtype."""
    for x in xs:
        if not isinstance(x, DevArray) or x.ndim != 2 or x.dtype != dtype_wanted or x.dtype not in D._FLOATS:
            return None
    return tuple(x._t for x in xs)


def _dot_vjp_0(ans, A, B):
    A_meta, B_meta = anp.metadata(A), anp.metadata(B)

    def vjp(g):
        if BatchMode.active:  # stacked matrix cotangents: one batched product with B^T shared by the batch
            if A_meta[1] != 2 or B_meta[1] != 2:
                raise NotBatchable
            return anp.astype(anp.matmul(g, anp.swapaxes(B, -1, -2)), A_meta[2])
        ts = _matrix_operands(A_meta[2], g, B) if A_meta[1] == 2 and B_meta[1] == 2 and _concrete(g, B) else None
        if ts is not None:
            return D.PendingProduct(ts[0], ts[1].t(), A_meta[2])  # added into A's accumulator by the contraction itself
        return dot_adjoint_0(B, g, A_meta, B_meta)

    return vjp


def _dot_vjp_1(ans, A, B):
    A_meta, B_meta = anp.metadata(A), anp.metadata(B)

    def vjp(g):
        if BatchMode.active:
            if A_meta[1] != 2 or B_meta[1] != 2:
                raise NotBatchable
            return anp.astype(anp.matmul(anp.swapaxes(A, -1, -2), g), B_meta[2])
        ts = _matrix_operands(B_meta[2], A, g) if A_meta[1] == 2 and B_meta[1] == 2 and _concrete(A, g) else None
        if ts is not None:
            return D.PendingProduct(ts[0].t(), ts[1], B_meta[2])
        return dot_adjoint_1(A, g, A_meta, B_meta)

    return vjp


defvjp(anp.dot, _dot_vjp_0, _dot_vjp_1)
defvjp(
    dot_adjoint_0,
    lambda ans, B, g, An, Bn: lambda A: dot_adjoint_1(A, g, An, Bn),
    lambda ans, B, g, An, Bn: lambda A: anp.dot(A, B),
)
defvjp(
    dot_adjoint_1,
    lambda ans, A, g, An, Bn: lambda B: dot_adjoint_0(B, g, An, Bn),
    lambda ans, A, g, An, Bn: lambda B: anp.dot(A, B),
)


def _matmul_cotangent(wrt_left, other, g, other_ndim, target_meta):
    """Cotangent of ``matmul(A, B)`` (numpy_vjps.py:567-612) for the left (``wrt_left``) or right operand, the
    other one being ``other``.  matmul treats a 1-d left operand as a single row and a 1-d right operand as a
    single column and drops that unit axis from its result; here the axis is put back on ``g`` (and on a 1-d
    ``other``), the cotangent is one stacked matrix product, ``g . B^T`` or ``A^T . g``, and the unit axis of a
    1-d target is dropped again.  Stacks that were broadcast are summed by ``unbroadcast``."""
    target_ndim = target_meta[1]
    if anp.ndim(g) == 0:  # vector times vector
        return unbroadcast(g * other, target_meta)
    left_is_vector = (target_ndim if wrt_left else other_ndim) == 1
    right_is_vector = (other_ndim if wrt_left else target_ndim) == 1
    if right_is_vector:
        g = anp.expand_dims(g, -1)              # the column axis of the result
    if left_is_vector:
        g = anp.expand_dims(g, -2)              # the row axis of the result
    if other_ndim == 1:
        other = anp.expand_dims(other, -1 if wrt_left else 0)   # B as a column / A as a row
    other_t = anp.swapaxes(other, -1, -2)
    out = anp.matmul(g, other_t) if wrt_left else anp.matmul(other_t, g)
    if target_ndim == 1:
        out = anp.squeeze(out, -2 if wrt_left else -1)
    return unbroadcast(out, target_meta)


def _matmul_adjoint_0(B, G, A_meta, B_ndim):
    return _matmul_cotangent(True, B, G, B_ndim, A_meta)


def _matmul_adjoint_1(A, G, A_ndim, B_meta):
    return _matmul_cotangent(False, A, G, A_ndim, B_meta)


def _matmul_vjp_0(ans, A, B):
    A_meta, B_ndim = anp.metadata(A), anp.ndim(B)

    def vjp(g):
        ts = _matrix_operands(A_meta[2], g, B) if A_meta[1] == 2 and B_ndim == 2 and _concrete(g, B) else None
        if ts is not None:  # matrices: the same pending product as for dot
            return D.PendingProduct(ts[0], ts[1].t(), A_meta[2])
        return _matmul_adjoint_0(B, g, A_meta, B_ndim)

    return vjp


def _matmul_vjp_1(ans, A, B):
    A_ndim, B_meta = anp.ndim(A), anp.metadata(B)

    def vjp(g):
        ts = _matrix_operands(B_meta[2], A, g) if A_ndim == 2 and B_meta[1] == 2 and _concrete(A, g) else None
        if ts is not None:
            return D.PendingProduct(ts[0].t(), ts[1], B_meta[2])
        return _matmul_adjoint_1(A, g, A_ndim, B_meta)

    return vjp


defvjp(anp.matmul, _matmul_vjp_0, _matmul_vjp_1)


def _split_axes(axes, A_ndim, B_ndim):
    axes0 = [axes[0]] if type(axes[0]) is int else list(axes[0])
    axes1 = [axes[1]] if type(axes[1]) is int else list(axes[1])
    summed = [onp.asarray(axes0, dtype="int64") % A_ndim, onp.asarray(axes1, dtype="int64") % B_ndim]
    other = [onp.delete(onp.arange(A_ndim), summed[0]), onp.delete(onp.arange(B_ndim), summed[1])]
    return summed, other


def _ints(a):
    return [int(i) for i in a]


@primitive
def tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim):
    """Adjoint of ``A -> tensordot(A, B, axes)`` (numpy_vjps.py:666-691): one MFMA contraction
    of permuted views plus a final axis permutation (a view)."""
    if B_ndim == 0:
        return D.arith_map(Op.MUL, G, B)
    G_axes = list(range(anp.ndim(G)))
    if type(axes) is int:
        axes = max(axes, 0)
        return anp.tensordot.fun(G, B, [G_axes[A_ndim - axes :], list(range(B_ndim))[axes:]])
    summed, other = _split_axes(axes, A_ndim, B_ndim)
    out = anp.tensordot.fun(G, B, [G_axes[len(other[0]) :], _ints(other[1])])
    perm = onp.argsort(onp.concatenate((other[0], summed[0][onp.argsort(summed[1])])))
    return anp.transpose.fun(out, _ints(perm))


@primitive
def tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim):
    """Adjoint of ``B -> tensordot(A, B, axes)`` (numpy_vjps.py:694-719)."""
    if A_ndim == 0:
        return D.arith_map(Op.MUL, G, A)
    G_axes = list(range(anp.ndim(G)))
    if type(axes) is int:
        axes = max(axes, 0)
        A_axes = list(range(A_ndim))
        return anp.tensordot.fun(A, G, [A_axes[: A_ndim - axes], G_axes[: A_ndim - axes]])
    summed, other = _split_axes(axes, A_ndim, B_ndim)
    out = anp.tensordot.fun(A, G, [_ints(other[0]), G_axes[: len(other[0])]])
    perm = onp.argsort(onp.concatenate((summed[1][onp.argsort(summed[0])], other[1])))
    return anp.transpose.fun(out, _ints(perm))


def _tensordot_vjp_0(ans, A, B, axes=2):
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    return lambda G: tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim)


def _tensordot_vjp_1(ans, A, B, axes=2):
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    return lambda G: tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim)


defvjp(anp.tensordot, _tensordot_vjp_0, _tensordot_vjp_1)
defvjp(
    tensordot_adjoint_0,
    lambda ans, B, G, axes, An, Bn: lambda A: tensordot_adjoint_1(A, G, axes, An, Bn),
    lambda ans, B, G, axes, An, Bn: lambda A: anp.tensordot(A, B, axes),
)
defvjp(
    tensordot_adjoint_1,
    lambda ans, A, G, axes, An, Bn: lambda B: tensordot_adjoint_0(B, G, axes, An, Bn),
    lambda ans, A, G, axes, An, Bn: lambda B: anp.tensordot(A, B, axes),
)
defvjp(
    anp.outer,
    lambda ans, a, b: lambda g: anp.dot(g, anp.ravel(b)),
    lambda ans, a, b: lambda g: anp.dot(anp.ravel(a), g),
)


def _grad_inner(argnum, ans, A, B):  # numpy_vjps.py:552-563
    A_ndim, B_ndim = anp.ndim(A), anp.ndim(B)
    axes = ([], []) if A_ndim == 0 or B_ndim == 0 else ([A_ndim - 1], [B_ndim - 1])
    if argnum == 0:
        return lambda G: tensordot_adjoint_0(B, G, axes, A_ndim, B_ndim)
    return lambda G: tensordot_adjoint_1(A, G, axes, A_ndim, B_ndim)


defvjp(anp.inner, partial(_grad_inner, 0), partial(_grad_inner, 1))


# ---- einsum (numpy_vjps.py:815-860, subscript-string convention) ------------------------------------
def _einsum_spread(cot, have, want, extents):
    """The cotangent ``cot`` (axes named by the distinct letters ``have``) laid out with the axes ``want`` of an
    einsum operand of shape ``extents``.  A letter of ``want`` missing from ``have`` was summed over by the forward
    pass without meeting any other operand: every position along it receives the same value (a broadcast).  A
    letter that ``want`` repeats read a diagonal going forward: its cotangent goes back onto that diagonal, zeros
    elsewhere (a product with an identity matrix placed on the two axes)."""
    distinct = "".join(dict.fromkeys(want))
    size = {c: extents[want.index(c)] for c in distinct}
    if have != distinct:
        cot = anp.reshape(cot, tuple(size[c] if c in have else 1 for c in distinct))
        cot = anp.broadcast_to(cot, tuple(size[c] for c in distinct))
    labels = list(distinct)
    for c in distinct:
        times = want.count(c)
        if times == 1:
            continue
        if times > 2:
            raise NotImplementedError(f"einsum: index {c!r} repeated {times} times in one operand")
        at = labels.index(c)
        # x[..., i, ...] -> y[..., i, j, ...] = x[..., i, ...] * (i == j)
        delta = anp.reshape(anp.eye(size[c]), (1,) * at + (size[c], size[c]) + (1,) * (len(labels) - at - 1))
        cot = anp.expand_dims(cot, at + 1) * delta
        labels.insert(at + 1, c)
    # labels now holds every axis of `want`, repeated letters adjacent: permute into `want`'s order
    order, used = [], [False] * len(labels)
    for c in want:
        k = next(i for i, (l, u) in enumerate(zip(labels, used)) if l == c and not u)
        used[k] = True
        order.append(k)
    return cot if order == list(range(len(order))) else anp.transpose(cot, order)


def _grad_einsum(argnum, ans, operands_, kwargs):
    """numpy_vjps.py:815-857, both calling conventions at once: the cotangent of operand k is the einsum of the
    output cotangent with all other operands, onto k's own letters."""
    target_meta = anp.metadata(operands_[argnum])
    position = argnum - 1 if isinstance(operands_[0], str) else argnum // 2

    def vjp(g):
        in_subs, out_subs, arrays = anp.parse_einsum_input(*operands_)
        subs = in_subs.split(",")
        wanted = subs[position]
        others = [a for k, a in enumerate(arrays) if k != position]
        other_subs = [sx for k, sx in enumerate(subs) if k != position]
        seen_elsewhere = set(out_subs).union(*other_subs)
        reachable = "".join(dict.fromkeys(c for c in wanted if c in seen_elsewhere))
        cot = anp.einsum(",".join([out_subs] + other_subs) + "->" + reachable, g, *others)
        return unbroadcast(_einsum_spread(cot, reachable, wanted, target_meta[0]), target_meta)

    return vjp


defvjp_argnum(anp.einsum, _grad_einsum)


# ---- concatenate / array construction (numpy_vjps.py:750-759, 922-938) -----------------------
def _grad_concatenate_args(argnum, ans, axis_args, kwargs):
    axis, args = axis_args[0], axis_args[1:]
    sizes = [anp.shape(a)[axis] for a in args[:argnum]]
    start = sum(sizes[:-1])
    idxs = [slice(None)] * anp.ndim(ans)
    idxs[axis] = slice(start, start + sizes[-1])
    return lambda g: g[(slice(None),) * BatchMode.active + tuple(idxs)]


defvjp_argnum(anp.concatenate_args, _grad_concatenate_args)
defvjp_argnum(anp.array_from_args, lambda argnum, ans, args, kwargs: lambda g: g[(slice(None),) * BatchMode.active + (argnum - 2,)])


def _grad_array_from_scalar_or_array(ans, array_args, array_kwargs, scarray):
    ndmin = array_kwargs.get("ndmin", 0)
    scarray_ndim = anp.ndim(scarray)
    if ndmin > scarray_ndim:
        return lambda g: anp.squeeze(g, axis=tuple(range(ndmin - scarray_ndim)))
    return lambda g: g


defvjp(anp._array_from_scalar_or_array, _grad_array_from_scalar_or_array, argnums=(2, 3))
# numpy_vjps.py:240-244: each sample is a fixed mix of the two end points; the mixing weights come from linspace itself
# (float64, as there, whatever the end points' precision)
defvjp(
    anp.linspace,
    lambda ans, start, stop, num=50, endpoint=True, dtype=None: lambda g: anp.dot(anp.linspace(1.0, 0.0, num, endpoint), g),
    lambda ans, start, stop, num=50, endpoint=True, dtype=None: lambda g: anp.dot(anp.linspace(0.0, 1.0, num, endpoint), g),
)
# numpy_vjps.py:88-89: every output element is the fill value, so its cotangent is their sum
defvjp(anp.full, lambda ans, shape, fill_value, dtype=None: lambda g: anp.sum(g), argnums=(1,))


# ---- indexing (numpy_vjps.py:941-954) --------------------------------------------------------
@primitive
def untake(x, idx, vs):
    """Cotangent of ``A[idx]``: a sparse object whose ``mut_add`` scatters ``x`` into a dense
    buffer - a strided in-place add for slices, the ordered scatter-add kernel (numpy.add.at
    order, bit for bit) for integer-array indices."""

    def mut_add(A):
        return anp.scatter_add(A, idx, x)

    return SparseObject(vs, mut_add)


def _only_inserts_unit_axes(idx):
    """True for indices made of ``None``, ``...`` and full slices: ``b[None, :]``, ``c[:, None]``."""
    items = idx if isinstance(idx, tuple) else (idx,)
    for it in items:
        if it is None or it is Ellipsis:
            continue
        if isinstance(it, slice) and it.start is None and it.stop is None and it.step is None:
            continue
        return False
    return True


def _grad_getitem(ans, A, idx):
    # numpy_vjps.py:954: untake(g, idx, vspace(A)), a sparse cotangent that add_outgrads scatters into zeros.
    # An index that only inserts unit axes selects every element exactly once, so that scatter is
    # `zeros + g` with A's shape: the cotangent itself, reshaped (nothing is launched).
    vs = vspace(A)

    def stacked(g):
        # cotangents stacked along a leading axis: the same selection behind a full slice, scattered into a
        # buffer with the batch axis in front (basic indices only: array indices would reorder result axes)
        if not anp._is_basic_index(idx):
            raise NotBatchable
        items = idx if isinstance(idx, tuple) else (idx,)
        wide = vspace(anp.zeros((anp.shape(g)[0],) + tuple(vs.shape), dtype=vs.dtype))
        return untake(g, (slice(None),) + tuple(items), wide)

    if _only_inserts_unit_axes(idx):
        shape, dtype = vs.shape, vs.dtype

        def vjp(g):
            if BatchMode.active:
                return _shaped_like(g, shape) if isinstance(g, DevArray) and g.dtype == dtype else stacked(g)
            if isinstance(g, DevArray) and g.dtype == dtype:
                return anp.reshape.fun(g, shape)
            return untake(g, idx, vs)

        return vjp
    return lambda g: stacked(g) if BatchMode.active else untake(g, idx, vs)


defvjp(func(DevArrayBox.__getitem__), _grad_getitem)
defvjp(untake, lambda ans, x, idx, _: lambda g: g[idx])


def _unpad(array, width):
    # numpy_vjps.py:957-967
    idxs = tuple(slice(l, -u or None) for l, u in anp.pad_widths(width, anp.ndim(array)))
    return array[idxs]


def pad_vjp(ans, array, pad_width, mode, **kwargs):
    # numpy_vjps.py:970-975
    assert mode == "constant", "Only constant mode padding is supported."
    return lambda g: _unpad(g, pad_width)


defvjp(anp.pad, pad_vjp)


# ---- rules that take cotangents stacked along a leading batch axis (core.batched_backward_pass) --------
# Elementwise rules broadcast the saved operands against the stacked cotangent as they are; the helpers
# they share (unbroadcast, repeat_to_match_shape, _shaped_like) leave the batch axis alone while
# BatchMode.active is set.  Everything not listed is replayed slice by slice.
batch_safe(
    anp.add, anp.subtract, anp.multiply, anp.true_divide, anp.power, anp.maximum, anp.minimum, anp.fmax, anp.fmin,
    anp.negative, anp.exp, anp.log, anp.tanh, anp.sinh, anp.cosh, anp.sin, anp.cos, anp.sqrt, anp.square,
    anp.reciprocal, anp.log1p, anp.expm1, anp.abs, anp.fabs, anp.logaddexp, anp.logaddexp2, anp.sinc, anp.remainder,
    anp.arctan2, anp.hypot, anp.exp2, anp.log2, anp.log10, anp.tan, anp.arcsin, anp.arccos, anp.arctan, anp.arcsinh,
    anp.arccosh, anp.arctanh, anp.rad2deg, anp.deg2rad, anp.clip, anp.nan_to_num, anp._where3, anp.astype,
    anp.reshape, anp.ravel, anp.expand_dims, anp.squeeze, anp.sum, anp._primitive_mean, anp.dot,
    anp.real, anp.real_if_close, anp.conjugate, anp.swapaxes, anp.moveaxis, anp.transpose, anp.atleast_1d,
    anp.atleast_2d, anp.atleast_3d, anp.broadcast_to, func(DevArrayBox.__getitem__), anp.concatenate_args,
    anp.array_from_args,
)
