"""The device array namespace: NumPy-named functions on ``DevArray`` wrapped as primitives.

Counterpart of the reference's autograd/numpy/numpy_wrapper.py:25-236 for the part of NumPy the
hot path uses.  Each differentiable function is a ``primitive`` whose raw implementation
launches HIP kernels; shape queries are never traced; list-taking functions are routed through
``concatenate_args`` / ``array_from_args`` so boxes inside Python lists are seen.
"""

import builtins
import numbers

import numpy as onp
import torch

from .. import _lib
from ..extend import notrace_primitive, primitive
from ..tracer import box_types as _box_types
from ..tracer import getval as _getval
from ..tracer import trace_stack as _trace_stack
from . import devarray as D
from .._lib import Cmp, Op, Red
from .devarray import DevArray

# constants and dtypes
pi, e, inf, nan, newaxis = onp.pi, onp.e, onp.inf, onp.nan, None
euler_gamma = onp.euler_gamma
float32, float64, bool_ = onp.float32, onp.float64, onp.bool_
dtype, __version__ = onp.dtype, onp.__version__
ndarray = DevArray


def _int_type(cls):
    """NumPy's integer scalar type, which also casts a device array or a box around one (untraced: an integer
    has no tangent).  The reference subclasses the integer types for the same reason, numpy_wrapper.py:18-22 and
    42-43; as a dtype the subclass means its parent."""

    def make(kind, value=0, *args):
        from ..tracer import getval

        value = getval(value)
        return D.astype(value, cls) if isinstance(value, DevArray) else cls(value, *args)

    return type(cls.__name__, (cls,), {"__new__": make, "__doc__": cls.__doc__})


int8, int16, int32, int64 = onp.int8, onp.int16, _int_type(onp.int32), _int_type(onp.int64)  # (the device holds the last two)


def _wrap(raw, name):
    raw.__name__ = name
    raw.__qualname__ = name
    return primitive(raw)


# ---- elementwise ----------------------------------------------------------------------------
def _unary(op, name):
    def raw(x):
        return D.float_map(op, x)

    return _wrap(raw, name)


negative = _wrap(lambda x: D.arith_map(Op.NEG, x), "negative")
exp = _unary(Op.EXP, "exp")
log = _unary(Op.LOG, "log")
tanh = _unary(Op.TANH, "tanh")
sinh = _unary(Op.SINH, "sinh")
cosh = _unary(Op.COSH, "cosh")
sin = _unary(Op.SIN, "sin")
cos = _unary(Op.COS, "cos")
sqrt = _unary(Op.SQRT, "sqrt")
log1p = _unary(Op.LOG1P, "log1p")
expm1 = _unary(Op.EXPM1, "expm1")
reciprocal = _unary(Op.RECIPROCAL, "reciprocal")
exp2 = _unary(Op.EXP2, "exp2")
log2 = _unary(Op.LOG2, "log2")
log10 = _unary(Op.LOG10, "log10")
tan = _unary(Op.TAN, "tan")
arcsin = _unary(Op.ARCSIN, "arcsin")
arccos = _unary(Op.ARCCOS, "arccos")
arctan = _unary(Op.ARCTAN, "arctan")
arcsinh = _unary(Op.ARCSINH, "arcsinh")
arccosh = _unary(Op.ARCCOSH, "arccosh")
arctanh = _unary(Op.ARCTANH, "arctanh")
fabs = _wrap(lambda x: D.float_map(Op.ABS, x), "fabs")
# numpy's loops multiply by the constant 180/pi resp. pi/180
rad2deg = degrees = _wrap(lambda x: D.float_map(Op.MUL, x, 180.0 / onp.pi), "rad2deg")
deg2rad = radians = _wrap(lambda x: D.float_map(Op.MUL, x, onp.pi / 180.0), "deg2rad")
square = _wrap(lambda x: D.arith_map(Op.SQUARE, x), "square")
abs = absolute = _wrap(lambda x: D.arith_map(Op.ABS, x), "abs")  # noqa: A001
sign = _wrap(lambda x: D.arith_map(Op.SIGN, x), "sign")


def _rounding(op, name):
    def raw(x, decimals=0, out=None):
        if decimals != 0:
            raise NotImplementedError(f"{name}: only decimals=0 is supported on the device")
        x = D.asarray(x)
        return D.map_op(op, x.dtype, x) if x.dtype in D._FLOATS else x

    return _wrap(raw, name)


floor = _rounding(Op.FLOOR, "floor")
ceil = _rounding(Op.CEIL, "ceil")
rint = _rounding(Op.RINT, "rint")
round = around = _rounding(Op.RINT, "round")  # noqa: A001
trunc = fix = _rounding(Op.TRUNC, "trunc")


def _binary(op, name, floating=False):
    fn = D.float_map if floating else D.arith_map

    def raw(x, y):
        return fn(op, x, y)

    return _wrap(raw, name)


add = _binary(Op.ADD, "add")
subtract = _binary(Op.SUB, "subtract")
multiply = _binary(Op.MUL, "multiply")
divide = true_divide = _binary(Op.DIV, "true_divide", floating=True)
power = _binary(Op.POW, "power")
maximum = _binary(Op.MAXIMUM, "maximum")
minimum = _binary(Op.MINIMUM, "minimum")
fmax = _binary(Op.FMAX, "fmax")
fmin = _binary(Op.FMIN, "fmin")
arctan2 = _binary(Op.ARCTAN2, "arctan2", floating=True)
hypot = _binary(Op.HYPOT, "hypot", floating=True)
logaddexp = _binary(Op.LOGADDEXP, "logaddexp", floating=True)
mod = remainder = _binary(Op.REMAINDER, "remainder", floating=True)
logaddexp2 = _binary(Op.LOGADDEXP2, "logaddexp2", floating=True)
nan_to_num = _unary(Op.NAN_TO_NUM, "nan_to_num")


@primitive
def clip(a, a_min, a_max):
    """``numpy.clip`` with scalar or array bounds: minimum(maximum(a, a_min), a_max)."""
    a = D.asarray(a)
    dt = D._float_dtype(D.result_dtype(a, a_min, a_max))
    return D.map_op(Op.MINIMUM, dt, D.map_op(Op.MAXIMUM, dt, a, a_min), a_max)


def _compare(cmp, name):
    def raw(x, y):
        return D.compare(cmp, x, y)

    return _wrap(raw, name)


equal = _compare(Cmp.EQ, "equal")
not_equal = _compare(Cmp.NE, "not_equal")
less = _compare(Cmp.LT, "less")
less_equal = _compare(Cmp.LE, "less_equal")
greater = _compare(Cmp.GT, "greater")
greater_equal = _compare(Cmp.GE, "greater_equal")


@primitive
def _where3(c, x, y):
    dt = D._float_dtype(D.result_dtype(x, y))
    if isinstance(c, (list, tuple, onp.ndarray)):  # a host mask
        c = D.asarray(onp.asarray(c))
    if isinstance(c, DevArray):
        c = D.astype(c, dt) if c.dtype != dt else c
    else:
        c = 1.0 if c else 0.0
    return D.map_op(Op.WHERE, dt, c, x, y)


def where(condition, *args, **kwargs):
    """``numpy.where(c, x, y)``, or ``numpy.nonzero(c)`` when called with the condition alone.  Keeps native Python
    types when no operand is an array or a box, as the reference does (autograd/numpy/__init__.py:13-39): the
    ``power`` rule calls ``where(y, y - 1, 1.0)`` with a Python exponent and needs a Python float back."""
    from ..tracer import isbox

    if not args and not kwargs:
        return nonzero(condition)
    if len(args) + len(kwargs) != 2 or not set(kwargs) <= {"x", "y"}:
        raise ValueError("either both or neither of x and y should be given")
    x = args[0] if args else kwargs["x"]
    y = args[1] if len(args) > 1 else kwargs["y"]

    def arrayish(v):
        if isinstance(v, (DevArray, onp.ndarray, onp.generic)) or isbox(v):
            return True
        return type(v) in (list, tuple) and builtins.any(arrayish(item) for item in v)

    if not (arrayish(condition) or arrayish(x) or arrayish(y)):
        if type(condition) in (list, tuple) or type(x) in (list, tuple) or type(y) in (list, tuple):
            return onp.where(condition, x, y).tolist()
        return x if condition else y
    return _where3(condition, x, y)


def _truth(a):
    """Operand for a logical op: 1.0 / 0.0 array (or Python float) from any array or scalar."""
    from ..tracer import getval

    a = getval(a)
    if isinstance(a, DevArray):
        return D.astype(D.compare(Cmp.NE, a, 0.0) if a.dtype != D._BOOL else a, onp.float64)
    return 1.0 if a else 0.0


def logical_and(a, b):
    """Non-differentiable (numpy_vjps.py:13-68); used by the ``clip`` rule."""
    return D.compare(Cmp.NE, D.map_op(Op.MUL, onp.dtype("float64"), _truth(a), _truth(b)), 0.0)


def logical_or(a, b):
    return D.compare(Cmp.NE, D.map_op(Op.ADD, onp.dtype("float64"), _truth(a), _truth(b)), 0.0)


def logical_not(a):
    return D.compare(Cmp.EQ, _truth(a), 0.0)


def logical_xor(a, b):
    return D.compare(Cmp.NE, _truth(a), _truth(b))


def isnan(x):
    from ..tracer import getval

    x = D.asarray(getval(x))
    return D.compare(Cmp.NE, x, x)


def isinf(x):
    from ..tracer import getval

    x = D.asarray(getval(x))
    return D.compare(Cmp.EQ, D.float_map(Op.ABS, x), onp.inf)


def isfinite(x):
    from ..tracer import getval

    x = D.asarray(getval(x))
    return D.compare(Cmp.LT, D.float_map(Op.ABS, x), onp.inf)  # NaN compares false


def isposinf(x):
    from ..tracer import getval

    return D.compare(Cmp.EQ, D.asarray(getval(x)), onp.inf)


def isneginf(x):
    from ..tracer import getval

    return D.compare(Cmp.EQ, D.asarray(getval(x)), -onp.inf)


def _truth_reduced(a, red, axis, keepdims):
    truth = _truth(a)
    if not isinstance(truth, DevArray):
        truth = D.full((), truth, onp.dtype(onp.float64))
    axes = D.normalize_axes(axis, truth.ndim)
    return D.map_reduce(Op.COPY, red, truth.dtype, (truth,), axes, keepdims)


def all(a, axis=None, keepdims=False):  # noqa: A001
    """Non-differentiable truth tests (numpy_vjps.py:13-68): the minimum / maximum / sum of the 0-1 array."""
    return D.compare(Cmp.NE, _truth_reduced(a, Red.MIN, axis, keepdims), 0.0)


def any(a, axis=None, keepdims=False):  # noqa: A001
    return D.compare(Cmp.NE, _truth_reduced(a, Red.MAX, axis, keepdims), 0.0)


def count_nonzero(a, axis=None, keepdims=False):
    """Counts are exact in float64 below 2**53; returned as int64 like NumPy's."""
    return D.astype(_truth_reduced(a, Red.SUM, axis, keepdims), onp.int64)


def isclose(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """|a - b| <= atol + rtol * |b| where both are finite, equality elsewhere (numpy.isclose)."""
    from ..tracer import getval

    a, b = D.asarray(getval(a)), D.asarray(getval(b))
    dt = D._float_dtype(D.result_dtype(a, b))
    f64 = onp.dtype(onp.float64)
    gap = D.map_op(Op.ABS, dt, D.map_op(Op.SUB, dt, a, b))
    bound = D.map_op(Op.ADD, dt, D.map_op(Op.MUL, dt, D.map_op(Op.ABS, dt, b), float(rtol)), float(atol))
    near = D.astype(D.compare(Cmp.LE, gap, bound), f64)
    finite = D.map_op(Op.MUL, f64, D.astype(isfinite(a), f64), D.astype(isfinite(b), f64))
    same = D.astype(D.compare(Cmp.EQ, a, b), f64)
    # finite pairs by the tolerance, the rest (infinities) by equality
    verdict = D.map_op(Op.WHERE, f64, finite, near, same)
    if equal_nan:
        both_nan = D.map_op(Op.MUL, f64, D.astype(isnan(a), f64), D.astype(isnan(b), f64))
        verdict = D.map_op(Op.MAXIMUM, f64, verdict, both_nan)
    return D.compare(Cmp.NE, verdict, 0.0)


def array_equal(a1, a2, equal_nan=False):
    """A Python bool (reads one element back): same shape and all elements equal."""
    from ..tracer import getval

    a1, a2 = D.asarray(getval(a1)), D.asarray(getval(a2))
    if a1.shape != a2.shape:
        return False
    if a1.size == 0:
        return True
    f64 = onp.dtype(onp.float64)
    same = D.astype(D.compare(Cmp.EQ, a1, a2), f64)
    if equal_nan:
        same = D.map_op(Op.MAXIMUM, f64, same, D.map_op(Op.MUL, f64, D.astype(isnan(a1), f64), D.astype(isnan(a2), f64)))
    return bool(all(same))


def _arg_extreme(red, name):
    def raw(a, axis=None, out=None, keepdims=False):
        """Index of the first extreme element, or of the first NaN if there is one: min over the axis of
        where(x == extreme or x is NaN, position, n) (positions are exact in float64 below 2**53).
        Non-differentiable (numpy_vjps.py:22-23)."""
        from ..tracer import getval

        x = D.asarray(getval(a))
        if x.dtype not in D._FLOATS:
            x = D.astype(x, onp.float64)
        if axis is None:
            x = ravel.fun(x)
            ax = 0
        else:
            ax = int(axis) % x.ndim
        n = x.shape[ax]
        if n == 0:
            raise ValueError(f"attempt to get {name} of an empty sequence")
        best = D.map_reduce(Op.COPY, red, x.dtype, (x,), (ax,), True)
        hit = D.compare(Cmp.EQ, x, best)
        view = [1] * x.ndim
        view[ax] = n
        pos = D.from_numpy(onp.arange(n, dtype=onp.float64).reshape(view))
        f64 = onp.dtype("float64")
        cand = D.map_op(Op.WHERE, f64, D.astype(hit, f64), pos, float(n))
        # a NaN makes the extreme NaN, which equals nothing: NumPy then reports the first NaN
        cand = D.map_op(Op.WHERE, f64, D.astype(D.compare(Cmp.NE, x, x), f64), pos, cand)
        idx = D.map_reduce(Op.COPY, Red.MIN, f64, (cand,), (ax,), bool(keepdims) and axis is not None)
        return D.astype(idx, onp.int64)

    raw.__name__ = raw.__qualname__ = name
    return raw


argmax = _arg_extreme(Red.MAX, "argmax")
argmin = _arg_extreme(Red.MIN, "argmin")


# ---- astype / copies --------------------------------------------------------------------------
@primitive
def astype(A, dtype, order="K", casting="unsafe", subok=True, copy=True):
    return D.astype(A, dtype)


_astype = astype


# ---- reductions ---------------------------------------------------------------------------------
def _reduction(red, name):
    def raw(x, axis=None, keepdims=False, dtype=None, out=None, **kwargs):
        if type(x) in (tuple, list) and builtins.all(isinstance(e, (int, onp.integer)) for e in x):
            # shape arithmetic on a tuple of Python ints (np.prod(shape)) stays a host integer, usable in slices
            return getattr(onp, name)(x, axis=axis, dtype=dtype, keepdims=keepdims)
        x = D.asarray(x)
        dt = D._float_dtype(x.dtype) if dtype is None else onp.dtype(dtype)
        return D.map_reduce(Op.COPY, red, dt, (x,), D.normalize_axes(axis, x.ndim), keepdims)

    return _wrap(raw, name)


sum = _reduction(Red.SUM, "sum")  # noqa: A001
prod = _reduction(Red.PROD, "prod")
max = amax = _reduction(Red.MAX, "max")  # noqa: A001
min = amin = _reduction(Red.MIN, "min")  # noqa: A001


@primitive
def _primitive_mean(x, axis=None, keepdims=False, dtype=None, out=None, **kwargs):
    x = D.asarray(x)
    axes = D.normalize_axes(axis, x.ndim)
    dt = D._float_dtype(x.dtype)
    total = D.map_reduce(Op.COPY, Red.SUM, dt, (x,), axes, keepdims)
    count = 1
    for a in axes:
        count *= x.shape[a]
    return D.map_op(Op.DIV, dt, total, float(count))


_primitive_mean.__name__ = "mean"


def mean(a, *args, **kwargs):
    if type(a) in (list, tuple):
        a = array(a)
    return _primitive_mean(a, *args, **kwargs)


# ---- shape-only functions (views: no kernel unless a copy is unavoidable) -----------------------
def _view_or_copy(x, shape):
    try:
        return x._view(lambda t: t.view(shape))
    except RuntimeError:
        return DevArray(D.contiguous(x)._t.view(shape), x.dtype)


def _norm_shape(shape, size):
    if isinstance(shape, (numbers.Integral, onp.integer)):
        shape = (int(shape),)
    shape = [int(s) for s in shape]
    if shape.count(-1) > 1:
        raise ValueError("can only specify one unknown dimension")
    if -1 in shape:
        known = 1
        for s in shape:
            if s != -1:
                known *= s
        if known == 0 or size % known:
            raise ValueError(f"cannot reshape array of size {size} into shape {tuple(shape)}")
        shape[shape.index(-1)] = size // known
    total = 1
    for s in shape:
        total *= s
    if total != size:
        raise ValueError(f"cannot reshape array of size {size} into shape {tuple(shape)}")
    return tuple(shape)


def _check_order(order):
    if order not in (None, "C"):
        raise NotImplementedError("only C order is supported on the device")


@primitive
def reshape(x, shape, order=None):
    _check_order(order)
    x = D.asarray(x)
    return _view_or_copy(x, _norm_shape(shape, x.size))


@primitive
def ravel(x, order=None):
    _check_order(order)
    x = D.asarray(x)
    return _view_or_copy(x, (x.size,))


@primitive
def expand_dims(x, axis):
    x = D.asarray(x)
    axes = (axis,) if isinstance(axis, (numbers.Integral, onp.integer)) else tuple(axis)
    nd = x.ndim + len(axes)
    axes = sorted(a % nd for a in axes)
    def expand(t):
        for a in axes:
            t = t.unsqueeze(a)
        return t

    return x._view(expand)


@primitive
def squeeze(x, axis=None):
    x = D.asarray(x)
    if axis is None:
        return x._view(lambda t: t.squeeze())
    axes = (axis,) if isinstance(axis, (numbers.Integral, onp.integer)) else tuple(axis)
    axes = sorted((a % x.ndim for a in axes), reverse=True)
    for a in axes:
        if x.shape[a] != 1:
            raise ValueError("cannot select an axis to squeeze out which has size not equal to one")

    def drop(t):
        for a in axes:
            t = t.squeeze(a)
        return t

    return x._view(drop)


@primitive
def transpose(x, axes=None):
    x = D.asarray(x)
    if axes is None:
        axes = tuple(range(x.ndim))[::-1]
    axes = tuple(int(a) % x.ndim for a in axes) if x.ndim else ()
    return x._view(lambda t: t.permute(axes) if t.dim() else t)


@primitive
def swapaxes(x, axis1, axis2):
    x = D.asarray(x)
    return x._view(lambda t: t.transpose(axis1, axis2))


@primitive
def moveaxis(x, source, destination):
    x = D.asarray(x)
    return x._view(lambda t: torch.movedim(t, source, destination))


@primitive
def broadcast_to(x, shape):
    x = D.asarray(x)
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
    return x._view(lambda t: t.expand(shape))


def _atleast(n):
    def raw(*arys):
        res = []
        for a in arys:
            a = D.asarray(a)
            def lift(t):
                if n >= 1 and t.dim() == 0:
                    t = t.reshape(1)
                if n >= 2 and t.dim() == 1:
                    t = t.unsqueeze(0)
                if n >= 3 and t.dim() == 2:
                    t = t.unsqueeze(2)
                return t

            res.append(a._view(lift))
        return res[0] if len(res) == 1 else res

    return _wrap(raw, f"atleast_{n}d")


atleast_1d, atleast_2d, atleast_3d = _atleast(1), _atleast(2), _atleast(3)


@primitive
def repeat(x, repeats, axis=None):
    x = D.asarray(x)
    if not isinstance(repeats, (numbers.Integral, onp.integer)):
        raise NotImplementedError("repeat: only an integer repeat count is supported on the device")
    repeats = int(repeats)
    if axis is None:
        x = ravel.fun(x)
        axis = 0
    axis %= x.ndim
    # out viewed as (..., n, repeats, ...) = x broadcast along a new axis
    shp = x.shape
    wide = shp[: axis + 1] + (repeats,) + shp[axis + 1 :]
    widened = x._view(lambda t: t.unsqueeze(axis + 1).expand(wide))
    out = D.map_op(Op.COPY, x.dtype, widened) if x.dtype in D._FLOATS else D.astype_copy(D.plain(widened))
    final = x.shape[:axis] + (x.shape[axis] * repeats,) + x.shape[axis + 1 :]
    return DevArray(out._t.view(final), x.dtype)


def _merged_stride(extents, strides):
    """The one stride that walks axes of these extents and strides as if they were a single axis (0 for a
    broadcast group), or None when there is none."""
    stride, span = None, 1  # span: elements covered by the axes seen so far (innermost first)
    for extent, st in zip(reversed(extents), reversed(strides)):
        if extent == 1:
            continue
        if stride is None:
            stride = st
        elif st != stride * span:
            return None
        span *= extent
    return 0 if stride is None else stride


def _concat_pieces(arrs, axis, dt):
    """The pieces of a concatenation as (tensor, extent, outer stride, axis stride, inner stride), or None when
    a piece is not a plain strided view (a pending map that is not a launch-free constant, another dtype)."""
    pieces = []
    for a in arrs:
        if a.dtype != dt:
            return None
        if type(a) is not DevArray and type(a) is not D.LazyDevArray:
            a = D.plain(a)  # a pending expression, product or reduction: computed now, joined from where it lands
        if type(a) is DevArray:
            t = a._t
        elif type(a) is D.LazyDevArray and a._scale == 1.0 and a._shift is None and a._ascale is None and a._producer is None:
            t = a._raw  # a constant: one shared element seen through stride-0 axes
        else:
            return None
        extents, strides = tuple(t.shape), t.stride()
        so = _merged_stride(extents[:axis], strides[:axis])
        si = _merged_stride(extents[axis + 1:], strides[axis + 1:])
        if so is None or si is None:
            return None
        if extents[axis]:
            pieces.append((t, extents[axis], so, strides[axis], si))
    return pieces if pieces else None


@primitive
def concatenate_args(axis, *args):
    arrs = [D.asarray(a) for a in args]
    dt = D.result_dtype(*arrs)
    if axis is None:
        arrs = [ravel.fun(a) for a in arrs]
        axis = 0
    nd = arrs[0].ndim
    if nd == 0:
        raise ValueError("zero-dimensional arrays cannot be concatenated")
    axis %= nd
    total = 0
    for a in arrs:
        if a.ndim != nd or a.shape[:axis] != arrs[0].shape[:axis] or a.shape[axis + 1 :] != arrs[0].shape[axis + 1 :]:
            raise ValueError("all the input array dimensions except for the concatenation axis must match exactly")
        total += a.shape[axis]
    shape = arrs[0].shape[:axis] + (total,) + arrs[0].shape[axis + 1 :]
    out = D.empty(shape, dt)
    if 2 <= len(arrs) <= _lib.MAX_CONCAT and dt in D._FLOATS and out.size:
        pieces = _concat_pieces(arrs, axis, dt)
        if pieces is not None:  # every piece is a strided (outer, extent, inner) view: one launch for all of them
            outer = 1
            for extent in shape[:axis]:
                outer *= extent
            _lib.concat(_lib.DTYPE_CODE[dt], outer, out.size // (outer * total), pieces, out._t)
            return out
    start = 0
    for a in arrs:
        n = a.shape[axis]
        if n:
            dst = DevArray(out._t.narrow(axis, start, n), dt)
            if dt in D._FLOATS:
                D.map_op(Op.COPY, dt, a, out=dst)
            else:
                _lib.cast(_lib.DTYPE_CODE[a.dtype], _lib.DTYPE_CODE[dt], dst.shape, dst._t, a._t)
        start += n
    return out


def concatenate(arr_list, axis=0):
    return concatenate_args(axis, *arr_list)


def _with_rank(m, n, lift):
    """``atleast_nd(m)``, skipping the call (and, for a traced array, the tape node of an identity) when ``m`` is an
    array that has ``n`` dimensions already."""
    return m if isinstance(_getval(m), DevArray) and ndim(m) >= n else lift(m)


def vstack(tup):
    return concatenate([_with_rank(m, 2, atleast_2d) for m in tup], axis=0)


row_stack = vstack


def hstack(tup):
    arrs = [_with_rank(m, 1, atleast_1d) for m in tup]
    if arrs[0].ndim == 1:
        return concatenate(arrs, 0)
    return concatenate(arrs, 1)


@primitive
def _array_from_scalar_or_array(array_args, array_kwargs, scalar):
    dtype = array_kwargs.get("dtype", array_args[0] if array_args else None)
    out = D.asarray(scalar, dtype)
    ndmin = array_kwargs.get("ndmin", 0)
    while out.ndim < ndmin:
        out = DevArray(out._t.unsqueeze(0), out.dtype)
    return out


@primitive
def array_from_args(array_args, array_kwargs, *args):
    dtype = array_kwargs.get("dtype", array_args[0] if array_args else None)
    parts = [D.asarray(a) for a in args]
    dt = onp.dtype(dtype) if dtype is not None else D.result_dtype(*parts)
    return concatenate_args.fun(0, *[DevArray(p._t.unsqueeze(0), p.dtype) for p in parts]) if parts else D.empty((0,), dt)


def array(A, *args, **kwargs):
    """``numpy.array``: host data is uploaded; lists that contain boxes stay differentiable."""
    from ..tracer import getval, isbox

    if isbox(A) and type(getval(A)) in (list, tuple):
        # a traced sequence (the reference asks autograd.builtins.type, which sees through boxes,
        # numpy_wrapper.py:83-88): its elements come out of the box one by one, traced
        return array_from_args(args, kwargs, *map(array, A))
    if type(A) in (list, tuple):
        flat_has_dev = _contains_dev_or_box(A)
        if flat_has_dev:
            return array_from_args(args, kwargs, *map(array, A))
        return D.asarray(onp.array(A, *args, **kwargs))
    if isbox(A) or isinstance(A, DevArray):
        return _array_from_scalar_or_array(args, kwargs, A)
    return D.asarray(onp.array(A, *args, **kwargs))


def _contains_dev_or_box(seq):
    from ..tracer import isbox

    for item in seq:
        if isinstance(item, DevArray) or isbox(item):
            return True
        if isinstance(item, (list, tuple)) and _contains_dev_or_box(item):
            return True
    return False


def asarray(a, dtype=None):
    from ..tracer import isbox

    if isbox(a):
        return a if dtype is None else astype(a, dtype)
    return D.asarray(a, dtype)


def stack(arrays, axis=0):
    arrays = [array(a) for a in arrays]
    if not arrays:
        raise ValueError("need at least one array to stack")
    if len({a.shape for a in arrays}) != 1:
        raise ValueError("all input arrays must have the same shape")
    nd = arrays[0].ndim + 1
    if not -nd <= axis < nd:
        raise IndexError(f"axis {axis} out of bounds [-{nd}, {nd})")
    axis %= nd
    sl = (slice(None),) * axis + (None,)
    return concatenate([a[sl] for a in arrays], axis=axis)


def column_stack(tup):
    """1-d inputs become columns, the rest are joined along axis 1 (numpy_wrapper.py:73-80)."""
    columns = []
    for v in tup:
        a = array(v)
        columns.append(reshape(a, (-1, 1)) if ndim(a) < 2 else a)
    return concatenate(columns, 1)


def select(condlist, choicelist, default=0):
    """``numpy.select``: the first condition that holds picks the choice (numpy_wrapper.py:58-60 assembles the result
    element by element on the host; here it is a chain of ``where`` from the last condition to the first)."""
    condlist, choicelist = list(condlist), list(choicelist)
    if len(condlist) != len(choicelist):
        raise ValueError("list of cases must be same length as list of conditions")
    if not condlist:
        raise ValueError("select with an empty condition list is not possible")
    out = default
    for cond, choice in zip(reversed(condlist), reversed(choicelist)):
        if _getval(choice) is not choice:
            # (a cast to its own dtype: the reference hands every traced choice its cotangent in the choice's dtype,
            # where the rule of `where` alone would leave a float32 one in float64)
            choice = astype(choice, result_type(choice))
        out = where(array(cond), choice, out)
    return out


def append(arr, values, axis=None):
    """``numpy.append`` through ``concatenate`` (numpy_wrapper.py:139-147): both operands flattened when no axis is given."""
    if axis is None:
        return concatenate((ravel(array(arr)), ravel(array(values))), axis=0)
    return concatenate((array(arr), values), axis=axis)


class _Joiner:
    """``r_[...]`` and ``c_[...]`` (numpy_wrapper.py:153-169) for arrays, scalars and ranges: ranges are expanded on
    the host, every item is raised to ``min_ndim`` dimensions (new unit axes last) and the items are joined along
    ``axis``.  The string directives of NumPy's index tricks are not taken."""

    def __init__(self, name, axis, min_ndim):
        self._name, self._axis, self._min_ndim = name, axis, min_ndim

    def __getitem__(self, items):
        items = items if type(items) is tuple else (items,)
        pieces = []
        for item in items:
            if isinstance(item, str):
                raise NotImplementedError(f"{self._name}[...] takes arrays, scalars and ranges, not string directives")
            piece = D.from_numpy(onp.r_[item]) if type(item) is slice else array(item)
            if ndim(piece) < self._min_ndim:
                piece = reshape(piece, shape(piece) + (1,) * (self._min_ndim - ndim(piece)))
            pieces.append(piece)
        if not pieces:
            return D.from_numpy(onp.r_[()])
        traced = [_getval(item) is not item for item in items]
        if builtins.any(traced):
            # the reference lets NumPy build an object array around the boxes and unpacks it element by element
            # (numpy_wrapper.py:91-97, 153-169).  Untraced items arrive there as Python numbers, which makes the
            # result float64 even when every array was float32; and every traced item gets its cotangent back in
            # its own dtype.  Casting the traced items first gives both.
            final = onp.result_type(*[result_type(piece) for piece in pieces])
            if not builtins.all(traced) and final == onp.float32:
                final = onp.dtype(onp.float64)
            pieces = [astype(piece, final) if is_traced and result_type(piece) != final else piece
                      for piece, is_traced in zip(pieces, traced)]
        return concatenate(pieces, axis=self._axis)


r_, c_ = _Joiner("r_", 0, 1), _Joiner("c_", -1, 2)


# ---- indexing -----------------------------------------------------------------------------------
def _is_basic_index(idx):
    items = idx if isinstance(idx, tuple) else (idx,)
    for it in items:
        if it is None or it is Ellipsis or type(it) is slice or type(it) is int:
            continue
        if isinstance(it, (numbers.Integral, onp.integer, slice)):
            continue
        return False
    return True


def _plain(idx):
    items = idx if isinstance(idx, tuple) else (idx,)
    return tuple(i if (i is None or type(i) is slice or type(i) is int or i is Ellipsis)
                 else (int(i) if isinstance(i, (numbers.Integral, onp.integer)) else i) for i in items)


_INDEX_PLANS = {}
_INDEX_PLAN_LIMIT = 512


def _index_key(idx):
    """Hashable identity of an index made of host data (ints, slices, None, Ellipsis, lists, NumPy arrays);
    None when it holds anything else (a device array)."""
    items = idx if isinstance(idx, tuple) else (idx,)
    key = []
    for it in items:
        if it is None or it is Ellipsis or isinstance(it, (int, onp.integer, bool, onp.bool_)):
            key.append(it)
        elif isinstance(it, slice):
            key.append(("s", it.start, it.stop, it.step))
        elif isinstance(it, (list, onp.ndarray)):
            arr = onp.asarray(it)
            if arr.dtype.kind not in "iub":
                raise IndexError("arrays used as indices must be of integer (or boolean) type")
            key.append(("a", arr.shape, arr.dtype.str, arr.tobytes()))
        else:
            return None
    return (isinstance(idx, tuple), tuple(key))


def _to_host_index(idx):
    """``idx`` with lists turned into NumPy arrays (an empty one is an empty INTEGER index, as NumPy reads it)
    and device arrays brought to the host (a synchronising transfer: their VALUES decide which elements are
    taken, and for boolean masks even how many)."""
    def one(it):
        if isinstance(it, DevArray):
            return it.numpy()
        if isinstance(it, list):
            if builtins.any(isinstance(e, DevArray) for e in it):
                it = [e.numpy() if isinstance(e, DevArray) else e for e in it]
            arr = onp.asarray(it)
            return arr.astype(onp.int64) if arr.size == 0 else arr
        return it

    return tuple(one(it) for it in idx) if isinstance(idx, tuple) else one(idx)


def _flat_positions(shape, idx):
    """int64 array shaped like ``A[idx]`` (for ``A`` of ``shape``) holding the flat (row-major) position in ``A``
    of every selected element.  NumPy itself applies the index, to stride-0 views of the axis coordinates: that
    costs memory for the RESULT only and brings NumPy's indexing rules along (broadcast of index arrays, where
    their axes land in the result, boolean masks, out-of-range errors)."""
    flat = None
    stride = 1
    strides = []
    for extent in reversed(shape):
        strides.append(stride)
        stride *= extent
    strides.reverse()
    for axis, extent in enumerate(shape):
        coords = onp.arange(extent, dtype=onp.int64).reshape((1,) * axis + (extent,) + (1,) * (len(shape) - axis - 1))
        picked = onp.broadcast_to(coords, shape)[idx]
        flat = picked * strides[axis] if flat is None else flat + picked * strides[axis]
    if flat is None:  # 0-d array: only (), ... and None can index it
        flat = onp.zeros((), dtype=onp.int64)[idx]
    return onp.asarray(flat, dtype=onp.int64, order="C")


class _IndexPlan:
    """What ``A[idx]`` with an advanced index selects from an array of one shape, resident on the device, and the
    stable order of the selection that the ordered scatter of the cotangent needs.  Built once per (shape, index)
    and kept while the cache has room, so repeated evaluations and recorded graphs do no host work and no
    transfers for it.

    One integer vector on the leading axis (``X[batch_rows]``) is kept as rows: ``n`` row numbers and rows of
    ``inner`` elements each.  Every other index form is the flat position of every selected ELEMENT (``inner`` = 1).
    """

    __slots__ = ("shape", "positions", "n", "_order", "n_rows", "inner", "nbytes")

    def __init__(self, shape, idx):
        rows = idx if not isinstance(idx, tuple) else (idx[0] if len(idx) == 1 else None)
        if isinstance(rows, onp.ndarray) and rows.ndim == 1 and rows.dtype.kind in "iu" and len(shape) >= 1:
            extent = shape[0]
            rows = rows.astype(onp.int64)
            if rows.size and (rows.min() < -extent or rows.max() >= extent):
                bad = rows[(rows < -extent) | (rows >= extent)][0]
                raise IndexError(f"index {bad} is out of bounds for axis 0 with size {extent}")
            flat = onp.where(rows < 0, rows + extent, rows)
            inner = 1
            for s in shape[1:]:
                inner *= s
            self.shape = (flat.size,) + tuple(shape[1:])
            self.n_rows, self.inner = extent, inner
        else:
            flat = _flat_positions(shape, idx)
            self.shape = flat.shape
            total = 1
            for s in shape:
                total *= s
            self.n_rows, self.inner = total, 1
        self.n = flat.size
        self.positions = D.from_numpy(flat.reshape(-1))
        # equal destinations keep their order of appearance, which is the order numpy.add.at adds them in
        self._order = D.from_numpy(onp.argsort(flat.reshape(-1), kind="stable").astype(onp.int64))
        self.nbytes = 16 * flat.size

    def order(self):
        return self._order


_INDEX_PLAN_BYTES = [0]
_INDEX_PLAN_BUDGET = 64 << 20      # device memory the kept plans may hold
_INDEX_PLAN_LARGEST = 8 << 20      # a plan beyond this is built, used and dropped (fresh minibatch rows every step)


def _index_plan(shape, idx):
    idx = _to_host_index(idx)
    big = builtins.sum(it.nbytes for it in (idx if isinstance(idx, tuple) else (idx,)) if isinstance(it, onp.ndarray)) > (1 << 20)
    if big:
        return _IndexPlan(tuple(shape), idx)  # (hashing a large index costs what building the plan costs)
    key = (tuple(shape), _index_key(idx))
    plan = _INDEX_PLANS.pop(key, None)
    if plan is None:
        plan = _IndexPlan(tuple(shape), idx)
        if plan.nbytes > _INDEX_PLAN_LARGEST:
            return plan
        _INDEX_PLAN_BYTES[0] += plan.nbytes
        # least recently used plans make room (a dict keeps insertion order; a hit re-inserts its key at the end)
        while _INDEX_PLANS and (_INDEX_PLAN_BYTES[0] > _INDEX_PLAN_BUDGET or len(_INDEX_PLANS) >= _INDEX_PLAN_LIMIT):
            oldest = next(iter(_INDEX_PLANS))
            _INDEX_PLAN_BYTES[0] -= _INDEX_PLANS.pop(oldest).nbytes
    _INDEX_PLANS[key] = plan
    return plan


def _device_rows(idx):
    """The index when it is a device-resident 1-d integer array (rows of the leading axis, chosen by data that
    never leaves the device); None otherwise."""
    if isinstance(idx, DevArray) and idx.ndim == 1 and idx.dtype in (D._I64, onp.dtype("int32")):
        return idx if idx.dtype == D._I64 else D.astype(idx, D._I64)
    return None


def _positive_steps(idx, shape):
    """``(idx_up, axes)``: a basic index whose slices all step upwards and select the same elements as
    ``idx``, and the axes of the result along which that selection is reversed to give ``A[idx]``
    (device views cannot have negative strides; a reversal is one gather)."""
    items = list(idx if isinstance(idx, tuple) else (idx,))
    if not builtins.any(isinstance(it, slice) and it.step is not None and it.step < 0 for it in items):
        return idx, ()
    if builtins.any(it is Ellipsis for it in items):
        k = [it is Ellipsis for it in items].index(True)
        consumed = len([it for it in items if it is not None and it is not Ellipsis])
        items[k : k + 1] = [slice(None)] * (len(shape) - consumed)
    up, axes, src_axis, res_axis = [], [], 0, 0
    for it in items:
        if it is None:
            up.append(None)
            res_axis += 1
            continue
        if src_axis >= len(shape):
            raise IndexError("too many indices for array")
        if isinstance(it, slice):
            if it.step is not None and it.step < 0:
                picked = range(*it.indices(shape[src_axis]))
                it = slice(picked[-1], picked[0] + 1, -picked.step) if len(picked) else slice(0, 0, 1)
                axes.append(res_axis)
            res_axis += 1
        up.append(it)
        src_axis += 1
    return tuple(up), tuple(axes)


def _in_memory_order(x, axis):
    """``(tensor, axis, restore)`` for a kernel that wants a contiguous operand and works along one axis.

    A transposed (axis-permuted) view of a contiguous array is handed over in its memory order, with the
    axis renamed accordingly, so that no transposing copy is made; ``restore`` turns the kernel's result
    (same layout) back into an array with ``x``'s shape.  Anything else is copied to row-major order first."""
    t = x._h()  # layout only: pending arithmetic, if any, is written out below, already in memory order
    dtype = x.dtype
    if not t.is_contiguous() and t.dim() > 1 and 0 not in t.stride():
        order = sorted(range(t.dim()), key=lambda d: -t.stride(d))
        if t.permute(order).is_contiguous():
            back = [order.index(d) for d in range(t.dim())]
            tm = D.plain(x._view(lambda u: u.permute(order)))._t
            if tm.is_contiguous():
                return tm, order.index(axis), lambda out: DevArray(out.permute(back), dtype)
    return D.contiguous(D.plain(x))._t, axis, lambda out: DevArray(out, dtype)


def _reverse_axes(x, axes):
    """``x`` reversed along ``axes`` (a new array), one copy kernel per axis."""
    for axis in axes:
        n = x.shape[axis]
        if n <= 1 or x.size == 0:
            continue
        if x.dtype not in D._FLOATS:
            raise NotImplementedError("reversal of non-floating arrays")
        src, ax, restore = _in_memory_order(x, axis)
        shp = tuple(src.shape)
        outer, inner = int(onp.prod(shp[:ax], dtype=onp.int64)), int(onp.prod(shp[ax + 1 :], dtype=onp.int64))
        out = _lib.empty(shp, x.dtype)
        _lib.reverse(_lib.DTYPE_CODE[x.dtype], src, outer, n, inner, out)
        x = restore(out)
    return x


def _gather(A, positions, n_rows, inner, out_shape):
    if A.dtype not in D._FLOATS:
        raise NotImplementedError("gather of non-floating arrays")
    src = D.contiguous(A)
    out = D.empty(out_shape, A.dtype)
    if out.size:
        _lib.take_rows(_lib.DTYPE_CODE[A.dtype], src._t, n_rows, inner, positions._t, positions.size, out._t)
    return out


def take(A, idx):
    """``A[idx]``: views for basic indices (plus one gather per axis sliced backwards); one gather kernel for
    every other NumPy index form (integer arrays and lists on any axes, mixed with slices and integers, boolean
    masks), driven by a device-resident table of flat positions that is built once per (shape, index)."""
    if _is_basic_index(idx):
        pidx, backwards = _positive_steps(_plain(idx), A.shape)
        if type(A) is D.LazyDevArray and _trace_stack.top < 0 and not builtins.any(A._raw.stride()):
            A._t  # outside any trace a lazy fill (zeros / ones) is written out before it is viewed: an item assignment through the view then reaches it
        if D._fusion.pending(A) and A.ndim == 1 and not backwards and D._fusion.ENABLED:
            rows = _leading_rows(pidx, A.shape)
            if rows is not None and rows[1] > rows[0]:
                return D._fusion.slice_of(A, rows[0], rows[1])  # a slice of a vector that is still an expression stays one
        if type(A) is D.PendingProduct and not backwards and D._fusion.ENABLED:
            part = _part_of_product(A, pidx)
            if part is not None:
                return part
        picked = A._view(lambda t: t[pidx])
        return _reverse_axes(picked, backwards) if backwards else picked
    if A.ndim == 0:
        raise IndexError("too many indices for array")
    rows = _device_rows(idx)
    if rows is not None:  # data-dependent rows: the index stays on the device (out-of-range values are the caller's to avoid)
        inner = 1
        for s in A.shape[1:]:
            inner *= s
        return _gather(A, rows, A.shape[0], inner, (rows.size,) + A.shape[1:])
    plan = _index_plan(A.shape, idx)
    return _gather(A, plan.positions, plan.n_rows, plan.inner, plan.shape)


def _part_of_product(P, pidx):
    """``P[r0:r1, c0:c1]`` of a matrix product that has not run yet, as the product of the factors' rows and columns
    (nothing runs; None when this is not such a slice).  The cotangent of an `hstack` hands each piece its columns of the
    stacked cotangent (numpy_vjps.py:783-788 `grad_concatenate_args`); when that cotangent is `G . W^T` only the columns
    of a traced piece are ever read (a recurrent net's state between its input and the column of ones), so only they
    are contracted, and the product stays one that a sum or a tanh rule can still take into its own launch.  Slices of
    less than half of an axis are views of the whole product as before: several small pieces of one product are cheaper
    contracted together."""
    if P.computed() or P._more or P._out is not None:
        return None
    if type(pidx) is not tuple:
        pidx = (pidx,)
    if len(pidx) > 2 or not builtins.all(type(i) is slice for i in pidx):
        return None
    rows, cols = P.shape
    r0, r1, rs = pidx[0].indices(rows)
    c0, c1, cs = pidx[1].indices(cols) if len(pidx) == 2 else (0, cols, 1)
    if rs != 1 or cs != 1 or r1 <= r0 or c1 <= c0 or (r1 - r0, c1 - c0) == (rows, cols):
        return None
    if 2 * (r1 - r0) < rows or 2 * (c1 - c0) < cols:
        return None
    return D.PendingProduct(P._left[r0:r1], P._right[:, c0:c1], P.dtype)


def assign_items(A, idx, value):
    """``A[idx] = value`` on a plain device array: data preparation outside any trace, the way examples/rnn.py:86
    fills its one-hot batches.  Basic indices with forward steps write through the strided view in one launch; a
    boolean mask of the array's own shape with a scalar value is one in-place select.  Arrays that share their memory
    by construction (broadcast views, borrowed accumulators) get a buffer of their own first.  Inside a traced
    function arrays stay immutable, as in the reference: a box has no item assignment and a boxed value cannot be
    stored into an array."""
    from ..tracer import isbox
    from .vspaces import is_broadcast_view

    if isbox(value) or isbox(idx):
        raise TypeError("a traced value cannot be assigned into an array: build the result with concatenate / where")
    D.ITEM_WRITES += 1
    if type(A) is D.LazyDevArray:
        if A._view_of_pending and (A._scale != 1.0 or A._shift is not None or A._ascale is not None) and builtins.any(A._raw.stride()):
            # `y = 1 - x; v = y[1:]; v[:] = 0`: in NumPy the write reaches y; here y's value does not exist in memory yet and
            # v would get a buffer of its own.  A wrong result without a word is worse than an error.
            raise ValueError("item assignment into a view of an array whose arithmetic is still pending would not reach "
                             "that array; assign into the array itself, or take the view of np.settle(array)")
        A._t  # pending arithmetic (a lazy fill, say) is written out: from here on the array is its own buffer
    elif type(A) is not DevArray:
        raise TypeError("item assignment needs a plain device array; this one is a cotangent still being formed "
                        "(np.settle gives a plain one)")
    if A._borrowed or is_broadcast_view(A):
        own = D.contiguous(D.copy(DevArray(A._t, A.dtype)))._t
        A._t, A._borrowed = own, False
        if type(A) is D.LazyDevArray:
            A._raw = own
    dtype = A.dtype
    if _is_basic_index(idx):
        pidx, backwards = _positive_steps(_plain(idx), A.shape)
        if backwards:
            raise NotImplementedError("item assignment through a slice that steps backwards")
        target = DevArray(A._t[pidx], dtype)
        source = D.asarray(value, dtype)
        if type(source) is not DevArray:
            source = D.plain(source)
        if onp.broadcast_shapes(source.shape, target.shape) != target.shape:
            raise ValueError(f"could not broadcast input array from shape {source.shape} into shape {target.shape}")
        if target.size == 0:
            return
        if dtype in D._FLOATS:
            D.map_op(Op.COPY, dtype, source, out=target)
        else:
            code = _lib.DTYPE_CODE[dtype]
            _lib.cast(code, code, target.shape, target._t, source._t.expand(target.shape))
        return
    mask = idx if isinstance(idx, DevArray) else (onp.asarray(idx) if isinstance(idx, (list, onp.ndarray)) else None)
    scalar = isinstance(value, (numbers.Number, onp.generic)) or (isinstance(value, (DevArray, onp.ndarray)) and value.ndim == 0)
    if mask is not None and mask.dtype == onp.bool_ and tuple(mask.shape) == A.shape and scalar and dtype in D._FLOATS:
        mask = D.astype(D.asarray(mask), dtype)
        whole = DevArray(A._t, dtype)
        D.map_op(Op.WHERE, dtype, mask, D.asarray(value, dtype) if not isinstance(value, numbers.Number) else float(value), whole, out=whole)
        return
    raise NotImplementedError("item assignment takes basic indices (integers, forward slices, newaxis, ellipsis) or a boolean "
                              "mask of the array's shape with a scalar value")


def _leading_rows(idx, shape):
    """(start, stop) when the basic index ``idx`` selects rows start:stop of the leading axis with
    step 1 and every other axis in full; None otherwise."""
    if isinstance(idx, slice):
        first, rest = idx, ()
    elif isinstance(idx, tuple) and idx and isinstance(idx[0], slice):
        first, rest = idx[0], idx[1:]
    else:
        return None
    if not shape or builtins.any(not (isinstance(r, slice) and r == slice(None)) for r in rest):
        return None
    start, stop, step = first.indices(shape[0])
    return (start, stop if stop > start else start) if step == 1 else None  # (this module's max is the array reduction)


def scatter_add(A, idx, x):
    """In place ``numpy.add.at(A, idx, x)`` on a freshly allocated, contiguous ``A``.

    Basic indices: a strided in-place add on the view (every destination gets exactly one
    addend).  Integer array on axis 0: the ordered scatter kernel, which adds repeated
    destinations sequentially in index order like ``numpy.add.at``.
    """
    from .vspaces import is_broadcast_view, is_shared_zero

    basic = _is_basic_index(idx)
    if basic:
        idx, backwards = _positive_steps(_plain(idx), A.shape)
        if backwards:  # A[::-1] += x  is  A[::1] += x reversed
            x = _reverse_axes(D.asarray(broadcast_to.fun(D.asarray(x, A.dtype), tuple(A._t[idx].shape))), backwards)
    if (basic and A.ndim == 1 and D._fusion.ENABLED and A.dtype in D._FLOATS and isinstance(x, DevArray) and x.dtype == A.dtype
            and not is_shared_zero(A)):
        rows = _leading_rows(idx, A.shape)
        if rows is not None and rows[1] > rows[0] and x.shape == (rows[1] - rows[0],):
            node = D._fusion.added_into(A, rows[0], x, take)  # stays an expression: the sum joins whatever reads it
            if node is not None:
                return node
    if A._borrowed or type(A) is not DevArray or is_broadcast_view(A) or is_shared_zero(A):  # not this accumulator's own memory yet: allocate it
        if is_shared_zero(A):
            if basic:
                # into zeros the sum is 0 + x, so the destination is never read back; and when the
                # view covers every element (b[None, :], c[:, None], full slices) the zero fill
                # is skipped as well
                probe = A._t[_plain(idx)]
                full_cover = probe.numel() == A._t.numel() and probe.dim() >= A._t.dim()
                if full_cover and isinstance(x, DevArray) and x.dtype == A.dtype and x.shape == tuple(probe.shape):
                    # basic indices cannot permute: the view is A with unit axes inserted, so 0 + x is x
                    # with A's shape.  Borrowed like any `zeros + g` (vspaces._mut_add): nothing is launched
                    shape = A.shape
                    acc = x._view(lambda t: t.reshape(shape))
                    acc._borrowed = True
                    return acc
                rows = None if full_cover else _leading_rows(idx, A.shape)
                if (rows is not None and A.ndim == 1 and D._fusion.ENABLED and isinstance(x, DevArray) and x.dtype == A.dtype
                        and A.dtype in D._FLOATS and x.shape == (rows[1] - rows[0],) and rows[1] > rows[0]):
                    # a vector's x[a:b]: the padded cotangent stays an expression (its zeros are never written; the program
                    # that finally needs it reads x's operands at moved addresses)
                    node = D._fusion.padded(x, rows[0], A.shape[0], A.dtype)
                    if node is not None:
                        return node
                if full_cover or rows is not None:
                    A = D.empty(A.shape, A.dtype)
                    if rows is not None:
                        # x[1:], x[:-1], x[a:b]: only the rows outside the range need zeros (two short fills),
                        # not the whole array
                        code = _lib.DTYPE_CODE[A.dtype]
                        for part in (A._t[:rows[0]], A._t[rows[1]:]):
                            if part.numel():
                                _lib.fill(code, part, 0.0)
                else:
                    A = D.zeros(A.shape, A.dtype)
                D.map_op(Op.ADD, A.dtype, 0.0, x, out=DevArray(A._t[_plain(idx)], A.dtype))
                return A
            A = D.zeros(A.shape, A.dtype)
        else:
            A = D.copy(A)
    if basic:
        view = DevArray(A._t[_plain(idx)], A.dtype)
        D.map_op(Op.ADD, A.dtype, view, x, out=view)
        return A
    if not A._t.is_contiguous():
        raise AssertionError("scatter destination must be contiguous")
    code = _lib.DTYPE_CODE[A.dtype]
    rows = _device_rows(idx)
    if rows is not None:
        # a device-resident index: its stable order comes from the counting sort on the device (keys as float64,
        # exact below 2^53), the runs of equal destination are found by the scatter kernel itself
        n = rows.size
        if n == 0:
            return A
        inner = 1
        for s in A.shape[1:]:
            inner *= s
        if n > 65536:
            raise NotImplementedError("scatter through a device-resident index of more than 65536 entries")
        # negative rows count from the end; a row outside [-n, n) stays outside (the gather reads NaN for it, the
        # scatter drops its addends: neither touches memory)
        as_float = D.astype(rows, D._F64)
        wrapped = D.map_op(Op.WHERE, D._F64, D.astype(D.compare(Cmp.LT, as_float, 0.0), D._F64),
                           D.map_op(Op.ADD, D._F64, as_float, float(A.shape[0])), as_float)
        keys = D.astype(wrapped, D._I64)
        order = D.empty((n,), D._I64)
        _lib.sort_rows(_lib.DTYPE_CODE[D._F64], D.contiguous(wrapped)._t, 1, n, None, order._t, None)
        target = (n,) + A.shape[1:]
        src = D.asarray(x, A.dtype)
        if src.shape != target:
            src = DevArray(src._h().expand(target), src.dtype) if type(src) is DevArray else broadcast_to.fun(src, target)
        src = D.contiguous(src)
        _lib.scatter_add_rows(code, A._t, A.shape[0], inner, src._t, keys._t, order._t, None, n)
        return A
    plan = _index_plan(A.shape, idx)
    if plan.n == 0:
        return A
    src = D.asarray(x, A.dtype)
    if src.shape != plan.shape:
        src = broadcast_to.fun(src, plan.shape)
    src = D.contiguous(D.plain(src))
    _lib.scatter_add_rows(code, A._t, plan.n_rows, plan.inner, src._t, plan.positions._t, plan.order()._t, None, plan.n)
    return A


def pad_widths(pad_width, ndim):
    """``pad_width`` in any of numpy.pad's spellings -> ((before, after),) * ndim of Python ints."""
    w = onp.asarray(pad_width)
    if w.dtype.kind not in "iu":
        raise TypeError("`pad_width` must be of integral type.")
    return tuple((int(b), int(a)) for b, a in onp.broadcast_to(w, (ndim, 2)))


@primitive
def pad(array, pad_width, mode="constant", **kwargs):
    """Zero padding (numpy.pad, constant mode): one fill and one strided copy into the interior."""
    if mode != "constant" or builtins.any(v != 0 for v in onp.ravel(kwargs.get("constant_values", 0))) or set(kwargs) - {"constant_values"}:
        raise NotImplementedError("pad: only mode='constant' with zeros is supported on the device")
    x = D.asarray(array)
    widths = pad_widths(pad_width, x.ndim)
    if builtins.any(b < 0 or a < 0 for b, a in widths):
        raise ValueError("index can't contain negative values")
    out = D.zeros(tuple(n + b + a for n, (b, a) in zip(x.shape, widths)), x.dtype)
    if x.size:
        inner = out._t[tuple(slice(b, b + n) for n, (b, _) in zip(x.shape, widths))]
        if x.dtype in D._FLOATS:
            D.map_op(Op.COPY, x.dtype, x, out=DevArray(inner, x.dtype))
        else:
            code = _lib.DTYPE_CODE[x.dtype]
            _lib.cast(code, code, x.shape, inner, x._t)
    return out


# ---- contractions -------------------------------------------------------------------------------
def _dot_raw(a, b):
    a, b = D.asarray(a) if not D.is_scalar(a) else a, D.asarray(b) if not D.is_scalar(b) else b
    if D.is_scalar(a) or D.is_scalar(b) or a.ndim == 0 or b.ndim == 0:
        return D.arith_map(Op.MUL, a, b)
    dt = D._float_dtype(D.result_dtype(a, b))
    a = D.astype(a, dt) if a.dtype != dt else a
    b = D.astype(b, dt) if b.dtype != dt else b
    if a.ndim == 1 and b.ndim == 1:
        if a.shape != b.shape:
            raise ValueError(f"shapes {a.shape} and {b.shape} not aligned")
        return D.map_reduce(Op.MUL, Red.SUM, dt, (a, b), (0,), False)
    if b.ndim == 1:  # (..., K) . (K,) -> (...): row map-reduce, bandwidth bound
        if a.shape[-1] != b.shape[0]:
            raise ValueError(f"shapes {a.shape} and {b.shape} not aligned")
        return D.map_reduce(Op.MUL, Red.SUM, dt, (a, b), (a.ndim - 1,), False)
    if a.ndim == 1:  # (K,) . (..., K, N) -> (..., N)
        if a.shape[0] != b.shape[-2]:
            raise ValueError(f"shapes {a.shape} and {b.shape} not aligned")
        a_col = DevArray(a._t.reshape((1,) * (b.ndim - 2) + (a.shape[0], 1)), dt)
        return D.map_reduce(Op.MUL, Red.SUM, dt, (a_col, b), (b.ndim - 2,), False)
    if a.shape[-1] != b.shape[-2]:
        raise ValueError(f"shapes {a.shape} and {b.shape} not aligned: {a.shape[-1]} (dim {a.ndim - 1}) != {b.shape[-2]} (dim {b.ndim - 2})")
    if a.ndim == 2 and b.ndim == 2:
        if D._fusion.ENABLED and a.shape[0] and b.shape[1]:
            # left pending: a bias and an activation that follow can then ride in the contraction's epilogue
            return D.note_forward_product(D.PendingProduct(a._t, b._t, dt))
        return DevArray(D.gemm2d(a._t, b._t, dt), dt)
    # numpy.dot on higher ranks: sum over last axis of a and second-to-last of b
    return _tensordot_raw(a, b, axes=((a.ndim - 1,), (b.ndim - 2,)))


dot = _wrap(_dot_raw, "dot")


def _matmul_raw(a, b):
    a, b = D.asarray(a), D.asarray(b)
    if a.ndim == 0 or b.ndim == 0:
        raise ValueError("matmul: Input operand does not have enough dimensions")
    if a.ndim <= 2 and b.ndim <= 2:
        return _dot_raw(a, b)
    dt = D._float_dtype(D.result_dtype(a, b))
    a = D.astype(a, dt) if a.dtype != dt else a
    b = D.astype(b, dt) if b.dtype != dt else b
    ta, tb = a._t, b._t
    a_vec, b_vec = ta.dim() == 1, tb.dim() == 1
    if a_vec:
        ta = ta.unsqueeze(0)
    if b_vec:
        tb = tb.unsqueeze(1)
    batch = D.broadcast_shapes(tuple(ta.shape[:-2]), tuple(tb.shape[:-2]))
    ta = ta.expand(batch + tuple(ta.shape[-2:]))
    tb = tb.expand(batch + tuple(tb.shape[-2:]))
    M, K = ta.shape[-2:]
    N = tb.shape[-1]

    def flat(t, rows, cols):
        # (batch..., rows, cols) -> (B, rows, cols) keeping stride-0 batch axes when one axis suffices
        try:
            return t.view((-1, rows, cols)) if len(batch) != 1 else t
        except RuntimeError:
            return D.contiguous(DevArray(t, dt))._t.view((-1, rows, cols))

    fa, fb = flat(ta, M, K), flat(tb, K, N)
    c = D.gemm_batched(fa, fb, dt).view(batch + (M, N))
    if a_vec:
        c = c.squeeze(-2)
    if b_vec:
        c = c.squeeze(-1)
    return DevArray(c, dt)


matmul = _wrap(_matmul_raw, "matmul")


def _tensordot_raw(a, b, axes=2):
    a, b = D.asarray(a), D.asarray(b)
    dt = D._float_dtype(D.result_dtype(a, b))
    a = D.astype(a, dt) if a.dtype != dt else a
    b = D.astype(b, dt) if b.dtype != dt else b
    if isinstance(axes, (numbers.Integral, onp.integer)):
        n = int(axes)
        if n < 0:
            n = 0
        axes_a, axes_b = list(range(a.ndim - n, a.ndim)), list(range(n))
    else:
        axes_a, axes_b = axes
        axes_a = [axes_a] if isinstance(axes_a, (numbers.Integral, onp.integer)) else list(axes_a)
        axes_b = [axes_b] if isinstance(axes_b, (numbers.Integral, onp.integer)) else list(axes_b)
    axes_a = [int(x) % a.ndim for x in axes_a] if a.ndim else []
    axes_b = [int(x) % b.ndim for x in axes_b] if b.ndim else []
    if len(axes_a) != len(axes_b) or builtins.any(a.shape[i] != b.shape[j] for i, j in zip(axes_a, axes_b)):
        raise ValueError("shape-mismatch for sum")
    free_a = [d for d in range(a.ndim) if d not in axes_a]
    free_b = [d for d in range(b.ndim) if d not in axes_b]
    M = 1
    for d in free_a:
        M *= a.shape[d]
    N = 1
    for d in free_b:
        N *= b.shape[d]
    K = 1
    for d in axes_a:
        K *= a.shape[d]
    at = a._t.permute(free_a + axes_a) if a.ndim else a._t
    bt = b._t.permute(axes_b + free_b) if b.ndim else b._t
    a2 = _view_or_copy(DevArray(at, dt), (M, K))._t
    b2 = _view_or_copy(DevArray(bt, dt), (K, N))._t
    out_shape = tuple(a.shape[d] for d in free_a) + tuple(b.shape[d] for d in free_b)
    c = D.gemm2d(a2, b2, dt)
    return DevArray(c.view(out_shape), dt)


tensordot = _wrap(_tensordot_raw, "tensordot")


@primitive
def outer(a, b):
    a, b = ravel.fun(D.asarray(a)), ravel.fun(D.asarray(b))
    return D.arith_map(Op.MUL, DevArray(a._t.unsqueeze(1), a.dtype), DevArray(b._t.unsqueeze(0), b.dtype))


# ---- the remaining array functions with rules in the reference's table (numpy_vjps.py:193-216, 352-405,
# ---- 552-566, 855-872): views where NumPy gives views, one copy kernel otherwise ------------------------
def _identity_primitive(name):
    return _wrap(lambda x: D.asarray(x), name)


# real arrays only: these are the identity (numpy_vjps.py:207-213 reduce to passing g through)
real = _identity_primitive("real")
real_if_close = _identity_primitive("real_if_close")
conj = conjugate = _identity_primitive("conjugate")


def _copy_into(dst, src):
    """dst[...] = src with the device copy kernel (cast when the types differ)."""
    if dst.dtype in D._FLOATS and src.dtype in D._FLOATS:
        D.map_op(Op.COPY, dst.dtype, src, out=dst)
    else:
        _lib.cast(_lib.DTYPE_CODE[src.dtype], _lib.DTYPE_CODE[dst.dtype], dst.shape, dst._t, D.plain(src)._t)


@primitive
def roll(x, shift, axis=None):
    x = D.asarray(x)
    if not isinstance(shift, (numbers.Integral, onp.integer)) or not (axis is None or isinstance(axis, numbers.Integral)):
        raise NotImplementedError("roll: one integer shift along one axis (or the flattened array) is supported")
    if axis is None:
        return reshape.fun(roll.fun(ravel.fun(x), shift, 0), x.shape)
    axis = D.normalize_axes(axis, x.ndim)[0]
    n = x.shape[axis]
    out = D.empty(x.shape, x.dtype)
    s = int(shift) % n if n else 0
    for dst0, src0, m in ((s, 0, n - s), (0, n - s, s)):
        if m and x.size:
            _copy_into(DevArray(out._t.narrow(axis, dst0, m), x.dtype), DevArray(D.plain(x)._t.narrow(axis, src0, m), x.dtype))
    return out


@primitive
def cumsum(x, axis=None):
    """Running sums, added in index order like NumPy's (bit-identical): one line per thread."""
    x = D.asarray(x)
    if x.dtype not in D._FLOATS:
        raise NotImplementedError("cumsum: floating-point arrays only on the device")
    if axis is None:
        x, axis = D.asarray(ravel.fun(x)), 0
    (axis,) = D.normalize_axes(axis, x.ndim)
    if x.size == 0:
        return D.empty(x.shape, x.dtype)
    src, ax, restore = _in_memory_order(x, axis)
    shp = tuple(src.shape)
    out = _lib.empty(shp, x.dtype)
    outer, inner = int(onp.prod(shp[:ax], dtype=onp.int64)), int(onp.prod(shp[ax + 1 :], dtype=onp.int64))
    _lib.cumsum(_lib.DTYPE_CODE[x.dtype], src, outer, shp[ax], inner, out)
    return restore(out)


def _split_views(ary, sections, axis, even):
    ary = D.asarray(ary)
    (axis,) = D.normalize_axes(axis, ary.ndim)
    n = ary.shape[axis]
    if isinstance(sections, (numbers.Integral, onp.integer)):
        k = int(sections)
        if k <= 0:
            raise ValueError("number sections must be larger than 0.")
        if even and n % k:
            raise ValueError("array split does not result in an equal division")
        each, extra = divmod(n, k)
        bounds = [0]
        for i in range(k):
            bounds.append(bounds[-1] + each + (1 if i < extra else 0))
    else:
        bounds = [0] + [int(b) for b in sections] + [n]
    pieces = []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        lo, hi = slice(lo, hi).indices(n)[:2]
        pieces.append(D.plain(ary)._view(lambda t, lo=lo, hi=hi: t.narrow(axis, lo, hi - lo if hi > lo else 0)))
    return pieces


split = _wrap(lambda ary, indices_or_sections, axis=0: _split_views(ary, indices_or_sections, axis, True), "split")
array_split = _wrap(lambda ary, indices_or_sections, axis=0: _split_views(ary, indices_or_sections, axis, False),
                    "array_split")
vsplit = _wrap(lambda ary, indices_or_sections: _split_views(ary, indices_or_sections, 0, True), "vsplit")
hsplit = _wrap(lambda ary, indices_or_sections: _split_views(
    ary, indices_or_sections, 1 if D.asarray(ary).ndim > 1 else 0, True), "hsplit")
dsplit = _wrap(lambda ary, indices_or_sections: _split_views(ary, indices_or_sections, 2, True), "dsplit")


@primitive
def diff(a, n=1, axis=-1):
    a = D.asarray(a)
    (axis,) = D.normalize_axes(axis, a.ndim)
    if n < 0:
        raise ValueError("order must be non-negative but got " + repr(n))
    for _ in range(int(n)):
        m = a.shape[axis]
        hi = D.plain(a)._view(lambda t: t.narrow(axis, 1, m - 1) if m else t)
        lo = D.plain(a)._view(lambda t: t.narrow(axis, 0, m - 1) if m else t)
        a = D.arith_map(Op.SUB, hi, lo)
    return a


@primitive
def sinc(x):
    """sin(pi x) / (pi x) the way NumPy evaluates it: x == 0 is moved to 1e-20 first."""
    x = D.asarray(x)
    dt = D._float_dtype(x.dtype)
    moved = D.map_op(Op.WHERE, dt, D.astype(D.compare(Cmp.EQ, x, 0.0), dt), 1.0e-20, x)
    y = D.map_op(Op.MUL, dt, onp.pi, moved)
    return D.map_op(Op.DIV, dt, D.map_op(Op.SIN, dt, y), y)


@primitive
def cross(a, b, axisa=-1, axisb=-1, axisc=-1, axis=None):
    """Vector product of 3-vectors (NumPy's own evaluation order: each component is one product minus another)."""
    if axis is not None:
        axisa = axisb = axisc = axis
    a, b = D.asarray(a), D.asarray(b)
    a, b = D.asarray(moveaxis.fun(a, axisa, -1)), D.asarray(moveaxis.fun(b, axisb, -1))
    if a.shape[-1] != 3 or b.shape[-1] != 3:
        raise NotImplementedError("cross: 3-vectors only on the device")
    part = lambda v, k: v._view(lambda t: t[..., k])  # noqa: E731
    comps = []
    for i, j in ((1, 2), (2, 0), (0, 1)):
        comps.append(D.arith_map(Op.SUB, D.arith_map(Op.MUL, part(a, i), part(b, j)),
                                 D.arith_map(Op.MUL, part(a, j), part(b, i))))
    out = stack(comps, axis=-1)
    return moveaxis.fun(out, -1, axisc)


@primitive
def rollaxis(a, axis, start=0):
    a = D.asarray(a)
    n = a.ndim
    (axis,) = D.normalize_axes(axis, n)
    if start < 0:
        start += n
    if not 0 <= start < n + 1:
        raise onp.exceptions.AxisError(f"'start' arg requires {-n} <= start < {n + 1}, but {start - n if start < 0 else start} was passed in")
    if axis < start:
        start -= 1
    if axis == start:
        return a
    order = list(range(n))
    order.remove(axis)
    order.insert(start, axis)
    return transpose.fun(a, order)


# ---- sorting (numpy_vjps.py:773-802): a stable counting sort on the device; rules move cotangents and tangents
# ---- through the permutation with `_reorder`, whose own rule is the inverse permutation --------------------
def _sorted_lines(x, axis, want):
    """Sort along ``axis``; ``want`` names the results: "sorted", "order" (argsort), "rank" (its inverse)."""
    x = D.asarray(x)
    if x.dtype not in D._FLOATS:
        raise NotImplementedError("sort: floating-point arrays only on the device")
    if axis is None:
        x, axis = D.asarray(ravel.fun(x)), 0
    if x.ndim == 0:
        raise onp.exceptions.AxisError(axis, 0)
    (axis,) = D.normalize_axes(axis, x.ndim)
    last = x.ndim - 1
    lines = D.contiguous(D.plain(D.asarray(moveaxis.fun(x, axis, last))))
    n = lines.shape[-1]
    rows = lines.size // n if n else 0
    i64 = onp.dtype(onp.int64)
    outs = {"sorted": D.empty(lines.shape, x.dtype) if "sorted" in want else None,
            "order": D.empty(lines.shape, i64) if "order" in want else None,
            # long rows are counted in slices that accumulate into the rank array: it is always handed over then
            "rank": D.empty(lines.shape, i64) if "rank" in want or n >= 2048 else None}
    if lines.size:
        _lib.sort_rows(_lib.DTYPE_CODE[x.dtype], lines._t, rows, n, *(None if outs[k] is None else outs[k]._t
                                                                      for k in ("sorted", "order", "rank")))
    back = lambda a: a if axis == last else D.asarray(moveaxis.fun(a, last, axis))  # noqa: E731
    return tuple(back(outs[k]) for k in want)


@primitive
def sort(a, axis=-1, kind=None, order=None):
    if order is not None:
        raise NotImplementedError("sort: structured-array fields are not supported on the device")
    return _sorted_lines(a, axis, ("sorted",))[0]


@primitive
def partition(a, kth, axis=-1, kind="introselect", order=None):
    """A full sort: it satisfies numpy.partition's contract for every ``kth``."""
    if order is not None:
        raise NotImplementedError("partition: structured-array fields are not supported on the device")
    return _sorted_lines(a, axis, ("sorted",))[0]


def argsort(a, axis=-1, kind=None, order=None):
    from ..tracer import getval

    return _sorted_lines(getval(a), axis, ("order",))[0]


def argpartition(a, kth, axis=-1, kind="introselect", order=None):
    from ..tracer import getval

    return _sorted_lines(getval(a), axis, ("order",))[0]


def sort_permutations(x, axis=-1):
    """(order, rank) along ``axis``: ``take_along_axis(x, order, axis)`` is sorted and ``rank`` is the inverse
    permutation of every line."""
    from ..tracer import getval

    return _sorted_lines(getval(x), axis, ("order", "rank"))


@primitive
def _reorder(x, index, inverse, axis=0):
    """``take_along_axis(x, index, axis)`` for an ``index`` that permutes every line and is already on the device
    (``inverse`` holds the inverse permutations, used by the rule).  The index comes from the sort kernel, so it
    is not read back for a bounds check."""
    x = D.asarray(x)
    if x.ndim > 1:
        (axis,) = D.normalize_axes(axis, x.ndim)
        last = x.ndim - 1
        lines = D.contiguous(D.plain(D.asarray(moveaxis.fun(x, axis, last))))
        n = lines.shape[-1]
        rows = lines.size // n if n else 0
        # flat positions: the line's offset plus the place within it (exact in float64 below 2**53)
        f64 = onp.dtype(onp.float64)
        within = D.astype(D.contiguous(D.asarray(moveaxis.fun(index, axis, last))), f64)
        starts = D.from_numpy((onp.arange(rows, dtype=onp.float64) * n).reshape(lines.shape[:-1] + (1,)))
        flat = D.astype(D.map_op(Op.ADD, f64, within, starts), onp.int64)
        out = D.empty(lines.shape, x.dtype)
        if lines.size:
            _lib.take_rows(_lib.DTYPE_CODE[x.dtype], lines._t, lines.size, 1, flat._t, lines.size, out._t)
        return out if axis == last else D.asarray(moveaxis.fun(out, last, axis))
    x = D.contiguous(D.plain(x))
    n = x.shape[0]
    out = D.empty(x.shape, x.dtype)
    if x.size:
        _lib.take_rows(_lib.DTYPE_CODE[x.dtype], x._t, n, x.size // n, index._t, n, out._t)
    return out


@primitive
def flip(m, axis=None):
    m = D.asarray(m)
    return _reverse_axes(m, D.normalize_axes(axis, m.ndim))


@primitive
def flipud(m):
    m = D.asarray(m)
    if m.ndim < 1:
        raise ValueError("Input must be >= 1-d.")
    return flip.fun(m, 0)


@primitive
def fliplr(m):
    m = D.asarray(m)
    if m.ndim < 2:
        raise ValueError("Input must be >= 2-d.")
    return flip.fun(m, 1)


@primitive
def rot90(m, k=1, axes=(0, 1)):
    m = D.asarray(m)
    if len(axes) != 2:
        raise ValueError("len(axes) must be 2.")
    (a0,), (a1,) = D.normalize_axes(axes[0], m.ndim), D.normalize_axes(axes[1], m.ndim)
    if a0 == a1:
        raise ValueError("Axes must be different.")
    k = int(k) % 4
    if k == 0:
        return m
    if k == 2:
        return flip.fun(m, (a0, a1))
    turned = D.asarray(swapaxes.fun(m, a0, a1))
    # a quarter turn is a transposition and one reversal (numpy.rot90: k=1 reverses axis a1 first, k=3 reverses it after)
    return flip.fun(turned, a0 if k == 1 else a1)


@primitive
def diagonal(A, offset=0, axis1=0, axis2=1):
    A = D.asarray(A)
    return D.plain(A)._view(lambda t: torch.diagonal(t, int(offset), axis1, axis2))


@primitive
def make_diagonal(D_, offset=0, axis1=0, axis2=1):
    """Zeros with ``D_`` written on the diagonal of the last two axes (numpy_wrapper.py:172-185: only that
    placement exists, and the zeros are float64 whatever ``D_`` is)."""
    if not (offset == 0 and axis1 == -1 and axis2 == -2):
        raise NotImplementedError(
            "Currently make_diagonal only supports offset=0, axis1=-1, axis2=-2"
        )
    d = D.asarray(D_)
    out = D.zeros(d.shape + (d.shape[-1],), onp.dtype(onp.float64))
    if d.size:
        _copy_into(DevArray(torch.diagonal(out._t, 0, -1, -2), out.dtype), d)
    return out


@primitive
def diag(x, k=0):
    x = D.asarray(x)
    k = int(k)
    if x.ndim == 2:
        return D.plain(x)._view(lambda t: torch.diagonal(t, k))
    if x.ndim != 1:
        raise ValueError("Input must be 1- or 2-d.")
    n = x.shape[0] + (k if k >= 0 else -k)
    out = D.zeros((n, n), x.dtype)
    if x.size:
        _copy_into(DevArray(torch.diagonal(out._t, k), x.dtype), x)
    return out


@primitive
def trace(x, offset=0):
    x = D.asarray(x)
    if x.ndim < 2:
        raise ValueError("diag requires an array of at least two dimensions")
    return sum.fun(diagonal.fun(x, offset), axis=-1)


def _triangle(x, k, lower):
    x = D.asarray(x)
    if x.ndim < 2:
        x = D.asarray(broadcast_to.fun(x, (x.shape[0] if x.ndim else 1,) * 2))
    if x.dtype not in D._FLOATS:
        raise NotImplementedError("tril/triu: floating-point arrays only on the device")
    rows, cols = x.shape[-2:]
    src = D.contiguous(D.plain(x))
    out = D.empty(x.shape, x.dtype)
    _lib.triangle(_lib.DTYPE_CODE[x.dtype], src._t, int(onp.prod(x.shape[:-2], dtype=onp.int64)), rows, cols, int(k), lower,
                  out._t)
    return out


tril = _wrap(lambda x, k=0: _triangle(x, k, True), "tril")
triu = _wrap(lambda x, k=0: _triangle(x, k, False), "triu")


@primitive
def tile(x, reps):
    x = D.asarray(x)
    reps = (int(reps),) if isinstance(reps, (numbers.Integral, onp.integer)) else tuple(int(r) for r in reps)
    nd = builtins.max(len(reps), x.ndim)
    reps = (1,) * (nd - len(reps)) + reps
    shp = (1,) * (nd - x.ndim) + x.shape
    # out viewed as (r0, n0, r1, n1, ...) = x broadcast along the r axes
    lifted, wide, final = [], [], []
    for r, n in zip(reps, shp):
        lifted += [1, n]
        wide += [r, n]
        final.append(r * n)
    widened = D.plain(x)._view(lambda t: t.reshape(lifted).expand(wide))
    out = D.copy(widened) if onp.prod(wide) else D.empty(tuple(wide), x.dtype)
    return DevArray(out._t.view(final), x.dtype)


@primitive
def kron(a, b):
    a, b = D.asarray(a), D.asarray(b)
    nd = builtins.max(a.ndim, b.ndim)
    sa, sb = (1,) * (nd - a.ndim) + a.shape, (1,) * (nd - b.ndim) + b.shape
    la, lb, final = [], [], []
    for n, m in zip(sa, sb):
        la += [n, 1]
        lb += [1, m]
        final.append(n * m)
    out = D.arith_map(Op.MUL, D.plain(a)._view(lambda t: t.reshape(la)), D.plain(b)._view(lambda t: t.reshape(lb)))
    return DevArray(D.contiguous(out)._t.view(final), out.dtype)


@primitive
def inner(a, b):
    if onp.ndim(a) == 0 or onp.ndim(b) == 0:  # a Python scalar stays weakly typed in the product
        return D.arith_map(Op.MUL, a, b)
    a, b = D.asarray(a), D.asarray(b)
    return _tensordot_raw(a, b, axes=([a.ndim - 1], [b.ndim - 1]))


# ---- einsum (subscript-string convention) -> sums, permutations and batched MFMA GEMMs ----------------
def parse_einsum_input(*args):
    """``(input subscripts, output subscripts, array operands)`` of an einsum call in either convention
    (subscript string, or operands alternating with sublists), letters only: NumPy's own parser (the
    reference wraps the same routine, numpy_wrapper.py:194-195) run on shape-only stand-ins, so no operand
    is copied to the host; it also spells out an ellipsis as letters."""
    try:
        from numpy._core.einsumfunc import _parse_einsum_input
    except ImportError:  # NumPy 1.x
        from numpy.core.einsumfunc import _parse_einsum_input
    from ..tracer import getval

    def stand_in(a):
        return onp.broadcast_to(onp.zeros((), onp.float32), shape(getval(a)))

    if isinstance(args[0], str):
        arrays = tuple(args[1:])
        spec = [args[0]] + [stand_in(a) for a in arrays]
    else:
        n = len(args) // 2
        arrays = tuple(args[0:2 * n:2])
        spec = [stand_in(a) if i % 2 == 0 and i < 2 * n else a for i, a in enumerate(args)]
    in_subs, out_subs, _ = _parse_einsum_input(spec)
    return in_subs, out_subs, arrays


def _einsum_diagonals(x, subs):
    """A letter repeated within one operand's subscripts reads a diagonal: the operand as a strided view with
    that letter once (its axis last, as ``torch.diagonal`` puts it).  Returns (view, subscripts)."""
    while True:
        dup = next((c for c in subs if subs.count(c) > 1), None)
        if dup is None:
            return x, subs
        p = subs.index(dup)
        q = subs.index(dup, p + 1)
        if x.shape[p] != x.shape[q]:
            raise ValueError(f"einsum: dimensions in operand for collapsing index {dup!r} don't match ({x.shape[p]} != {x.shape[q]})")
        x = x._view(lambda t: torch.diagonal(t, 0, p, q))
        subs = "".join(c for i, c in enumerate(subs) if i not in (p, q)) + dup


def _einsum_sum_out(x, subs, drop):
    """Sum the axes of ``x`` labelled by the letters in ``drop``."""
    axes = tuple(i for i, c in enumerate(subs) if c in drop)
    if not axes:
        return x, subs
    x = D.map_reduce(Op.COPY, Red.SUM, x.dtype, (x,), axes, False)
    return x, "".join(c for c in subs if c not in drop)


def _einsum_pair(a, sa, b, sb, keep):
    """Contract two labelled operands; letters in ``keep`` survive.  Returns (array, labels)."""
    a, sa = _einsum_sum_out(a, sa, {c for c in sa if c not in sb and c not in keep})
    b, sb = _einsum_sum_out(b, sb, {c for c in sb if c not in sa and c not in keep})
    size = {}
    for x, sx in ((a, sa), (b, sb)):
        for c, n in zip(sx, x.shape):
            if size.get(c, 1) == 1:
                size[c] = n
            elif n not in (1, size[c]):
                raise ValueError(f"einsum: operands could not be broadcast together on subscript {c!r}")
    batch = [c for c in sa if c in sb and c in keep]
    contracted = [c for c in sa if c in sb and c not in keep]
    free_a = [c for c in sa if c not in sb]
    free_b = [c for c in sb if c not in sa]

    def arrange(x, sx, order):
        x = transpose.fun(x, [sx.index(c) for c in order])
        full = tuple(size[c] for c in order)
        return broadcast_to.fun(x, full) if x.shape != full else x

    def prod(letters):
        n = 1
        for c in letters:
            n *= size[c]
        return n

    Bn, M, K, N = prod(batch), prod(free_a), prod(contracted), prod(free_b)
    a3 = _view_or_copy(arrange(a, sa, batch + free_a + contracted), (Bn, M, K))
    b3 = _view_or_copy(arrange(b, sb, batch + contracted + free_b), (Bn, K, N))
    dt = a.dtype
    c = D.gemm_batched(D.plain(a3)._t, D.plain(b3)._t, dt)
    out_subs = batch + free_a + free_b
    return DevArray(c.view(tuple(size[c_] for c_ in out_subs)), dt), "".join(out_subs)


@primitive
def einsum(*operands, **kwargs):
    """``numpy.einsum`` in both calling conventions (subscript string; operands alternating with sublists):
    a letter repeated within one operand is read as a diagonal (a strided view), then operands are
    contracted pairwise from the left, each pair as a batched GEMM on permuted views; letters that appear
    nowhere else are summed out first."""
    if kwargs:
        raise NotImplementedError(f"einsum: keyword arguments {sorted(kwargs)} are not supported on the device")
    in_subs, out_subs, arrays = parse_einsum_input(*operands)
    subs = in_subs.split(",")
    arrays = [D.asarray(a) for a in arrays]
    dt = D._float_dtype(D.result_dtype(*arrays))
    arrays = [D.astype(a, dt) if a.dtype != dt else a for a in arrays]
    if len(set(out_subs)) != len(out_subs):
        raise ValueError("einsum: output subscripts may name an index only once")
    for k in range(len(arrays)):
        arrays[k], subs[k] = _einsum_diagonals(arrays[k], subs[k])
    cur, cur_subs = arrays[0], subs[0]
    for k in range(1, len(arrays)):
        keep = set(out_subs).union(*subs[k + 1:]) if k + 1 < len(arrays) else set(out_subs)
        cur, cur_subs = _einsum_pair(cur, cur_subs, arrays[k], subs[k], keep)
    cur, cur_subs = _einsum_sum_out(cur, cur_subs, {c for c in cur_subs if c not in out_subs})
    if cur_subs != out_subs:
        cur = transpose.fun(cur, [cur_subs.index(c) for c in out_subs])
    if type(cur) is not DevArray or not cur._t.is_contiguous():
        cur = D.copy(cur) if cur.dtype in D._FLOATS else cur  # a diagonal or permuted view of an input: NumPy returns a new array
    return copy_if_input(cur, arrays)


def copy_if_input(x, inputs):
    """``x`` itself unless it is one of ``inputs`` (a primitive must not return its argument object)."""
    for a in inputs:
        if x is a:
            return D.alias(x)
    return x


# ---- non-differentiable helpers ---------------------------------------------------------------
def _meta_of(A):
    if isinstance(A, DevArray):
        return A.shape, A.ndim, A.dtype, False
    if type(A) in (list, tuple):
        A = onp.asarray(A)  # (result_type would read a nested list as a structured dtype)
    return onp.shape(A), onp.ndim(A), onp.result_type(A), onp.iscomplexobj(A)


# `metadata`, `shape` and `ndim` run dozens of times per step of a traced loop (every rule that reshapes or unbroadcasts
# asks): they unbox and read the attributes themselves instead of going through the generic wrapper.
def metadata(A):
    while type(A) in _box_types:
        A = A._value
    if isinstance(A, DevArray):
        return A.shape, A.ndim, A.dtype, False
    return _meta_of(A)


def shape(A):
    while type(A) in _box_types:
        A = A._value
    if isinstance(A, DevArray):
        return A.shape
    return _meta_of(A)[0]


def ndim(A):
    while type(A) in _box_types:
        A = A._value
    if isinstance(A, DevArray):
        return A.ndim
    return _meta_of(A)[1]


metadata._is_primitive = shape._is_primitive = ndim._is_primitive = True


@notrace_primitive
def result_type(*xs):
    return D.result_dtype(*xs) if len(xs) > 1 else _meta_of(xs[0])[2]


@notrace_primitive
def size(A):
    return A.size if isinstance(A, DevArray) else onp.size(A)


@notrace_primitive
def iscomplexobj(A):
    return False if isinstance(A, DevArray) else onp.iscomplexobj(A)


@notrace_primitive
def isscalar(A):
    return onp.isscalar(A)


def zeros(shape, dtype=float):
    return D.constant(shape, 0.0, dtype)


def ones(shape, dtype=float):
    return D.constant(shape, 1.0, dtype)


@primitive
def full(shape, fill_value, dtype=None):
    """``numpy.full``; differentiable in ``fill_value`` (argument 1), which may be a 0-d device array."""
    if isinstance(fill_value, DevArray):
        shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
        src = fill_value if dtype is None else astype(fill_value, dtype)
        return D.contiguous(broadcast_to(reshape(src, ()), shape))
    if dtype is None or not isinstance(fill_value, (int, float)) or isinstance(fill_value, bool):
        return D.full(shape, fill_value, dtype)
    return D.constant(shape, fill_value, dtype)


def empty(shape, dtype=float):
    return D.empty(shape, dtype)


def settle(x):
    """``x`` with any deferred arithmetic done (a pending affine map written out, a deferred contraction or
    logsumexp cotangent computed); tuples, lists and dicts are walked.  The package's own differential operators do
    this to every derivative they hand back; it is for callers that obtained a value some other way (a tracer of
    another package hosting the value type) and want its kernels inside their own timed region."""
    from ..tracer import getval

    x = getval(x)
    kind = type(x)
    if kind is tuple or kind is list:
        return kind(settle(item) for item in x)
    if kind is dict:
        return {key: settle(item) for key, item in x.items()}
    finish = getattr(kind, "_settled", None)
    return finish(x) if finish is not None else x


@notrace_primitive
def zeros_like(a, dtype=None):
    s, _, dt, _ = _meta_of(a)
    return D.constant(s, 0.0, dtype or dt)


@notrace_primitive
def full_like(a, fill_value, dtype=None):
    s, _, dt, _ = _meta_of(a)
    return D.full(s, fill_value, onp.dtype(dtype or dt))


@notrace_primitive
def empty_like(a, dtype=None):
    s, _, dt, _ = _meta_of(a)
    return D.empty(s, onp.dtype(dtype or dt))


@notrace_primitive
def ones_like(a, dtype=None):
    s, _, dt, _ = _meta_of(a)
    return D.constant(s, 1.0, dtype or dt)


@primitive
def linspace(start, stop, num=50, endpoint=True, dtype=None):
    """``numpy.linspace``.  Host numbers give an uploaded constant; a device-resident end point is
    taken through NumPy's own arithmetic, ``arange(num) * ((stop - start) / div) + start`` with the
    last sample set to ``stop``, in the dtype NumPy would choose."""
    if not (isinstance(start, DevArray) or isinstance(stop, DevArray)):
        return D.from_numpy(onp.linspace(start, stop, num, endpoint=endpoint), dtype)
    num = int(num)
    if num < 0:
        raise ValueError("Number of samples, %s, must be non-negative." % num)
    div = num - 1 if endpoint else num
    ends = [v.dtype if isinstance(v, DevArray) else v for v in (start, stop)]
    steps = D.from_numpy(onp.arange(num, dtype=onp.result_type(ends[0], ends[1], float(num))))
    step = (stop - start) / div if div > 0 else (stop - start)
    samples = steps * step + start
    if endpoint and num > 1:
        samples = concatenate([samples[:-1], reshape(stop + 0.0 * start, (1,))])
    return samples if dtype is None else astype(samples, dtype)


def gradient(f, *varargs, axis=None, edge_order=1):
    """``numpy.gradient`` with unit spacing: central differences inside, one-sided ones at both
    ends, built from slices so that it differentiates to any order (the reference gives it a
    hand-written cotangent, numpy_vjps.py:297-342, and only supports ``axis`` too)."""
    if varargs or edge_order != 1:
        raise NotImplementedError("The only optional argument currently supported for np.gradient is axis.")
    nd = ndim(f)
    if axis is None:
        axes = tuple(range(nd))
    elif isinstance(axis, numbers.Integral):
        axes = (int(axis),)
    else:
        axes = tuple(int(a) for a in axis)
    axes = tuple(a + nd if a < 0 else a for a in axes)
    extents = shape(f)
    outs = []
    for a in axes:
        if not 0 <= a < nd:
            raise onp.exceptions.AxisError(a, nd)
        if extents[a] < 2:
            raise ValueError(
                "Shape of array too small to calculate a numerical gradient, "
                "at least (edge_order + 1) elements are required."
            )

        def cut(lo, hi, a=a):
            return f[(slice(None),) * a + (slice(lo, hi),)]

        pieces = [cut(1, 2) - cut(0, 1)]
        if extents[a] > 2:
            pieces.append((cut(2, None) - cut(None, -2)) / 2.0)
        pieces.append(cut(-1, None) - cut(-2, -1))
        outs.append(concatenate(pieces, axis=a))
    if len(axes) == 1 and (axis is None or isinstance(axis, numbers.Integral)):
        return outs[0]
    from ..builtins import tuple as traced_tuple  # (a traced container: the derivatives stay visible to the caller's trace)

    return traced_tuple(outs)


def arange(*args, **kwargs):
    return D.from_numpy(onp.arange(*args, **kwargs))


def eye(N, M=None, k=0, dtype=float):
    """Made on the device (a zero fill and ones written along the diagonal view), so that rules that need an
    identity, like the cotangent of ``trace``, launch kernels only and can be recorded into a graph."""
    dt = onp.dtype(dtype)
    if dt not in D._FLOATS:
        return D.from_numpy(onp.eye(N, M, k, dtype=dtype))
    out = D.zeros((int(N), int(N if M is None else M)), dt)
    diagonal_view = torch.diagonal(out._t, int(k))
    if diagonal_view.numel():
        D.map_op(Op.COPY, dt, D.ones((), dt), out=DevArray(diagonal_view, dt))
    return out


to_numpy = D.to_numpy


def synchronize():
    _lib.synchronize()


# ---- what device arrays, being real, make trivial; and the functions whose result SHAPE depends on the data ----
@primitive
def imag(x):
    """The imaginary part of a real array: zeros (its cotangent too, numpy_vjps.py:220)."""
    s, _, dt, _ = _meta_of(x)
    return D.constant(s, 0.0, D._float_dtype(dt))


@primitive
def angle(x):
    """``numpy.angle`` of a real array: pi where it is negative, else 0 (piecewise constant: numpy_vjps.py:224
    gives a zero cotangent for real arguments)."""
    x = D.asarray(x)
    dt = D._float_dtype(x.dtype)
    return D.map_op(Op.WHERE, dt, D.astype(D.compare(Cmp.LT, x, 0.0), dt), float(onp.pi), 0.0)


def isreal(x):
    from ..tracer import getval

    return D.full(_meta_of(getval(x))[0], True, onp.bool_)


def iscomplex(x):
    from ..tracer import getval

    return D.full(_meta_of(getval(x))[0], False, onp.bool_)


def floor_divide(a, b):
    """``numpy.floor_divide`` (no derivative, numpy_vjps.py:13-68), the way NumPy forms it: the quotient of
    ``a - remainder(a, b)`` and ``b`` is a whole number up to rounding, so it is rounded to the nearest; a zero
    divisor gives ``a / b``."""
    from ..tracer import getval

    a, b = getval(a), getval(b)
    whole = rint.fun(true_divide.fun(subtract.fun(a, remainder.fun(a, b)), b))
    return _where3.fun(D.compare(Cmp.EQ, D.asarray(b) if isinstance(b, DevArray) else b, 0.0), true_divide.fun(a, b), whole)


def array_equiv(a1, a2):
    """A Python bool (reads one element back): the shapes broadcast and all elements are equal."""
    from ..tracer import getval

    a1, a2 = D.asarray(getval(a1)), D.asarray(getval(a2))
    try:
        D.broadcast_shapes(a1.shape, a2.shape)
    except ValueError:
        return False
    hit = D.compare(Cmp.EQ, a1, a2)
    return True if hit.size == 0 else bool(to_numpy(min.fun(D.astype(hit, onp.float64))) == 1.0)


def _on_the_host(name):
    """Functions whose result shape depends on the values (``nonzero`` and friends; none has a derivative,
    numpy_vjps.py:13-68): the operands are read back, NumPy answers, the integer results are uploaded.  A
    synchronising transfer, so they cannot be recorded into a graph."""
    fun = getattr(onp, name)

    def raw(*args, **kwargs):
        from ..tracer import getval

        host = [to_numpy(getval(a)) if isinstance(getval(a), DevArray) else getval(a) for a in args]
        out = fun(*host, **kwargs)
        if isinstance(out, tuple):
            return tuple(D.from_numpy(onp.ascontiguousarray(o)) for o in out)
        return D.from_numpy(onp.ascontiguousarray(out))

    raw.__name__ = raw.__qualname__ = name
    return raw


nonzero, flatnonzero, argwhere, searchsorted = (_on_the_host(n) for n in ("nonzero", "flatnonzero", "argwhere", "searchsorted"))


def allclose(a, b, rtol=1e-05, atol=1e-08):
    from ..tracer import getval

    return bool(onp.allclose(to_numpy(getval(a)), to_numpy(getval(b)), rtol=rtol, atol=atol))


def _var_forward(x, axis=None, ddof=0, keepdims=False, **kwargs):
    x = D.asarray(x)
    axes = D.normalize_axes(axis, x.ndim)
    dt = D._float_dtype(x.dtype)
    n = 1
    for d in axes:
        n *= x.shape[d]
    mu = _primitive_mean.fun(x, axis=axis, keepdims=True)
    centered = D.map_op(Op.SUB, dt, x, mu)
    total = D.map_reduce(Op.SQUARE, Red.SUM, dt, (centered,), axes, keepdims)
    return D.map_op(Op.DIV, dt, total, float(n - ddof))


_primitive_var = _wrap(_var_forward, "var")
_primitive_std = _wrap(lambda x, axis=None, ddof=0, keepdims=False, **kw: D.float_map(
    Op.SQRT, _var_forward(x, axis=axis, ddof=ddof, keepdims=keepdims)), "std")


def var(a, *args, **kwargs):
    if type(a) in (list, tuple):
        a = array(a)
    return _primitive_var(a, *args, **kwargs)


def std(a, *args, **kwargs):
    if type(a) in (list, tuple):
        a = array(a)
    return _primitive_std(a, *args, **kwargs)


# ---- names that never touch array data ---------------------------------------------------------------
def meshgrid(*xi, copy=True, sparse=False, indexing="xy"):
    """Coordinate matrices as broadcast views of the 1-d inputs (``numpy.meshgrid``; the reference wraps it without a
    rule, here it differentiates through ``reshape`` and ``broadcast_to``).  ``copy`` is accepted for NumPy's
    signature: device arrays are never written in place, so views serve either way."""
    if indexing not in ("xy", "ij"):
        raise ValueError("Valid values for `indexing` are 'xy' and 'ij'.")
    nd = len(xi)
    grids = []
    for position, x in enumerate(xi):
        extents = [1] * nd
        extents[position] = -1
        grids.append(reshape(ravel(array(x)), tuple(extents)))
    if indexing == "xy" and nd > 1:
        grids[0], grids[1] = reshape(grids[0], (1, -1) + (1,) * (nd - 2)), reshape(grids[1], (-1, 1) + (1,) * (nd - 2))
    if not sparse:
        full = onp.broadcast_shapes(*(shape(g) for g in grids)) if grids else ()
        grids = [broadcast_to(g, full) for g in grids]
    return tuple(grids)


def identity(n, dtype=float):
    return eye(n, dtype=dtype)


# floating-point error state, printing, dtype arithmetic and index helpers are NumPy's own: they take no array data
for _name in ("seterr geterr errstate set_printoptions get_printoptions printoptions finfo iinfo issubdtype promote_types "
              "can_cast broadcast_shapes s_ index_exp iterable unravel_index ravel_multi_index generic number inexact "
              "floating integer signedinteger unsignedinteger float16 double single uint8 uint16 uint32 uint64 intp int_").split():
    globals()[_name] = getattr(onp, _name)
del _name
