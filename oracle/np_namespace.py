"""NumPy functions wrapped as primitives of the repository's tracer (oracle side).

Restates the part of the reference's autograd/numpy/numpy_wrapper.py that the
hot path uses: every listed NumPy callable becomes a ``primitive`` (25-52),
shape queries are never traced (18, 188-190), list-taking functions are routed
through ``concatenate_args`` / ``array_from_args`` so that boxes inside Python
lists are seen (57-107).  TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

import numpy as _np

from autograd_amd.extend import notrace_primitive, primitive

# --- every NumPy callable below is wrapped once; aliases share the wrapper ---------
_WRAPPED = """
add subtract multiply divide true_divide power negative positive mod remainder
exp exp2 expm1 log log2 log10 log1p sin cos tan sinh cosh tanh arcsin arccos arctan
arcsinh arccosh arctanh sqrt square abs absolute fabs reciprocal sign maximum minimum
fmax fmin logaddexp hypot arctan2 where clip nan_to_num real imag conj conjugate
rad2deg degrees deg2rad radians
sum mean prod max min amax amin var std cumsum
reshape ravel expand_dims squeeze transpose swapaxes moveaxis atleast_1d atleast_2d
atleast_3d repeat tile split array_split vsplit hsplit dsplit rollaxis rot90 diff cross sinc logaddexp2 broadcast_to roll flipud fliplr diag diagonal trace tril triu
dot matmul tensordot inner outer einsum kron
astype
floor ceil round rint around fix trunc all any argmax argmin argsort argpartition sort partition nonzero
count_nonzero searchsorted floor_divide logical_and logical_or logical_not logical_xor
isfinite isinf isnan allclose isclose array_equal greater greater_equal less less_equal
equal not_equal iscomplex size isscalar isreal zeros_like ones_like empty_like full_like
zeros ones empty full eye identity arange linspace asarray copy pad gradient
""".split()

_by_identity = {}
for _name in _WRAPPED:
    _obj = getattr(_np, _name)
    if id(_obj) not in _by_identity:
        _by_identity[id(_obj)] = primitive(_obj)
    globals()[_name] = _by_identity[id(_obj)]

for _name in ("ndim", "shape", "iscomplexobj", "result_type"):
    globals()[_name] = notrace_primitive(getattr(_np, _name))

# constants and dtypes pass through unchanged
pi, e, inf, nan, newaxis = _np.pi, _np.e, _np.inf, _np.nan, _np.newaxis
float16, float32, float64 = _np.float16, _np.float32, _np.float64
int32, int64, bool_ = _np.int32, _np.int64, _np.bool_
ndarray = _np.ndarray

ufunc_wrappers = {
    getattr(_np, n): globals()[n] for n in _WRAPPED if isinstance(getattr(_np, n), _np.ufunc)
}

_primitive_mean, _primitive_var, _primitive_std = mean, var, std  # noqa: F821
_astype = astype  # noqa: F821


def parse_einsum_input(*args):  # numpy_wrapper.py:194-195
    from numpy._core.einsumfunc import _parse_einsum_input

    return _parse_einsum_input(args)


@notrace_primitive
def metadata(A):
    return _np.shape(A), _np.ndim(A), _np.result_type(A), _np.iscomplexobj(A)


@primitive
def concatenate_args(axis, *args):
    return _np.concatenate(args, axis).view(_np.ndarray)


def concatenate(arr_list, axis=0):
    return concatenate_args(axis, *arr_list)


def vstack(tup):
    return concatenate([atleast_2d(m) for m in tup], axis=0)  # noqa: F821


def hstack(tup):
    arrs = [atleast_1d(m) for m in tup]  # noqa: F821
    return concatenate(arrs, 0 if arrs[0].ndim == 1 else 1)


@primitive
def _array_from_scalar_or_array(array_args, array_kwargs, scalar):
    return _np.array(scalar, *array_args, **array_kwargs)


@primitive
def array_from_args(array_args, array_kwargs, *args):
    return _np.array(args, *array_args, **array_kwargs)


def array(A, *args, **kwargs):
    if type(A) in (list, tuple):
        return array_from_args(args, kwargs, *map(array, A))
    return _array_from_scalar_or_array(args, kwargs, A)


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


def select(condlist, choicelist, default=0):  # numpy_wrapper.py:58-60: assembled element by element
    raw_array = _np.select(list(condlist), list(choicelist), default=default)
    return array(list(raw_array.ravel())).reshape(raw_array.shape)


def column_stack(tup):  # numpy_wrapper.py:73-80
    arrays = []
    for v in tup:
        arr = array(v)
        if arr.ndim < 2:
            arr = array(arr, ndmin=2).T
        arrays.append(arr)
    return concatenate(arrays, 1)


def _wrap_if_boxes_inside(raw_array):  # numpy_wrapper.py:91-97 (without the warning)
    if raw_array.dtype is _np.dtype("O"):
        return array_from_args((), {}, *raw_array.ravel()).reshape(raw_array.shape)
    return raw_array


def append(arr, values, axis=None):  # numpy_wrapper.py:139-147
    arr = array(arr)
    if axis is None:
        if ndim(arr) != 1:  # noqa: F821
            arr = ravel(arr)  # noqa: F821
        values = ravel(array(values))  # noqa: F821
        axis = ndim(arr) - 1  # noqa: F821
    return concatenate((arr, values), axis=axis)


class _RClass:  # numpy_wrapper.py:153-159: NumPy builds an object array around the boxes, which is then unpacked
    def __getitem__(self, args):
        return _wrap_if_boxes_inside(_np.r_[args])


class _CClass:  # numpy_wrapper.py:162-169
    def __getitem__(self, args):
        return _wrap_if_boxes_inside(_np.c_[args])


r_, c_ = _RClass(), _CClass()

_raw_where = where  # noqa: F821


@primitive
def make_diagonal(D, offset=0, axis1=0, axis2=1):  # numpy_wrapper.py:172-185
    if not (offset == 0 and axis1 == -1 and axis2 == -2):
        raise NotImplementedError("Currently make_diagonal only supports offset=0, axis1=-1, axis2=-2")
    out = _np.zeros(D.shape + (D.shape[-1],))
    out_diagonal = _np.diagonal(out, offset, axis1, axis2)
    out_diagonal.flags.writeable = True
    out_diagonal[...] = D
    return out


def where(condition, *args, **kwargs):  # noqa: F811
    """Keep native Python types when no operand is an array or a box
    (reference autograd/numpy/__init__.py:13-39): the ``power`` rule calls
    ``where(y, y - 1, 1.0)`` with a Python exponent and must get a Python float."""
    from autograd_amd.tracer import Box

    def arrayish(v):
        if isinstance(v, (Box, _np.ndarray, _np.generic)):
            return True
        return isinstance(v, (list, tuple)) and any(arrayish(i) for i in v)

    if not args and not kwargs:
        return _raw_where(condition)
    if len(args) + len(kwargs) != 2:
        raise ValueError("either both or neither of x and y should be given")
    x = args[0] if args else kwargs.get("x")
    y = args[1] if len(args) > 1 else kwargs.get("y")
    res = _raw_where(condition, x, y)
    if arrayish(condition) or arrayish(x) or arrayish(y):
        return res
    return res.tolist() if isinstance(res, _np.ndarray) else res
