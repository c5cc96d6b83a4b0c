"""ndarray box and vspace for the oracle's NumPy value type.

Restates the reference's autograd/numpy/numpy_boxes.py:12-189 (operator
overloads route to the wrapped namespace; ``__getitem__`` is itself a
primitive; NumPy ufuncs called on a box are redirected through
``__array_ufunc__``) and autograd/numpy/numpy_vspaces.py:7-75.
TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

import numpy as np

from autograd_amd.extend import Box, VSpace, primitive

from . import np_namespace as anp

Box.__array_priority__ = 90.0


def _route(name, swap=False):
    fn = getattr(anp, name)
    if swap:
        return lambda self, other: fn(other, self)
    return lambda self, other: fn(self, other)


class ArrayBox(Box):
    __slots__ = []
    __array_priority__ = 100.0
    _namespace = staticmethod(lambda: anp)

    @primitive
    def __getitem__(A, idx):
        return A[idx]

    shape = property(lambda self: anp.shape(self._value))
    ndim = property(lambda self: anp.ndim(self._value))
    size = property(lambda self: anp.size(self._value))
    dtype = property(lambda self: anp.result_type(self._value))
    T = property(lambda self: anp.transpose(self))

    def __array_namespace__(self, *, api_version=None):
        return anp

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        # ndarray.__mul__(box) etc. arrive here through NumPy's override protocol
        if method != "__call__" or "out" in kwargs:
            return NotImplemented
        wrapper = anp.ufunc_wrappers.get(ufunc)
        if wrapper is None:
            return NotImplemented
        return wrapper(*inputs, **kwargs)

    def __len__(self):
        return len(self._value)

    def __hash__(self):
        return id(self)

    def astype(self, *args, **kwargs):
        return anp._astype(self, *args, **kwargs)

    def __neg__(self):
        return anp.negative(self)

    def __abs__(self):
        return anp.abs(self)

    __add__, __radd__ = _route("add"), _route("add", True)
    __sub__, __rsub__ = _route("subtract"), _route("subtract", True)
    __mul__, __rmul__ = _route("multiply"), _route("multiply", True)
    __pow__, __rpow__ = _route("power"), _route("power", True)
    __mod__, __rmod__ = _route("mod"), _route("mod", True)
    __truediv__, __rtruediv__ = _route("true_divide"), _route("true_divide", True)
    __matmul__, __rmatmul__ = _route("matmul"), _route("matmul", True)
    __eq__, __ne__ = _route("equal"), _route("not_equal")
    __gt__, __ge__ = _route("greater"), _route("greater_equal")
    __lt__, __le__ = _route("less"), _route("less_equal")


ArrayBox.register(np.ndarray)
for _t in (np.float64, np.float32, np.float16, np.longdouble, np.complex64, np.complex128):
    ArrayBox.register(_t)

for _m in (
    "all any argmax argmin argsort nonzero searchsorted round "
    "clip cumsum diagonal max mean min prod ravel repeat squeeze std sum swapaxes "
    "trace transpose var"
).split():
    setattr(ArrayBox, _m, getattr(anp, _m))
ArrayBox.flatten = anp.ravel


def _box_reshape(x, *args, **kwargs):
    if isinstance(args[0], int):
        return anp.reshape(x, args, **kwargs)
    return anp.reshape(x, *args, **kwargs)


ArrayBox.reshape = _box_reshape


class ArrayVSpace(VSpace):
    def __init__(self, value):
        value = np.asarray(value)
        self.shape = value.shape
        self.dtype = value.dtype

    @property
    def size(self):
        return np.prod(self.shape)

    @property
    def ndim(self):
        return len(self.shape)

    def zeros(self):
        return np.zeros(self.shape, dtype=self.dtype)

    def ones(self):
        return np.ones(self.shape, dtype=self.dtype)

    def standard_basis(self):
        for idxs in np.ndindex(*self.shape):
            vect = np.zeros(self.shape, dtype=self.dtype)
            vect[idxs] = 1
            yield vect

    def randn(self):
        return np.array(np.random.randn(*self.shape)).astype(self.dtype)

    def _inner_prod(self, x, y):
        return np.dot(np.ravel(x), np.ravel(y))


VSpace.register(np.ndarray, ArrayVSpace)  # real arrays only: no workload of the path is complex
for _t in (np.float64, np.float32, np.float16, np.longdouble):
    ArrayVSpace.register(_t)
