"""``DevArrayBox``: the tracer box for device arrays.

Same routing as the reference's ArrayBox (autograd/numpy/numpy_boxes.py:12-189): operators
and array methods call the namespace primitives, ``__getitem__`` is itself a primitive, and
attributes that are not differentiable (shape, dtype, ...) pass through to the value.  The
same operator table is installed on ``DevArray`` so unboxed values go through the same
primitives (and therefore the same kernels).
"""

from ..extend import Box, primitive
from . import wrapper as anp
from .devarray import DevArray, FusedResult, LazyDevArray, LseCotangent, PendingProduct, PendingReduce
from .fusion import ExprArray


def _route(name, swap=False):
    fn = getattr(anp, name)
    if swap:
        return lambda self, other: fn(other, self)
    return lambda self, other: fn(self, other)


_OPERATORS = {
    "__neg__": lambda self: anp.negative(self),
    "__abs__": lambda self: anp.abs(self),
    "__pos__": lambda self: self,
    "__add__": _route("add"),
    "__radd__": _route("add", True),
    "__sub__": _route("subtract"),
    "__rsub__": _route("subtract", True),
    "__mul__": _route("multiply"),
    "__rmul__": _route("multiply", True),
    "__truediv__": _route("true_divide"),
    "__rtruediv__": _route("true_divide", True),
    "__pow__": _route("power"),
    "__rpow__": _route("power", True),
    "__mod__": _route("remainder"),
    "__rmod__": _route("remainder", True),
    "__matmul__": _route("matmul"),
    "__rmatmul__": _route("matmul", True),
    "__eq__": _route("equal"),
    "__ne__": _route("not_equal"),
    "__gt__": _route("greater"),
    "__ge__": _route("greater_equal"),
    "__lt__": _route("less"),
    "__le__": _route("less_equal"),
}


def _reshape_method(x, *args, **kwargs):
    # x.reshape(5, 4) and x.reshape((5, 4)) are both allowed (numpy_vjps.py:762-771)
    if isinstance(args[0], int):
        return anp.reshape(x, args, **kwargs)
    return anp.reshape(x, *args, **kwargs)


_METHODS = {
    name: getattr(anp, name)
    for name in "sum mean max min prod ravel repeat reshape squeeze swapaxes transpose astype dot diagonal trace".split()
}
_METHODS["reshape"] = _reshape_method
_METHODS["flatten"] = anp.ravel


class DevArrayBox(Box):
    __slots__ = []
    __array_priority__ = 300.0
    __array_ufunc__ = DevArray.__array_ufunc__  # numpy.exp(box), ndarray <op> box: the namespace's (traced) function
    _namespace = staticmethod(lambda: __import__("autograd_amd.numpy", fromlist=["numpy"]))

    @primitive
    def __getitem__(A, idx):
        return anp.take(A, idx)

    shape = property(lambda self: anp.shape(self._value))
    ndim = property(lambda self: anp.ndim(self._value))
    size = property(lambda self: anp.size(self._value))
    dtype = property(lambda self: anp.result_type(self._value))
    T = property(lambda self: anp.transpose(self))

    def __array_namespace__(self, *, api_version=None):
        return self._namespace()

    def __len__(self):
        return len(self._value)

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def __hash__(self):
        return id(self)

    def __setitem__(self, idx, value):
        raise TypeError("boxed arrays are immutable: item assignment is not supported")


for _name, _fn in {**_OPERATORS, **_METHODS}.items():
    setattr(DevArrayBox, _name, _fn)
    setattr(DevArray, _name, _fn)  # plain device arrays take the same operators and methods (nothing to trace)

# unboxed values index through the same function (a plain call: nothing to trace)
DevArray.__getitem__ = lambda self, idx: anp.take(self, idx)
DevArray.__hash__ = object.__hash__
DevArrayBox.__hash__ = lambda self: id(self)

DevArrayBox.register(DevArray)
DevArrayBox.register(LazyDevArray)
DevArrayBox.register(PendingProduct)
DevArrayBox.register(LseCotangent)
DevArrayBox.register(FusedResult)
DevArrayBox.register(ExprArray)
DevArrayBox.register(PendingReduce)
DevArrayBox.register(float)


def _box_host_value(value, trace, node):
    """A host ``ndarray`` or NumPy scalar handed to a differential operator (``grad(f)(numpy_array)``, as callers such
    as ``scipy.optimize.minimize`` do) is uploaded once where it enters the trace; everything downstream, the
    gradient included, is a device array."""
    from .devarray import from_numpy

    import numpy as onp

    return DevArrayBox(from_numpy(onp.asarray(value)), trace, node)


def _register_host_values():
    from .. import _host

    if _host.HOST:
        return  # the hosting package boxes host arrays itself, as host arrays
    import numpy as onp

    for host_type in (onp.ndarray, onp.float64, onp.float32):
        # (only where nothing else has claimed host arrays as a value type of its own: a CPU array library
        # registered on this tracer, before or after this import, keeps them)
        Box.type_mappings.setdefault(host_type, _box_host_value)


_register_host_values()
