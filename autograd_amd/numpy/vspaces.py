"""``DevArrayVSpace``: the vector space of device arrays.

Counterpart of the reference's ArrayVSpace (autograd/numpy/numpy_vspaces.py:7-37).  The
accumulation hooks used by ``add_outgrads`` (autograd/core.py:185-205) launch kernels:
``_add`` allocates a fresh buffer, ``_mut_add`` updates the (always freshly allocated,
never aliased) accumulator in place.
"""

import numpy as onp

from .. import _lib
from .._lib import Op, Red
from ..extend import VSpace
from . import devarray as D
from . import fusion as _fusion
from .devarray import DevArray, LazyDevArray


_ZEROS = {}


def _shared_zero(dtype):
    z = _ZEROS.get(dtype)
    if z is None:
        z = _ZEROS[dtype] = D.zeros((), dtype)
        D.KNOWN_SCALARS[z._t.data_ptr()] = 0.0
    return z


_ONES = {}


def _shared_one(dtype):
    o = _ONES.get(dtype)
    if o is None:
        o = _ONES[dtype] = D.ones((), dtype)
        D.KNOWN_SCALARS[o._t.data_ptr()] = 1.0
    return o


_SEED_VIEWS = {}


def _seed_view(one, shape, dtype):
    """The shared zero (or one) seen through ``shape``: a stride-0 view that nothing ever writes, so the view itself
    is shared too (making one costs a few microseconds of a gradient evaluation that makes several)."""
    key = (one, shape, dtype)
    t = _SEED_VIEWS.get(key)
    if t is None:
        if len(_SEED_VIEWS) >= 1024:
            _SEED_VIEWS.clear()
        t = _SEED_VIEWS[key] = (_shared_one(dtype) if one else _shared_zero(dtype))._t.expand(shape)
    return t


def is_broadcast_view(x):
    """True when some axis of extent > 1 has stride 0: several indices share one element."""
    t = x._h()
    if t.numel() <= 1:
        return False
    for extent, stride in zip(t.shape, t.stride()):
        if stride == 0 and extent > 1:
            return True
    return False


def is_shared_zero(x):
    if type(x) is not DevArray:
        return False
    z = _ZEROS.get(x.dtype)
    return z is not None and x._t.data_ptr() == z._t.data_ptr()


class DevArrayVSpace(VSpace):
    def __init__(self, value):
        if isinstance(value, DevArray):
            self.shape = value.shape
            self.dtype = value.dtype
        else:
            value = onp.asarray(value)
            self.shape = value.shape
            self.dtype = value.dtype

    @property
    def size(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def ndim(self):
        return len(self.shape)

    def zeros(self):
        """A zero cotangent.  Accumulators start from it (core.py:212-215, 238-241 of the
        reference: ``vs.zeros()`` then ``+=``), so it is returned as a stride-0 view of one shared
        zero: creating it writes nothing, and the first ``x_prev + x_new`` reads it from a
        register instead of streaming a zero-filled buffer.  It is never written in place:
        ``_mut_add`` and the scatter rule allocate the real buffer when they meet it."""
        if self.size == 0:
            return D.zeros(self.shape, self.dtype)
        return DevArray(_seed_view(0, self.shape, self.dtype), self.dtype)

    def ones(self):
        """The seed cotangent of ``elementwise_grad`` (differential_operators.py:41-49 of the reference
        seeds ``vs.ones()``): like ``zeros``, a stride-0 view of one shared element, so seeding a
        backward pass writes nothing and the first rule reads the seed from a register."""
        if self.size == 0:
            return D.ones(self.shape, self.dtype)
        return DevArray(_seed_view(1, self.shape, self.dtype), self.dtype)

    def standard_basis(self):
        for idxs in onp.ndindex(*self.shape):
            vect = D.zeros(self.shape, self.dtype)
            cell = vect._t[idxs] if idxs else vect._t
            _lib.fill(_lib.DTYPE_CODE[self.dtype], cell, 1.0)  # a single element is always contiguous
            yield vect

    def stacked_standard_basis(self):
        """All ``size`` standard basis vectors stacked along a new leading axis: an identity matrix viewed
        as ``(size,) + shape`` (one launch instead of ``size`` fills)."""
        from . import wrapper as anp

        eye = anp.eye(self.size, dtype=self.dtype)
        return eye._view(lambda t: t.reshape((self.size,) + tuple(self.shape)))

    def randn(self):
        # host RNG (numpy.random, as the reference) so seeded tests see the same draws
        return D.from_numpy(onp.array(onp.random.randn(*self.shape)).astype(self.dtype))

    def _add(self, x, y):
        if type(x) is D.PendingProduct and type(y) is D.PendingProduct and not x.computed() and not y.computed() \
                and x.dtype == y.dtype and x.shape == y.shape:
            acc = x.sum_started()  # two matrix cotangents whose contractions have not run: a sum of products (neither is touched)
            acc.add_product(y)
            return acc
        return D.map_op(Op.ADD, D._float_dtype(D.result_dtype(x, y)), x, y)

    def _mut_add(self, x, y):
        """``x += y`` for an accumulator ``x`` (reference core.py:262-264).

        ``zeros() + y`` is ``y``: instead of streaming ``y`` through an add with zero, the
        accumulator borrows ``y``'s memory and is marked ``_borrowed``; the next contribution
        then goes out of place (same traffic as an in-place add), so the borrowed array - which
        may also be a tape value or another node's cotangent - is never written."""
        if not isinstance(x, DevArray):
            return self._add(x, y)
        if type(y) is D.PendingProduct and not y.computed() and y.dtype == x.dtype and y.shape == x.shape:
            # a matrix cotangent whose contraction has not run yet: run it into the accumulator
            if is_shared_zero(x):
                return y.sum_started()  # 0 + G: the accumulator collects the products and contracts once, when read
            if type(x) is D.PendingProduct and not x.computed() and x._more is not None:
                x.add_product(y)
                return x
            if type(x) is DevArray and not x._borrowed and not is_broadcast_view(x) and x._t.is_contiguous():
                y.add_into(x._t)
                return x
        if is_shared_zero(x):
            if isinstance(y, DevArray) and y.shape == x.shape and y.dtype == x.dtype:
                acc = D.alias(y)
                acc._borrowed = True
                return acc
            res = self._add(x, y)  # the shared zero is never written
            return D.astype(res, x.dtype) if isinstance(res, DevArray) and res.dtype != x.dtype else res
        if isinstance(y, DevArray) and y.dtype != x.dtype and D.result_dtype(x, y) != x.dtype:
            # numpy.add(x, y, out=x) of the reference (numpy_vspaces.py:33-34 through core.py:262-264)
            # adds in the promoted dtype and stores in x's: a float64 cotangent accumulated into a
            # float32 leaf comes out float32
            return D.astype(self._add(x, y), x.dtype)
        if x._borrowed or type(x) is not DevArray or is_broadcast_view(x) or _fusion.pending(y):
            return self._add(x, y)  # (a pending addend: the sum joins its expression instead of forcing it into memory first)
        if isinstance(y, DevArray) and y.shape != x.shape and D.broadcast_shapes(x.shape, y.shape) != x.shape:
            return self._add(x, y)
        return D.map_op(Op.ADD, x.dtype, x, y, out=x)

    def _scalar_mul(self, x, a):
        return D.arith_map(Op.MUL, x, a)

    def _inner_prod(self, x, y):
        x, y = D.asarray(x), D.asarray(y)
        dt = D._float_dtype(D.result_dtype(x, y))
        return D.map_reduce(Op.MUL, Red.SUM, dt, (x, y), tuple(range(max(x.ndim, y.ndim))), False)


DevArrayVSpace.register(DevArray)
DevArrayVSpace.register(LazyDevArray)
DevArrayVSpace.register(D.PendingProduct)
DevArrayVSpace.register(D.LseCotangent)
DevArrayVSpace.register(D.FusedResult)
DevArrayVSpace.register(_fusion.ExprArray)
DevArrayVSpace.register(D.PendingReduce)
DevArrayVSpace.register(float)


def _register_host_values():
    from .. import _host

    if not _host.HOST:  # (under a hosting package host arrays keep that package's vector space)
        for host_type in (onp.ndarray, onp.float64, onp.float32):
            VSpace.mappings.setdefault(host_type, DevArrayVSpace)  # (unless another array library on this tracer owns them)


_register_host_values()
