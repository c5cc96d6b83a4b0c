"""``DevArray``: the device-resident array value type, and the raw (untraced) operations on it.

A ``DevArray`` is an immutable n-d array in MI355X HBM.  It is a thin wrapper around a
``torch.Tensor`` used only as a memory handle: shape, strides and offset are the tensor's
view metadata (slicing, reshaping, transposing and broadcasting are views and launch
nothing), and every arithmetic operation launches a kernel of ``libagmi.so`` on torch's
current stream.  It plays the role ``numpy.ndarray`` plays for the reference
(autograd/numpy/numpy_boxes.py:12-189 boxes ndarrays; ``DevArrayBox`` boxes these).

dtype promotion follows NumPy 2 (NEP 50): Python scalars are weak, arrays and NumPy
scalars are strong.
"""

import math
import numbers
import weakref

import numpy as onp
import torch

from .. import _lib
from .._lib import Op, Red

_FLOATS = (onp.dtype("float32"), onp.dtype("float64"))
_F64 = onp.dtype("float64")
_BOOL = onp.dtype("bool")
_I64 = onp.dtype("int64")


ITEM_WRITES = 0  # counts item assignments (``x[idx] = v``): what caches an array by identity checks before trusting its contents


class DevArray:
    """n-d array in GPU memory; arithmetic is hand-written HIP kernels."""

    __slots__ = ("_t", "dtype", "_borrowed", "_shape_tuple")
    __array_priority__ = 200.0

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        """A NumPy ufunc applied to a device array (``numpy.abs(x)``, ``host_array * x``, ``numpy.float64(2) * x``)
        runs the namespace's function of the same name on the device; anything else (``out=``, ``.reduce`` ...)
        is declined, which NumPy reports as a TypeError."""
        if method != "__call__" or kwargs:
            return NotImplemented
        from . import wrapper

        fn = getattr(wrapper, ufunc.__name__, None)
        return NotImplemented if fn is None else fn(*inputs)

    def __init__(self, tensor, dtype=None):
        self._t = tensor
        self.dtype = dtype if dtype is not None else _lib.NUMPY_DTYPE[tensor.dtype]
        # True on an array whose memory another value reads: an accumulator initialised from a cotangent (0 + g kept
        # as g), or the operand of arithmetic that is still pending.  In-place accumulation and item assignment
        # then go to fresh memory instead
        self._borrowed = False
        self._shape_tuple = None  # filled by the first `shape` (asked many times per launch; arrays never change)

    # ---- metadata ----------------------------------------------------------------------
    @property
    def shape(self):
        s = self._shape_tuple
        if s is None:
            s = self._shape_tuple = tuple(self._t.shape)
        return s

    @property
    def ndim(self):
        return self._t.dim()

    @property
    def size(self):
        return self._t.numel()

    @property
    def strides(self):
        item = self.dtype.itemsize
        return tuple(s * item for s in self._t.stride())

    @property
    def T(self):
        from . import wrapper

        return wrapper.transpose(self)

    def __len__(self):
        if self._t.dim() == 0:
            raise TypeError("len() of unsized object")
        return self._t.shape[0]

    def __iter__(self):
        if self._t.dim() == 0:
            raise TypeError("iteration over a 0-d array")
        return (self[i] for i in range(self._t.shape[0]))

    # ---- host transfer (synchronises) ------------------------------------------------------
    def numpy(self):
        """Copy to a host ``numpy.ndarray`` (blocks until the stream has produced the data)."""
        _lib.check_not_capturing("DevArray.numpy()")
        return self._t.cpu().numpy()

    def __array__(self, dtype=None, copy=None):
        a = self.numpy()
        return a.astype(dtype) if dtype is not None else a

    def item(self):
        if self._t.numel() != 1:
            raise ValueError("can only convert an array of size 1 to a Python scalar")
        _lib.check_not_capturing("DevArray.item()")
        return self._t.item()

    def __float__(self):
        return float(self.item())

    def __int__(self):
        return int(self.item())

    def __index__(self):
        if self.dtype.kind not in "iu" or self._t.numel() != 1:
            raise TypeError("only integer scalar arrays can be converted to a scalar index")
        return int(self.item())

    def __bool__(self):
        if self._t.numel() != 1:
            raise ValueError("The truth value of an array with more than one element is ambiguous.")
        return bool(self.item())

    def __repr__(self):
        return f"DevArray({self.numpy()!r}, device='{self._t.device}')"

    __str__ = __repr__
    __hash__ = object.__hash__

    def __setitem__(self, idx, value):
        from . import wrapper

        wrapper.assign_items(self, idx, value)

    # ---- view helpers ---------------------------------------------------------------------
    def _h(self):
        """The tensor that carries shape, strides and storage (metadata only: never its values)."""
        return self._t

    def _view(self, fn):
        """``fn`` (a view operation on a tensor: slicing, reshaping, permuting ...) applied to this array."""
        return DevArray(fn(self._t), self.dtype)

    def _settled(self):
        """This array with no arithmetic pending (see ``core.settle``)."""
        return self

    # ---- operators and methods are attached by wrapper.py (they are traced primitives) ------


class LazyDevArray(DevArray):
    """``raw * scale * ascale + shift`` not yet written to memory.

    Negation, arithmetic with a Python scalar, and products / sums with a BROADCAST array operand
    (``A * b[None, :] + c[:, None]``, a bias added to a matrix product) return one of these instead
    of launching a kernel (see ``_fold``); the next kernel that reads it applies the steps on load,
    each one rounded on its own, so the value is bit-for-bit what the eager passes would have
    stored.  ``scale`` is a Python float; ``ascale`` is None or a tensor of ``raw``'s shape (a
    stride-0 view of the broadcast operand); ``shift`` is None, a Python float or such a tensor.
    Code that is unaware of all this reads ``_t`` as on any ``DevArray``: the first such read writes
    the value to a fresh buffer (one copy kernel) and keeps it.
    """

    __slots__ = ("_raw", "_scale", "_shift", "_ascale", "_producer", "_view_of_pending")

    def __init__(self, raw, dtype, scale, shift, ascale=None, producer=None):
        self._raw = raw
        # the matrix product whose (still empty) result buffer `raw` is, while that product has not run: whatever
        # first needs this value runs it, possibly together with the pending steps (a dense layer's bias and
        # activation go into the contraction's epilogue, see `fusion._dense_layer`)
        self._producer = producer
        self._view_of_pending = False  # True on a view taken of an array whose arithmetic was still pending
        self.dtype = dtype
        self._borrowed = False
        self._scale = scale    # Python float, representable in dtype; 1.0 = no multiply
        self._ascale = ascale  # tensor shaped like raw, or None
        self._shift = shift    # Python float or tensor shaped like raw; None = no add (x + 0.0 is not x for -0.0)
        self._shape_tuple = None

    def __getattr__(self, name):
        # only reached when a slot is unset: `_t` before the value has been written out
        if name != "_t":
            raise AttributeError(name)
        raw = self._raw
        out = _lib.empty(tuple(raw.shape), self.dtype)
        _lib.elementwise(Op.COPY, _lib.DTYPE_CODE[self.dtype], tuple(raw.shape), (out,), (self._affine(),))
        self._t = out
        # from here on the value lives in `out`: later readers take it from there (an identity map)
        self._raw, self._scale, self._shift, self._ascale = out, 1.0, None, None
        return out

    def _affine(self):
        if self._producer is not None:
            self._produce()
        return _lib.Affine(self._raw, self._scale, self._shift, self._ascale)

    def _produce(self):
        """Fill the storage (the matrix product it waits for runs now)."""
        product, self._producer = self._producer, None
        product._t

    @property
    def shape(self):
        s = self._shape_tuple
        if s is None:
            s = self._shape_tuple = tuple(self._raw.shape)
        return s

    @property
    def ndim(self):
        return self._raw.dim()

    @property
    def size(self):
        return self._raw.numel()

    @property
    def strides(self):
        item = self.dtype.itemsize
        return tuple(s * item for s in self._raw.stride())

    def __len__(self):
        if self._raw.dim() == 0:
            raise TypeError("len() of unsized object")
        return self._raw.shape[0]

    def __iter__(self):
        if self._raw.dim() == 0:
            raise TypeError("iteration over a 0-d array")
        return (self[i] for i in range(self._raw.shape[0]))

    def _h(self):
        return self._raw

    def _settled(self):
        return DevArray(self._t, self.dtype)

    def _view(self, fn):
        """The same view operation on the storage and on the array-valued steps (they have the
        storage's shape); when one of them cannot be viewed that way the value is written out."""
        asc, sh = self._ascale, self._shift
        if sh is None and asc is None and self._scale == 1.0:
            if self._producer is not None:
                self._produce()
            return DevArray(fn(self._raw), self.dtype)  # nothing pending (the value has been written out): a plain view
        try:
            view = LazyDevArray(fn(self._raw), self.dtype, self._scale,
                                fn(sh) if isinstance(sh, torch.Tensor) else sh,
                                fn(asc) if asc is not None else None, self._producer)
            view._view_of_pending = True
            return view
        except RuntimeError:
            return DevArray(fn(self._t), self.dtype)


class PendingProduct(DevArray):
    """The matrix product ``left @ right`` of two 2-d tensors, not yet computed.

    The cotangent rules of ``dot`` return one of these for matrix operands.  A cotangent usually
    ends up added to an accumulator (the weight matrix of a recurrent net receives one per time
    step); ``DevArrayVSpace._mut_add`` then runs the contraction with beta = 1 straight into the
    accumulator (``add_into``) instead of writing a temporary that an add kernel reads back.  The
    sum is the same to the bit: the kernel's epilogue adds C to the very accumulators it would
    otherwise have stored.  Anything else that touches the value reads ``_t`` as on any
    ``DevArray``; the first such read computes the product and keeps it.
    """

    __slots__ = ("_left", "_right", "_shape", "_out", "_more", "__weakref__")

    def __init__(self, left, right, dtype):
        self._left, self._right = left, right
        self._shape = (left.shape[0], right.shape[1])
        self.dtype = dtype
        self._borrowed = False
        self._out = None
        self._more = None  # further (left, right) pairs whose products are added to this one (see `sum_started`)

    def __getattr__(self, name):
        # only reached when a slot is unset: `_t` before the product has been computed
        if name != "_t":
            raise AttributeError(name)
        if self._more:
            out = self._sum_of_products()
        elif self._out is None:
            out = gemm2d(self._left, self._right, self.dtype)
        else:
            out = gemm2d(self._left, self._right, self.dtype, out=self._out)
        self._t = out
        self._left = self._right = self._out = self._more = None
        return out

    def sum_started(self):
        """A new pending value that starts a sum of products with this one: the accumulator of a matrix cotangent.

        A weight matrix used at every step of a recurrence receives one product per step, ``cat_t.T @ G_t``
        (numpy_vjps.py:615-638 through core.py:185-205).  Run one by one they are as many small contractions as
        there are steps, each a launch whose duration is mostly latency; the sum of all of them is ONE
        contraction over the stacked operands, ``[cat_0; cat_1; ...].T @ [G_0; G_1; ...]``.  The accumulator
        therefore only collects the operand pairs (``add_product``) and contracts when its value is read."""
        acc = PendingProduct(self._left, self._right, self.dtype)
        acc._more = list(self._more) if self._more else []
        return acc

    def add_product(self, other):
        """``self += other`` for two pending products of one shape (``self`` came from ``sum_started``)."""
        self._more.append((other._left, other._right))
        if other._more:
            self._more.extend(other._more)

    def _sum_of_products(self):
        terms = [(self._left, self._right)] + self._more
        out = self._out if self._out is not None else _lib.empty(self._shape, self.dtype)
        M, N = self._shape
        # The stacked form: every left factor the transpose of a row-major (K_i, M) matrix, every right factor a
        # row-major (K_i, N) matrix (the weight cotangents of `dot`), at least four of them.
        stackable = len(terms) >= 4 and M and N and all(
            l.stride(0) == 1 and l.stride(1) == M and r.is_contiguous() and l.shape[1] for l, r in terms)
        if not stackable:
            gemm2d(terms[0][0], terms[0][1], self.dtype, out=out)
            for l, r in terms[1:]:
                gemm2d(l, r, self.dtype, out=out, beta=1.0)
            return out
        total = sum(l.shape[1] for l, _ in terms)
        lefts, rights = _lib.empty((total, M), self.dtype), _lib.empty((total, N), self.dtype)
        code = _lib.DTYPE_CODE[self.dtype]
        for k in range(0, len(terms), _lib.MAX_CONCAT):
            group = terms[k:k + _lib.MAX_CONCAT]
            begin = sum(l.shape[1] for l, _ in terms[:k])
            rows = sum(l.shape[1] for l, _ in group)
            _lib.concat(code, 1, M, [(l, l.shape[1], 0, M, 1) for l, _ in group], lefts[begin:begin + rows])
            _lib.concat(code, 1, N, [(r, r.shape[0], 0, N, 1) for _, r in group], rights[begin:begin + rows])
        return gemm2d(lefts.t(), rights, self.dtype, out=out)

    def _buffer(self):
        """The memory the product will be written to (allocated now, filled when the product runs)."""
        if self._left is None:
            return self._t
        out = self._out
        if out is None:
            out = self._out = _lib.empty(self._shape, self.dtype)
        return out

    def _h(self):
        return self._buffer()

    def with_activation(self, bias, act_out):
        """Run the product with ``act_out = tanh(product + bias)`` formed in the contraction's epilogue; False when the
        fused kernel does not take these operands (nothing has run then)."""
        if not self._shape[0] or not self._shape[1] or not self._left.shape[1] or self._more:
            return False
        out = self._buffer()
        code = _lib.DTYPE_CODE[self.dtype]
        # Another forward product that has not run (the output head of the step before, which reads the state this
        # layer reads): it waits for nothing this layer produces, so its tiles ride in this launch instead of
        # being a link of their own in the chain of launches.  Refused unless both are the kernel's: nothing has run.
        mate = _forward_mate(self)
        if mate is not None:
            mate_out = mate._buffer()
            if _lib.gemm_fused(code, self._left, self._right, out, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=act_out,
                               beside=(mate._left, mate._right, mate_out)):
                mate._t = mate_out
                mate._left = mate._right = mate._out = mate._more = None
                self._t = out
                self._left = self._right = self._out = None
                return True
        if not _lib.gemm_fused(code, self._left, self._right, out, _lib.EPILOGUE_BIAS_TANH, bias=bias, out=act_out):
            return False
        self._t = out
        self._left = self._right = self._out = None
        return True

    def into_tanh_cotangent(self, x, bias, out):
        """``out = (left @ right) / cosh(x + bias)**2`` in one launch (the product itself stays uncomputed); False when
        the fused kernel does not take these operands."""
        if not self._shape[0] or not self._shape[1] or not self._left.shape[1]:
            return False
        code = _lib.DTYPE_CODE[self.dtype]
        if not self._more:
            return _lib.gemm_fused(code, self._left, self._right, out, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x)
        # A sum of products (the state of a recurrent net receives one cotangent from the next step and one from the
        # output head): all but the last are contracted into `out`, the last one adds what `out` holds to its
        # accumulators (beta = 1) before the tanh rule is applied to them.
        if len(self._more) > 3 or x.data_ptr() == out.data_ptr():
            return False
        terms = [(self._left, self._right)] + self._more
        last_left, last_right = terms[-1]
        M, N = self._shape
        K = last_left.shape[1]
        # (checked before anything runs, so that a refusal leaves nothing half done: the fused kernel wants a unit stride
        # in each operand, spans below 2 GiB, and no cut of a very long K across blocks when it also reads C)
        if not K or (last_left.stride(0) != 1 and last_left.stride(1) != 1) or (last_right.stride(0) != 1 and last_right.stride(1) != 1) \
                or max(last_left.numel(), last_right.numel(), M * N) >= 1 << 28 or last_left.stride(0) < 0 or last_left.stride(1) < 0 \
                or last_right.stride(0) < 0 or last_right.stride(1) < 0 or (K > 4096 and -(-M // 64) * -(-N // 64) < 128):
            return False
        if len(terms) == 2:
            # two products of one shape: one launch when each would be cut over the waves of a block (the kernel then
            # gives the two launches' bits); refused for anything else, and nothing has run
            first_left, first_right = terms[0]
            if first_left.shape[1] and _lib.gemm_fused(code, first_left, first_right, out, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x,
                                                       second=(last_left, last_right)):
                return True
        for k, (l, r) in enumerate(terms[:-1]):
            gemm2d(l, r, self.dtype, out=out, beta=1.0 if k else 0.0)
        if not _lib.gemm_fused(code, last_left, last_right, out, _lib.EPILOGUE_TANH_VJP, bias=bias, x=x, beta=1.0):
            raise RuntimeError("the fused contraction refused operands that were checked against its limits")
        return True

    def computed(self):
        return self._left is None

    def fresh(self):
        """The product in a buffer of the caller's own (nothing is kept here)."""
        if self._more:
            kept, self._out = self._out, None
            out = self._sum_of_products()
            self._out = kept
            return DevArray(out, self.dtype)
        return DevArray(gemm2d(self._left, self._right, self.dtype), self.dtype)

    def add_into(self, acc):
        """``acc += left @ right`` for a contiguous tensor ``acc`` of this shape and dtype."""
        gemm2d(self._left, self._right, self.dtype, out=acc, beta=1.0)
        for l, r in self._more or ():
            gemm2d(l, r, self.dtype, out=acc, beta=1.0)

    @property
    def shape(self):
        return self._shape

    @property
    def ndim(self):
        return 2

    @property
    def size(self):
        return self._shape[0] * self._shape[1]

    @property
    def strides(self):
        return (self._shape[1] * self.dtype.itemsize, self.dtype.itemsize)

    def __len__(self):
        return self._shape[0]

    def __iter__(self):
        return (self[i] for i in range(self._shape[0]))

    def _settled(self):
        return DevArray(self._t, self.dtype)


# the last few products that `dot` left pending (weakly held): candidates to ride in another layer's launch
_FORWARD_PRODUCTS = []


def note_forward_product(product):
    """Remember a forward matrix product that has not run (see ``PendingProduct.with_activation``)."""
    if len(_FORWARD_PRODUCTS) >= 3:
        del _FORWARD_PRODUCTS[0]
    _FORWARD_PRODUCTS.append((weakref.ref(product), _lib.CAPTURING))
    return product


def _forward_mate(product):
    for k in range(len(_FORWARD_PRODUCTS) - 1, -1, -1):
        ref, while_recording = _FORWARD_PRODUCTS[k]
        other = ref()
        if other is None or other.computed():
            del _FORWARD_PRODUCTS[k]
            continue
        # (a product from outside a graph that is being recorded is not taken into it: the recorded launch runs at the
        # replays, and whoever reads the product outside would find a buffer that nothing has written yet)
        if other is not product and while_recording == _lib.CAPTURING and not other._more and other.dtype == product.dtype \
                and other._shape[0] and other._shape[1] and other._left.shape[1]:
            del _FORWARD_PRODUCTS[k]
            return other
    return None


class LseCotangent(DevArray):
    """``g * exp(x - ans)`` for ``ans = logsumexp(x, axis=1)`` of a matrix ``x``: the cotangent of ``x``, not yet written.

    The rules that run next on the tape usually need this matrix only to reduce or rescale it: its row
    sums (an offset that was broadcast along the rows), its product with a factor that was broadcast
    down the columns, the column sums of its product with the matrix the factor multiplied.  Each such
    consumer (``row_sums`` / ``scaled_by`` / ``col_sums_with``) gets a :class:`FusedResult`, whose memory
    exists but whose values do not yet; the first time any of them is read, ONE kernel
    (``agmi_lse_cotangent_fused``) walks ``x``'s storage once and produces all of them, and this
    matrix itself never reaches memory.  Anything else reads ``_t`` as on any ``DevArray`` and gets it
    written out by the elementwise rule kernel.
    """

    __slots__ = ("_g", "_x", "_ans", "_shape", "_wanted")

    def __init__(self, g_k, x, ans_k, dtype):
        self._g, self._x, self._ans = g_k, x, ans_k
        self._shape = x.shape
        self.dtype = dtype
        self._borrowed = False
        self._wanted = {}  # kind -> (operand tensor or None, output tensor)

    def __getattr__(self, name):
        if name != "_t":
            raise AttributeError(name)
        self.run()
        self._t = out = map_op(Op.LSE_VJP, self.dtype, self._g, 1.0, self._x, self._ans)._t
        return out

    @staticmethod
    def eligible(g_k, x, ans_k, dtype):
        """The layouts the fused kernel covers: a row-major matrix (its pending map, if any, made of
        row or column vectors) reduced along its rows; everything in one floating dtype."""
        if dtype not in _FLOATS or x.dtype != dtype or x.ndim != 2 or type(x) not in (DevArray, LazyDevArray):
            return False
        h = x._h()
        vec = 16 // dtype.itemsize
        if h.shape[0] == 0 or h.shape[1] == 0 or h.shape[1] % vec or h.stride(1) != 1:
            return False
        if type(x) is LazyDevArray:
            for aux in (x._ascale, x._shift):
                if isinstance(aux, torch.Tensor) and not (aux.stride(1) == 0 or (aux.stride(1) == 1 and aux.stride(0) == 0)):
                    return False
        for v in (g_k, ans_k):
            if type(v) is not DevArray or v.dtype != dtype or v.shape != (h.shape[0], 1):
                return False
        return True

    def computed(self):
        return _has_value(self)

    # ---- consumers ----------------------------------------------------------------------
    def _request(self, kind, operand, out_shape):
        if kind in self._wanted:
            held, out = self._wanted[kind]
            if held is operand or (held is not None and operand is not None and held.data_ptr() == operand.data_ptr()
                                   and held.stride() == operand.stride()):
                return FusedResult(self, out)
            self.run()  # a second consumer of the same kind with another operand: a pass of its own
        out = _lib.empty(out_shape, self.dtype)
        self._wanted[kind] = (operand, out)
        return FusedResult(self, out)

    def row_sums(self):
        """``sum(self, axis=1, keepdims=True)``"""
        return self._request("row_sums", None, (self._shape[0], 1))

    def scaled_by(self, factor):
        """``factor * self`` for a tensor ``factor`` broadcast down the columns (strides (0, 1)); None when it is not."""
        if factor.dim() != 2 or factor.shape[1] != self._shape[1] or factor.stride(0) != 0 or factor.stride(1) != 1:
            return None
        return self._request("scaled", factor, self._shape)

    def col_sums_with(self, other):
        """``sum(other * self, axis=0, keepdims=True)`` when ``other`` is the very storage ``x`` is a map of; else None."""
        h = self._x._h()
        if (type(other) is not DevArray or other.dtype != self.dtype or other._t.data_ptr() != h.data_ptr()
                or other._t.shape != h.shape or other._t.stride() != h.stride()):
            return None
        return self._request("col_sums", None, (1, self._shape[1]))

    def run(self):
        """Produce every result asked for so far (one pass over ``x``'s storage)."""
        wanted, self._wanted = self._wanted, {}
        if not wanted:
            return
        x = self._x
        operand = x._affine() if type(x) is LazyDevArray else x._t
        rs = wanted.get("row_sums")
        sc = wanted.get("scaled")
        cs = wanted.get("col_sums")
        ok = _lib.lse_cotangent(_lib.DTYPE_CODE[self.dtype], operand, self._ans._t, self._g._t,
                                row_sums=rs[1] if rs else None, col_factor=sc[0] if sc else None,
                                scaled=sc[1] if sc else None, col_sums=cs[1] if cs else None)
        if ok:
            return
        # a layout the fused kernel does not take after all: write the matrix out, then the plain kernels
        full = DevArray(self._t, self.dtype)
        if rs:
            map_reduce_into(Op.COPY, rs[1], (full,), (1,))
        if sc:
            map_op(Op.MUL, self.dtype, DevArray(sc[0], self.dtype), full, out=DevArray(sc[1], self.dtype))
        if cs:
            map_reduce_into(Op.MUL, cs[1], (DevArray(self._x._h(), self.dtype), full), (0,))

    @property
    def shape(self):
        return self._shape

    @property
    def ndim(self):
        return 2

    @property
    def size(self):
        return self._shape[0] * self._shape[1]

    @property
    def strides(self):
        return (self._shape[1] * self.dtype.itemsize, self.dtype.itemsize)

    def __len__(self):
        return self._shape[0]

    def __iter__(self):
        return (self[i] for i in range(self._shape[0]))

    def _settled(self):
        return DevArray(self._t, self.dtype)


def _has_value(a):
    try:
        object.__getattribute__(a, "_t")
        return True
    except AttributeError:
        return False


class FusedResult(DevArray):
    """A result of :class:`LseCotangent`'s fused pass: its memory is allocated (so views, reshapes and
    shape queries work), its values arrive when anything first reads ``_t`` of any such result."""

    __slots__ = ("_source", "_out")

    def __init__(self, source, out):
        self._source, self._out = source, out
        self.dtype = source.dtype
        self._borrowed = False
        self._shape_tuple = None

    def __getattr__(self, name):
        if name != "_t":
            raise AttributeError(name)
        self._source.run()
        self._t = out = self._out
        self._source = None
        return out

    @property
    def shape(self):
        s = self._shape_tuple
        if s is None:
            s = self._shape_tuple = tuple(self._out.shape)
        return s

    @property
    def ndim(self):
        return self._out.dim()

    @property
    def size(self):
        return self._out.numel()

    @property
    def strides(self):
        item = self.dtype.itemsize
        return tuple(s * item for s in self._out.stride())

    def __len__(self):
        if self._out.dim() == 0:
            raise TypeError("len() of unsized object")
        return self._out.shape[0]

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def _h(self):
        return self._out

    def _settled(self):
        return DevArray(self._t, self.dtype)

    def _view(self, fn):
        if _has_value(self):
            return DevArray(fn(self._t), self.dtype)
        return FusedResult(self._source, fn(self._out))  # still waiting for the same pass


def map_reduce_into(op, out_t, xs, axes):
    """``sum over axes of op(xs...)`` written to the tensor ``out_t`` (kept-dims shape)."""
    dtype = _lib.NUMPY_DTYPE[out_t.dtype]
    ops = _limit_aux(tuple(_operand(x, dtype) for x in xs), dtype)
    shape = _bshape(ops)
    ops = tuple(_expand(t, shape) for t in ops)
    mask = [d in axes for d in range(len(shape))]
    if not _lib.map_reduce(op, Red.SUM, _lib.DTYPE_CODE[dtype], shape, mask, out_t, ops):
        raise _lib.AgmiError("map_reduce_into: unsupported layout")


def plain(x):
    """``x`` with any pending arithmetic written out (a no-op for everything else)."""
    return DevArray(x._t, x.dtype) if type(x) in _DEFERRED else x


_DEFERRED = (LazyDevArray, PendingProduct, LseCotangent, FusedResult)


def in_memory(x):
    """``x`` as a plain device array when its value already lies in memory (a deferred value that has been
    computed: no launch, no copy); ``x`` itself otherwise."""
    kind = type(x)
    if kind is DevArray or kind is LazyDevArray or kind not in _DEFERRED:
        return x
    return DevArray(x._t, x.dtype) if _has_value(x) else x


def alias(x):
    """A second handle on ``x``'s storage (and pending map)."""
    return x._view(lambda t: t)


def _is_pow2(c):
    """A power of two of modest size.  Multiplying by one is exact unless the product leaves the normal
    range, so merging it into a pending factor is bit-for-bit the eager result for every element whose
    eager intermediates stay normal; keeping the exponent within +-8 keeps a chain of merged factors from
    carrying values across the underflow or overflow threshold that the eager passes would have hit
    (``(x * 2**-60) * 2**60`` is two real passes, as in NumPy)."""
    return c != 0.0 and math.isfinite(c) and math.frexp(c)[0] in (0.5, -0.5) and 2.0**-8 <= abs(c) <= 2.0**8


def _representable(v, dtype):
    return math.isfinite(v) and (dtype == _F64 or float(onp.float32(v)) == v)


def _state(a):
    """(raw tensor, scalar scale, array scale, shift) of a device array."""
    if type(a) is LazyDevArray:
        if a._producer is not None:
            a._produce()
        return a._raw, a._scale, a._ascale, a._shift
    return a._t, 1.0, None, None


def _state_and_producer(a):
    """``_state`` without running a matrix product that has not run yet: its result buffer and the product."""
    if type(a) is LazyDevArray:
        return a._raw, a._scale, a._ascale, a._shift, a._producer
    if type(a) is PendingProduct and not a.computed():
        return a._buffer(), 1.0, None, None, a
    return a._t, 1.0, None, None, None


def _fold(op, dtype, xs):
    """``op(xs)`` as a pending map ``raw * scale * ascale + shift`` of its array operand, or None.

    Folded only when the kernel's fixed step order (scalar factor, array factor, offset), each step
    rounded on its own, gives bit-for-bit the value of the eager passes (for elements whose eager
    intermediates are neither subnormal nor overflowing; see ``_is_pow2``):
    * negation: always (it commutes with rounding), unless an array-valued offset is pending;
    * a Python-scalar factor: when it, or the pending scalar factor, is a power of two (that
      multiply is then exact) - and only a power of two once an array factor or an offset is pending;
    * a Python-scalar offset, or an array offset: when no offset is pending;
    * an array factor: when no array factor and no offset is pending.
    Scalars are Python floats/ints (weak in NumPy's promotion: converted to the array's dtype
    first).  An array operand qualifies when it is BROADCAST against the other one (strictly fewer
    elements, same dtype): the other operand's storage stays the `raw` of the result.
    """
    if op == Op.NEG:
        (a,) = xs
        c = None
        swapped = False
    elif len(xs) == 2:
        a, c = xs
        swapped = False
        if isinstance(c, DevArray) and isinstance(a, DevArray):
            if a._h().shape == c._h().shape:
                return None  # a true elementwise binary operation
            if c.size > a.size:
                a, c, swapped = c, a, True
            return _fold_array(op, dtype, a, c, swapped)
        if type(c) is not float and type(c) is not int:
            a, c, swapped = c, a, True
            if type(c) is not float and type(c) is not int:
                return None
    else:
        return None
    if not isinstance(a, DevArray) or a.dtype != dtype:
        return None
    raw, s, asc, t, producer = _state_and_producer(a)
    array_shift = isinstance(t, torch.Tensor)
    if c is not None:
        c = float(c) if dtype == _F64 else float(onp.float32(c))
    if op == Op.NEG:
        if array_shift:
            return None
        s, t = -s, (None if t is None else -t)
    elif op == Op.MUL or (op == Op.DIV and not swapped and _is_pow2(c)):
        if op == Op.DIV:
            c = 1.0 / c
        if t is None and asc is None:
            if not (_is_pow2(s) or _is_pow2(c)):  # one of the two multiplies is exact
                return None
            s = s * c
        elif _is_pow2(c) and not array_shift:
            s = s * c
            if t is not None:
                t2 = t * c
                if not _representable(t2, dtype) or (t2 == 0.0) != (t == 0.0):
                    return None
                t = t2
        else:
            return None
        if s != s or not (_representable(s, dtype) or math.isinf(s)):
            return None
    elif op == Op.ADD:
        if t is not None:
            return None
        t = c
    elif op == Op.SUB:
        if t is not None:
            return None
        if swapped:  # c - x = (-x) + c
            s, t = -s, c
        else:  # x - c = x + (-c)
            t = -c
    else:
        return None
    a._borrowed = True  # the result reads `a`'s memory when it is consumed: an item assignment into `a` must not reach it
    if s == 1.0 and t is None and asc is None and producer is None:
        return DevArray(raw, dtype)
    return LazyDevArray(raw, dtype, s, t, asc, producer)


def _fold_array(op, dtype, a, c, swapped):
    """``_fold`` for two array operands: ``c`` is broadcast against ``a`` (``swapped``: ``c`` was the
    left operand)."""
    if a.dtype != dtype or c.dtype != dtype or dtype not in _FLOATS:
        return None
    if c.size >= a.size or a.size == 0 or broadcast_shapes(a.shape, c.shape) != a.shape:
        return None
    raw, s, asc, t, producer = _state_and_producer(a)
    if t is not None:
        return None  # an offset is the last step
    if type(c) is LazyDevArray or c.ndim > a.ndim:
        c = plain(c)
    vec = c._t.expand(a.shape)
    if op == Op.MUL and asc is not None or op not in (Op.MUL, Op.ADD) and not (op == Op.SUB and swapped):
        return None
    a._borrowed = c._borrowed = True  # (both are read when the result is consumed; see `_fold`)
    if op == Op.MUL:
        return LazyDevArray(raw, dtype, s, None, vec, producer)
    if op == Op.ADD:
        return LazyDevArray(raw, dtype, s, vec, asc, producer)
    return LazyDevArray(raw, dtype, -s, vec, asc, producer)  # c - a = (-a) + c


_FOLDABLE = frozenset({Op.NEG, Op.MUL, Op.ADD, Op.SUB, Op.DIV})


def is_scalar(x):
    return type(x) is float or type(x) is int or (isinstance(x, (numbers.Number, onp.generic)) and not isinstance(x, DevArray))


# --------------------------------------------------------------------------------------------
# construction
# --------------------------------------------------------------------------------------------
def _np_dtype(dtype):
    return None if dtype is None else onp.dtype(dtype)


def from_numpy(a, dtype=None):
    """Upload a host array (one H2D copy; no arithmetic)."""
    a = onp.asarray(a, dtype=dtype)
    if a.dtype not in _lib.DTYPE_CODE:
        if a.dtype.kind == "f":
            a = a.astype(onp.float64 if a.dtype.itemsize > 4 else onp.float32)
        elif a.dtype.kind in "iu":
            a = a.astype(onp.int64)
        else:
            raise TypeError(f"dtype {a.dtype} is not supported on the device")
    if not a.flags.c_contiguous or not a.flags.writeable:
        a = onp.array(a, order="C")  # (ascontiguousarray would turn a 0-d array into 1-d)
    _lib.check_not_capturing("uploading a host array")
    t = torch.from_numpy(a).to(_lib.device())
    return DevArray(t, a.dtype)


def asarray(x, dtype=None):
    """Device array from a DevArray (no copy), host array, nested list or scalar."""
    dtype = _np_dtype(dtype)
    if isinstance(x, DevArray):
        return x if dtype is None or dtype == x.dtype else astype(x, dtype)
    if isinstance(x, (numbers.Number, onp.generic)):
        dt = dtype or (onp.asarray(x).dtype if isinstance(x, onp.generic) else (_F64 if not isinstance(x, (bool, int)) else onp.asarray(x).dtype))
        if dt in _FLOATS:
            return full((), float(x), dt)
        return from_numpy(onp.asarray(x), dt)
    if isinstance(x, (list, tuple)) and any(isinstance(e, DevArray) for e in x):
        from . import wrapper

        return wrapper.stack([asarray(e) for e in x])
    return from_numpy(x, dtype)


def to_numpy(x):
    if isinstance(x, DevArray):
        return x.numpy()
    return onp.asarray(x)


def empty(shape, dtype=_F64):
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
    dtype = onp.dtype(dtype)
    return DevArray(_lib.empty(shape, dtype), dtype)


def full(shape, fill_value, dtype=None):
    dtype = onp.dtype(dtype) if dtype is not None else onp.asarray(fill_value).dtype
    if dtype.kind == "i" and dtype not in _lib.DTYPE_CODE:
        dtype = _I64
    out = empty(shape, dtype)
    _lib.fill(_lib.DTYPE_CODE[dtype], out._t, fill_value)
    return out


def zeros(shape, dtype=_F64):
    return full(shape, 0.0, onp.dtype(dtype))


def ones(shape, dtype=_F64):
    return full(shape, 1.0, onp.dtype(dtype))


_CONSTANTS = {}
_CONSTANT_VIEWS = {}
KNOWN_SCALARS = {}  # data pointer of a one-element array that is never written -> its value (shared zeros / ones / constants)


def constant(shape, value, dtype):
    """An array of ``shape`` filled with ``value`` that costs no launch to make: a stride-0 view of one
    shared element, wrapped as a pending map (``LazyDevArray``) so that kernels read it through broadcast
    strides and only code that needs the memory itself (an in-place update, a contiguous operand) has
    it written out, once, on its first ``_t``.  Floating dtypes only; others get a real fill."""
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(int(s) for s in shape)
    dtype = onp.dtype(dtype)
    n = 1
    for extent in shape:
        n *= extent
    if dtype not in _FLOATS or n == 0 or not shape:
        return full(shape, value, dtype)
    key = (dtype, float(value))
    seen = _CONSTANT_VIEWS.get((key, shape))
    if seen is not None:
        return LazyDevArray(seen, dtype, 1.0, None)
    one = _CONSTANTS.get(key)
    if one is None:
        if len(_CONSTANTS) > 64:
            return full(shape, value, dtype)
        one = _CONSTANTS[key] = full((), float(value), dtype)._t
        KNOWN_SCALARS[one.data_ptr()] = float(value)
    if len(_CONSTANT_VIEWS) >= 1024:
        _CONSTANT_VIEWS.clear()
    # (the view of the shared element is shared as well: nothing ever writes through it, and a loop that makes the same
    # column of ones at every step saves the view's few microseconds each time)
    seen = _CONSTANT_VIEWS[(key, shape)] = one.expand(shape)
    return LazyDevArray(seen, dtype, 1.0, None)


# --------------------------------------------------------------------------------------------
# operand preparation
# --------------------------------------------------------------------------------------------
def result_dtype(*operands):
    """NumPy-2 result type of an operation on ``operands`` (Python scalars are weak)."""
    args = []
    first = None
    same = True
    for x in operands:
        if isinstance(x, DevArray):
            if first is None:
                first = x.dtype
            elif x.dtype != first:
                same = False
            args.append(x.dtype)
        elif isinstance(x, onp.ndarray):
            same = False
            args.append(x.dtype)
        elif isinstance(x, onp.generic):
            same = False
            args.append(x.dtype)
        elif isinstance(x, (bool, int, float)):
            args.append(x)
        else:
            same = False
            args.append(onp.asarray(x).dtype)
    if first is not None and same and first in _FLOATS:
        return first  # fast path: weak scalars never change a float array's dtype
    return onp.result_type(*args)


def _float_dtype(dt):
    """dtype a floating ufunc (exp, true_divide, ...) computes in for input dtype ``dt``."""
    if dt in _FLOATS:
        return dt
    if dt.kind == "f":
        return onp.dtype("float32") if dt.itemsize <= 4 else _F64
    return _F64


def astype(x, dtype):
    dtype = onp.dtype(dtype)
    if not isinstance(x, DevArray):
        return asarray(x, dtype)
    if dtype == x.dtype:
        return copy(x)
    if dtype not in _lib.DTYPE_CODE:
        raise TypeError(f"dtype {dtype} is not supported on the device")
    out = empty(x.shape, dtype)
    _lib.cast(_lib.DTYPE_CODE[x.dtype], _lib.DTYPE_CODE[dtype], x.shape, out._t, x._t)
    return out


def _operand(x, dtype):
    """tensor (of ``dtype``) or Python float for a kernel input slot."""
    if isinstance(x, DevArray):
        if x.dtype != dtype:
            x = astype(x, dtype)
        elif type(x) is LazyDevArray:
            return x._affine()
        return x._t
    if type(x) is float or type(x) is int or isinstance(x, (numbers.Number, onp.generic)):  # (exact types first: the ABC test is slow)
        return float(x)
    return asarray(x, dtype)._t


def broadcast_shapes(a, b):
    """NumPy broadcasting of two shape tuples (plain tuple arithmetic: this sits on the launch path)."""
    if a == b:
        return a
    if len(a) < len(b):
        a, b = b, a
    pad = len(a) - len(b)
    out = list(a)
    for i, sb in enumerate(b):
        sa = a[pad + i]
        if sa == sb or sb == 1:
            continue
        if sa == 1:
            out[pad + i] = sb
        else:
            raise ValueError(f"operands could not be broadcast together with shapes {a} {b}")
    return tuple(out)


def _bshape(operands):
    shape = None
    for t in operands:
        if type(t) is _lib.Affine:
            t = t.t
        if isinstance(t, torch.Tensor):
            s = tuple(t.shape)
            if shape is None:
                shape = s
            elif s != shape:
                shape = broadcast_shapes(shape, s)
    return shape


def _expand(t, shape):
    if isinstance(t, torch.Tensor):
        if tuple(t.shape) != shape:
            return t.expand(shape)
    elif type(t) is _lib.Affine and tuple(t.t.shape) != shape:
        sh, asc = t.shift, t.ascale
        return _lib.Affine(t.t.expand(shape), t.scale, sh.expand(shape) if isinstance(sh, torch.Tensor) else sh,
                           asc.expand(shape) if asc is not None else None)
    return t


def _n_aux(t):
    return (t.ascale is not None) + isinstance(t.shift, torch.Tensor)


def _limit_aux(ops, dtype):
    """A launch takes at most ``_lib.MAX_AUX`` array-valued steps: write out the operands that carry
    the most of them until the rest fits."""
    total = 0
    for t in ops:
        if type(t) is _lib.Affine:
            total += _n_aux(t)
    if total <= _lib.MAX_AUX:
        return ops
    ops = list(ops)
    while total > _lib.MAX_AUX:
        k = max(range(len(ops)), key=lambda i: _n_aux(ops[i]) if type(ops[i]) is _lib.Affine else 0)
        total -= _n_aux(ops[k])
        t = ops[k]
        ops[k] = LazyDevArray(t.t, dtype, t.scale, t.shift, t.ascale)._t
    return tuple(ops)


def _lift_scalars(operands, dtype):
    """All operands are by-value scalars: put the first on the device as a 0-d array."""
    return (full((), operands[0], dtype)._t,) + tuple(operands[1:])


_fusion = None  # the module that defers elementwise steps (``fusion.py`` sets it when it is imported)


def map_op(op, dtype, *xs, out=None, n_out=1):
    """Elementwise ``op`` on broadcast operands; returns DevArray (or a tuple).

    Negation and arithmetic with one Python scalar launch nothing when the result can be kept as
    a pending affine map of the operand (``_fold``); any other single-result step is returned as a
    pending expression node (``fusion.ExprArray``) that is evaluated, together with the steps that
    follow it, when something first needs its memory."""
    if out is None:
        fuse = n_out == 1 and _fusion is not None and _fusion.ENABLED
        if fuse:
            for x in xs:
                if (type(x) is _fusion.ExprArray and x._args is not None) or (type(x) is PendingReduce and x._call is not None):
                    # an operand that is itself pending (an expression, or a reduction of one: the value of a traced
                    # loss, which `grad` never reads): no map can be folded into it
                    node = _fusion.make(op, dtype, xs)
                    if node is not None:
                        return node
                    break
        if op in _FOLDABLE:
            folded = _fold(op, dtype, xs)
            if folded is not None:
                return folded
        if fuse:
            node = _fusion.make(op, dtype, xs)
            if node is not None:
                return node
    elif type(out) is not DevArray:
        raise TypeError("map_op: `out` must be a plain device array")
    ops = _limit_aux(tuple(_operand(x, dtype) for x in xs), dtype)
    shape = _bshape(ops)
    if shape is None:
        ops = _lift_scalars(ops, dtype)
        shape = ()
    if out is not None:
        shape = out.shape  # the operands are broadcast to the destination (they may all be smaller)
    ops = tuple(_expand(t, shape) for t in ops)
    code = _lib.DTYPE_CODE[dtype]
    if out is not None:
        _lib.elementwise(op, code, shape, (out._t,), ops)
        return out
    outs = tuple(_lib.empty(shape, dtype) for _ in range(n_out))
    _lib.elementwise(op, code, shape, outs, ops)
    if n_out == 1:
        return DevArray(outs[0], dtype)
    return tuple(DevArray(t, dtype) for t in outs)


def float_map(op, *xs):
    """Floating ufunc: compute in the promoted floating dtype."""
    return map_op(op, _float_dtype(result_dtype(*xs)), *xs)


def arith_map(op, *xs):
    """add/subtract/multiply/...: promoted dtype, computed in floating point.

    Integer and bool arrays are promoted to float64 (integer arithmetic has no kernels:
    the differentiable path is floating point)."""
    return map_op(op, _float_dtype(result_dtype(*xs)), *xs)


def copy(x):
    return map_op(Op.COPY, x.dtype, x) if x.dtype in _FLOATS else astype_copy(x)


def astype_copy(x):
    out = empty(x.shape, x.dtype)
    code = _lib.DTYPE_CODE[x.dtype]
    _lib.cast(code, code, x.shape, out._t, x._t)
    return out


def contiguous(x):
    x = plain(x) if type(x) is PendingProduct else in_memory(x)  # a computed product is contiguous already
    return x if type(x) is DevArray and x._t.is_contiguous() else copy(x)


def compare(cmp, a, b):
    dt = _float_dtype(result_dtype(a, b))
    ops = tuple(x.t if type(x) is _lib.Affine else x
                for x in (_operand(plain(a), dt), _operand(plain(b), dt)))  # the compare kernel applies no map
    shape = _bshape(ops)
    if shape is None:
        ops = _lift_scalars(ops, dt)
        shape = ()
    ops = tuple(_expand(t, shape) for t in ops)
    out = empty(shape, _BOOL)
    _lib.compare(cmp, _lib.DTYPE_CODE[dt], shape, out._t, ops)
    return out


# --------------------------------------------------------------------------------------------
# reductions
# --------------------------------------------------------------------------------------------
def normalize_axes(axis, ndim):
    if axis is None:
        return tuple(range(ndim))
    if type(axis) is int or isinstance(axis, (numbers.Integral, onp.integer)):
        axis = (int(axis),)
    axes = tuple(sorted({int(a) % ndim if ndim else 0 for a in axis}))
    for a in axis:
        if not -max(ndim, 1) <= int(a) < max(ndim, 1):
            raise onp.exceptions.AxisError(int(a), ndim)  # NumPy's own exception (a ValueError and an IndexError)
    return axes


def reduce_shape(shape, axes, keepdims):
    if keepdims:
        return tuple(1 if d in axes else s for d, s in enumerate(shape))
    return tuple(s for d, s in enumerate(shape) if d not in axes)


_IDENTITY = {Red.SUM: 0.0, Red.PROD: 1.0}


class PendingReduce(DevArray):
    """A reduction of pending elementwise expressions, not yet run: the forward value of a traced ``sum`` is often
    never read (``grad`` keeps the cotangents only), and running it would force its operand expression into memory
    first.  Reading ``_t`` runs it."""

    __slots__ = ("_call", "_shape")

    def __init__(self, call, shape, dtype):
        self._call, self._shape = call, shape
        self.dtype = dtype
        self._borrowed = False
        self._shape_tuple = shape

    def __getattr__(self, name):
        if name != "_t":
            raise AttributeError(name)
        self._t = out = _map_reduce_now(*self._call)._t
        self._call = None
        return out

    @property
    def shape(self):
        return self._shape

    @property
    def ndim(self):
        return len(self._shape)

    @property
    def size(self):
        n = 1
        for s in self._shape:
            n *= s
        return n

    @property
    def strides(self):
        return DevArray(self._t, self.dtype).strides

    def __len__(self):
        if not self._shape:
            raise TypeError("len() of unsized object")
        return self._shape[0]

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def _h(self):
        return self._t

    def _settled(self):
        return DevArray(self._t, self.dtype)

    def _view(self, fn):
        return DevArray(fn(self._t), self.dtype)


_DEFERRED = _DEFERRED + (PendingReduce,)


def _kept(x):
    """An operand as a deferred reduction keeps it: the array is marked as read by something pending (an item assignment
    then moves the ARRAY's handle to a buffer of its own) and the reduction holds a handle of its own on the memory as it
    is now."""
    if isinstance(x, DevArray):
        x._borrowed = True
        kind = type(x)
        if kind is DevArray:
            return DevArray(x._t, x.dtype)
        if kind is LazyDevArray:
            return LazyDevArray(x._raw, x.dtype, x._scale, x._shift, x._ascale, x._producer)
    return x


def map_reduce(op, red, dtype, xs, axes, keepdims, shape=None):
    """``RED_axes op(xs...)`` with ``xs`` broadcast to ``shape`` (default: their broadcast); left pending while an
    operand is a pending expression (see :class:`PendingReduce`)."""
    if _fusion is not None and _fusion.ENABLED:
        for x in xs:
            if type(x) is _fusion.ExprArray and x._args is not None:
                full = shape
                if full is None:
                    full = ()
                    for y in xs:
                        if isinstance(y, DevArray) and y.shape != full:
                            full = broadcast_shapes(full, y.shape)
                axes = tuple(axes)
                return PendingReduce((op, red, dtype, tuple([_kept(y) for y in xs]), axes, keepdims, shape),
                                     reduce_shape(full, axes, keepdims), dtype)
        if red == Red.SUM and op == Op.COPY and len(xs) == 1 and shape is None and isinstance(xs[0], DevArray):
            # The sum of a whole array, the last step of most losses: `grad` never reads its value (the cotangent of a sum
            # needs none of it), so it runs when something does (`value_and_grad`, a print, arithmetic on the scalar).
            x = xs[0]
            axes = tuple(axes)
            if len(axes) == x.ndim and x.size > 0:
                return PendingReduce((op, red, dtype, (_kept(x),), axes, keepdims, None), reduce_shape(x.shape, axes, keepdims), dtype)
    return _map_reduce_now(op, red, dtype, xs, axes, keepdims, shape)


def _map_reduce_now(op, red, dtype, xs, axes, keepdims, shape=None):
    if len(xs) == 1 and _fusion is not None and type(xs[0]) is _fusion.ExprArray and xs[0]._args is not None \
            and red == Red.SUM and (op == Op.COPY or op == Op.NEG) and xs[0].dtype == dtype:
        # The reduction of a pending `a * b` (or +, -, /) of arrays in memory: the reduction kernel forms the
        # product itself, element by element as the elementwise kernel would, so the expression need not be
        # written out for it (the sum's own rule, `-sum(g * t)` of a log-softmax, reads it once more at most,
        # inside the program that consumes it).  -sum(x) = sum(-x) exactly.
        inner = _fusion.lone_binary(xs[0])
        if inner is not None and (shape is None or tuple(shape) == xs[0].shape):
            iop, (a, b) = inner
            if op == Op.NEG:  # the sign goes to the operands, where it is a pending factor of the load (exact)
                neg = lambda v: -v if type(v) is float else map_op(Op.NEG, dtype, v)  # noqa: E731
                if iop == Op.SUB:
                    a, b = b, a
                elif iop == Op.ADD:
                    a, b = neg(a), neg(b)
                else:
                    a = neg(a)
            return _map_reduce_now(iop, red, dtype, (a, b), axes, keepdims, shape=xs[0].shape)
    ops = _limit_aux(tuple(_operand(x, dtype) for x in xs), dtype)
    if shape is None:
        shape = _bshape(ops)
    if shape is None:
        ops = _lift_scalars(ops, dtype)
        shape = ()
    ops = tuple(_expand(t, shape) for t in ops)
    nd = len(shape)
    axes = tuple(axes)
    mask = [d in axes for d in range(nd)]
    kept_shape = reduce_shape(shape, axes, True)
    out_t = _lib.empty(kept_shape, dtype)
    n_reduced = 1
    for d in axes:
        n_reduced *= shape[d]
    code = _lib.DTYPE_CODE[dtype]
    if out_t.numel() == 0:
        pass
    elif n_reduced == 0:
        if red not in _IDENTITY:
            raise ValueError("zero-size array to reduction operation which has no identity")
        _lib.fill(code, out_t, _IDENTITY[red])
    elif not _lib.map_reduce(op, red, code, shape, mask, out_t, ops):
        if any(type(t) is _lib.Affine and (t.ascale is not None or isinstance(t.shift, torch.Tensor)) for t in ops):
            # broadcast operands of pending maps can keep reduced axes from merging: write those out, retry
            settled = [LazyDevArray(t.t, dtype, t.scale, t.shift, t.ascale)._settled() if type(t) is _lib.Affine
                       else _rewrap(t, dtype) for t in ops]
            return _map_reduce_now(op, red, dtype, settled, axes, keepdims, shape=shape)
        # reduced axes interleaved with kept ones: one group of adjacent axes at a time
        if red == Red.LOGSUMEXP:
            raise NotImplementedError("logsumexp over non-adjacent axes of a non-contiguous layout")
        if op == Op.COPY and isinstance(ops[0], torch.Tensor) and ops[0].is_contiguous():
            cur = DevArray(ops[0], dtype)  # nothing to apply or lay out first: reduce the operand itself
        else:
            cur = plain(map_op(op, dtype, *[_rewrap(t, dtype) for t in ops]))  # (written out: the reduction below must not take it apart again)
        for group in _adjacent_groups(axes):
            cur = _map_reduce_now(Op.COPY, red, dtype, (cur,), group, True)
        out_t = cur._t
    out = DevArray(out_t, dtype)
    if not keepdims and axes:
        out = DevArray(out_t.reshape(reduce_shape(shape, axes, False)), dtype)
    return out


def _rewrap(t, dtype):
    if isinstance(t, torch.Tensor):
        return DevArray(t, dtype)
    if type(t) is _lib.Affine:
        return LazyDevArray(t.t, dtype, t.scale, t.shift, t.ascale)
    return t


def _adjacent_groups(axes):
    groups, cur = [], []
    for a in axes:
        if cur and a != cur[-1] + 1:
            groups.append(tuple(cur))
            cur = []
        cur.append(a)
    if cur:
        groups.append(tuple(cur))
    return groups


# --------------------------------------------------------------------------------------------
# contractions
# --------------------------------------------------------------------------------------------
def gemm2d(a, b, dtype, out=None, beta=0.0):
    """``a @ b`` for 2-d tensors of ``dtype`` (any strides) -> contiguous (M, N) tensor."""
    M, K = a.shape
    K2, N = b.shape
    if K != K2:
        raise ValueError(f"shapes {tuple(a.shape)} and {tuple(b.shape)} not aligned: {K} (dim 1) != {K2} (dim 0)")
    c = out if out is not None else _lib.empty((M, N), dtype)
    if M and N:
        _lib.gemm(_lib.DTYPE_CODE[dtype], 1, M, N, K, 1.0, a, a.stride(0), a.stride(1), 0, b, b.stride(0),
                  b.stride(1), 0, beta, c, max(N, 1), 0)
    return c


def gemm_batched(a, b, dtype):
    """(B, M, K) @ (B, K, N) with broadcastable (possibly stride-0) batch axes."""
    Bn, M, K = a.shape
    _, K2, N = b.shape
    if K != K2:
        raise ValueError(f"matmul: inner dimensions differ ({K} vs {K2})")
    c = _lib.empty((Bn, M, N), dtype)
    if Bn and M and N:
        _lib.gemm(_lib.DTYPE_CODE[dtype], Bn, M, N, K, 1.0, a, a.stride(1), a.stride(2), a.stride(0), b,
                  b.stride(1), b.stride(2), b.stride(0), 0.0, c, max(N, 1), M * N)
    return c
