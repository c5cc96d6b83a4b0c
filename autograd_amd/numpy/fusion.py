"""Deferred elementwise expressions: chains of rules evaluated as ONE kernel launch.

The rules of a backward pass are mostly elementwise (autograd/numpy/numpy_vjps.py:76-93, 139-143,
157-191 of the reference: ``y * g``, ``g / y``, ``-g * x / y**2``, ``ans * g``, and between them the
cotangent sums of autograd/core.py:185-205).  ``devarray.map_op`` is the single door every such
step goes through; instead of launching, it returns an :class:`ExprArray`: a node that names the
operation and its operands.  Nothing runs until something needs the memory (a contraction, a
reduction, a gather, a host transfer, ``core.settle`` at the end of a backward pass).  At that
moment the pending nodes under the value are written down as a straight-line program over a small
register file and handed to ``agmi_program``, which reads each leaf array once, keeps every
intermediate in registers and writes only what was asked for.  Values that the forward pass saved
for its rules are recomputed inside the program instead of being stored and read back.

Every step of a program is the functor of the one-rule kernel, rounded on its own, so the result
is bit for bit what the separate launches give (``ENABLED = False`` runs exactly those; the GPU
tests compare the two).

What ends a chain: an operand of another shape (a pending operand is written out before it is
broadcast), another dtype, more pending nodes than ``MAX_CONE``, and anything that is not
elementwise.
"""

import math
import os
import sys

import numpy as onp

from .. import _lib
from .._lib import Op, Red
from . import devarray as D
from .devarray import DevArray, LazyDevArray

from .. import _host

# off under a hosting `autograd` (AUTOGRAD_AMD_HOST): that package's make_vjp hands cotangents back as they are, and
# never completes a pending expression for the caller
ENABLED = os.environ.get("AUTOGRAD_AMD_FUSE", "1").strip() not in ("0", "") and not _host.HOST
MAX_CONE = 192  # pending nodes under one value before its largest pending operand is written out

_F32 = onp.dtype("float32")

# operands each op takes (single-result ops: everything a program may contain)
ARITY = {}
for _name in ("COPY NEG EXP LOG TANH SINH COSH SIN COS SQRT SQUARE ABS SIGN RECIPROCAL LOG1P EXPM1 EXP2 LOG2 LOG10 TAN "
              "ARCSIN ARCCOS ARCTAN ARCSINH ARCCOSH ARCTANH FLOOR CEIL RINT TRUNC NAN_TO_NUM").split():
    ARITY[getattr(Op, _name)] = 1
for _name in ("ADD SUB MUL DIV POW MAXIMUM MINIMUM FMAX FMIN ARCTAN2 HYPOT LOGADDEXP REMAINDER LOGADDEXP2 TANH_VJP "
              "RECIPROCAL_VJP SQRT_VJP SIN_VJP COS_VJP SINH_VJP COSH_VJP SQUARE_VJP LOG1P_VJP EXPM1_VJP "
              "EQUAL_AS_FLOAT").split():
    ARITY[getattr(Op, _name)] = 2
for _name in "WHERE DIV_VJP1 POW_VJP0 POW_VJP1 ABS_VJP MUL_ADD MUL_MUL MUL_SUB MUL_RSUB ADD_MUL SUB_MUL".split():
    ARITY[getattr(Op, _name)] = 3
for _name in "LSE_VJP CHOOSE_VJP EXTREMUM_VJP".split():
    ARITY[getattr(Op, _name)] = 4

# pseudo-op of a program: the sum of its operand over each row of a two-axis index space, at every index of the row
ROWSUM = _lib.PROGRAM_ROWSUM
ROWLSE = _lib.PROGRAM_ROWLSE  # the same for the logsumexp of a row
ARITY[ROWSUM] = ARITY[ROWLSE] = 1
_CHAINED_INTO_MUL = {Op.MUL: Op.MUL_MUL, Op.ADD: Op.ADD_MUL, Op.SUB: Op.SUB_MUL}
CHAINED = os.environ.get("AUTOGRAD_AMD_FUSE_CHAINED", "1").strip() not in ("0", "")  # (off: for measurements)
ROWSUM_WIDEST = {onp.dtype("float32"): 512, onp.dtype("float64"): 256}  # one wave's tile of the program kernel

COUNTS = {"programs": 0, "instructions": 0, "single": 0, "unfused": 0, "layers": 0}  # what ran (tests and profiles read it)


class ExprArray(DevArray):
    """``op(*args)`` not yet computed.  ``args`` are device arrays (plain, pending, or with a pending
    affine map) of this node's dtype whose shapes broadcast to this node's, and Python floats.
    Reading ``_t`` evaluates the node together with every pending node under it."""

    __slots__ = ("_op", "_args", "_shape", "_out", "_cone", "_lo")

    def __init__(self, op, args, shape, dtype, cone):
        self._op, self._args, self._shape = op, args, shape
        self.dtype = dtype
        self._borrowed = False
        self._shape_tuple = shape
        self._out = None
        self._cone = cone  # upper bound on the number of pending nodes under (and including) this one

    def __getattr__(self, name):
        # only reached when a slot is unset: `_t` before the value has been computed
        if name != "_t":
            raise AttributeError(name)
        evaluate((self,))
        return self._out

    def _buffer(self):
        out = self._out
        if out is None:
            out = self._out = _lib.empty(self._shape, self.dtype)
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
        item = self.dtype.itemsize
        return tuple(s * item for s in self._buffer().stride())

    def __len__(self):
        if not self._shape:
            raise TypeError("len() of unsized object")
        return self._shape[0]

    def __iter__(self):
        if not self._shape:
            raise TypeError("iteration over a 0-d array")
        return (self[i] for i in range(self._shape[0]))

    def _h(self):
        return self._buffer()

    def _settled(self):
        return DevArray(self._t, self.dtype)

    def _view(self, fn):
        return DevArray(fn(self._t), self.dtype)

    @staticmethod
    def _settle_group(values):
        evaluate(values)


def pending(x):
    return type(x) is ExprArray and x._args is not None


_REDUCIBLE = (Op.MUL, Op.ADD, Op.SUB, Op.DIV)


def lone_binary(x):
    """(op, operands) when the pending expression ``x`` is one binary arithmetic rule over operands that are in memory
    (or scalars), all of ``x``'s dtype; None otherwise."""
    if x._op not in _REDUCIBLE or len(x._args) != 2:
        return None
    for a in x._args:
        if isinstance(a, DevArray):
            if pending(a) or a.dtype != x.dtype or type(a) not in (DevArray, LazyDevArray):
                return None
        elif type(a) is not float:
            return None
    return x._op, tuple(x._args)


def make(op, dtype, xs):
    """``op(*xs)`` as a pending node, or None when the step has to run the ordinary way."""
    arity = ARITY.get(op)
    if arity is None or arity != len(xs) or dtype not in D._FLOATS:
        return None
    args = []
    shape = None
    for x in xs:
        if isinstance(x, DevArray):
            if x.dtype != dtype:
                x = D.astype(x, dtype)
            s = x.shape
            if shape is None:
                shape = s
            elif s != shape:
                shape = D.broadcast_shapes(shape, s)
            args.append(x)
        elif type(x) is float or type(x) is int or D.is_scalar(x):
            args.append(float(x))
        else:
            return None
    if shape is None or len(shape) > _lib.MAX_DIMS:
        return None
    wide = 0
    for s in shape:
        if s == 0:
            return None
        if s > 1:
            wide += 1
    if wide > 6:
        return None  # more axes than the strided kernels index when none of them merge: said at once, by the ordinary path
    cone = 1
    for k, x in enumerate(args):
        kind = type(x)
        if kind is float:
            continue
        if kind is D.PendingReduce and x._call is not None:
            node = _row_sums(x, shape, dtype)
            if node is not None:
                args[k] = node
                cone += node._cone
                continue
        if kind is ExprArray and x._args is not None:
            if x._shape != shape:
                x._t  # a pending operand is written out before it is broadcast: programs work on one shape
            else:
                cone += x._cone
        x._borrowed = True  # read when the result is evaluated: in-place accumulation and item assignment must not reach it
        # an item assignment into a borrowed array moves THAT handle to a buffer of its own: the node keeps a handle on
        # the memory as it is now
        if kind is DevArray:
            args[k] = DevArray(x._t, dtype)
        elif kind is LazyDevArray:
            args[k] = LazyDevArray(x._raw, dtype, x._scale, x._shift, x._ascale, x._producer)
    if cone > MAX_CONE:
        node = ExprArray(op, tuple(args), shape, dtype, cone)
        cone = node._cone = len(_post_order((node,)))
        while cone > MAX_CONE:
            big = None
            for x in args:
                if pending(x) and (big is None or x._cone > big._cone):
                    big = x
            big._t
            cone = node._cone = len(_post_order((node,)))
        return node
    return ExprArray(op, tuple(args), shape, dtype, cone)


def rows_fit_a_wave(shape, dtype):
    """Whether a reduction over the rows of ``shape`` can be formed inside a program: two axes, a row within one wave's
    tile of the program kernel, and a shape whose rows the reduction kernel gives to a group of lanes (the order of
    additions the program follows)."""
    if len(shape) != 2 or dtype not in ROWSUM_WIDEST:
        return False
    rows, cols = shape
    return 2 <= cols <= ROWSUM_WIDEST[dtype] and (cols <= 64 or rows >= 64)


def _row_sums(x, shape, dtype):
    """Row sums that have not run (``x``: a pending ``sum(e, axis=1, keepdims=True)``, the unbroadcast of a cotangent)
    about to be broadcast back over the rows they came from: a node of the full shape that the program kernel forms
    inside the chain (``g - exp(x - lse) * sum(g, axis=1)`` of a log-softmax is then one launch instead of a
    reduction plus a program).  Only for the shapes whose rows the reduction kernel gives to a group of lanes: the
    program adds in that kernel's order, so the value does not depend on which of the two ran.  None otherwise."""
    op, red, rdtype, xs, axes, _keepdims, full = x._call
    if len(xs) != 1 or rdtype != dtype or len(shape) != 2:
        return None
    if not (red == Red.SUM and (op == Op.COPY or op == Op.NEG)) and not (red == Red.LOGSUMEXP and op == Op.COPY):
        return None
    src = xs[0]
    rows, cols = shape
    if not isinstance(src, DevArray) or src.shape != shape or src.dtype != dtype or x.shape != (rows, 1) \
            or tuple(axes) not in ((1,), (-1,)) or (full is not None and tuple(full) != shape):
        return None
    if not rows_fit_a_wave(shape, dtype):
        return None
    node = ExprArray(ROWSUM if red == Red.SUM else ROWLSE, (src,), shape, dtype, 1 + (src._cone if pending(src) else 0))
    if op == Op.NEG:
        node = ExprArray(Op.NEG, (node,), shape, dtype, node._cone + 1)
    return node


def _post_order(roots):
    """The pending nodes under ``roots``, every node after the nodes it reads."""
    order, seen = [], set()
    stack = [(r, 0) for r in reversed(roots)]
    while stack:
        node, k = stack.pop()
        if k == 0:
            if id(node) in seen:
                continue
            seen.add(id(node))
        args = node._args
        n = len(args)
        while k < n:
            a = args[k]
            k += 1
            if type(a) is ExprArray and a._args is not None and id(a) not in seen:
                stack.append((node, k))
                stack.append((a, 0))
                break
        else:
            order.append(node)
    return order


def evaluate(values):
    """Compute every pending node among ``values`` (nodes of one shape and dtype share a launch)."""
    groups = {}
    for v in values:
        if type(v) is ExprArray and v._args is not None:
            groups.setdefault((v._shape, v.dtype), {})[id(v)] = v
    for group in groups.values():
        _run(list(group.values()))


def _finish(node):
    node._t = node._buffer()
    node._args = None


def _run(roots):
    order = _post_order(roots)
    if len(order) == 1 and order[0]._op != SHIFT:
        if not _dense_layer(order[0]):
            _single(order[0])
        return
    if len(roots) > _lib.PROGRAM_MAX_OUTPUTS:
        half = len(roots) // 2
        _run(roots[:half])
        _run([r for r in roots[half:] if r._args is not None])
        return
    program = _program_for(roots, order)
    if program is None:
        # too long, too many leaves or too many live values for one program: write a node from the middle of the
        # order out first (everything it needs comes before it), then try again with that node as a leaf
        if len(roots) > 1:
            half = len(roots) // 2
            _run(roots[:half])
            _run([r for r in roots[half:] if r._args is not None])
            return
        if len(order) > 1:
            # the node whose own expression is closest to half of this one
            half, pick = len(order) / 2.0, order[0]
            for node in order[:-1]:
                if abs(min(node._cone, len(order)) - half) < abs(min(pick._cone, len(order)) - half):
                    pick = node
            _run([pick])
            _run(roots)
            return
        program = False
    if program is not False:
        leaves, imms, words, n_regs, shifted, masks = program
        root = roots[0]
        shape, dtype = root._shape, root.dtype
        outs = tuple(r._buffer() for r in roots)
        if shifted is None:
            leaves = tuple(t if tuple(t.shape) == shape else t.expand(shape) for t in leaves)
        if _lib.program(_lib.DTYPE_CODE[dtype], shape, outs, leaves, imms, words, n_regs, shifted, masks):
            COUNTS["programs"] += 1
            COUNTS["instructions"] += len(words)
            for r in roots:
                _finish(r)
            return
    # a layout the program kernel does not cover (more than two axes left after merging, a strided innermost
    # axis): the steps run one by one
    COUNTS["unfused"] += 1
    for node in order:
        if node._args is not None:
            _single(node)


def _row_vector(t, shape):
    """The contiguous vector behind a tensor of ``shape`` that repeats one row (strides (0, 1)); None otherwise."""
    if tuple(t.shape) != shape or t.stride(0) != 0 or (t.stride(1) != 1 and shape[1] != 1):
        return None
    return t[0]


def _dense_layer(node):
    """A lone ``tanh`` over a matrix product that has not run yet (plus a pending bias), or the tanh rule applied to
    one (the cotangent ``G . W^T`` of examples/neural_net.py:33-35 under autograd/numpy/numpy_vjps.py:178, 615-624),
    goes into the contraction's epilogue: one launch for the layer.  False: not that shape (nothing has run)."""
    op = node._op
    if node.dtype != _F32 or len(node._shape) != 2:
        return False
    if op == Op.TANH:
        a = node._args[0]
        if type(a) is D.PendingProduct and not a.computed():
            product, bias = a, None
        elif type(a) is LazyDevArray and a._producer is not None and a._scale == 1.0 and a._ascale is None:
            product = a._producer
            raw = a._raw
            if product.computed() or raw.data_ptr() != product._buffer().data_ptr() or tuple(raw.shape) != product.shape \
                    or not raw.is_contiguous():
                return False
            bias = a._shift
            if bias is not None:
                if type(bias) is float:
                    return False
                bias = _row_vector(bias, node._shape)
                if bias is None:
                    return False
        else:
            return False
        if product.shape != node._shape or not product.with_activation(bias, node._buffer()):
            return False
        if type(a) is LazyDevArray:
            a._producer = None
    elif op == Op.TANH_VJP:
        g, x = node._args
        if type(g) is not D.PendingProduct or g.computed() or g.shape != node._shape:
            return False
        x = D.in_memory(x)  # (a forward product that has run is a plain array by now)
        bias = None
        if type(x) is DevArray:
            xt = x._t
        elif type(x) is LazyDevArray and x._scale == 1.0 and x._ascale is None and type(x._shift) is not float:
            xt = D._state(x)[0]  # (runs the forward product first if it never ran)
            if x._shift is not None:
                bias = _row_vector(x._shift, node._shape)
                if bias is None:
                    return False
        else:
            return False
        if tuple(xt.shape) != node._shape or (xt.stride(1) != 1 and node._shape[1] != 1) or xt.stride(0) < node._shape[1]:
            return False
        if not g.into_tanh_cotangent(xt, bias, node._buffer()):
            return False
    else:
        return False
    COUNTS["layers"] += 1
    _finish(node)
    return True


def _single(node):
    """One node by the ordinary kernels (its operands are computed first)."""
    dtype = node.dtype
    if node._op == SHIFT:
        _single_shift(node)
        return
    if node._op == ROWSUM or node._op == ROWLSE:
        sums = D._map_reduce_now(Op.COPY, Red.SUM if node._op == ROWSUM else Red.LOGSUMEXP, dtype, (node._args[0],), (1,), True)
        _lib.elementwise(Op.COPY, _lib.DTYPE_CODE[dtype], node._shape, (node._buffer(),), (D._expand(sums._t, node._shape),))
        COUNTS["single"] += 1
        _finish(node)
        return
    ops = D._limit_aux(tuple(D._operand(a, dtype) for a in node._args), dtype)
    shape = node._shape
    ops = tuple(D._expand(t, shape) for t in ops)
    _lib.elementwise(node._op, _lib.DTYPE_CODE[dtype], shape, (node._buffer(),), ops)
    COUNTS["single"] += 1
    _finish(node)


def _single_shift(node):
    """A shifted vector by the ordinary kernels: zeros outside, one copy inside."""
    dtype = node.dtype
    code = _lib.DTYPE_CODE[dtype]
    src = D._operand(D.plain(node._args[0]), dtype)
    if type(src) is _lib.Affine:
        src = LazyDevArray(src.t, dtype, src.scale, src.shift, src.ascale)._t
    out = node._buffer()
    n, m, lo = node._shape[0], src.shape[0], node._lo
    begin, end = max(lo, 0), min(lo + m, n)
    end = max(end, begin)
    outside = node._args[1]
    if outside is not None:
        rest = D.plain(outside)._t
    for at, part in ((0, out[:begin]), (end, out[end:])):
        if part.numel():
            if outside is None:
                _lib.fill(code, part, 0.0)
            else:
                _lib.elementwise(Op.COPY, code, tuple(part.shape), (part,), (rest[at:at + part.shape[0]],))
    if end > begin:
        _lib.elementwise(Op.COPY, code, (end - begin,), (out[begin:end],), (src[begin - lo:end - lo],))
    COUNTS["single"] += 1
    _finish(node)


class _TooBig(Exception):
    pass


class _Unsupported(Exception):
    pass


def _emit(roots):
    """``(leaf tensors, the shift each is read at, immediates, instruction words, registers, whether vectors are read at
    shifted positions (see :func:`shifted`), masks)`` of the program that computes ``roots``; None when it does not fit
    the kernel's limits.

    The nodes are first written down in static single assignment form, one instruction per distinct
    subexpression, with three rewrites that change no bit of any result: negations are carried as a sign on the
    value and absorbed by the sums, products and quotients that consume them (``(-a) + b`` is ``b - a``,
    ``(-a) * b`` is ``-(a * b)``, a negated immediate is another immediate); a product whose only reader is a sum
    becomes one multiply-add instruction of two roundings; ``x * 1.0`` is ``x``.  Instructions nothing reads are
    dropped, then registers are assigned by liveness."""
    dtype = roots[0].dtype
    KNOWN = D.KNOWN_SCALARS
    n_out = roots[0]._shape[0] if len(roots[0]._shape) == 1 else None
    single = dtype == _F32
    itemsize = dtype.itemsize
    leaves, leaf_ids, leaf_where = [], {}, []
    imms, imm_ids = [], {}
    masks = []
    # a value is ("L", k) / ("I", k) / ("X", k): leaf k, immediate k, result of instruction k; ("N", v) is minus v
    instrs = []   # (op, operand values, mask index or None)
    numbered = {}  # the same: one instruction for equal subexpressions
    memo = {}      # (id(node), shift) -> value
    any_shift = [False]
    limit = 4 * _lib.PROGRAM_MAX_INSTRUCTIONS  # (before dead instructions are dropped; bounds the work on a hopeless cone)

    def leaf(t, shift):
        if KNOWN:
            c = KNOWN.get(t.data_ptr())
            if c is not None and (t.numel() == 1 or builtins_all_zero(t.stride())):
                return imm(c)  # a shared constant (the seed of elementwise_grad, a zeros / ones array): no load
        vector = t.dim() == 1 and t.numel() > 1 and t.stride(0) == 1
        if shift:
            if not vector:
                if t.numel() == 1 or builtins_all_zero(t.stride()):
                    shift = 0  # one element for every index: nothing to shift
                else:
                    raise _Unsupported
            else:
                any_shift[0] = True
        if vector and n_out is not None and t.shape[0] != n_out:
            any_shift[0] = True  # (a slice that starts at index 0: read in place, but not over its whole extent)
        # (unit-stride vectors are told apart by address alone: in a program all of them span the root's extent,
        # or are read at shifted positions inside one storage)
        # (told apart by storage and position in it, not by address: two storages that happen to lie back to back
        # must not look like one vector read at two shifts, or the program would depend on where the allocator put them)
        key = (t.data_ptr() - t.storage_offset() * itemsize, t.storage_offset() + shift) if vector \
            else (t.data_ptr(), t.stride(), tuple(t.shape))
        v = leaf_ids.get(key)
        if v is None:
            if len(leaves) >= 4 * _lib.PROGRAM_MAX_LEAVES:
                raise _TooBig
            v = leaf_ids[key] = ("L", len(leaves))
            leaves.append(t)
            leaf_where.append(shift)
        return v

    def imm(c):
        c = float(onp.float32(c)) if single else float(c)
        key = (c, bool(onp.signbit(c))) if c == 0.0 else c  # -0.0 and 0.0 are different immediates; NaN never equals itself: not shared
        v = imm_ids.get(key)
        if v is None:
            v = ("I", len(imms))
            if c == c:
                imm_ids[key] = v
            imms.append(c)
        return v

    def emit(op, *srcs, mask=None):
        key = (op, srcs, mask)
        v = numbered.get(key)
        if v is None:
            if len(instrs) >= limit:
                raise _TooBig
            v = numbered[key] = ("X", len(instrs))
            instrs.append(key)
        return v

    def real(v):
        """``v`` as a value that exists: a carried sign becomes a negation (or the negated immediate)."""
        if v[0] != "N":
            return v
        base = v[1]
        return imm(-imms[base[1]]) if base[0] == "I" else emit(Op.NEG, base)

    def minus(v):
        if v[0] == "N":
            return v[1]
        if v[0] == "I":
            return imm(-imms[v[1]])
        return ("N", v)

    def signed(negative, op, *bases):
        """``op(bases)`` with the sign its operands carried; an immediate among them takes the sign."""
        if negative:
            for k, b in enumerate(bases):
                if b[0] == "I" and (op != Op.DIV_VJP1 or k < 2):
                    flipped = bases[:k] + (imm(-imms[b[1]]),) + bases[k + 1:]
                    return ins_plain(op, *flipped)
            return ("N", ins_plain(op, *bases))
        return ins_plain(op, *bases)

    def ins_plain(op, *srcs):
        if op == Op.MUL:
            # x * 1.0 is x, bit for bit (the cotangent seeds of elementwise_grad are ones); x * -1.0 is -x
            for me, other in ((1, 0), (0, 1)):
                if srcs[me][0] == "I":
                    c = imms[srcs[me][1]]
                    if c == 1.0:
                        return srcs[other]
                    if c == -1.0:
                        return minus(srcs[other])
        elif op == Op.DIV and srcs[1][0] == "I" and imms[srcs[1][1]] == 1.0:
            return srcs[0]
        return emit(op, *srcs)

    def ins(op, *srcs, mask=None):
        if mask is not None:
            inside, rest = srcs
            if inside[0] == "N" and (rest[0] == "N" or rest[0] == "I"):
                # a select commutes with the sign when both sides carry it (minus an immediate is an immediate)
                return ("N", emit(op, inside[1], minus(rest), mask=mask))
            return emit(op, real(inside), real(rest), mask=mask)
        if op == Op.NEG:
            return minus(srcs[0])
        na = srcs[0][0] == "N"
        if op == Op.ADD or op == Op.SUB:
            a, b = srcs
            if op == Op.SUB:
                b = minus(b)  # a - b is a + (-b), the very same operation
            nb = b[0] == "N"
            if not na and not nb:
                return emit(Op.ADD, a, b)
            if na and nb:
                return emit(Op.SUB, real(a), b[1])   # (-a) + (-b): one negation stays, the other becomes the subtraction
            if na:
                return emit(Op.SUB, b, a[1])         # (-a) + b = b - a
            return emit(Op.SUB, a, b[1])             # a + (-b) = a - b
        if op == Op.MUL or op == Op.DIV:
            a, b = srcs
            nb = b[0] == "N"
            return signed(na != nb, op, a[1] if na else a, b[1] if nb else b)
        if op == Op.SQUARE or op == Op.ABS:
            return emit(op, srcs[0][1] if na else srcs[0])
        if op == Op.RECIPROCAL or op == ROWSUM:  # (a row's sum of negated terms is minus its sum, bit for bit)
            return signed(na, op, srcs[0][1] if na else srcs[0])
        if op == Op.DIV_VJP1:  # ((-g) * x) / (y * y)
            g, x, y = srcs
            nx = x[0] == "N"
            return signed(na != nx, op, g[1] if na else g, x[1] if nx else x, y[1] if y[0] == "N" else y)
        return ins_plain(op, *[real(v) for v in srcs])

    def masked(v, rest, lo, hi):
        rng = (lo, hi)
        if rng in masks:
            k = masks.index(rng)
        else:
            if len(masks) >= _lib.PROGRAM_MAX_MASKS:
                raise _TooBig
            k = len(masks)
            masks.append(rng)
        return ins(_lib.PROGRAM_MASK, v, rest, mask=k)

    def power(x, e):
        """``pow_like_numpy(x, e)`` for an exponent known here: the short cuts NumPy takes become the plain
        operations they are (same bits), so that the general routine stays out of the program."""
        if e == 2.0:
            return ins(Op.SQUARE, x)
        if e == 1.0:
            return x
        if e == 0.0:
            return imm(1.0)
        if e == -1.0:
            return ins(Op.RECIPROCAL, x)
        if e == 0.5:
            return ins(Op.SQRT, x)
        return ins(Op.POW, x, imm(e))

    def value(a, shift):
        """The register value that holds ``a[i + shift]`` at output index ``i``."""
        if type(a) is float:
            return imm(a)
        if type(a) is ExprArray and a._args is not None:
            key = (id(a), shift)
            v = memo.get(key)
            if v is not None:
                return v
            op = a._op
            if op == SHIFT:
                src, outside = a._args
                lo, m = a._lo, src.shape[0]
                v = value(src, shift - lo)
                first, behind = lo - shift, lo - shift + m  # the output indices that fall inside `src`
                if first > 0 or behind < n_out:
                    rest = imm(0.0) if outside is None else value(outside, shift)
                    v = masked(v, rest, max(first, 0), min(behind, n_out))
            else:
                srcs = tuple(value(arg, shift) for arg in a._args)
                if op == Op.POW and srcs[1][0] == "I":
                    v = power(srcs[0], imms[srcs[1][1]])
                elif op == Op.POW_VJP0 and srcs[2][0] == "I":
                    # (g * y) * x**where(y, y - 1, 1), the exponent formed in the array's precision as the functor does
                    y = imms[srcs[2][1]]
                    e = float(onp.float32(y) - onp.float32(1.0)) if single else y - 1.0
                    v = ins(Op.MUL, ins(Op.MUL, srcs[0], srcs[2]), power(srcs[1], e if y != 0.0 else 1.0))
                else:
                    v = ins(op, *srcs)
            memo[key] = v
            return v
        if type(a) is LazyDevArray:
            raw, scale, ascale, offset = D._state(a)
            v = leaf(raw, shift)
            if scale != 1.0:
                v = ins(Op.MUL, v, imm(scale))
            if ascale is not None:
                v = ins(Op.MUL, v, leaf(ascale, shift))
            if offset is not None:
                v = ins(Op.ADD, v, imm(offset) if type(offset) is float else leaf(offset, shift))
            return v
        return leaf(a._t, shift)

    try:
        root_values = [real(value(r, 0)) for r in roots]
        # every root is the result of an instruction of its own (a root that came out as a leaf, an immediate or
        # another root's value gets a copy: the kernel stores registers, and each output once)
        seen = set()
        for k, v in enumerate(root_values):
            if v[0] != "X" or v in seen:
                root_values[k] = v = emit(Op.COPY, v, mask=("root", k))
            seen.add(v)
    except _TooBig:
        return None

    # A product, sum or difference that only one sum, difference or product reads travels with its reader: one
    # instruction with three operands (the first rule rounded, then the second, as the two instructions would be).
    # What an interpreted instruction costs is operand moves and dispatch, hardly the arithmetic.
    uses = {}
    for _op, srcs, _mask in instrs:
        for v in srcs:
            uses[v] = uses.get(v, 0) + 1
    for v in root_values:
        uses[v] = uses.get(v, 0) + 1
    if CHAINED:
        for k, (op, srcs, mask) in enumerate(instrs):
            if mask is not None or (op != Op.ADD and op != Op.SUB and op != Op.MUL):
                continue
            for me, other in ((0, 1), (1, 0)):
                p = srcs[me]
                if p[0] != "X" or uses.get(p) != 1:
                    continue
                pop, psrcs, pmask = instrs[p[1]]
                if pmask is not None:
                    continue
                if pop == Op.SQUARE:
                    pop, psrcs = Op.MUL, (psrcs[0], psrcs[0])  # x * x, the very same product
                if op == Op.MUL:
                    both = _CHAINED_INTO_MUL.get(pop)
                elif pop != Op.MUL:
                    continue
                elif op == Op.ADD:
                    both = Op.MUL_ADD
                else:
                    both = Op.MUL_SUB if me == 0 else Op.MUL_RSUB
                if both is None:
                    continue
                instrs[k] = (both, (psrcs[0], psrcs[1], srcs[other]), None)
                uses[p] = 0
                break
    # drop what nothing reads (from the roots backwards), then number leaves, immediates and instructions anew
    needed = set(root_values)
    for k in range(len(instrs) - 1, -1, -1):
        if ("X", k) in needed:
            needed.update(instrs[k][1])
    kept = [k for k in range(len(instrs)) if ("X", k) in needed]
    used_leaves = [k for k in range(len(leaves)) if ("L", k) in needed]
    used_imms = [k for k in range(len(imms)) if ("I", k) in needed]
    if (len(kept) > _lib.PROGRAM_MAX_INSTRUCTIONS - len(roots) or len(used_leaves) > _lib.PROGRAM_MAX_LEAVES
            or len(used_imms) > _lib.PROGRAM_MAX_IMMEDIATES):
        return None
    rename = {("L", k): ("L", n) for n, k in enumerate(used_leaves)}
    rename.update({("I", k): ("I", n) for n, k in enumerate(used_imms)})
    rename.update({("X", k): ("X", n) for n, k in enumerate(kept)})
    instrs = [(instrs[k][0], tuple(rename[v] for v in instrs[k][1]), instrs[k][2]) for k in kept]
    root_values = [rename[v] for v in root_values]
    leaf_where = [leaf_where[k] for k in used_leaves]
    leaves = [leaves[k] for k in used_leaves]
    imms = [imms[k] for k in used_imms]

    n_leaf, n_imm, n_ins = len(leaves), len(imms), len(instrs)
    need_shifted = bool(any_shift[0] or masks)
    # last use of every value (instruction index; stores come after all instructions)
    last = {}
    for k, (_op, srcs, _mask) in enumerate(instrs):
        for s in srcs:
            last[s] = k
    for v in root_values:
        last[v] = n_ins
    row_sums = builtins_any_rowsum(instrs)
    for n_regs in ([16] if single or row_sums else [8, 16]):  # (8 float32 registers are indexed by a chain of selects in the kernel: slower than 16)
        if n_leaf + n_imm > n_regs:
            continue
        reg = {("L", k): k for k in range(n_leaf)}
        for k in range(n_imm):
            reg[("I", k)] = n_regs - 1 - k
        free = list(range(n_regs - 1 - n_imm, n_leaf - 1, -1))  # popped from the low end
        words = []
        ok = True
        for k, (op, srcs, mask) in enumerate(instrs):
            regs = [reg[s] for s in srcs]
            for s in dict.fromkeys(srcs):  # (each once, in operand order: the same words in every process)
                if s[0] != "I" and last[s] == k:
                    free.append(reg[s])
            if not free:
                ok = False
                break
            dst = free.pop()
            reg[("X", k)] = dst
            if op == _lib.PROGRAM_MASK:
                w = op | dst << 8 | regs[0] << 12 | mask << 16 | regs[1] << 20  # inside value, range, outside value
            else:
                w = op | dst << 8
                for pos, r in enumerate(regs):
                    w |= r << (12 + 4 * pos)
            words.append(w)
        if not ok:
            continue
        for out_index, v in enumerate(root_values):
            r = reg[v]
            words.append(_lib.PROGRAM_STORE | r << 8 | r << 12 | out_index << 16)
        return leaves, leaf_where, imms, words, n_regs, need_shifted, masks
    return None


def _bind(leaves, leaf_where, n_out, itemsize, need_shifted):
    """The leaf tensors as the kernel takes them, and per leaf ``(shift, lo, hi)`` for a one-axis program with vectors read
    at shifted positions (None otherwise): every vector leaf comes with the indices at which its (moved) address stays
    inside its storage; whatever lies outside a vector's own extent is masked by the program."""
    if not need_shifted:
        return leaves, None
    shifted_leaves, bound = [], []
    for t, shift in zip(leaves, leaf_where):
        if t.dim() == 1 and t.numel() > 1 and t.stride(0) == 1:
            first = t.storage_offset() + shift
            total = t.untyped_storage().nbytes() // itemsize
            shifted_leaves.append((shift, -first, total - first))
            bound.append(t)
        elif t.numel() == 1 or builtins_all_zero(t.stride()):
            shifted_leaves.append((0, 0, n_out))
            bound.append(t.as_strided((n_out,), (0,)))
        else:
            raise _Unsupported
    return bound, shifted_leaves


# ---- emitted programs are kept ---------------------------------------------------------------------------------
# Writing a program down (the walk, the rewrites, the register assignment) costs tens of microseconds for a three-step
# expression and hundreds for a Hessian-vector product, every evaluation, although a loop evaluates the same
# expressions over and over.  What the emitted program depends on is written down as a key: the nodes in order with
# their operations and operands, where an operand is another node (by position), a scalar (by value), or an array in
# memory (by shape, strides, which distinct array it is, and where it lies in which storage, since vectors of one
# storage are merged when a shift makes them coincide).  Equal keys give equal programs; only the tensors differ, and
# those are bound again from the walk.
_PROGRAMS = {}
_PROGRAM_LIMIT = 2048
CACHE = os.environ.get("AUTOGRAD_AMD_FUSE_CACHE", "1").strip() not in ("0", "")
VERIFY = os.environ.get("AUTOGRAD_AMD_FUSE_VERIFY", "").strip() not in ("0", "")  # re-emit on every hit and compare


def _signature(roots, order):
    """``(key, tensors)``: the key described above and the distinct leaf tensors in the order the key numbers them;
    None when an operand is of a kind the key does not describe."""
    KNOWN = D.KNOWN_SCALARS
    itemsize = roots[0].dtype.itemsize
    index = {}
    for k, n in enumerate(order):
        index[id(n)] = k
    tensors, ident, bases = [], {}, {}

    def leaf_desc(t):
        ptr, stride, shape = t.data_ptr(), t.stride(), tuple(t.shape)
        if KNOWN:
            c = KNOWN.get(ptr)
            if c is not None and (t.numel() == 1 or builtins_all_zero(stride)):
                return ("k", c, math.copysign(1.0, c))
        key = (ptr, stride, shape)
        k = ident.get(key)
        if k is None:
            k = ident[key] = len(tensors)
            tensors.append(t)
        off = t.storage_offset()
        base = ptr - off * itemsize
        b = bases.get(base)
        if b is None:
            b = bases[base] = len(bases)
        return ("l", k, shape, stride, b, off)

    def desc(a):
        kind = type(a)
        if kind is float:
            return ("f", a, math.copysign(1.0, a))
        if a is None:
            return None
        if kind is ExprArray and a._args is not None:
            return ("n", index[id(a)])
        if kind is LazyDevArray:
            raw, scale, ascale, offset = D._state(a)
            if offset is not None:
                offset = ("f", offset, math.copysign(1.0, offset)) if type(offset) is float else leaf_desc(offset)
            return ("z", leaf_desc(raw), scale, None if ascale is None else leaf_desc(ascale), offset)
        if not isinstance(a, DevArray):
            raise _Unsupported
        return leaf_desc(a._t)

    parts = []
    try:
        for n in order:
            parts.append((n._op, n._lo if n._op == SHIFT else 0, tuple([desc(a) for a in n._args])))
        where = tuple([index[id(r)] for r in roots])
    except (_Unsupported, KeyError, TypeError):
        return None
    for n in order:
        if n._args is None:
            return None  # reading a deferred operand ran part of this very expression: described as it no longer is
    return (roots[0].dtype, roots[0]._shape, where, tuple(parts)), tensors


def _program_for(roots, order):
    """``_emit`` and ``_bind`` through the cache: ``(leaves, imms, words, n_regs, shifted, masks)``, None (does not fit
    one program) or False (a layout the kernel does not cover)."""
    root = roots[0]
    n_out = root._shape[0] if len(root._shape) == 1 else None
    itemsize = root.dtype.itemsize
    sig = _signature(roots, order) if CACHE else None
    if sig is not None:
        key, tensors = sig
        hit = _PROGRAMS.get(key)
        if hit is not None:
            if hit[0] != "ok":
                return None if hit[0] == "none" else False
            _, slots, where, imms, words, n_regs, need_shifted, masks = hit
            leaves, shifted = _bind([tensors[k] for k in slots], where, n_out, itemsize, need_shifted)
            if VERIFY:
                _verify(roots, (leaves, imms, words, n_regs, shifted, masks), n_out, itemsize)
            return leaves, imms, words, n_regs, shifted, masks
    try:
        emitted = _emit(roots)
        if emitted is not None:
            raw, where, imms, words, n_regs, need_shifted, masks = emitted
            leaves, shifted = _bind(raw, where, n_out, itemsize, need_shifted)
    except _Unsupported:
        emitted = False
    if sig is not None:
        if len(_PROGRAMS) >= _PROGRAM_LIMIT:
            _PROGRAMS.clear()
        if emitted is None:
            _PROGRAMS[key] = ("none",)
        elif emitted is False:
            _PROGRAMS[key] = ("unsupported",)
        else:
            ident = {}
            for k, t in enumerate(tensors):
                ident[(t.data_ptr(), t.stride(), tuple(t.shape))] = k
            try:
                slots = tuple([ident[(t.data_ptr(), t.stride(), tuple(t.shape))] for t in raw])
            except KeyError:
                slots = None  # (a leaf the key's walk did not see: leave this expression uncached)
            if slots is not None:
                _PROGRAMS[key] = ("ok", slots, tuple(where), list(imms), list(words), n_regs, need_shifted, list(masks))
    if emitted is None or emitted is False:
        return emitted
    return leaves, imms, words, n_regs, shifted, masks


def _verify(roots, bound, n_out, itemsize):
    raw, where, imms, words, n_regs, need_shifted, masks = _emit(roots)
    leaves, shifted = _bind(raw, where, n_out, itemsize, need_shifted)
    got_leaves, got_imms, got_words, got_regs, got_shifted, got_masks = bound
    same = (list(got_words) == list(words) and got_regs == n_regs and list(got_masks) == list(masks)
            and [repr(c) for c in got_imms] == [repr(c) for c in imms] and got_shifted == shifted
            and len(got_leaves) == len(leaves)
            and all(a.data_ptr() == b.data_ptr() and a.stride() == b.stride() and a.shape == b.shape
                    for a, b in zip(got_leaves, leaves)))
    if not same:
        raise AssertionError("a kept program differs from the one emitted for the same expression")


def slice_of(A, start, stop):
    """``A[start:stop]`` of a pending vector ``A`` as a pending node (nothing is written out)."""
    return shifted(A, -start, stop - start)


def padded(x, start, n, dtype):
    """``zeros(n)`` with ``0.0 + x`` added into ``[start : start + len(x)]`` (the cotangent of ``x = y[start:stop]``,
    formed the way the scatter rule forms it, sign of zero included) as a pending node; None when ``x`` cannot
    take part in a program."""
    inner = make(Op.ADD, dtype, (0.0, x))
    if inner is None or inner._shape != x.shape:
        return None
    return shifted(inner, start, n)


def added_into(A, start, x, take):
    """``A`` with ``x`` added into ``A[start : start + len(x)]`` (``numpy.add.at`` through a slice of a vector) as
    a pending node; ``take(A, slice)`` gives that slice of ``A``.  None when the sum cannot take part in a program."""
    m = x.shape[0]
    inner = make(Op.ADD, A.dtype, (take(A, slice(start, start + m)), x))
    if inner is None or inner._shape != (m,):
        return None
    return shifted(inner, start, A.shape[0], outside=A)


def builtins_any_rowsum(instrs):
    for instr in instrs:
        if instr[0] == ROWSUM or instr[0] == ROWLSE:
            return True
    return False


def builtins_all_zero(strides):
    for s in strides:
        if s != 0:
            return False
    return True


SHIFT = -1  # pseudo-op of a shifted vector


def shifted(src, lo, n, outside=None):
    """The vector of length ``n`` that holds ``src[i - lo]`` at index ``i`` where that exists and ``outside[i]`` (zero
    when None) elsewhere, as a pending node: a slice of a pending vector (``lo = -start``) and the zero-padded vector that the cotangent of
    a slice is (``untake`` of ``x[a:b]``, autograd/numpy/numpy_vjps.py:919-950: ``lo = a``) are both this.  The
    program kernel reads the leaves under such a node at moved addresses, so ``x[1:]``, ``x[:-1]`` and the
    cotangents scattered back through them cost no pass of their own."""
    cone = 1 + (src._cone if pending(src) else 0)
    src._borrowed = True
    if outside is not None:
        outside._borrowed = True
        if pending(outside):
            cone += outside._cone
    node = ExprArray(SHIFT, (src, outside), (n,), src.dtype, cone)
    node._lo = lo
    return node


D._DEFERRED = D._DEFERRED + (ExprArray,)
D._fusion = sys.modules[__name__]
