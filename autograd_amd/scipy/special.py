"""``logsumexp`` on device arrays, with its reverse- and forward-mode rules.

Counterpart of the reference's autograd/scipy/special.py:119-147, whose forward is
``scipy.special.logsumexp``.  Forward: one single-pass reduction kernel over (max, scaled sum)
pairs.  Reverse, concrete operands: one fused kernel ``g * b * exp(x - ans)`` that reads ``g``
and ``ans`` through broadcast strides, so neither is ever materialised at full size (the
reference materialises both); for the rows of a matrix the cotangent is not written at all until
the rules that consume it have run (``devarray.LseCotangent``).  Forward mode: the same functor fused into a sum.
"""

import numbers

from .._lib import Op, Red
from ..core import BatchMode, batch_safe
from ..extend import defjvp, defvjp, primitive
from ..numpy import devarray as D
from ..numpy import fusion
from ..numpy import wrapper as np
from ..numpy.vjps import _concrete, repeat_to_match_shape


@primitive
def logsumexp(x, axis=None, b=1.0, keepdims=False):
    x = D.asarray(x)
    axes = D.normalize_axes(axis, x.ndim)
    if (type(b) is float or isinstance(b, numbers.Number)) and b == 1.0:
        dt = D._float_dtype(x.dtype)
        if keepdims and axes == (1,) and x.dtype == dt and fusion.ENABLED and fusion.rows_fit_a_wave(x.shape, dt):
            # The log-softmax of a layer's rows (reference examples/rnn.py:50-52, examples/neural_net.py:24-28:
            # x - logsumexp(x, axis=1, keepdims=True)): the value is only ever read back by the chains around it, the
            # subtraction and the rule g * exp(x - ans), and a program forms the logsumexp of a short row itself
            # (bit for bit the reduction kernel's value).  So nothing runs here; a reader of the value itself runs it.
            return D.PendingReduce((Op.COPY, Red.LOGSUMEXP, dt, (D._kept(x),), axes, True, None), (x.shape[0], 1), dt)
        return D.map_reduce(Op.COPY, Red.LOGSUMEXP, dt, (x,), axes, keepdims)
    # weighted form, the way scipy evaluates it: m = max(x), log(sum(b * exp(x - m))) + m, with weights of either
    # sign (a negative total gives NaN, as there).  Two passes over x: the maximum, then the weighted sum
    # fused into its reduction.
    if not isinstance(b, numbers.Number):
        b = D.asarray(b)
        if D.broadcast_shapes(x.shape, b.shape) != x.shape:
            x = np.broadcast_to.fun(x, D.broadcast_shapes(x.shape, b.shape))
            axes = D.normalize_axes(axis, x.ndim)
    dt = D._float_dtype(D.result_dtype(x, b))
    top = D.map_reduce(Op.COPY, Red.MAX, dt, (x,), axes, True)
    top = np._where3.fun(np.isfinite(top), top, 0.0)  # all -inf, or an inf / NaN present: no shift
    total = D.map_reduce(Op.LSE_VJP, Red.SUM, dt, (1.0, b, x, top), axes, True)
    out = np.add.fun(np.log.fun(total), top)
    if keepdims:
        return out
    return np.reshape.fun(out, tuple(n for d, n in enumerate(x.shape) if d not in axes))


def _keep(a, shape, axis, keepdims):
    """Reduced-shape array ``a`` viewed with the reduced axes kept as size 1."""
    if keepdims or len(shape) == 0:
        return a
    axes = D.normalize_axes(axis, len(shape))
    new_shape = tuple(1 if d in axes else s for d, s in enumerate(shape))
    return a._view(lambda t: t.reshape(new_shape))


def _make_grad_logsumexp(ans, x, axis=None, b=1.0, keepdims=False):
    shape, dtype = np.shape(x), np.result_type(x)

    def vjp(g):
        if BatchMode.active:
            # cotangents stacked along a leading axis: plain broadcasting against the kept-dims form of `ans`
            g_repeated, _ = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
            axes = D.normalize_axes(axis, len(shape))
            ans_kept = ans if keepdims or not shape else np.reshape(ans, tuple(1 if d in axes else n for d, n in enumerate(shape)))
            return g_repeated * b * np.exp(x - ans_kept)
        if _concrete(g, ans, x, b):
            g_k = _keep(D.asarray(g), shape, axis, keepdims)
            ans_k = _keep(ans, shape, axis, keepdims)
            dt = D._float_dtype(D.result_dtype(g_k, x, ans_k))
            if (type(b) is float and b == 1.0 and len(shape) == 2 and D.normalize_axes(axis, 2) == (1,)
                    and D.LseCotangent.eligible(g_k, x, ans_k, dt)):
                # rows of a matrix: the cotangent stays unwritten until its consumers are known; the usual
                # ones (row sums, a rescaled copy, column sums of a product) then come out of one pass
                return D.LseCotangent(g_k, x, ans_k, dt)
            return D.map_op(Op.LSE_VJP, dt, g_k, b, x, ans_k)
        g_repeated, _ = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        ans_repeated, _ = repeat_to_match_shape(ans, shape, dtype, axis, keepdims)
        return g_repeated * b * np.exp(x - ans_repeated)

    return vjp


defvjp(logsumexp, _make_grad_logsumexp)
batch_safe(logsumexp)


def _fwd_grad_logsumexp(g, ans, x, axis=None, b=1.0, keepdims=False):
    shape = np.shape(x)
    if _concrete(g, ans, x, b):
        ans_k = _keep(ans, shape, axis, keepdims)
        dt = D._float_dtype(D.result_dtype(g, x, ans_k))
        return D.map_reduce(Op.LSE_VJP, Red.SUM, dt, (g, b, x, ans_k), D.normalize_axes(axis, len(shape)), keepdims)
    if not keepdims:
        if isinstance(axis, int):
            ans = np.expand_dims(ans, axis)
        elif isinstance(axis, tuple):
            for ax in sorted(axis):
                ans = np.expand_dims(ans, ax)
    return np.sum(g * b * np.exp(x - ans), axis=axis, keepdims=keepdims)


defjvp(logsumexp, _fwd_grad_logsumexp)
