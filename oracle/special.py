"""logsumexp for the oracle's NumPy value type.

Forward is SciPy's ``scipy.special.logsumexp`` wrapped as a primitive, the
rules restate the reference's autograd/scipy/special.py:119-147.
TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

import scipy.special

from autograd_amd.extend import defjvp, defvjp, primitive

from . import np_namespace as np
from .np_vjps import repeat_to_match_shape

logsumexp = primitive(scipy.special.logsumexp)


def _make_grad_logsumexp(ans, x, axis=None, b=1.0, keepdims=False):
    shape, dtype = np.shape(x), np.result_type(x)

    def vjp(g):
        g_repeated, _ = repeat_to_match_shape(g, shape, dtype, axis, keepdims)
        ans_repeated, _ = repeat_to_match_shape(ans, shape, dtype, axis, keepdims)
        return g_repeated * b * np.exp(x - ans_repeated)

    return vjp


defvjp(logsumexp, _make_grad_logsumexp)


def _fwd_grad_logsumexp(g, ans, x, axis=None, b=1.0, keepdims=False):
    if not keepdims:
        if isinstance(axis, int):
            ans = np.expand_dims(ans, axis)
        elif isinstance(axis, tuple):
            for ax in sorted(axis):
                ans = np.expand_dims(ans, ax)
    return np.sum(g * b * np.exp(x - ans), axis=axis, keepdims=keepdims)


defjvp(logsumexp, _fwd_grad_logsumexp)
