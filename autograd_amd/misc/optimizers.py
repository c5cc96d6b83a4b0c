"""Gradient-based optimizers whose state and parameters stay on the device.

Same functions, signatures and arithmetic as the reference (autograd/misc/optimizers.py:15-75):
``sgd``, ``rmsprop`` and ``adam`` take ``grad(x, i)``, an initial point that may be any nest of
containers of device arrays, an optional ``callback(x, i, g)`` and the hyper-parameters, and
return the final point in the structure of the initial one.  Each iteration's update is ONE
fused kernel (``agmi_optimizer_step``) over the flat parameter vector instead of 6-12 whole-array
passes; element arithmetic follows the reference's expressions in order, including NumPy's
dtype promotion: the state starts as float64 ``zeros``/``ones`` (optimizers.py:38, 53, 64-65), so
state and updated parameters are float64 whatever dtype the initial point has.
"""

import numpy as onp

from .. import _lib
from ..numpy import devarray as D
from ..wrap_util import wraps
from .flatten import flatten


def unflatten_optimizer(optimize):
    """Takes an optimizer that operates on flat 1-d device arrays and returns a wrapped version
    that handles trees of nested containers (lists/tuples/dicts) with arrays/scalars at the
    leaves (optimizers.py:15-31)."""

    @wraps(optimize)
    def _optimize(grad, x0, callback=None, *args, **kwargs):
        _x0, unflatten = flatten(x0)
        _grad = lambda x, i: flatten(grad(unflatten(x), i))[0]  # noqa: E731
        if callback:
            _callback = lambda x, i, g: callback(unflatten(x), i, unflatten(g))  # noqa: E731
        else:
            _callback = None
        return unflatten(optimize(_grad, _x0, _callback, *args, **kwargs))

    return _optimize


_F64 = onp.dtype("float64")


def _flat(a, what):
    a = D.plain(D.asarray(a))
    if a.ndim != 1 or a.dtype not in D._FLOATS:
        raise TypeError(f"{what} must be a flat float32/float64 device array, got shape {a.shape} dtype {a.dtype}")
    return D.contiguous(a)


def _step(kind, x, g, s0, s1, hyper):
    """x_new (fresh float64 array; earlier iterates a callback may have kept stay valid)."""
    x, g = _flat(x, "the parameter vector"), _flat(g, "the gradient")
    if g.shape != x.shape:
        raise ValueError(f"gradient of shape {g.shape} for parameters of shape {x.shape}")
    out = D.empty(x.shape, _F64)
    if x.size:
        _lib.optimizer_step(kind, x._t, g._t, s0._t, None if s1 is None else s1._t, out._t, hyper)
    return out


@unflatten_optimizer
def sgd(grad, x, callback=None, num_iters=200, step_size=0.1, mass=0.9):
    """Stochastic gradient descent with momentum.
    grad() must have signature grad(x, i), where i is the iteration number."""
    velocity = D.zeros((len(x),), _F64)
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        x = _step(_lib.OPT_SGD, x, g, velocity, None, (mass, 1.0 - mass, step_size))
    return x


@unflatten_optimizer
def rmsprop(grad, x, callback=None, num_iters=100, step_size=0.1, gamma=0.9, eps=10**-8):
    """Root mean squared prop: See Adagrad paper for details."""
    avg_sq_grad = D.ones((len(x),), _F64)
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        x = _step(_lib.OPT_RMSPROP, x, g, avg_sq_grad, None, (gamma, 1 - gamma, step_size, eps))
    return x


@unflatten_optimizer
def adam(grad, x, callback=None, num_iters=100, step_size=0.001, b1=0.9, b2=0.999, eps=10**-8):
    """Adam as described in http://arxiv.org/pdf/1412.6980.pdf.
    It's basically RMSprop with momentum and some correction terms."""
    m = D.zeros((len(x),), _F64)
    v = D.zeros((len(x),), _F64)
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        x = _step(_lib.OPT_ADAM, x, g, m, v,
                  (1 - b1, b1, 1 - b2, b2, 1 - b1 ** (i + 1), 1 - b2 ** (i + 1), step_size, eps))
    return x
