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
    """An optimizer written for flat 1-d device vectors -> one that takes any nest of lists, tuples and dicts
    with arrays or scalars at the leaves: the point, the gradients and what the callback sees are flattened
    and unflattened at the boundary (optimizers.py:15-31)."""

    @wraps(optimize)
    def on_containers(grad, x0, callback=None, *args, **kwargs):
        flat_x0, unflatten = flatten(x0)

        def flat_grad(x, i):
            return flatten(grad(unflatten(x), i))[0]

        flat_callback = None
        if callback:

            def flat_callback(x, i, g):
                return callback(unflatten(x), i, unflatten(g))

        return unflatten(optimize(flat_grad, flat_x0, flat_callback, *args, **kwargs))

    return on_containers


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


def _descend(grad, x, callback, num_iters, kind, state, hyper_at):
    """The loop all three optimizers share: gradient at (x, i), the callback sees (x, i, g) before the
    update, then one fused update kernel; ``hyper_at(i)`` gives the iteration's scalars."""
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        x = _step(kind, x, g, state[0], state[1], hyper_at(i))
    return x


@unflatten_optimizer
def sgd(grad, x, callback=None, num_iters=200, step_size=0.1, mass=0.9):
    """Gradient descent with momentum: velocity = mass * velocity - (1 - mass) * g; x += step_size * velocity.
    ``grad(x, i)`` receives the iteration number (optimizers.py:33-45)."""
    velocity = D.zeros((len(x),), _F64)
    return _descend(grad, x, callback, num_iters, _lib.OPT_SGD, (velocity, None),
                    lambda i: (mass, 1.0 - mass, step_size))


@unflatten_optimizer
def rmsprop(grad, x, callback=None, num_iters=100, step_size=0.1, gamma=0.9, eps=10**-8):
    """RMSprop: a running average of squared gradients (started at one) scales each step
    (optimizers.py:48-59)."""
    mean_square = D.ones((len(x),), _F64)
    return _descend(grad, x, callback, num_iters, _lib.OPT_RMSPROP, (mean_square, None),
                    lambda i: (gamma, 1 - gamma, step_size, eps))


@unflatten_optimizer
def adam(grad, x, callback=None, num_iters=100, step_size=0.001, b1=0.9, b2=0.999, eps=10**-8):
    """Adam (Kingma & Ba, arXiv:1412.6980): bias-corrected running first and second moments
    (optimizers.py:62-75)."""
    moments = (D.zeros((len(x),), _F64), D.zeros((len(x),), _F64))
    return _descend(grad, x, callback, num_iters, _lib.OPT_ADAM, moments,
                    lambda i: (1 - b1, b1, 1 - b2, b2, 1 - b1 ** (i + 1), 1 - b2 ** (i + 1), step_size, eps))
