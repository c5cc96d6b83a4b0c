"""CPU restatement of the reference's container flattening and optimizers.  TEST INFRASTRUCTURE.

Follows autograd/misc/flatten.py:11-35 and autograd/misc/optimizers.py:15-75 line by line on the
oracle's NumPy namespace (``oracle.anp``), so that on the same inputs it computes what the
reference computes, including NumPy's dtype promotion (the optimizers' state is float64).
Pinned by tests/golden/reference_next.npz, written by the real reference.
"""

import oracle.anp as np
from autograd_amd import make_vjp
from autograd_amd.builtins import type
from autograd_amd.wrap_util import wraps


def flatten(value):  # misc/flatten.py:11-17
    unflatten, flat_value = make_vjp(_flatten)(value)
    return flat_value, unflatten


def _flatten(value):  # misc/flatten.py:20-27
    t = type(value)
    if t in (list, tuple):
        return _concatenate(map(_flatten, value))
    elif t is dict:
        return _concatenate(_flatten(value[k]) for k in sorted(value))
    else:
        return np.ravel(value)


def _concatenate(lst):  # misc/flatten.py:30-32
    lst = list(lst)
    return np.concatenate(lst) if lst else np.array([])


def unflatten_optimizer(optimize):  # misc/optimizers.py:15-31
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


@unflatten_optimizer
def sgd(grad, x, callback=None, num_iters=200, step_size=0.1, mass=0.9):  # misc/optimizers.py:34-47
    velocity = np.zeros(len(x))
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        velocity = mass * velocity - (1.0 - mass) * g
        x = x + step_size * velocity
    return x


@unflatten_optimizer
def rmsprop(grad, x, callback=None, num_iters=100, step_size=0.1, gamma=0.9, eps=10**-8):  # misc/optimizers.py:50-60
    avg_sq_grad = np.ones(len(x))
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        avg_sq_grad = avg_sq_grad * gamma + g**2 * (1 - gamma)
        x = x - step_size * g / (np.sqrt(avg_sq_grad) + eps)
    return x


@unflatten_optimizer
def adam(grad, x, callback=None, num_iters=100, step_size=0.001, b1=0.9, b2=0.999, eps=10**-8):  # misc/optimizers.py:63-75
    m = np.zeros(len(x))
    v = np.zeros(len(x))
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        m = (1 - b1) * g + b1 * m
        v = (1 - b2) * (g**2) + b2 * v
        mhat = m / (1 - b1 ** (i + 1))
        vhat = v / (1 - b2 ** (i + 1))
        x = x - step_size * mhat / (np.sqrt(vhat) + eps)
    return x
