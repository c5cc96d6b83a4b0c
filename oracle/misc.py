"""CPU restatement of the reference's container flattening and optimizers.  TEST INFRASTRUCTURE.

Restates autograd/misc/flatten.py:11-35 and autograd/misc/optimizers.py:15-75 on the oracle's NumPy
namespace (``oracle.anp``): the same nesting of concatenations and, in the update formulas, the same
NumPy expressions in the same order, so that on the same inputs it computes what the reference
computes to the bit, including NumPy's dtype promotion (the optimizers' state is float64).
Pinned by tests/golden/reference_next.npz, written by the real reference.
"""

import oracle.anp as np
from autograd_amd import make_vjp
from autograd_amd.builtins import type
from autograd_amd.wrap_util import wraps


# ---- flatten (misc/flatten.py:11-35) ---------------------------------------------------------------
def _joined(parts):
    """One vector from the flattened children; an empty container gives an empty float64 vector (30-32)."""
    parts = list(parts)
    if not parts:
        return np.array([])
    return np.concatenate(parts)


def _flatten(value):
    """Depth first, every container level joined on its own; dict values in sorted-key order (20-27)."""
    kind = type(value)
    if kind is dict:
        return _joined(_flatten(value[key]) for key in sorted(value))
    if kind in (list, tuple):
        return _joined(_flatten(item) for item in value)
    return np.ravel(value)


def flatten(value):
    """``(flat vector, unflatten)``: unflatten is the cotangent map of the flattening (11-17)."""
    unflatten, flat = make_vjp(_flatten)(value)
    return flat, unflatten


# ---- optimizers (misc/optimizers.py:15-75) -------------------------------------------------------
def unflatten_optimizer(optimize):
    """Lift an optimizer on flat vectors to nested containers (15-31)."""

    @wraps(optimize)
    def lifted(grad, x0, callback=None, *args, **kwargs):
        flat_x0, unflatten = flatten(x0)
        flat_callback = (lambda x, i, g: callback(unflatten(x), i, unflatten(g))) if callback else None
        return unflatten(optimize(lambda x, i: flatten(grad(unflatten(x), i))[0], flat_x0, flat_callback, *args, **kwargs))

    return lifted


def _run(grad, x, callback, num_iters, update):
    """Iteration shared by the three optimizers: gradient, callback on (x, i, g), then the update."""
    for i in range(num_iters):
        g = grad(x, i)
        if callback:
            callback(x, i, g)
        x = update(x, g, i)
    return x


@unflatten_optimizer
def sgd(grad, x, callback=None, num_iters=200, step_size=0.1, mass=0.9):
    state = {"velocity": np.zeros(len(x))}  # optimizers.py:38

    def update(x, g, i):  # optimizers.py:43-44
        state["velocity"] = mass * state["velocity"] - (1.0 - mass) * g
        return x + step_size * state["velocity"]

    return _run(grad, x, callback, num_iters, update)


@unflatten_optimizer
def rmsprop(grad, x, callback=None, num_iters=100, step_size=0.1, gamma=0.9, eps=10**-8):
    state = {"mean_square": np.ones(len(x))}  # optimizers.py:53

    def update(x, g, i):  # optimizers.py:58-59
        state["mean_square"] = state["mean_square"] * gamma + g**2 * (1 - gamma)
        return x - step_size * g / (np.sqrt(state["mean_square"]) + eps)

    return _run(grad, x, callback, num_iters, update)


@unflatten_optimizer
def adam(grad, x, callback=None, num_iters=100, step_size=0.001, b1=0.9, b2=0.999, eps=10**-8):
    state = {"m": np.zeros(len(x)), "v": np.zeros(len(x))}  # optimizers.py:64-65

    def update(x, g, i):  # optimizers.py:70-74: moment estimates, their bias correction, the step
        state["m"] = (1 - b1) * g + b1 * state["m"]
        state["v"] = (1 - b2) * (g**2) + b2 * state["v"]
        m_corrected = state["m"] / (1 - b1 ** (i + 1))
        v_corrected = state["v"] / (1 - b2 ** (i + 1))
        return x - step_size * m_corrected / (np.sqrt(v_corrected) + eps)

    return _run(grad, x, callback, num_iters, update)
