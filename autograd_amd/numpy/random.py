"""``autograd_amd.numpy.random``: NumPy's host generators, results uploaded to the device.

The reference wraps ``numpy.random`` unchanged (autograd/numpy/random.py:1-5) so that user code
writes ``npr.RandomState(0).randn(m, n)``; draws are not differentiable.  Here the same generators
run on the host - the same seed gives the same numbers as with the reference - and every array
they return is uploaded once and handed back as a device array (float64 unless the generator
says otherwise, as in NumPy).  Scalars stay Python/NumPy scalars.
"""

import numpy as _onp
import numpy.random as _npr

from .devarray import from_numpy as _from_numpy


def _upload(result):
    if isinstance(result, _onp.ndarray) and result.dtype.kind in "fiub":
        return _from_numpy(result)
    if isinstance(result, tuple):
        return tuple(_upload(r) for r in result)
    return result


def _host(x):
    from .devarray import DevArray

    return x.numpy() if isinstance(x, DevArray) else x


def _wrap(fn):
    def wrapped(*args, **kwargs):
        return _upload(fn(*[_host(a) for a in args], **{k: _host(v) for k, v in kwargs.items()}))

    wrapped.__name__ = getattr(fn, "__name__", "random_function")
    wrapped.__doc__ = getattr(fn, "__doc__", None)
    return wrapped


class RandomState:
    """``numpy.random.RandomState`` whose array draws land on the device."""

    def __init__(self, *args, **kwargs):
        self._rs = _npr.RandomState(*args, **kwargs)

    def __getattr__(self, name):
        attr = getattr(self._rs, name)
        return _wrap(attr) if callable(attr) else attr


for _name in (
    "rand randn random random_sample uniform normal standard_normal randint permutation choice beta gamma "
    "exponential binomial poisson laplace logistic lognormal multivariate_normal"
).split():
    globals()[_name] = _wrap(getattr(_npr, _name))

seed = _npr.seed
get_state = _npr.get_state
set_state = _npr.set_state


def shuffle(x):
    raise TypeError("device arrays are immutable: use permutation() instead of shuffle()")
