"""Flatten nested containers of device arrays into one flat device vector and back.

Same contract as the reference (autograd/misc/flatten.py:11-35): ``flatten(value)`` returns the
1-d vector and an ``unflatten`` function, built as the VJP of the flattening so that both
directions are differentiable; dict values are taken in sorted-key order.  Everything stays in
HBM: flattening is one strided copy kernel per leaf into the result (``concatenate``),
unflattening is slice + reshape views and launches nothing.
"""

import autograd_amd.numpy as np
from autograd_amd import make_vjp
from autograd_amd.builtins import type


def flatten(value):
    """Flattens any nesting of tuples, lists, or dicts, with device arrays or scalars inside.
    Returns a 1-d device array and an unflatten function."""
    unflatten, flat_value = make_vjp(_flatten)(value)
    return flat_value, unflatten


def _flatten(value):
    t = type(value)
    if t in (list, tuple):
        return _concatenate(map(_flatten, value))
    elif t is dict:
        return _concatenate(_flatten(value[k]) for k in sorted(value))
    else:
        return np.ravel(value)


def _concatenate(lst):
    lst = list(lst)
    return np.concatenate(lst) if lst else np.array([])


def flatten_func(func, example):
    _ex, unflatten = flatten(example)
    _func = lambda _x, *args: flatten(func(unflatten(_x), *args))[0]  # noqa: E731
    return _func, unflatten, _ex
