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


def _leaves_in_order(value):
    """The leaves of ``value`` from left to right, each as a 1-d array (boxes stay boxes)."""
    kind = type(value)  # sees through boxes
    if kind is dict:
        children = [value[key] for key in sorted(value)]
    elif kind is list or kind is tuple:
        children = value
    else:
        return [np.ravel(value)]
    found = []
    for child in children:
        found.extend(_leaves_in_order(child))
    # an empty container flattens to an empty float64 vector (and promotes its neighbours like one)
    return found if found else [np.array([])]


def _flatten(value):
    pieces = _leaves_in_order(value)
    return pieces[0] if len(pieces) == 1 and type(value) not in (list, tuple, dict) else np.concatenate(pieces)


def flatten(value):
    """Flattens any nesting of tuples, lists, or dicts, with device arrays or scalars inside.
    Returns a 1-d device array and an unflatten function: unflattening a vector is the cotangent map
    of flattening, which hands every leaf its slice in the leaf's shape."""
    unflatten, flat = make_vjp(_flatten)(value)
    return flat, unflatten


def flatten_func(func, example):
    """``func`` on containers -> the same function on flat vectors (and the flat example)."""
    flat_example, unflatten = flatten(example)

    def on_vectors(flat, *args):
        return flatten(func(unflatten(flat), *args))[0]

    return on_vectors, unflatten, flat_example
