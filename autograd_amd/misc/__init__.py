"""Helpers either side of the gradient evaluation: container flattening and optimizers
(autograd/misc/__init__.py of the reference exports ``flatten`` and ``const_graph``)."""

from .flatten import flatten, flatten_func  # noqa: F401
from .tracers import const_graph  # noqa: F401
