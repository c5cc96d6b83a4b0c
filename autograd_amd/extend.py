"""Extension API: everything needed to add a primitive or a value type.

The names the reference exposes from autograd/extend.py:2-16, taken from where they are defined here.
"""

from . import core as _core
from . import tracer as _tracer

_FROM_CORE = ("VSpace vspace SparseObject VJPNode JVPNode defvjp defvjp_argnum defvjp_argnums "
              "defjvp defjvp_argnum defjvp_argnums def_linear").split()
_FROM_TRACER = "Box primitive notrace_primitive register_notrace".split()

for _name in _FROM_CORE:
    globals()[_name] = getattr(_core, _name)
for _name in _FROM_TRACER:
    globals()[_name] = getattr(_tracer, _name)

__all__ = _FROM_CORE + _FROM_TRACER
