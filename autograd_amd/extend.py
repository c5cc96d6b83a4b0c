"""Extension API: everything needed to add a primitive or a value type.

Same names as the reference's autograd/extend.py:2-16.
"""

from .core import (  # noqa: F401
    JVPNode,
    SparseObject,
    VJPNode,
    VSpace,
    def_linear,
    defjvp,
    defjvp_argnum,
    defjvp_argnums,
    defvjp,
    defvjp_argnum,
    defvjp_argnums,
    vspace,
)
from .tracer import Box, notrace_primitive, primitive, register_notrace  # noqa: F401
