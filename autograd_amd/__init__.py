"""MI355X-native execution path for autograd-style differentiation.

The tracer, the differential operators and the extension API have the
reference's names and semantics (autograd/__init__.py:1-24); array values live
on the GPU as ``autograd_amd.numpy`` device arrays whose operations and
derivative rules launch hand-written HIP kernels.

    import autograd_amd.numpy as np
    from autograd_amd import grad, elementwise_grad, make_hvp
"""

from .builtins import dict, isinstance, list, tuple, type  # noqa: A004,F401
from .differential_operators import (  # noqa: F401
    checkpoint,
    deriv,
    elementwise_grad,
    grad,
    grad_and_aux,
    grad_named,
    hessian,
    hessian_tensor_product,
    hessian_vector_product,
    holomorphic_grad,
    jacobian,
    make_ggnvp,
    make_hvp,
    make_jvp,
    make_jvp_reversemode,
    make_vjp,
    multigrad_dict,
    tensor_jacobian_product,
    value_and_grad,
    vector_jacobian_product,
)
from .extend import primitive  # noqa: F401
from .graphs import capture  # noqa: F401

__version__ = "0.1.0"
