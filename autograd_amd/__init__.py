"""MI355X-native execution path for autograd-style differentiation.

The tracer, the differential operators and the extension API have the
reference's names and semantics (autograd/__init__.py:1-24); array values live
on the GPU as ``autograd_amd.numpy`` device arrays whose operations and
derivative rules launch hand-written HIP kernels.

    import autograd_amd.numpy as np
    from autograd_amd import grad, elementwise_grad, make_hvp
"""

from . import _host

_host.install()  # an installed HIPS/autograd may host the value type instead of this package's own tracer

from . import _compiled  # noqa: E402

_compiled.install()  # the host-side modules come from their compiled copies when those are built and current

from . import differential_operators as _operators  # noqa: E402
from .builtins import dict, isinstance, list, tuple, type  # noqa: A004,E402,F401
from .core import primitive_with_deprecation_warnings as primitive  # noqa: E402,F401
from .graphs import capture  # noqa: E402,F401

# the differential operators of autograd/__init__.py:1-22, under the same names
_OPERATORS = ("grad elementwise_grad value_and_grad grad_and_aux grad_named multigrad_dict deriv holomorphic_grad "
              "jacobian hessian make_vjp make_jvp make_jvp_reversemode make_hvp make_ggnvp hessian_tensor_product "
              "hessian_vector_product tensor_jacobian_product vector_jacobian_product checkpoint").split()
for _name in _OPERATORS:
    globals()[_name] = getattr(_operators, _name)

__version__ = "0.1.0"
