"""``import oracle.anp as np``: the oracle's traced NumPy namespace, fully wired.

Importing this module registers the ndarray box/vspace and every rule.
TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

from . import np_boxes, np_jvps, np_vjps  # noqa: F401  (registration side effects)
from .np_namespace import *  # noqa: F401,F403
from .np_namespace import (  # noqa: F401
    _array_from_scalar_or_array,
    _astype,
    _primitive_mean,
    _primitive_std,
    _primitive_var,
    array,
    array_from_args,
    concatenate,
    concatenate_args,
    hstack,
    metadata,
    stack,
    vstack,
    where,
)
from .np_vjps import untake  # noqa: F401
from .special import logsumexp  # noqa: F401
