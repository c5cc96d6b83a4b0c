"""``import autograd_amd.numpy as np``: NumPy-named functions on MI355X device arrays.

The counterpart of ``autograd.numpy`` (reference autograd/numpy/__init__.py): every function
is a traced primitive with reverse- and forward-mode rules; values are ``DevArray`` s in HBM and
every arithmetic step is a hand-written HIP kernel.  Host data enters with ``np.asarray`` /
``np.array`` (one upload) and leaves with ``np.to_numpy`` (or ``DevArray.numpy()``).
"""

from . import boxes, vspaces, vjps, jvps  # noqa: F401  (registration side effects; order matters)
from .boxes import DevArrayBox  # noqa: F401
from .devarray import DevArray, from_numpy  # noqa: F401
from .vspaces import DevArrayVSpace  # noqa: F401
from .wrapper import *  # noqa: F401,F403
from .wrapper import (  # noqa: F401
    __version__,
    _array_from_scalar_or_array,
    _astype,
    _primitive_mean,
    _primitive_std,
    _primitive_var,
    abs,
    max,
    min,
    sum,
)
from .vjps import untake  # noqa: F401
from . import random  # noqa: E402,F401  (``np.random`` without a separate import, autograd/numpy/__init__.py:6)
