"""Which tracer hosts the device value type.

By default the package runs on its own tracer (``tracer.py``, ``core.py``).  With

    AUTOGRAD_AMD_HOST=autograd

in the environment before the first import, an installed HIPS/autograd hosts it instead: the names
``autograd_amd.tracer / core / extend / builtins`` then resolve to the installed package's modules, so that

* ``DevArrayBox.register(DevArray)`` and ``DevArrayVSpace.register(DevArray)`` (numpy/boxes.py, numpy/vspaces.py)
  are the calls of autograd/tracer.py:176-180 and autograd/core.py:281-286 on the reference's own tables,
* every rule in numpy/vjps.py, numpy/jvps.py, scipy/special.py and scipy/signal.py is attached with the
  reference's ``defvjp`` / ``defjvp`` (autograd/core.py:45-81, 162-183), and
* ``autograd.grad`` and the other operators of autograd/differential_operators.py differentiate programs written
  against ``autograd_amd.numpy`` with the reference's ``trace`` / ``backward_pass``, side by side with
  ``autograd.numpy`` programs on host arrays.  This package's own operators (``autograd_amd.grad`` ...) run on the
  hosting core too; they differ from the reference's only where those are tied to host NumPy (``jacobian`` stacks
  its rows with ``autograd.numpy``, differential_operators.py:57-75, which brings device arrays to the host).

What this package's own core adds on top of the reference's is switched off under a foreign host: cotangents are
not stacked for ``jacobian`` (the reference's loop runs instead) and the cyclic collector is left alone.
"""

import os
import sys
import types

HOST = os.environ.get("AUTOGRAD_AMD_HOST", "").strip()


def _reference_core(package):
    import autograd.core as rcore

    core = types.ModuleType(package + ".core", "autograd.core plus inert stand-ins for the stacked backward pass")
    core.__dict__.update({k: v for k, v in vars(rcore).items() if not k.startswith("__")})

    class NotBatchable(Exception):
        pass

    class BatchMode:
        active = 0  # never set: the hosting core has no stacked pass

    def batch_safe(*primitives):
        return None

    def make_vjp_and_batched(fun, x):
        pull_back, ans = rcore.make_vjp(fun, x)
        return pull_back, None, ans  # no stacked pass under the hosting core: callers loop over basis vectors

    core.NotBatchable, core.BatchMode, core.batch_safe = NotBatchable, BatchMode, batch_safe
    core.make_vjp_and_batched = make_vjp_and_batched
    return core


def install():
    """Alias this package's tracer modules to the hosting package's.  Must run before they are first imported."""
    if not HOST:
        return None
    if HOST != "autograd":
        raise ImportError(f"AUTOGRAD_AMD_HOST={HOST!r}: the only foreign host is 'autograd'")
    package = __name__.rsplit(".", 1)[0]
    already = [m for m in ("tracer", "core", "extend") if package + "." + m in sys.modules]
    if already:
        raise ImportError("AUTOGRAD_AMD_HOST must be set before autograd_amd is first imported")
    import autograd
    import autograd.builtins
    import autograd.extend
    import autograd.tracer

    sys.modules[package + ".tracer"] = autograd.tracer
    sys.modules[package + ".core"] = _reference_core(package)
    sys.modules[package + ".extend"] = autograd.extend
    sys.modules[package + ".builtins"] = autograd.builtins
    return autograd
