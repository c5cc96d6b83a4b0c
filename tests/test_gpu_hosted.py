"""The device value type hosted by an installed HIPS/autograd instead of this package's own tracer.

With ``AUTOGRAD_AMD_HOST=autograd`` the package registers ``DevArrayBox`` / ``DevArrayVSpace`` through the
reference's ``Box.register`` / ``VSpace.register`` (autograd/tracer.py:176-180, autograd/core.py:281-286) and
attaches its rules with the reference's ``defvjp`` / ``defjvp``; ``autograd.grad`` then differentiates device
programs.  Needs the ``autograd`` package to be importable, so it is skipped where it is not installed.  The
choice of host is made at import time: the check runs in a child process.
"""

import importlib.util
import os
import subprocess
import sys

import pytest

PROGRAM = r"""
import numpy as onp
import autograd, autograd.numpy as anp, autograd.scipy.special as rspecial
import autograd_amd as ag, autograd_amd.numpy as dnp
from autograd_amd.scipy.special import logsumexp
from autograd.tracer import Box
from autograd.core import VSpace

assert issubclass(dnp.DevArrayBox, Box) and issubclass(dnp.DevArrayVSpace, VSpace)
assert Box.type_mappings[dnp.DevArray] is dnp.DevArrayBox and dnp.DevArray in VSpace.mappings
rs = onp.random.RandomState(0)
A, b, c = rs.randn(50, 70), rs.randn(70), rs.randn(50)

def program(np, lse):
    return lambda A, b, c: (np.sum(np.tanh(A * b[None, :] + c[:, None]) ** 2) + np.sum(lse(A * 2.0, axis=1))
                            + np.sum(np.dot(A, b) * c))

want = autograd.grad(program(anp, rspecial.logsumexp), (0, 1, 2))(A, b, c)
got = autograd.grad(program(dnp, logsumexp), (0, 1, 2))(dnp.asarray(A), dnp.asarray(b), dnp.asarray(c))
for w, g in zip(want, got):
    assert onp.allclose(g.numpy(), w, rtol=1e-12, atol=1e-13), onp.abs(g.numpy() - w).max()
x = rs.randn(6)
H = ag.hessian(lambda v: dnp.sum(dnp.sin(v) * v[::-1]))(dnp.asarray(x))  # stays on the device
assert onp.allclose(H.numpy(), autograd.hessian(lambda v: anp.sum(anp.sin(v) * v[::-1]))(x), rtol=1e-12, atol=1e-13)
assert onp.allclose(ag.grad(program(dnp, logsumexp))(dnp.asarray(A), dnp.asarray(b), dnp.asarray(c)).numpy(), want[0], rtol=1e-12, atol=1e-13)
tangent = autograd.make_jvp(lambda v: dnp.tanh(v) * 2.0)(dnp.asarray(x))(dnp.asarray(onp.ones(6)))[1]
assert onp.allclose(tangent.numpy(), 2.0 / onp.cosh(x) ** 2, rtol=1e-12)
tree = autograd.grad(lambda p: dnp.sum(p["w"] ** 2) + dnp.sum(p["v"][0]))({"w": dnp.asarray(x), "v": [dnp.asarray(x)]})
assert onp.allclose(tree["w"].numpy(), 2 * x) and onp.allclose(tree["v"][0].numpy(), 1.0)
print("hosted ok")
"""


@pytest.mark.gpu
@pytest.mark.skipif(importlib.util.find_spec("autograd") is None, reason="HIPS/autograd is not installed here")
def test_device_arrays_differentiate_under_the_installed_autograd():
    env = dict(os.environ, AUTOGRAD_AMD_HOST="autograd")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env["PYTHONPATH"] = root + os.pathsep + env.get("PYTHONPATH", "")
    done = subprocess.run([sys.executable, "-c", PROGRAM], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "hosted ok" in done.stdout, done.stderr[-2000:]


def test_an_unknown_host_is_refused_at_import():
    env = dict(os.environ, AUTOGRAD_AMD_HOST="somethingelse")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env["PYTHONPATH"] = root + os.pathsep + env.get("PYTHONPATH", "")
    done = subprocess.run([sys.executable, "-c", "import autograd_amd"], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode != 0 and "AUTOGRAD_AMD_HOST" in done.stderr
