"""The compiled copies of the host-side modules (``autograd_amd/_compiled.py``, ``build_host.py``): they are used
only while they match their sources, and the interpreted sources are what runs otherwise."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MANIFEST = os.path.join(ROOT, "autograd_amd", "_ext", "manifest.json")

PROBE = r"""
import json, autograd_amd, autograd_amd.tracer as T, autograd_amd.numpy.wrapper as W
from autograd_amd import _compiled
from autograd_amd.numpy.devarray import broadcast_shapes
assert broadcast_shapes((3, 1), (4,)) == (3, 4)
print(json.dumps({"status": _compiled.status(), "tracer": T.__file__, "wrapper": W.__file__}))
"""


def _probe(**env):
    full = dict(os.environ, PYTHONPATH=ROOT, **env)
    import torch  # noqa: F401  (see the GPU test below)

    done = subprocess.run([sys.executable, "-W", "ignore", "-c", PROBE], env=full, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr
    return json.loads(done.stdout.strip().splitlines()[-1])


def test_pure_python_on_request():
    seen = _probe(AUTOGRAD_AMD_PURE_PYTHON="1")
    assert seen["status"]["mode"] == "python" and seen["tracer"].endswith("tracer.py") and seen["wrapper"].endswith("wrapper.py")


@pytest.mark.skipif(not os.path.exists(MANIFEST), reason="host modules not compiled (python -m autograd_amd.build_host)")
def test_compiled_modules_are_served_while_they_match_their_sources(monkeypatch):
    from autograd_amd import _compiled, build_host

    with open(MANIFEST) as f:
        manifest = json.load(f)
    assert set(manifest["modules"]) == {"autograd_amd." + name for name in build_host.MODULES}
    monkeypatch.delenv("AUTOGRAD_AMD_PURE_PYTHON", raising=False)
    seen = _probe(AUTOGRAD_AMD_PURE_PYTHON="")
    table, reason = _compiled._usable()
    if table is None:  # a source was edited after the build: everything must come from the sources
        assert seen["status"]["mode"] == "python" and seen["tracer"].endswith("tracer.py"), reason
    else:
        assert seen["status"]["mode"] == "compiled" and len(seen["status"]["modules"]) == len(build_host.MODULES)
        assert os.sep + "_ext" + os.sep in seen["tracer"] and os.sep + "_ext" + os.sep in seen["wrapper"]
    # one changed source switches every compiled module off
    real = _compiled.source_hash
    monkeypatch.setattr(_compiled, "source_hash", lambda path: "0" * 64 if path.endswith("util.py") else real(path))
    table, reason = _compiled._usable()
    assert table is None and "changed after it was compiled" in reason  # (names util.py, or a source edited since the build)
    monkeypatch.setenv("AUTOGRAD_AMD_PURE_PYTHON", "1")
    assert _compiled._usable() == (None, "AUTOGRAD_AMD_PURE_PYTHON is set")


DIGEST = r"""
import hashlib, json
import numpy as onp
import autograd_amd as ag, autograd_amd.numpy as np
from autograd_amd import _compiled, configs
from autograd_amd.scipy.special import logsumexp

be = configs.device_backend()
digest = hashlib.sha256()
out = configs.run_config("bcast", be, configs.bcast_inputs(rows=96, cols=200))
for key in sorted(out):
    digest.update(onp.ascontiguousarray(out[key]).tobytes())
inp = configs.rnn_inputs(seq_len=5, batch=3, input_size=4, state_size=6, output_size=4)
grads = configs.rnn_program(be)["grad"](configs.tree_map(be.put, inp["params"]), be.put(inp["inputs"]), be.put(inp["targets"]))
for key in sorted(grads):
    digest.update(grads[key].numpy().tobytes())
x = np.array(onp.linspace(-1.0, 1.0, 7))
H = ag.hessian(lambda v: np.sum(np.tanh(v) * v[::-1]) + logsumexp(v * 2.0))(x)
J = ag.make_jvp(lambda v: np.sin(v) @ v)(x)(np.ones(7))[1]
digest.update(H.numpy().tobytes() + J.numpy().tobytes())
print(json.dumps({"mode": _compiled.status()["mode"], "digest": digest.hexdigest()}))
"""


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(MANIFEST), reason="host modules not compiled (python -m autograd_amd.build_host)")
def test_compiled_and_interpreted_host_modules_give_the_same_bits():
    """The same sources, compiled or interpreted, launch the same kernels on the same operands: gradients of the
    broadcast + logsumexp workload and of a small recurrent net, a Hessian and a forward-mode product, bit for bit."""
    import torch  # noqa: F401  (loaded here first: on a fresh machine the first load takes minutes, the children then find it cached)

    seen = {}
    for pure in ("", "1"):
        env = dict(os.environ, PYTHONPATH=ROOT, AUTOGRAD_AMD_PURE_PYTHON=pure)
        done = subprocess.run([sys.executable, "-W", "ignore", "-c", DIGEST], env=env, capture_output=True, text=True, timeout=600)
        assert done.returncode == 0, done.stderr
        result = json.loads(done.stdout.strip().splitlines()[-1])
        seen[result["mode"]] = result["digest"]
    assert set(seen) == {"compiled", "python"} and seen["compiled"] == seen["python"], seen
