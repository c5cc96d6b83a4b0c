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
    done = subprocess.run([sys.executable, "-W", "ignore", "-c", PROBE], env=full, capture_output=True, text=True, timeout=120)
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
    assert table is None and "util.py changed" in reason
    monkeypatch.setenv("AUTOGRAD_AMD_PURE_PYTHON", "1")
    assert _compiled._usable() == (None, "AUTOGRAD_AMD_PURE_PYTHON is set")
