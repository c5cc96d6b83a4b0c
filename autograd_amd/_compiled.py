"""Compiled copies of the package's host-side modules.

Every eager evaluation is bound by the host: the tracer (autograd/tracer.py:44-99 of the reference, ``tracer.py``
here), the backward pass, the rule closures and the launch marshalling run a few thousand Python function calls per
evaluation, about 13 us per primitive, while the kernels they launch finish sooner.  ``build_host.py`` therefore
translates the same ``.py`` sources, unchanged, to C extension modules with Cython and puts them under
``autograd_amd/_ext/`` together with a manifest of the source hashes; this module makes ``import`` resolve the
listed names to those extensions.  The sources stay the single definition of the behaviour:

* a module is served from its compiled copy only while the manifest's hash of EVERY listed source equals the
  file's current hash (one edited source switches all of them off, with a warning, so stale code never runs);
* without the ``_ext`` folder, under another Python version, or with ``AUTOGRAD_AMD_PURE_PYTHON=1`` the ``.py``
  files are imported as usual;
* modules that a hosting ``autograd`` provides (``AUTOGRAD_AMD_HOST``) are already in ``sys.modules`` and are left
  alone.

``status()`` says which of the two is in use (``bench.py`` reports it).
"""

import hashlib
import importlib.abc
import importlib.machinery
import importlib.util
import json
import os
import sys
import warnings

_PACKAGE = __name__.rsplit(".", 1)[0]
_ROOT = os.path.dirname(os.path.abspath(__file__))
_DIR = os.path.join(_ROOT, "_ext")
_STATE = {"mode": "python", "reason": "not installed", "modules": ()}


def source_path(module):
    """``autograd_amd.numpy.wrapper`` -> ``<package dir>/numpy/wrapper.py``."""
    return os.path.join(_ROOT, *module.split(".")[1:]) + ".py"


def source_hash(path):
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


class _Finder(importlib.abc.MetaPathFinder):
    def __init__(self, table):
        self.table = table  # full module name -> path of its extension file

    def find_spec(self, fullname, path=None, target=None):
        file = self.table.get(fullname)
        if file is None:
            return None
        loader = importlib.machinery.ExtensionFileLoader(fullname, file)
        return importlib.util.spec_from_file_location(fullname, file, loader=loader)


def _usable():
    """``(table, reason)``: the extension file of every listed module, or None and why not."""
    if os.environ.get("AUTOGRAD_AMD_PURE_PYTHON", "").strip() not in ("", "0"):
        return None, "AUTOGRAD_AMD_PURE_PYTHON is set"
    manifest_path = os.path.join(_DIR, "manifest.json")
    if not os.path.exists(manifest_path):
        return None, "no compiled modules (run `python -m autograd_amd.build_host`)"
    with open(manifest_path) as f:
        manifest = json.load(f)
    if manifest.get("python") != sys.implementation.cache_tag:
        return None, f"compiled for {manifest.get('python')}, this is {sys.implementation.cache_tag}"
    table = {}
    for module, entry in manifest["modules"].items():
        file = os.path.join(_DIR, entry["file"])
        if not os.path.exists(file):
            return None, f"{entry['file']} is missing"
        if source_hash(source_path(module)) != entry["sha256"]:
            return None, f"{os.path.relpath(source_path(module), _ROOT)} changed after it was compiled (rebuild)"
        table[module] = file
    return table, ""


def install():
    """Serve the listed modules from their compiled copies.  Must run before they are first imported."""
    table, reason = _usable()
    if table is None:
        _STATE.update(mode="python", reason=reason, modules=())
        if "changed after" in reason or "missing" in reason:
            warnings.warn(f"autograd_amd: compiled host modules are not used: {reason}", stacklevel=2)
        return
    table = {name: file for name, file in table.items() if name not in sys.modules}
    sys.meta_path.insert(0, _Finder(table))
    _STATE.update(mode="compiled", reason="", modules=tuple(sorted(table)))


def status():
    """``{"mode": "compiled" | "python", "reason": ..., "modules": (...)}``."""
    return dict(_STATE)
