"""Translate the package's host-side modules to C extension modules (``python -m autograd_amd.build_host``).

The listed ``.py`` files are compiled as they are, with Cython in pure-Python mode (no annotations are used for
typing, every function keeps Python call semantics), into ``autograd_amd/_ext/`` next to a manifest of their
source hashes; ``_compiled.py`` serves them at import while the hashes still match.  User programs (``configs.py``,
anything a caller writes) are not in the list: they stay interpreted, as a caller's code would be.
"""

import json
import os
import shutil
import subprocess
import sys
import sysconfig
import tempfile
from concurrent.futures import ThreadPoolExecutor

from . import _compiled

# the tracer, the backward pass, the rule tables, the value type and the launch marshalling
MODULES = (
    "tracer", "core", "util", "wrap_util", "builtins", "differential_operators", "_lib",
    "numpy.devarray", "numpy.fusion", "numpy.wrapper", "numpy.vjps", "numpy.jvps", "numpy.boxes", "numpy.vspaces",
    "scipy.special", "scipy.signal", "misc.flatten", "misc.optimizers",
)
_DIRECTIVES = ("language_level=3", "annotation_typing=False", "binding=True", "always_allow_keywords=True")


def _compile_one(name, work, out_dir):
    full = f"{_compiled._PACKAGE}.{name}"
    source = _compiled.source_path(full)
    stem = name.replace(".", "_")
    c_file = os.path.join(work, stem + ".c")
    cython = [sys.executable, "-m", "cython", "--module-name", full, "-o", c_file]
    for directive in _DIRECTIVES:
        cython += ["-X", directive]
    subprocess.run(cython + [source], check=True)
    target = stem + sysconfig.get_config_var("EXT_SUFFIX")
    cc = os.environ.get("CC", "gcc")
    subprocess.run([cc, "-shared", "-fPIC", "-O2", "-fwrapv", "-fno-strict-aliasing", "-DNDEBUG", "-w",
                    "-I", sysconfig.get_paths()["include"], c_file, "-o", os.path.join(out_dir, target)], check=True)
    return full, {"file": target, "sha256": _compiled.source_hash(source)}


def build(jobs=None):
    """Compile every listed module; returns the manifest.  Replaces ``_ext/`` only when all of them built."""
    jobs = jobs or min(8, os.cpu_count() or 1)
    final = _compiled._DIR
    with tempfile.TemporaryDirectory() as work:
        staged = os.path.join(work, "staged")
        os.makedirs(staged)
        with ThreadPoolExecutor(jobs) as pool:
            built = dict(pool.map(lambda name: _compile_one(name, work, staged), MODULES))
        manifest = {"python": sys.implementation.cache_tag, "modules": built}
        with open(os.path.join(staged, "manifest.json"), "w") as f:
            json.dump(manifest, f, indent=1, sort_keys=True)
        shutil.rmtree(final, ignore_errors=True)
        shutil.copytree(staged, final)
    return manifest


def clean():
    shutil.rmtree(_compiled._DIR, ignore_errors=True)


if __name__ == "__main__":
    if sys.argv[1:] == ["clean"]:
        clean()
    else:
        print(f"compiled {len(build()['modules'])} host modules into {_compiled._DIR}")
