"""The CPU oracle reproduces the real reference bit for bit.

``tests/golden/reference_vectors.npz`` was written by HIPS/autograd itself (see
tests/golden/make_fixtures.py).  The oracle follows the reference's formulas,
operation order and replay/accumulation order, and runs on the same NumPy, so
every array must be IDENTICAL (values and dtype), not merely close.
"""

import os

import numpy as np
import pytest

from autograd_amd import configs
from cases import SMALL, extra_cases, flatten
from conftest import oracle_backend

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))


def _same(name, got):
    want = GOLD[name]
    got = np.asarray(got)
    assert got.dtype == want.dtype, f"{name}: dtype {got.dtype} != reference {want.dtype}"
    assert got.shape == want.shape, f"{name}: shape {got.shape} != reference {want.shape}"
    assert np.array_equal(got, want, equal_nan=True), (
        f"{name}: max |diff| {np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))}"
    )


@pytest.mark.parametrize("name", list(SMALL))
def test_workloads_bit_identical(name):
    be = oracle_backend()
    inputs = configs.CONFIG_INPUTS[name](**SMALL[name])
    store = {}
    flatten(name, configs.run_config(name, be, inputs), store)
    assert store, name
    for key, value in store.items():
        _same(key, value)


def test_extra_cases_bit_identical():
    store = {}
    flatten("extra", extra_cases(oracle_backend()), store)
    assert set(store) == {k for k in GOLD.files if k.startswith("extra/")}
    for key, value in store.items():
        _same(key, value)


def test_fixture_is_complete():
    keys = set(GOLD.files)
    for name in SMALL:
        assert any(k.startswith(name + "/") for k in keys), name
