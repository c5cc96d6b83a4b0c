"""The CPU oracle's flatten / optimizers / jacobian / hessian reproduce the real reference bit for bit.

``tests/golden/reference_next.npz`` was written by HIPS/autograd itself
(tests/golden/make_fixtures.py) on the cases of tests/golden/cases_next.py.
"""

import os
from types import SimpleNamespace

import numpy as np

import autograd_amd as ag
from cases import flatten
from cases_next import next_cases
from conftest import oracle_backend

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_next.npz"))


def oracle_ext():
    import oracle.misc as M
    from oracle.convolution import convolve

    return SimpleNamespace(flatten=M.flatten, sgd=M.sgd, rmsprop=M.rmsprop, adam=M.adam, jacobian=ag.jacobian,
                           hessian=ag.hessian, convolve=convolve, ag=ag, make_jvp_reversemode=ag.make_jvp_reversemode)


def test_next_cases_bit_identical():
    store = {}
    flatten("next", next_cases(oracle_backend(), oracle_ext()), store)
    assert set(store) == set(GOLD.files)
    for key, got in store.items():
        want, got = GOLD[key], np.asarray(got)
        assert got.dtype == want.dtype and got.shape == want.shape, (key, got.dtype, want.dtype, got.shape, want.shape)
        assert np.array_equal(got, want, equal_nan=True), (key, np.max(np.abs(got.astype(np.float64) - want)))


def test_flatten_promotes_mixed_leaves_like_numpy_concatenate():
    import oracle.anp as anp
    import oracle.misc as M

    flat, unflatten = M.flatten([np.ones(3, np.float32), np.ones(2)])
    assert flat.dtype == np.float64 and anp.shape(flat) == (5,)
    back = unflatten(flat)
    assert back[0].shape == (3,) and back[1].shape == (2,)
    empty, _ = M.flatten([])
    assert empty.shape == (0,)


def test_random_programs_bit_identical():
    """Gradients of 40 seeded random programs per precision (tests/golden/cases_random.py), all five
    inputs each, against the vectors the reference wrote: the restated rules, the accumulation
    order of fan-out and NumPy's promotion all have to agree for every bit to."""
    import oracle.anp as anp
    from cases_random import random_program_cases

    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_random.npz"))
    seeds = sorted({int(k.split("/")[2]) for k in gold.files})
    got = {}
    for dtype in (np.float64, np.float32):
        got.update(random_program_cases(anp, anp.logsumexp, ag.grad, lambda a: a, seeds, dtype))
    assert set(got) == set(gold.files) and len(got) == 400
    for key, g in got.items():
        g, want = np.asarray(g), gold[key]
        assert g.dtype == want.dtype and g.shape == want.shape, key
        assert np.array_equal(g, want, equal_nan=True), key
