"""Differential testing on random programs: device gradients vs the CPU oracle.

A seeded generator builds small programs out of the namespace's primitives (broadcasting
arithmetic with arrays, row/column vectors and Python scalars; unary ufuncs; views: transposes,
slices, reshapes; axis reductions; logsumexp; matrix products) and evaluates ``grad`` with
respect to every array input on both back ends.  The same Python function runs on both, so any
difference comes from the device value type: its kernels, its pending-map folding and view
propagation, its accumulation.  Tolerance: rtol 1e-9 of |ref| + max|ref| in float64 (device libm
and reduction order differ from NumPy's in the last bits and programs chain up to ~12 operations),
1e-4 in float32.
"""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu

from cases_random import make_program  # noqa: E402  (tests/golden is on sys.path, see conftest.py)


@pytest.mark.parametrize("dtype,rtol", [(onp.float64, 1e-9), (onp.float32, 1e-4)])
@pytest.mark.parametrize("block", range(6))
def test_random_programs_match_the_oracle(block, dtype, rtol):
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import oracle.anp as anp
    from autograd_amd.scipy.special import logsumexp as dlse

    for seed in range(block * 25, block * 25 + 25):
        program, inputs = make_program(seed)
        host = [a.astype(dtype) for a in inputs]
        argnums = tuple(range(len(host)))
        want = ag.grad(lambda *xs: program(anp, anp.logsumexp, *xs), argnums)(*host)
        want_val = program(anp, anp.logsumexp, *host)
        dev = [dnp.asarray(a) for a in host]
        got = ag.grad(lambda *xs: program(dnp, dlse, *xs), argnums)(*dev)
        got_val = float(program(dnp, dlse, *dev))
        if not onp.all(onp.isfinite(onp.asarray(want_val))) or not all(onp.all(onp.isfinite(w)) for w in want):
            continue  # the random program overflowed on the host as well: nothing to compare
        assert abs(got_val - float(want_val)) <= rtol * 10 * (abs(float(want_val)) + 1.0), (seed, got_val, want_val)
        # one scale for the whole program: a gradient that cancels analytically is rounding noise of the
        # size of the terms that cancelled, on either back end
        scale = max(float(onp.max(onp.abs(w))) if onp.size(w) else 0.0 for w in want)
        for k, (g, w) in enumerate(zip(got, want)):
            g = g.numpy()
            w = onp.asarray(w)
            assert g.shape == w.shape, (seed, k, g.shape, w.shape)
            assert g.dtype == w.dtype, (seed, k, g.dtype, w.dtype)
            err = onp.abs(g.astype(onp.float64) - w.astype(onp.float64))
            assert onp.all(err <= rtol * onp.abs(w) + rtol * scale + 1e-300), (seed, k, float(err.max()), float(scale))


def test_random_programs_hessian_vector_products_match_the_oracle():
    """Reverse-over-reverse and forward-over-reverse through the same random programs (float64)."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import oracle.anp as anp
    from autograd_amd.scipy.special import logsumexp as dlse

    checked = 0
    for seed in range(200, 240):
        program, inputs = make_program(seed)
        v = onp.random.RandomState(seed).randn(*inputs[0].shape)
        rest = inputs[1:]
        want_rev = ag.make_hvp(lambda a: program(anp, anp.logsumexp, a, *rest))(inputs[0])[0](v)
        if not onp.all(onp.isfinite(want_rev)):
            continue
        want_fwd = ag.make_jvp(ag.grad(lambda a: program(anp, anp.logsumexp, a, *rest)))(inputs[0])(v)[1]
        dev_rest = [dnp.asarray(a) for a in rest]
        A, V = dnp.asarray(inputs[0]), dnp.asarray(v)
        got_rev = ag.make_hvp(lambda a: program(dnp, dlse, a, *dev_rest))(A)[0](V).numpy()
        got_fwd = ag.make_jvp(ag.grad(lambda a: program(dnp, dlse, a, *dev_rest)))(A)(V)[1].numpy()
        scale = float(onp.max(onp.abs(want_rev))) + 1e-300
        for got, want in ((got_rev, want_rev), (got_fwd, want_fwd)):
            assert got.shape == want.shape and got.dtype == want.dtype, seed
            assert onp.all(onp.abs(got - want) <= 1e-8 * onp.abs(want) + 1e-8 * scale), (seed, float(onp.abs(got - want).max()), scale)
        checked += 1
    assert checked >= 30


def test_random_programs_match_the_reference_vectors():
    """The same generator, seeds the reference itself evaluated (tests/golden/reference_random.npz)."""
    import os

    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.special import logsumexp as dlse
    from cases_random import random_program_cases

    gold = onp.load(os.path.join(os.path.dirname(__file__), "golden", "reference_random.npz"))
    seeds = sorted({int(k.split("/")[2]) for k in gold.files})
    for dtype, rtol in ((onp.float64, 1e-9), (onp.float32, 1e-4)):
        got = random_program_cases(dnp, dlse, ag.grad, dnp.asarray, seeds, dtype)
        for seed in seeds:
            keys = [k for k in got if k.split("/")[2] == str(seed)]
            want = [gold[k] for k in keys]
            if not all(onp.all(onp.isfinite(w)) for w in want):
                continue
            scale = max(float(onp.max(onp.abs(w))) if w.size else 0.0 for w in want)
            for k, w in zip(keys, want):
                g = got[k].numpy()
                assert g.dtype == w.dtype and g.shape == w.shape, k
                assert onp.all(onp.abs(g.astype(onp.float64) - w) <= rtol * (onp.abs(w) + scale)), k
