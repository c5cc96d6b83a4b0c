"""Device parity for the components either side of the hot path (flatten, optimizers,
jacobian / hessian) against vectors written by the real reference (tests/golden/reference_next.npz).

Tolerances: flatten / unflatten are copies and views (bit-exact); everything that goes through a
device contraction or reduction: rtol 1e-5 (float32) / 1e-12 (float64) of |ref| + max|ref|.  The
fused optimizer update itself is checked bit for bit against the NumPy passes on identical inputs.
"""

import os
from types import SimpleNamespace

import numpy as onp
import pytest

from cases import flatten
from cases_next import next_cases

pytestmark = pytest.mark.gpu

GOLD = onp.load(os.path.join(os.path.dirname(__file__), "golden", "reference_next.npz"))


def device_ext():
    import autograd_amd as ag
    import autograd_amd.misc.optimizers as opt
    from autograd_amd.misc import flatten as dflatten
    from autograd_amd.scipy.signal import convolve

    return SimpleNamespace(flatten=dflatten, sgd=opt.sgd, rmsprop=opt.rmsprop, adam=opt.adam, jacobian=ag.jacobian,
                           hessian=ag.hessian, convolve=convolve, ag=ag, make_jvp_reversemode=ag.make_jvp_reversemode)


def test_next_cases_match_reference_vectors():
    from autograd_amd import configs

    be = configs.device_backend()
    store = {}
    flatten("next", configs.tree_map(be.get, next_cases(be, device_ext())), store)
    assert set(store) == set(GOLD.files)
    for key, got in store.items():
        want = GOLD[key]
        assert got.dtype == want.dtype and got.shape == want.shape, (key, got.dtype, want.dtype, got.shape, want.shape)
        if key.startswith("next/flatten/") and "grad" not in key:
            assert onp.array_equal(got, want), key
            continue
        # the rule sweep runs on float32 operands; where the reference's promotion makes a result float64, parts of
        # it were still computed in float32 (by the reference sub-expression by sub-expression, by a fused kernel
        # after promoting its operands), so float32 tolerance applies to its values; dtypes must match exactly
        from_f32 = (want.dtype == onp.float32 or "_f32" in key or key.startswith("next/sweep/")
                    or (key.startswith(("next/opt/sgd/", "next/opt/rmsprop/", "next/opt/adam")) and "f64" not in key))
        rtol = 1e-5 if from_f32 else 1e-12
        scale = onp.max(onp.abs(want)) if want.size else 0.0
        err = onp.abs(got.astype(onp.float64) - want.astype(onp.float64))
        ok = (err <= rtol * onp.abs(want) + rtol * scale) | (onp.isnan(got) & onp.isnan(want))
        assert onp.all(ok), (key, float(onp.nanmax(err)))


@pytest.mark.parametrize("xdt,gdt", [(onp.float32, onp.float32), (onp.float64, onp.float32), (onp.float64, onp.float64),
                                     (onp.float32, onp.float64)])
def test_fused_updates_are_bit_identical_to_the_numpy_passes(xdt, gdt):
    """One step of each optimizer on identical inputs: the kernel must round exactly like
    misc/optimizers.py:40-47, 54-59, 66-75 evaluated by NumPy."""
    import autograd_amd.numpy as dnp
    from autograd_amd import _lib
    from autograd_amd.numpy import devarray as D

    rs = onp.random.RandomState(3)
    n = 4099
    x, g = rs.randn(n).astype(xdt), (rs.randn(n) * 3).astype(gdt)
    s0, s1 = onp.abs(rs.randn(n)), onp.abs(rs.randn(n))
    X, G = dnp.asarray(x), dnp.asarray(g)

    def run(kind, hyper, two_states):
        S0, S1 = dnp.asarray(s0), (dnp.asarray(s1) if two_states else None)
        out = D.empty((n,), onp.float64)
        _lib.optimizer_step(kind, X._t, G._t, S0._t, None if S1 is None else S1._t, out._t, hyper)
        return out.numpy(), S0.numpy(), (S1.numpy() if two_states else None)

    mass, step = 0.8, 0.05
    vel = mass * s0 - (1.0 - mass) * g
    got = run(_lib.OPT_SGD, (mass, 1.0 - mass, step), False)
    assert onp.array_equal(got[1], vel) and onp.array_equal(got[0], x + step * vel)

    gamma, eps = 0.9, 10**-8
    avg = s0 * gamma + g**2 * (1 - gamma)
    got = run(_lib.OPT_RMSPROP, (gamma, 1 - gamma, step, eps), False)
    assert onp.array_equal(got[1], avg) and onp.array_equal(got[0], x - step * g / (onp.sqrt(avg) + eps))

    b1, b2, i = 0.9, 0.999, 6
    m = (1 - b1) * g + b1 * s0
    v = (1 - b2) * (g**2) + b2 * s1
    mhat, vhat = m / (1 - b1 ** (i + 1)), v / (1 - b2 ** (i + 1))
    got = run(_lib.OPT_ADAM, (1 - b1, b1, 1 - b2, b2, 1 - b1 ** (i + 1), 1 - b2 ** (i + 1), step, eps), True)
    assert onp.array_equal(got[1], m) and onp.array_equal(got[2], v)
    assert onp.array_equal(got[0], x - step * mhat / (onp.sqrt(vhat) + eps))


def test_training_loop_stays_on_the_device_and_converges():
    """adam on a least-squares problem: parameters, gradients and optimizer state never leave HBM
    (no host transfer happens inside the loop: it runs under the capture guard)."""
    import autograd_amd.numpy as dnp
    from autograd_amd import _lib, grad
    from autograd_amd.misc.optimizers import adam

    rs = onp.random.RandomState(0)
    A, y = rs.randn(64, 8), rs.randn(64)
    Ad, yd = dnp.asarray(A), dnp.asarray(y)
    loss = lambda p, i: dnp.sum((dnp.dot(Ad, p["w"]) + p["b"] - yd) ** 2) / 64.0  # noqa: E731
    p0 = {"w": dnp.asarray(onp.zeros(8)), "b": dnp.asarray(onp.zeros(()))}
    _lib.CAPTURING = True  # any .numpy()/.item()/upload inside the loop would raise
    try:
        p = adam(grad(loss), p0, num_iters=300, step_size=0.05)
    finally:
        _lib.CAPTURING = False
    w_star, *_ = onp.linalg.lstsq(onp.c_[A, onp.ones(64)], y, rcond=None)
    assert onp.allclose(onp.r_[p["w"].numpy(), p["b"].numpy()], w_star, atol=2e-2)
