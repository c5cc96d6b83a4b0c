"""``jacobian`` / ``hessian`` as ONE replay of the tape for all basis cotangents (stacked along a leading
axis), checked against the per-element loop of the reference (autograd/differential_operators.py:57-91),
which the CPU oracle still runs: its value type offers no stacked basis."""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu


def _programs(n, lse, put):
    rs = onp.random.RandomState(3)
    W, bvec, M2 = put(rs.randn(5, 3)), put(rs.randn(3)), put(rs.randn(3, 4))
    return {
        "elementwise": (lambda x: n.tanh(x) * x + n.exp(-x) / (1.0 + x * x), rs.randn(6)),
        "dense layer": (lambda x: n.tanh(n.dot(x, W) + bvec), rs.randn(4, 5)),
        "two layers": (lambda x: n.dot(n.tanh(n.dot(x, W) + bvec), M2) ** 2, rs.randn(2, 5)),
        "reductions": (lambda x: n.sum(x * x, axis=1) / (1.0 + n.mean(x, axis=0)[0]), rs.randn(3, 4)),
        "logsumexp": (lambda x: lse(x * 2.0, axis=1) - n.exp(x[:, 0]), rs.randn(4, 3)),
        "reshapes": (lambda x: n.reshape(n.sin(x), (6, 2)) * n.ravel(x)[:6, None], rs.randn(3, 4)),
        "0-d input": (lambda x: n.stack([x, x ** 2, n.sin(x)]), onp.array(0.7)),
        "broadcasts": (lambda x: (x[None, :] * x[:, None]) + x, rs.randn(4)),
        "vector dot": (lambda x: n.dot(x, bvec) * x, rs.randn(3)),           # a rule form replayed slice by slice
        "concatenate": (lambda x: n.concatenate([x * 2, n.cos(x)]), rs.randn(3)),
        "transposes": (lambda x: n.transpose(n.exp(x)) @ x, rs.randn(3, 2)),    # matmul: slice by slice
        "running sum": (lambda x: n.cumsum(x * x) * n.sort(x), rs.randn(5)),    # no batched rule at all
        "where and clip": (lambda x: n.where(x > 0, x * x, n.clip(x, -0.5, 0.5)) * n.maximum(x, 0.1), rs.randn(7)),
    }


def test_jacobian_and_hessian_match_the_per_element_loop():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import oracle.anp as anp
    from autograd_amd.scipy.special import logsumexp

    ref = _programs(anp, anp.logsumexp, lambda a: a)
    dev = _programs(dnp, logsumexp, dnp.asarray)
    for name, (f_ref, x0) in ref.items():
        f_dev = dev[name][0]
        want = ag.jacobian(f_ref)(x0)
        got = ag.jacobian(f_dev)(dnp.asarray(x0)).numpy()
        assert got.shape == want.shape and got.dtype == want.dtype, name
        assert onp.allclose(got, want, rtol=1e-12, atol=1e-12 * onp.max(onp.abs(want))), name
        if name in ("elementwise", "dense layer", "reductions", "logsumexp", "0-d input", "broadcasts", "where and clip"):
            want_h = ag.hessian(lambda x: anp.sum(f_ref(x) ** 2))(x0)
            got_h = ag.hessian(lambda x: dnp.sum(f_dev(x) ** 2))(dnp.asarray(x0)).numpy()
            assert got_h.shape == want_h.shape, name
            assert onp.allclose(got_h, want_h, rtol=1e-10, atol=1e-10 * onp.max(onp.abs(want_h))), name


def test_a_large_output_space_goes_through_in_blocks(monkeypatch):
    """The stacked cotangents of one replay are kept within a byte budget: with a budget of a few basis vectors the
    Jacobian comes out of several replays, row block by row block, and is the same array."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd import differential_operators as ops
    from autograd_amd.scipy.special import logsumexp

    progs = _programs(dnp, logsumexp, dnp.asarray)
    for name in ("dense layer", "logsumexp", "broadcasts", "running sum", "two layers"):
        f, x0 = progs[name]
        x = dnp.asarray(x0)
        whole = ag.jacobian(f)(x).numpy()
        n_out, n_in = whole.size // max(x0.size, 1), x0.size
        monkeypatch.setattr(ops, "JACOBIAN_BLOCK_BYTES", 3 * 16 * max(n_in, n_out) * 8)  # three basis vectors per replay
        blocks = ag.jacobian(f)(x).numpy()
        monkeypatch.undo()
        assert onp.array_equal(blocks, whole), name


def test_launch_count_of_a_jacobian_does_not_depend_on_the_output_size():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd import _lib
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(0)
    counts = {}
    for n_out in (8, 1024):
        W1, b1, W2 = dnp.asarray(rs.randn(16, 32)), dnp.asarray(rs.randn(32)), dnp.asarray(rs.randn(32, n_out))
        f = lambda x: logsumexp(dnp.dot(dnp.tanh(dnp.dot(x, W1) + b1), W2) * 0.5, axis=0) + dnp.sum(x) ** 2
        x = dnp.asarray(rs.randn(4, 16))
        ag.jacobian(f)(x)  # warm-up (one-time allocations)
        with _lib.KernelTimer() as kt:
            J = ag.jacobian(f)(x)
        counts[n_out] = len(kt.records)
        assert J.shape == (n_out, 4, 16)
        # one row against a plain gradient of that output
        k = n_out - 3
        row = ag.grad(lambda x: f(x)[k])(x)
        assert onp.allclose(J.numpy()[k], row.numpy(), rtol=1e-12, atol=1e-13)
    assert counts[8] == counts[1024], counts


def test_float32_jacobian_keeps_the_reference_dtypes():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import oracle.anp as anp

    x0 = onp.random.RandomState(1).randn(3, 4).astype(onp.float32)
    want = ag.jacobian(lambda x: anp.sum(anp.tanh(x) ** 2, axis=0) / 3.0)(x0)
    got = ag.jacobian(lambda x: dnp.sum(dnp.tanh(x) ** 2, axis=0) / 3.0)(dnp.asarray(x0)).numpy()
    assert got.dtype == want.dtype and got.shape == want.shape
    assert onp.allclose(got, want, rtol=1e-5, atol=1e-6)
