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

UNARY = ["tanh", "sin", "cos", "exp_small", "square", "negative", "sqrt_abs", "log1p_sq", "abs_shift"]


def _apply_unary(np, name, x):
    if name == "exp_small":
        return np.exp(x * 0.25)
    if name == "sqrt_abs":
        return np.sqrt(np.abs(x) + 1.0)
    if name == "log1p_sq":
        return np.log1p(x * x)
    if name == "abs_shift":
        return np.abs(x + 0.37)
    return getattr(np, name)(x)


def make_program(seed):
    """Returns (program(np, logsumexp, *arrays) -> scalar, list of host input arrays)."""
    rs = onp.random.RandomState(seed)
    m, n = int(rs.randint(2, 7)), int(rs.randint(2, 9))
    inputs = [rs.randn(m, n), rs.uniform(0.5, 1.5, n), rs.randn(m), rs.randn(n, m), rs.randn(m, n)]
    steps = []
    for _ in range(int(rs.randint(3, 12))):
        kind = rs.choice(["bin_full", "bin_row", "bin_col", "bin_scalar", "unary", "view", "dot", "mix"])
        steps.append((kind, int(rs.randint(0, 1 << 30))))
    tail = rs.choice(["sum", "lse_rows", "lse_cols", "mean_sq", "rowsum_weighted", "max_rows"])

    def program(np, logsumexp, A, b, c, D, E):
        x = A  # (m, n) throughout
        for kind, r in steps:
            q = onp.random.RandomState(r)
            op = q.choice(["add", "sub", "mul", "div"])
            if kind == "bin_full":
                other = E if q.rand() < 0.5 else np.transpose(D)
                x = {"add": x + other, "sub": other - x, "mul": x * other, "div": x / (other * other + 1.0)}[op]
            elif kind == "bin_row":
                x = {"add": x + b, "sub": b[None, :] - x, "mul": b * x, "div": x / b}[op]
            elif kind == "bin_col":
                col = c[:, None]
                x = {"add": col + x, "sub": x - col, "mul": x * col, "div": x / (col * col + 0.5)}[op]
            elif kind == "bin_scalar":
                s = float(q.choice([2.0, 0.5, -1.0, 3.0, 0.1, -0.75]))
                x = {"add": x + s, "sub": s - x, "mul": s * x, "div": x / s}[op]
            elif kind == "unary":
                x = _apply_unary(np, UNARY[q.randint(len(UNARY))], x)
            elif kind == "view":
                v = q.randint(4)
                if v == 0:
                    x = np.transpose(np.transpose(x) * 1.5)
                elif v == 1:
                    x = np.reshape(np.reshape(x, (x.shape[0] * x.shape[1],)) + 0.25, x.shape)
                elif v == 2:
                    x = x + np.sum(x[1:, :], axis=0) * 0.1 - x[0:1, :]
                else:
                    x = x * np.expand_dims(np.sum(x[:, ::2], axis=1), 1)
                    x = np.tanh(x * 0.1)
            elif kind == "dot":
                x = np.dot(np.dot(x, D), E) * 0.05 if q.rand() < 0.5 else np.dot(x, np.dot(D, x)) * 0.05
                x = np.tanh(x)
            else:  # the same value consumed several times in different forms (fan-out accumulation)
                y = x * b + c[:, None]
                x = y * 0.5 - np.transpose(np.transpose(y)) * y * 0.01 + np.sum(y, axis=1, keepdims=True) * 0.01
        if tail == "sum":
            return np.sum(x)
        if tail == "lse_rows":
            return np.sum(logsumexp(x, axis=1))
        if tail == "lse_cols":
            return np.sum(logsumexp(x * b + c[:, None], axis=0) * b)
        if tail == "mean_sq":
            return np.mean(x * x)
        if tail == "rowsum_weighted":
            return np.sum(np.sum(x, axis=1) * c)
        return np.sum(np.max(x, axis=1))

    return program, inputs


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
