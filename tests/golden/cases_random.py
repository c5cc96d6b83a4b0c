"""Seeded generator of small random programs over the traced NumPy namespace (broadcasting arithmetic
with arrays, row / column vectors and Python scalars; unary ufuncs; views; axis reductions;
logsumexp; matrix products; fan-out; reversals, rolls, running sums, triangles, pieces and
diagonals).  The same Python function runs on the reference (when
writing fixtures), the CPU oracle and the device.
"""

import numpy as onp

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
        kind = rs.choice(["bin_full", "bin_row", "bin_col", "bin_scalar", "unary", "view", "dot", "mix", "rearrange"])
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
            elif kind == "rearrange":  # shape-preserving uses of the array-function table
                v = q.randint(10)
                rows = x.shape[0]
                if v == 0:
                    x = np.roll(x, int(q.randint(-3, 4)), axis=int(q.randint(2))) + np.roll(x, 2) * 0.5
                elif v == 1:
                    x = x[::-1] * 0.5 + np.fliplr(x) - np.rot90(x, 2) * 0.25
                elif v == 2:
                    x = np.cumsum(x, axis=int(q.randint(2))) * 0.3 + np.reshape(np.cumsum(x), x.shape) * 0.01
                elif v == 3:
                    x = np.tile(x, (2, 1))[1 : 1 + rows] * b - x[:, ::-1]
                elif v == 4:
                    x = np.concatenate([np.diff(x, axis=1), x[:, :1]], axis=1) + np.tril(x) - 0.5 * np.triu(x, 1)
                elif v == 5:
                    head, rest = np.split(x, [1], axis=0)
                    x = np.concatenate([rest * 2.0, head], axis=0) + np.flipud(x) * 0.1
                elif v == 6:
                    x = np.dot(np.inner(x, x) * 0.05, x) + np.trace(np.dot(x, D)) * 0.01
                elif v == 7:
                    x = x + np.diag(np.dot(x, D))[:, None] * 0.1 + np.diag(np.diag(np.dot(x, D)))[:, :1] * 0.1
                elif v == 8:
                    x = np.sinc(x * 0.3) + np.logaddexp2(x, E) * 0.1
                else:
                    x = np.kron(x, b[:2])[:, ::2] * 0.5 + np.moveaxis(np.rollaxis(np.transpose(x), 1), 0, 0)
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


def random_program_cases(np, logsumexp, grad, put, seeds, dtype):
    """{key: gradient} for every input of every seeded program, evaluated on one back end."""
    out = {}
    tag = "f32" if dtype == onp.float32 else "f64"
    for seed in seeds:
        program, inputs = make_program(seed)
        host = [put(a.astype(dtype)) for a in inputs]
        with onp.errstate(all="ignore"):
            grads = grad(lambda *xs: program(np, logsumexp, *xs), tuple(range(len(host))))(*host)
        for k, g in enumerate(grads):
            out[f"random/{tag}/{seed}/{k}"] = g
    return out
