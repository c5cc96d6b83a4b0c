"""Arrays of more than 2^31 elements (8.6 GB in float32): the 64-bit index variants of the fill,
elementwise, row-broadcast and reduction kernels.  Values are chosen so that every result is known
in closed form; a wrong offset (a 32-bit wrap) lands on a different constant."""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu

COLS = 32768
ROWS = (1 << 16) + 3                      # ROWS * COLS = 2^31 + 98304 elements
N = ROWS * COLS


def test_more_than_two_to_the_31_elements():
    import torch

    import autograd_amd.numpy as dnp
    from autograd_amd import grad
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    free, _ = torch.cuda.mem_get_info()
    if free < 40 * (1 << 30):
        pytest.skip("needs 40 GB of free device memory")
    x = dnp.full((N,), 0.5, dtype=onp.float32)
    # mark the far end: positions beyond 2^31 must be addressed, not wrapped onto the start
    tail = dnp.asarray(onp.arange(1.0, 9.0, dtype=onp.float32))
    D.map_op(Op.COPY, x.dtype, tail, out=D.DevArray(x._t[N - 8:], x.dtype))  # arrays are immutable to users
    y = dnp.exp(x)                                         # flat kernel, 64-bit offsets
    assert onp.allclose(y[N - 8:].numpy(), onp.exp(onp.arange(1.0, 9.0, dtype=onp.float32)), rtol=1e-6)
    assert onp.allclose(y[(1 << 31) - 4:(1 << 31) + 4].numpy(), onp.exp(onp.float32(0.5)), rtol=1e-6)
    assert onp.allclose(y[:4].numpy(), onp.exp(onp.float32(0.5)), rtol=1e-6)
    total = float(dnp.sum(x))                              # two-stage reduction over > 2^31 elements
    want = 0.5 * (N - 8) + 36.0
    assert abs(total - want) <= 1e-6 * want
    del y

    X = dnp.reshape(x, (ROWS, COLS))
    b = dnp.asarray(onp.linspace(1.0, 2.0, COLS).astype(onp.float32))
    Z = dnp.tanh(X * b[None, :])                           # row kernel with a broadcast operand, 64-bit thread index
    last = Z[ROWS - 1, COLS - 8:].numpy()
    assert onp.allclose(last, onp.tanh(onp.arange(1.0, 9.0, dtype=onp.float32) * b.numpy()[-8:]), rtol=1e-6)
    assert onp.allclose(Z[ROWS - 2, :4].numpy(), onp.tanh(onp.float32(0.5) * b.numpy()[:4]), rtol=1e-6)
    colsum = dnp.sum(X, axis=0).numpy()                    # column reduction with 65539 rows of 32768
    want_cols = onp.full(COLS, 0.5 * ROWS, dtype=onp.float64)
    want_cols[-8:] += onp.arange(1.0, 9.0) - 0.5
    assert onp.allclose(colsum, want_cols, rtol=1e-6)
    rowsum = dnp.sum(X, axis=1)
    assert onp.allclose(rowsum[:3].numpy(), 0.5 * COLS, rtol=1e-6)
    assert onp.allclose(float(rowsum[ROWS - 1]), 0.5 * (COLS - 8) + 36.0, rtol=1e-6)
    del Z

    # the gradient path on the same array: d/dx sum(x * x) = 2x, the cotangent is a pending map on x itself
    g = grad(lambda a: dnp.sum(a * a))(x)
    assert onp.allclose(g[N - 8:].numpy(), 2.0 * onp.arange(1.0, 9.0), rtol=1e-6)
    assert onp.allclose(g[(1 << 31):(1 << 31) + 4].numpy(), 1.0, rtol=1e-6)
