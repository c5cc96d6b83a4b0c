"""``autograd_amd.scipy.signal.convolve`` and ``numpy.pad`` on the device against the CPU oracle
(oracle/convolution.py, itself bit-identical to the reference on tests/golden/reference_next.npz)
at sizes that reach every window-contraction kernel (LDS-staged tiles and one thread per position,
with filter-batch tiles of 1, 2, 4 and 8; one block per output) and the operand-copy path.

Tolerance: |got - want| <= rtol * (|want| + max|want|), rtol 1e-5 (float32) / 1e-12 (float64); the
summation order of a device contraction differs from numpy.einsum's.
"""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu


def _close(got, want, dtype):
    rtol = 1e-5 if dtype == onp.float32 else 1e-12
    assert got.dtype == want.dtype and got.shape == want.shape, (got.dtype, want.dtype, got.shape, want.shape)
    err = onp.abs(got.astype(onp.float64) - want.astype(onp.float64))
    bound = rtol * (onp.abs(want) + (onp.max(onp.abs(want)) if want.size else 0.0))
    assert onp.all(err <= bound), float(onp.max(err - bound))


def _both(kw, a, b, dtype):
    """value and both cotangents, device vs oracle"""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import oracle.anp as anp
    from autograd_amd import _lib
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    want = oconv(a, b, **kw)
    got = dconv(dnp.asarray(a), dnp.asarray(b), **kw)
    kernel = _lib.lib().agmi_last_kernel().decode()
    _close(got.numpy(), want, dtype)
    w = onp.random.RandomState(5).randn(*want.shape).astype(dtype)
    wd = dnp.asarray(w)
    gd = ag.grad(lambda x, y: dnp.sum(dconv(x, y, **kw) * wd), (0, 1))(dnp.asarray(a), dnp.asarray(b))
    go = ag.grad(lambda x, y: anp.sum(oconv(x, y, **kw) * w), (0, 1))(a, b)
    for d, o in zip(gd, go):
        _close(d.numpy(), o, dtype)
    return kernel


@pytest.mark.parametrize("dtype", [onp.float32, onp.float64])
def test_convnet_layer_forward_and_both_cotangents(dtype):
    rs = onp.random.RandomState(0)
    img, filt = rs.randn(8, 3, 14, 14).astype(dtype), rs.randn(3, 5, 5, 5).astype(dtype)
    kernel = _both(dict(axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode="valid"), img, filt, dtype)
    assert kernel.startswith("correlate_reduce")


@pytest.mark.parametrize("mode", ["full", "valid", "same"])
def test_long_one_dimensional_windows(mode):
    rs = onp.random.RandomState(1)
    _both(dict(mode=mode), rs.randn(300), rs.randn(200), onp.float64)
    _both(dict(mode=mode), rs.randn(2000).astype(onp.float32), rs.randn(700).astype(onp.float32), onp.float32)


@pytest.mark.parametrize("filters,tile", [(1, 1), (2, 2), (4, 4), (6, 8), (16, 8)])
def test_staged_tiles_with_filter_batch_tiles(filters, tile):
    import autograd_amd.numpy as dnp
    from autograd_amd import _lib
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    rs = onp.random.RandomState(2)
    img, filt = rs.randn(64, 2, 68, 68).astype(onp.float32), rs.randn(2, filters, 5, 5).astype(onp.float32)
    for mode in ("valid", "same"):
        kw = dict(axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode=mode)
        got = dconv(dnp.asarray(img), dnp.asarray(filt), **kw)
        assert _lib.lib().agmi_last_kernel().decode() == f"correlate_tiled<float, {tile}>"
        _close(got.numpy(), oconv(img, filt, **kw), onp.float32)


@pytest.mark.parametrize("dtype", [onp.float32, onp.float64])
def test_windows_too_large_to_stage_run_one_thread_per_position(dtype):
    import autograd_amd.numpy as dnp
    from autograd_amd import _lib
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    rs = onp.random.RandomState(7)
    img, filt = rs.randn(200, 200).astype(dtype), rs.randn(40, 40).astype(dtype)
    got = dconv(dnp.asarray(img), dnp.asarray(filt), mode="valid")
    assert _lib.lib().agmi_last_kernel().decode().startswith("correlate_positions<")
    _close(got.numpy(), oconv(img, filt, mode="valid"), dtype)


@pytest.mark.parametrize("mode", ["full", "valid", "same"])
def test_staged_tiles_on_ragged_shapes(mode):
    """Tile edges: outputs that are not multiples of the tile, images fewer than a tile holds, a third
    convolved axis, negative strides (the flips) and padding on every side."""
    rs = onp.random.RandomState(8)
    _both(dict(axes=([1, 2], [1, 2]), mode=mode), rs.randn(3, 13, 9), rs.randn(2, 4, 3), onp.float64)
    _both(dict(mode=mode), rs.randn(5, 7, 9).astype(onp.float32), rs.randn(2, 3, 2).astype(onp.float32), onp.float32)
    _both(dict(axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode=mode), rs.randn(5, 3, 17, 33), rs.randn(3, 7, 4, 6),
          onp.float64)
    _both(dict(mode=mode), rs.randn(1000), rs.randn(9), onp.float64)


def test_free_axes_that_do_not_merge_are_copied_once():
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    rs = onp.random.RandomState(3)
    base, w = rs.randn(3, 4, 8), rs.randn(2, 3)
    kw = dict(axes=([2], [1]), mode="full")
    got = dconv(dnp.transpose(dnp.asarray(base), (1, 0, 2)), dnp.asarray(w), **kw)
    _close(got.numpy(), oconv(base.transpose(1, 0, 2), w, **kw), onp.float64)
    # pending maps and mixed dtypes are written out / promoted before the launch
    lazy = dnp.asarray(base) * 2.0 + 1.0
    got = dconv(lazy, dnp.asarray(w.astype(onp.float32)), **kw)
    _close(got.numpy(), oconv(base * 2.0 + 1.0, w.astype(onp.float32), **kw), onp.float64)


def test_forward_mode_is_the_same_contraction():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    rs = onp.random.RandomState(4)
    a, b, t = rs.randn(4, 6), rs.randn(2, 3), rs.randn(4, 6)
    value, tangent = ag.make_jvp(lambda x: dconv(x, dnp.asarray(b), mode="same"))(dnp.asarray(a))(dnp.asarray(t))
    _close(value.numpy(), oconv(a, b, mode="same"), onp.float64)
    _close(tangent.numpy(), oconv(t, b, mode="same"), onp.float64)


def test_errors_match_the_reference():
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.signal import convolve as dconv

    a, b = dnp.asarray(onp.ones((4, 2))), dnp.asarray(onp.ones((2, 3)))
    with pytest.raises(ValueError, match="One array must be larger"):
        dconv(a, b, mode="valid")
    with pytest.raises(AssertionError, match="Mode circular undefined"):
        dconv(a, b, mode="circular")
    assert dconv(dnp.asarray(onp.ones((0, 3))), b, axes=([1], [1]), mode="full").shape == (0, 2, 5)


@pytest.mark.parametrize("dtype", [onp.float32, onp.float64])
def test_pad_and_its_rules_are_exact(dtype):
    import autograd_amd as ag
    import autograd_amd.numpy as dnp

    rs = onp.random.RandomState(6)
    x = rs.randn(3, 4).astype(dtype)
    for width in (1, (1, 2), ((2, 0), (0, 3)), ((0, 0), (0, 0))):
        want = onp.pad(x, width, mode="constant")
        assert onp.array_equal(dnp.pad(dnp.asarray(x), width, mode="constant").numpy(), want)
        w = rs.randn(*want.shape).astype(dtype)
        g = ag.grad(lambda z: dnp.sum(dnp.pad(z, width, mode="constant") * dnp.asarray(w)))(dnp.asarray(x))
        lo = [p[0] for p in onp.broadcast_to(onp.asarray(width), (2, 2))]
        assert onp.array_equal(g.numpy(), w[lo[0]:lo[0] + 3, lo[1]:lo[1] + 4])
    lazy = dnp.asarray(x) * 2.0
    assert onp.array_equal(dnp.pad(lazy, 1, mode="constant").numpy(), onp.pad(x * dtype(2.0), 1, mode="constant"))
    _, tangent = ag.make_jvp(lambda z: dnp.pad(z, 2, mode="constant"))(dnp.asarray(x))(dnp.asarray(x))
    assert onp.array_equal(tangent.numpy(), onp.pad(x, 2, mode="constant"))
    with pytest.raises(NotImplementedError):
        dnp.pad(dnp.asarray(x), 1, mode="reflect")
