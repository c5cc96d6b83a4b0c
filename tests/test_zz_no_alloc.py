"""``agmi_map_reduce_static``: the entry point for callers that cannot allocate device memory.

It must give, bit for bit, what ``agmi_map_reduce`` gives with a roomy caller-owned workspace
(same kernels, same summation tree), while staging partial results in the library's built-in
scratch array.  Every case below is a two-stage reduction (it really uses the scratch), called
through the C ABI twice in a row, the second time on a smaller input, so that stale partial
results of the first call would show up in the second.
"""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu


def _both(x, axis, op, red, extra=()):
    """Run the reduction of ``x`` (and ``extra`` operands of the fused map) over ``axis`` through the
    static entry point and through the workspace one; returns the two results as NumPy arrays."""
    import torch

    from autograd_amd import _lib

    _lib.lib()
    dev = _lib.device()
    code = _lib.DTYPE_CODE[onp.dtype(x.dtype)]
    ins = [torch.from_numpy(a).to(dev) for a in (x,) + tuple(extra)]
    kept = [n for d, n in enumerate(x.shape) if d != axis]
    mask = [d == axis for d in range(x.ndim)]
    results = []
    for entry in (_lib.map_reduce_static, _lib.map_reduce):
        out = torch.full(kept, float("nan"), dtype=ins[0].dtype, device=dev)
        view = out.unsqueeze(axis).expand(x.shape)
        assert entry(op, red, code, x.shape, mask, view, ins)
        results.append(out)
    torch.cuda.synchronize(dev)
    return [r.cpu().numpy() for r in results]


CASES = [
    # (dtype, first shape, second (smaller) shape, axis, reduction)
    ("float32", (4096, 2048), (1000, 300), 0, "sum"),        # column form, chunks across blocks
    ("float32", (8, 200000), (3, 70001), 1, "sum"),          # row form, several chunks per row
    ("float64", (2048, 1024), (515, 130), 0, "sum"),
    ("float32", (4096, 1024), (700, 200), 0, "logsumexp"),   # (max, scaled sum) pairs in the scratch
    ("float64", (4, 300000), (2, 50000), 1, "logsumexp"),
    ("float32", (2048, 512), (900, 64), 0, "max"),
]


@pytest.mark.parametrize("dtype,first,second,axis,red", CASES)
def test_static_scratch_matches_workspace_entry_point(dtype, first, second, axis, red):
    from autograd_amd._lib import Op, Red

    kind = {"sum": Red.SUM, "logsumexp": Red.LOGSUMEXP, "max": Red.MAX}[red]
    rs = onp.random.RandomState(7)
    for shape in (first, second):
        x = rs.randn(*shape).astype(dtype)
        got, want = _both(x, axis, Op.COPY, kind)
        assert got.dtype == want.dtype and got.shape == want.shape
        assert not onp.isnan(got).any()
        assert onp.array_equal(got, want), f"{shape}: static and workspace entry points differ"
        ref = {"sum": onp.sum, "max": onp.max}.get(red)
        if ref is not None:
            r = ref(x.astype(onp.float64), axis=axis)
            tol = 1e-5 if dtype == "float32" else 1e-12
            assert onp.all(onp.abs(got - r) <= tol * onp.abs(r) + tol * onp.max(onp.abs(r)))


def test_static_scratch_with_a_fused_rule_in_front_of_the_sum():
    from autograd_amd._lib import Op, Red

    rs = onp.random.RandomState(3)
    for shape in ((4096, 1024), (777, 96)):
        x = rs.randn(*shape).astype("float32")
        g = rs.randn(*shape).astype("float32")
        got, want = _both(x, 0, Op.MUL, Red.SUM, extra=(g,))
        assert onp.array_equal(got, want)
        r = onp.sum(x.astype(onp.float64) * g, axis=0)
        assert onp.all(onp.abs(got - r) <= 1e-5 * onp.abs(r) + 1e-5 * onp.max(onp.abs(r)))


def test_partial_results_beyond_the_scratch_are_rejected_and_later_calls_still_work():
    import torch

    from autograd_amd import _lib
    from autograd_amd._lib import Op, Red

    _lib.lib()
    dev = _lib.device()
    # float64 logsumexp over the rows of (256, 40000): two chunks of 40000 (max, sum) pairs = 1.28 MB
    x = torch.zeros((256, 40000), dtype=torch.float64, device=dev)
    out = torch.full((40000,), 7.0, dtype=torch.float64, device=dev)
    view = out.unsqueeze(0).expand(256, 40000)
    with pytest.raises(_lib.AgmiError) as err:
        _lib.map_reduce_static(Op.COPY, Red.LOGSUMEXP, _lib.DTYPE_CODE[onp.dtype("float64")], (256, 40000),
                               [True, False], view, [x])
    assert "code -3" in str(err.value) and "scratch" in str(err.value)
    torch.cuda.synchronize(dev)
    assert bool((out == 7.0).all()), "a rejected call must launch nothing"
    # the workspace entry point takes the same problem
    assert _lib.map_reduce(Op.COPY, Red.LOGSUMEXP, _lib.DTYPE_CODE[onp.dtype("float64")], (256, 40000),
                           [True, False], view, [x])
    torch.cuda.synchronize(dev)
    assert onp.allclose(out.cpu().numpy(), onp.log(256.0), rtol=1e-12)
    # and the static one keeps working afterwards
    rs = onp.random.RandomState(11)
    y = rs.randn(2048, 640).astype("float32")
    got, want = _both(y, 0, Op.COPY, Red.SUM)
    assert onp.array_equal(got, want)
