"""HIP-graph replay of differentiated functions: every replay must equal the eager evaluation.

The recorded graph holds exactly the kernels the eager tracer launched, so results are compared
bit for bit.  Each graph is replayed several times on new input values, with eager work and
device synchronisations between the replays.
"""

import numpy as onp
import pytest

from autograd_amd import configs
from tests.golden.cases import SMALL, flatten

pytestmark = pytest.mark.gpu


def _programs(name, be):
    """(function of device inputs, tuple of host input names) for workload ``name``."""
    if name == "tanh":
        prog = configs.tanh_program(be)
        return (lambda x: (prog["d1"](x), prog["d2"](x), prog["d3"](x))), ("x",)
    if name == "bcast":
        return configs.bcast_program(be)["grad"], ("A", "b", "c")
    if name == "mlp":
        return configs.mlp_program(be)["grad"], ("params", "X", "T")
    if name == "rnn":
        return configs.rnn_program(be)["grad"], ("params", "inputs", "targets")
    if name == "convnet":
        from autograd_amd.scipy.signal import convolve

        return configs.convnet_program(be, convolve)["grad"], ("params", "X", "T")
    prog = configs.rosen_program(be)
    return (lambda x, v: (prog["grad"](x), prog["hvp_rev"](x, v), prog["hvp_fwd"](x, v))), ("x", "v")


def _perturb(tree, rng):
    """New values of the same shapes/dtypes (one-hot and other exact-valued arrays: permuted rows)."""
    def leaf(a):
        a = onp.asarray(a)
        if a.size and onp.all(a == onp.round(a)) and a.ndim >= 2:
            return a[rng.permutation(a.shape[0])]
        return (a + 0.25 * rng.standard_normal(a.shape)).astype(a.dtype)
    return configs.tree_map(leaf, tree)


@pytest.mark.parametrize("name", ["tanh", "bcast", "mlp", "rnn", "rosen", "convnet"])
def test_replay_equals_eager_on_every_workload(name):
    import autograd_amd as ag
    import autograd_amd.numpy as dnp

    be = configs.device_backend()
    fun, keys = _programs(name, be)
    host = configs.convnet_inputs(batch=5) if name == "convnet" else configs.CONFIG_INPUTS[name](**SMALL[name])
    args = [configs.tree_map(be.put, host[k]) for k in keys]
    graphed = ag.capture(fun, *args)
    rng = onp.random.default_rng(5)
    for replay in range(4):
        if replay:
            host = {k: _perturb(host[k], rng) for k in keys}
            args = [configs.tree_map(be.put, host[k]) for k in keys]
        got, want = {}, {}
        flatten("", configs.tree_map(be.get, graphed(*args)), got)
        # eager work between replays: the eager evaluation itself plus an unrelated reduction
        flatten("", configs.tree_map(be.get, fun(*args)), want)
        float(dnp.sum(dnp.exp(dnp.asarray(onp.linspace(0.0, 1.0, 5000)))))
        dnp.synchronize()
        assert got.keys() == want.keys() and len(got) > 0
        for k in want:
            assert got[k].dtype == want[k].dtype and got[k].shape == want[k].shape, (name, replay, k)
            assert onp.array_equal(got[k], want[k], equal_nan=True), (name, replay, k)
        # same argument objects again: nothing is copied, the replay alone must reproduce it
        again = {}
        flatten("", configs.tree_map(be.get, graphed(*args)), again)
        for k in want:
            assert onp.array_equal(again[k], want[k], equal_nan=True), (name, replay, k, "second replay")


def test_capture_contract_errors():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp

    x = dnp.asarray(onp.linspace(-1.0, 1.0, 64))
    g = ag.capture(ag.elementwise_grad(lambda v: dnp.tanh(v) * 2.0), x)
    want = 2.0 / onp.cosh(onp.linspace(-1.0, 1.0, 64)) ** 2
    assert onp.allclose(g(x).numpy(), want, rtol=1e-14)
    with pytest.raises(TypeError):
        g(dnp.asarray(onp.zeros(65)))
    with pytest.raises(TypeError):
        g(dnp.asarray(onp.zeros(64, onp.float32)))
    with pytest.raises(TypeError):
        g(x, x)
    # outputs that alias an input buffer are detached from it
    ident = ag.capture(lambda v: v, x)
    first = ident(x).numpy()
    ident(dnp.asarray(onp.zeros(64)))
    assert onp.array_equal(first, onp.linspace(-1.0, 1.0, 64))
    # scalars are constants of the recording
    scaled = ag.capture(lambda v, s: dnp.exp(v * s), x, 3.0)
    assert onp.allclose(scaled(x, 3.0).numpy(), onp.exp(3.0 * onp.linspace(-1.0, 1.0, 64)), rtol=1e-14)
    with pytest.raises(ValueError):
        scaled(x, 2.0)
    # host transfers cannot be recorded: reported as such, and the library stays usable afterwards
    with pytest.raises(RuntimeError, match="cannot be recorded"):
        ag.capture(lambda v: dnp.exp(v) * float(dnp.sum(v)), x)
    assert onp.allclose(dnp.exp(x).numpy(), onp.exp(onp.linspace(-1.0, 1.0, 64)), rtol=1e-14)


def test_replay_of_random_programs_equals_eager():
    """Gradients of 40 random programs (pending maps, views, fan-out accumulation) recorded and replayed."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.special import logsumexp
    from cases_random import make_program

    for seed in range(300, 340):
        program, inputs = make_program(seed)
        fun = ag.grad(lambda *xs: program(dnp, logsumexp, *xs), tuple(range(len(inputs))))  # noqa: B023
        args = [dnp.asarray(a) for a in inputs]
        graphed = ag.capture(fun, *args)
        for trial in range(2):
            if trial:
                rs = onp.random.RandomState(seed + 1000)
                args = [dnp.asarray(a + 0.1 * rs.standard_normal(a.shape)) for a in inputs]
            got = [g.numpy() for g in graphed(*args)]
            want = [g.numpy() for g in fun(*args)]
            for g, w in zip(got, want):
                assert g.dtype == w.dtype and onp.array_equal(g, w, equal_nan=True), (seed, trial)


def test_replay_of_array_functions_equals_eager():
    """Running sums, reversals, triangles, rolls, pieces and the counting sort (with its atomically accumulated
    ranks) launch kernels only, so they can be recorded; every replay must equal the eager evaluation bit for bit."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp

    rs = onp.random.RandomState(17)
    w = dnp.asarray(rs.randn(3000))

    def f(x, v):
        y = dnp.cumsum(x, axis=1) * 1e-2 + dnp.cumsum(x, axis=0) * 1e-2 + dnp.reshape(dnp.cumsum(x), x.shape) * 1e-3
        y = y + dnp.tril(x) - x[::-1] + dnp.roll(x, 3, axis=1) + dnp.fliplr(x) + dnp.rot90(x, 2) * 0.5
        head, tail = dnp.split(y, [7], axis=0)
        y = dnp.concatenate([tail, head], axis=0) + dnp.trace(x) * 1e-2 + dnp.tile(x[:1], (x.shape[0], 1))
        return dnp.sum(y * y) + dnp.sum(dnp.sort(v) * w) + dnp.sum(dnp.diff(x, axis=1) ** 2)

    fun = ag.grad(f, (0, 1))
    hx, hv = rs.randn(70, 70), rs.randn(3000)
    graphed = ag.capture(fun, dnp.asarray(hx), dnp.asarray(hv))
    for trial in range(3):
        x, v = dnp.asarray(hx + 0.1 * trial * rs.randn(70, 70)), dnp.asarray(hv + trial * rs.randn(3000))
        got = [g.numpy() for g in graphed(x, v)]
        dnp.synchronize()
        want = [g.numpy() for g in fun(x, v)]
        for g, w_ in zip(got, want):
            assert g.dtype == w_.dtype and onp.array_equal(g, w_), trial


def test_gather_and_ordered_scatter_replay_from_a_graph():
    """``x[[0, 1, 0]]`` (the reference's repeated-index case, tests/test_numpy.py:887-890) and a device-resident
    row index inside a recorded evaluation: the index tables live on the device, so the replay needs no host
    work, and repeated destinations are still added in index order."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp

    rs = onp.random.default_rng(3)
    rows = dnp.asarray(onp.array([4, 0, 4, 2, 4], dtype=onp.int64))
    w = dnp.asarray(rs.standard_normal((5, 3)) * 1e3)

    def f(x, M):
        return dnp.sum(x[[0, 1, 0]] ** 2) + dnp.sum(M[rows] * w) + dnp.sum(M[[1, 1, 3], 1:] ** 3)

    g = ag.grad(f, (0, 1))
    x0, M0 = rs.standard_normal(3), rs.standard_normal((6, 3))
    graphed = ag.capture(g, dnp.asarray(x0), dnp.asarray(M0))
    for replay in range(4):
        x0, M0 = rs.standard_normal(3), rs.standard_normal((6, 3))
        got = graphed(dnp.asarray(x0), dnp.asarray(M0))
        got = [a.numpy().copy() for a in got]
        dnp.sum(dnp.asarray(M0) * 2.0).numpy()  # eager work and a synchronisation between replays
        want = g(dnp.asarray(x0), dnp.asarray(M0))
        for a, b in zip(got, want):
            assert onp.array_equal(a, b.numpy())
        dM = onp.zeros_like(M0)
        onp.add.at(dM, onp.array([4, 0, 4, 2, 4]), w.numpy())
        onp.add.at(dM, (onp.array([1, 1, 3]), slice(1, None)), 3 * M0[[1, 1, 3], 1:] ** 2)
        assert onp.allclose(got[1], dM, rtol=1e-12)


def test_an_argument_written_by_item_assignment_is_copied_again():
    """A replay skips the copy of an argument that is the same object as last time; an item assignment in between
    (``x[0] = ...`` outside any trace) must not be missed."""
    import autograd_amd as ag
    import autograd_amd.numpy as np

    x = np.array(onp.arange(6.0))
    g = ag.capture(ag.grad(lambda v: np.sum(np.sin(v) * v)), x)
    want = lambda h: onp.cos(h) * h + onp.sin(h)  # noqa: E731
    onp.testing.assert_allclose(g(x).numpy(), want(onp.arange(6.0)), rtol=1e-12)
    onp.testing.assert_allclose(g(x).numpy(), want(onp.arange(6.0)), rtol=1e-12)
    x[0] = 2.5
    x[4:] = onp.array([-1.0, 0.5])
    onp.testing.assert_allclose(g(x).numpy(), want(onp.array([2.5, 1.0, 2.0, 3.0, -1.0, 0.5])), rtol=1e-12)
