"""User programs written exactly like the reference's examples run on the device namespace.

``examples/neural_net.py`` (MLP + L2 prior through ``flatten`` + ``adam`` with a callback) with a
synthetic data set in place of the MNIST download, against the CPU oracle running the same
program on the same draws.
"""

import itertools

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu


def _program(np, npr, grad, flatten, adam, logsumexp, put):
    """examples/neural_net.py:16-110, data set replaced by seeded synthetic arrays."""

    def init_random_params(scale, layer_sizes, rs=None):
        rs = rs if rs is not None else npr.RandomState(0)
        return [(scale * rs.randn(m, n), scale * rs.randn(n)) for m, n in itertools.pairwise(layer_sizes)]

    def neural_net_predict(params, inputs):
        for W, b in params:
            outputs = np.dot(inputs, W) + b
            inputs = np.tanh(outputs)
        return outputs - logsumexp(outputs, axis=1, keepdims=True)

    def l2_norm(params):
        flattened, _ = flatten(params)
        return np.dot(flattened, flattened)

    def log_posterior(params, inputs, targets, L2_reg):
        log_prior = -L2_reg * l2_norm(params)
        log_lik = np.sum(neural_net_predict(params, inputs) * targets)
        return log_prior + log_lik

    def accuracy(params, inputs, targets):
        target_class = np.argmax(targets, axis=1)
        predicted_class = np.argmax(neural_net_predict(params, inputs), axis=1)
        return np.mean(predicted_class == target_class)

    layer_sizes = [20, 16, 12, 10]
    L2_reg, param_scale, batch_size, num_epochs, step_size = 1.0, 0.1, 32, 2, 0.001
    data = onp.random.RandomState(1)
    labels = data.randint(0, 10, 96)
    train_images = put(data.randn(96, 20))
    train_labels = put(onp.eye(10)[labels])
    init_params = init_random_params(param_scale, layer_sizes)
    num_batches = int(np.ceil(len(train_images) / batch_size))

    def batch_indices(iter):
        idx = iter % num_batches
        return slice(idx * batch_size, (idx + 1) * batch_size)

    def objective(params, iter):
        idx = batch_indices(iter)
        return -log_posterior(params, train_images[idx], train_labels[idx], L2_reg)

    log = []

    def print_perf(params, iter, gradient):
        if iter % num_batches == 0:
            log.append(float(accuracy(params, train_images, train_labels)))

    optimized = adam(grad(objective), init_params, step_size=step_size, num_iters=num_epochs * num_batches,
                     callback=print_perf)
    return optimized, log, float(objective(optimized, 0))


def test_neural_net_example_trains_like_the_reference():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import autograd_amd.numpy.random as dnpr
    import oracle.anp as anp
    import oracle.misc as omisc
    from autograd_amd.misc import flatten
    from autograd_amd.misc.optimizers import adam
    from autograd_amd.scipy.special import logsumexp

    got, got_log, got_obj = _program(dnp, dnpr, ag.grad, flatten, adam, logsumexp, dnp.asarray)
    want, want_log, want_obj = _program(anp, onp.random, ag.grad, omisc.flatten, omisc.adam, anp.logsumexp, lambda a: a)
    assert got_log == want_log and len(got_log) == 2
    assert abs(got_obj - want_obj) <= 1e-10 * abs(want_obj)
    for (gw, gb), (ww, wb) in zip(got, want):
        for g, w in ((gw, ww), (gb, wb)):
            g = g.numpy()
            assert g.dtype == w.dtype and g.shape == w.shape
            assert onp.allclose(g, w, rtol=1e-10, atol=1e-12)


def test_random_argmax_rounding_helpers():
    import autograd_amd.numpy as dnp
    import autograd_amd.numpy.random as dnpr

    a = dnpr.RandomState(3).randn(4, 5)
    assert onp.array_equal(a.numpy(), onp.random.RandomState(3).randn(4, 5))
    dnpr.seed(5)
    b = dnpr.uniform(-1, 1, (3,))
    onp.random.seed(5)
    assert onp.array_equal(b.numpy(), onp.random.uniform(-1, 1, (3,)))
    x = onp.random.RandomState(0).randn(7, 9)
    x[2, 3] = x[2, 5] = 10.0  # ties: first index wins
    X = dnp.asarray(x)
    for axis in (0, 1, None, -1):
        assert onp.array_equal(dnp.argmax(X, axis=axis).numpy(), onp.argmax(x, axis=axis))
        assert onp.array_equal(dnp.argmin(X, axis=axis).numpy(), onp.argmin(x, axis=axis))
    assert dnp.argmax(X, axis=1).dtype == onp.int64
    y = onp.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 2.4999, -0.0, onp.inf, onp.nan])
    Y = dnp.asarray(y)
    for name in ("floor", "ceil", "rint", "round", "trunc", "fix"):
        assert onp.array_equal(getattr(dnp, name)(Y).numpy(), getattr(onp, name)(y), equal_nan=True), name
    assert onp.array_equal(dnp.isnan(Y).numpy(), onp.isnan(y))
    assert onp.array_equal(dnp.isinf(Y).numpy(), onp.isinf(y))
    assert onp.array_equal(dnp.isfinite(Y).numpy(), onp.isfinite(y))
    from autograd_amd import grad

    assert float(grad(lambda v: dnp.sum(dnp.floor(v) * v))(Y[:3]).numpy()[0]) == -3.0  # floor is piecewise constant
