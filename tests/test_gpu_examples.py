"""User programs written exactly like the reference's examples run on the device namespace.

``examples/neural_net.py`` (MLP + L2 prior through ``flatten`` + ``adam`` with a callback) with a
synthetic data set in place of the MNIST download, against the CPU oracle running the same
program on the same draws; ``examples/convnet.py`` (LeNet-style stack of ``convolve`` + max pooling
layers trained by momentum SGD on a flat weight vector) likewise.
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


def _convnet(np, npr, grad, convolve, put):
    """examples/convnet.py:14-218 at reduced layer sizes, data set replaced by seeded synthetic arrays."""

    class WeightsParser:
        def __init__(self):
            self.idxs_and_shapes = {}
            self.N = 0

        def add_weights(self, name, shape):
            start = self.N
            self.N += np.prod(shape)
            self.idxs_and_shapes[name] = (slice(start, self.N), shape)

        def get(self, vect, name):
            idxs, shape = self.idxs_and_shapes[name]
            return np.reshape(vect[idxs], shape)

    def logsumexp(X, axis, keepdims=False):
        max_X = np.max(X)
        return max_X + np.log(np.sum(np.exp(X - max_X), axis=axis, keepdims=keepdims))

    def make_nn_funs(input_shape, layer_specs, L2_reg):
        parser = WeightsParser()
        cur_shape = input_shape
        for layer in layer_specs:
            N_weights, cur_shape = layer.build_weights_dict(cur_shape)
            parser.add_weights(layer, (N_weights,))

        def predictions(W_vect, inputs):
            cur_units = inputs
            for layer in layer_specs:
                cur_units = layer.forward_pass(cur_units, parser.get(W_vect, layer))
            return cur_units

        def loss(W_vect, X, T):
            log_prior = -L2_reg * np.dot(W_vect, W_vect)
            log_lik = np.sum(predictions(W_vect, X) * T)
            return -log_prior - log_lik

        return parser.N, predictions, loss

    class conv_layer:
        def __init__(self, kernel_shape, num_filters):
            self.kernel_shape, self.num_filters = kernel_shape, num_filters

        def forward_pass(self, inputs, param_vector):
            params = self.parser.get(param_vector, "params")
            biases = self.parser.get(param_vector, "biases")
            conv = convolve(inputs, params, axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode="valid")
            return conv + biases

        def build_weights_dict(self, input_shape):
            self.parser = WeightsParser()
            self.parser.add_weights("params", (input_shape[0], self.num_filters) + self.kernel_shape)
            self.parser.add_weights("biases", (1, self.num_filters, 1, 1))
            out_yx = tuple(a - b + 1 for a, b in zip(input_shape[1:], self.kernel_shape))
            return self.parser.N, (self.num_filters,) + out_yx

    class maxpool_layer:
        def __init__(self, pool_shape):
            self.pool_shape = pool_shape

        def build_weights_dict(self, input_shape):
            output_shape = list(input_shape)
            for i in [0, 1]:
                assert input_shape[i + 1] % self.pool_shape[i] == 0, "maxpool shape should tile input exactly"
                output_shape[i + 1] = input_shape[i + 1] // self.pool_shape[i]
            return 0, output_shape

        def forward_pass(self, inputs, param_vector):
            new_shape = inputs.shape[:2]
            for i in [0, 1]:
                pool_width = self.pool_shape[i]
                new_shape += (inputs.shape[i + 2] // pool_width, pool_width)
            result = inputs.reshape(new_shape)
            return np.max(np.max(result, axis=3), axis=4)

    class full_layer:
        def __init__(self, size):
            self.size = size

        def build_weights_dict(self, input_shape):
            input_size = np.prod(input_shape, dtype=int)
            self.parser = WeightsParser()
            self.parser.add_weights("params", (input_size, self.size))
            self.parser.add_weights("biases", (self.size,))
            return self.parser.N, (self.size,)

        def forward_pass(self, inputs, param_vector):
            params = self.parser.get(param_vector, "params")
            biases = self.parser.get(param_vector, "biases")
            if inputs.ndim > 2:
                inputs = inputs.reshape((inputs.shape[0], np.prod(inputs.shape[1:])))
            return self.nonlinearity(np.dot(inputs[:, :], params) + biases)

    class tanh_layer(full_layer):
        def nonlinearity(self, x):
            return np.tanh(x)

    class softmax_layer(full_layer):
        def nonlinearity(self, x):
            return x - logsumexp(x, axis=1, keepdims=True)

    input_shape = (1, 12, 12)
    layer_specs = [conv_layer((3, 3), 2), maxpool_layer((2, 2)), conv_layer((2, 2), 3), maxpool_layer((2, 2)),
                   tanh_layer(8), softmax_layer(4)]
    L2_reg, param_scale, learning_rate, momentum, batch_size = 1.0, 0.1, 1e-3, 0.9, 6
    data = onp.random.RandomState(2)
    images = put(data.rand(18, 1, 12, 12))
    labels = put(onp.eye(4)[data.randint(0, 4, 18)])
    N_weights, pred_fun, loss_fun = make_nn_funs(input_shape, layer_specs, L2_reg)
    loss_grad = grad(loss_fun)
    W = npr.RandomState(0).randn(N_weights) * param_scale
    cur_dir = np.zeros(N_weights)
    losses = []
    for epoch in range(2):
        for start in range(0, 18, batch_size):
            idxs = slice(start, start + batch_size)
            losses.append(float(loss_fun(W, images[idxs], labels[idxs])))
            grad_W = loss_grad(W, images[idxs], labels[idxs])
            cur_dir = momentum * cur_dir + (1.0 - momentum) * grad_W
            W -= learning_rate * cur_dir
    return W, losses, pred_fun(W, images)


def test_convnet_example_trains_like_the_reference():
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    import autograd_amd.numpy.random as dnpr
    import oracle.anp as anp
    from autograd_amd.scipy.signal import convolve as dconv
    from oracle.convolution import convolve as oconv

    got_W, got_losses, got_pred = _convnet(dnp, dnpr, ag.grad, dconv, dnp.asarray)
    want_W, want_losses, want_pred = _convnet(anp, onp.random, ag.grad, oconv, lambda a: a)
    assert len(got_losses) == 6 and onp.allclose(got_losses, want_losses, rtol=1e-11, atol=0)
    for g, w in ((got_W, want_W), (got_pred, want_pred)):
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
    x[1, 4] = x[1, 7] = x[5, 0] = onp.nan  # a NaN wins over every number, the first one in its line
    X = dnp.asarray(x)
    for axis in (0, 1, None):
        assert onp.array_equal(dnp.argmax(X, axis=axis).numpy(), onp.argmax(x, axis=axis))
        assert onp.array_equal(dnp.argmin(X, axis=axis).numpy(), onp.argmin(x, axis=axis))
    y = onp.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 2.4999, -0.0, onp.inf, onp.nan])
    Y = dnp.asarray(y)
    for name in ("floor", "ceil", "rint", "round", "trunc", "fix"):
        assert onp.array_equal(getattr(dnp, name)(Y).numpy(), getattr(onp, name)(y), equal_nan=True), name
    assert onp.array_equal(dnp.isnan(Y).numpy(), onp.isnan(y))
    assert onp.array_equal(dnp.isinf(Y).numpy(), onp.isinf(y))
    assert onp.array_equal(dnp.isfinite(Y).numpy(), onp.isfinite(y))
    from autograd_amd import grad

    assert float(grad(lambda v: dnp.sum(dnp.floor(v) * v))(Y[:3]).numpy()[0]) == -3.0  # floor is piecewise constant
