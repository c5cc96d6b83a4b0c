"""The five benchmark workloads, written once against an abstract array namespace.

Each workload is the user-level program (modelled on the reference's
examples/tanh.py:22-23, examples/neural_net.py:28-36, examples/rnn.py:20-61 and a
vectorised examples/rosenbrock.py:7-8) plus a seeded input generator.  A
``Backend`` bundles the array namespace and differential operators to run it
with: the device path (``device_backend()``), or any other implementation of
the same API supplied by the caller (the tests pass a NumPy one).

Inputs are always produced on the host with NumPy from
``numpy.random.RandomState(seed)`` in a fixed draw order, then handed to
``backend.put``; timing code must do that before the timed region.
"""

from collections import namedtuple

import numpy as onp

Backend = namedtuple(
    "Backend", "name np logsumexp grad elementwise_grad make_hvp make_jvp put get sync"
)


def device_backend():
    """The MI355X path: ``autograd_amd.numpy`` device arrays and HIP kernels."""
    import autograd_amd as ag
    import autograd_amd.numpy as dnp
    from autograd_amd.scipy.special import logsumexp

    return Backend(
        name="autograd_amd(HIP gfx950)",
        np=dnp,
        logsumexp=logsumexp,
        grad=ag.grad,
        elementwise_grad=ag.elementwise_grad,
        make_hvp=ag.make_hvp,
        make_jvp=ag.make_jvp,
        put=dnp.asarray,
        get=dnp.to_numpy,
        sync=dnp.synchronize,
    )


def tree_map(f, tree):
    if isinstance(tree, (list, tuple)):
        return type(tree)(tree_map(f, t) for t in tree)
    if isinstance(tree, dict):
        return {k: tree_map(f, v) for k, v in tree.items()}
    return f(tree)


def tree_leaves(tree):
    if isinstance(tree, (list, tuple)):
        return [leaf for t in tree for leaf in tree_leaves(t)]
    if isinstance(tree, dict):
        return [leaf for k in tree for leaf in tree_leaves(tree[k])]
    return [tree]


# --------------------------------------------------------------------------------------
# config 1: elementwise tanh derivatives, float64
# --------------------------------------------------------------------------------------
def tanh_inputs(n=4194304):
    return {"x": onp.linspace(-7.0, 7.0, n)}


def tanh_program(be):
    np = be.np

    def tanh(x):
        return (1.0 - np.exp(-2 * x)) / (1.0 + np.exp(-(2 * x)))

    eg = be.elementwise_grad
    return {
        "d1": eg(tanh),
        "d2": eg(eg(tanh)),
        "d3": eg(eg(eg(tanh))),
    }


# --------------------------------------------------------------------------------------
# config 2: broadcast + logsumexp + sum, float32
# --------------------------------------------------------------------------------------
def bcast_inputs(rows=8192, cols=4096, seed=0):
    rs = onp.random.RandomState(seed)
    A = rs.randn(rows, cols).astype(onp.float32)
    b = rs.uniform(0.5, 1.5, cols).astype(onp.float32)
    c = rs.randn(rows).astype(onp.float32)
    return {"A": A, "b": b, "c": c}


def bcast_program(be):
    np, logsumexp = be.np, be.logsumexp

    def L(A, b, c):
        return np.sum(logsumexp(A * b[None, :] + c[:, None], axis=1))

    return {"loss": L, "grad": be.grad(L, (0, 1, 2))}


# --------------------------------------------------------------------------------------
# config 3: MLP gradient, float32
# --------------------------------------------------------------------------------------
def mlp_inputs(batch=1024, layer_sizes=(784, 1024, 1024, 10), seed=0):
    rs = onp.random.RandomState(seed)
    X = rs.randn(batch, layer_sizes[0]).astype(onp.float32)
    labels = rs.randint(0, layer_sizes[-1], batch)
    T = (labels[:, None] == onp.arange(layer_sizes[-1])[None, :]).astype(onp.float32)
    params = []
    for m, n in zip(layer_sizes[:-1], layer_sizes[1:]):
        W = (0.1 * rs.randn(m, n)).astype(onp.float32)
        params.append((W, onp.zeros(n, onp.float32)))
    return {"X": X, "T": T, "params": params}


def mlp_program(be):
    np, logsumexp = be.np, be.logsumexp

    def predict(params, inputs):
        for W, b in params:
            outputs = np.dot(inputs, W) + b
            inputs = np.tanh(outputs)
        return outputs - logsumexp(outputs, axis=1, keepdims=True)

    def loss(params, X, T):
        return -np.sum(predict(params, X) * T)

    return {"loss": loss, "grad": be.grad(loss)}


# --------------------------------------------------------------------------------------
# config 4: vanilla tanh RNN driven by a Python loop, float32
# --------------------------------------------------------------------------------------
def rnn_inputs(seq_len=64, batch=256, input_size=128, state_size=512, output_size=128, seed=0, dtype=onp.float32):
    rs = onp.random.RandomState(seed)
    ids = rs.randint(0, input_size, (seq_len, batch))
    inputs = (ids[:, :, None] == onp.arange(input_size)[None, None, :]).astype(dtype)
    tids = rs.randint(0, output_size, (seq_len, batch))
    targets = (tids[:, :, None] == onp.arange(output_size)[None, None, :]).astype(dtype)
    params = {
        "init hiddens": (0.1 * rs.randn(1, state_size)).astype(dtype),
        "change": (0.1 * rs.randn(input_size + state_size + 1, state_size)).astype(dtype),
        "predict": (0.1 * rs.randn(state_size + 1, output_size)).astype(dtype),
    }
    return {"inputs": inputs, "targets": targets, "params": params}


def rnn_program(be):
    np, logsumexp = be.np, be.logsumexp

    def concat_and_multiply(weights, *args):
        cat_state = np.hstack(args + (np.ones((args[0].shape[0], 1), dtype=args[0].dtype),))
        return np.dot(cat_state, weights)

    def rnn_predict(params, inputs):
        def update_rnn(input, hiddens):
            return np.tanh(concat_and_multiply(params["change"], input, hiddens))

        def hiddens_to_output_probs(hiddens):
            output = concat_and_multiply(params["predict"], hiddens)
            return output - logsumexp(output, axis=1, keepdims=True)

        num_sequences = inputs.shape[1]
        hiddens = np.repeat(params["init hiddens"], num_sequences, axis=0)
        output = [hiddens_to_output_probs(hiddens)]
        for input in inputs:
            hiddens = update_rnn(input, hiddens)
            output.append(hiddens_to_output_probs(hiddens))
        return output

    def rnn_log_likelihood(params, inputs, targets):
        logprobs = rnn_predict(params, inputs)
        loglik = 0.0
        num_time_steps, num_examples, _ = inputs.shape
        for t in range(num_time_steps):
            loglik += np.sum(logprobs[t] * targets[t])
        return loglik / (num_time_steps * num_examples)

    def loss(params, inputs, targets):
        return -rnn_log_likelihood(params, inputs, targets)

    return {"loss": loss, "grad": be.grad(loss)}


# --------------------------------------------------------------------------------------
# config 5: Rosenbrock Hessian-vector product, float64
# --------------------------------------------------------------------------------------
def rosen_inputs(n=2**24, seed=0):
    rs = onp.random.RandomState(seed)
    x = rs.uniform(-2.0, 2.0, n)
    v = rs.randn(n)
    return {"x": x, "v": v}


def rosen_program(be):
    np = be.np

    def f(x):
        return np.sum(100 * (x[1:] - x[:-1] ** 2) ** 2 + (1 - x[:-1]) ** 2)

    def hvp_rev(x, v):
        """reverse-over-reverse, as the reference's make_hvp defines it"""
        return be.make_hvp(f)(x)[0](v)

    def hvp_fwd(x, v):
        """forward-over-reverse: JVP of the gradient"""
        return be.make_jvp(be.grad(f))(x)(v)[1]

    return {"f": f, "grad": be.grad(f), "hvp_rev": hvp_rev, "hvp_fwd": hvp_fwd}


# --------------------------------------------------------------------------------------
# beside the five configs: the LeNet-style stack of examples/convnet.py (conv 5x5x6, 2x2 max pool,
# conv 5x5x16, 2x2 max pool, tanh 120, tanh 84, log-softmax 10) on 28x28 images
# --------------------------------------------------------------------------------------
def convnet_inputs(batch=256, seed=0, dtype=onp.float64):
    rs = onp.random.RandomState(seed)
    shapes = {"c1": (1, 6, 5, 5), "b1": (1, 6, 1, 1), "c2": (6, 16, 5, 5), "b2": (1, 16, 1, 1),
              "w3": (256, 120), "b3": (120,), "w4": (120, 84), "b4": (84,), "w5": (84, 10), "b5": (10,)}
    params = {k: (0.1 * rs.randn(*shp)).astype(dtype) for k, shp in shapes.items()}
    X = rs.rand(batch, 1, 28, 28).astype(dtype)
    T = (rs.randint(0, 10, batch)[:, None] == onp.arange(10)[None, :]).astype(dtype)
    return {"params": params, "X": X, "T": T}


def convnet_program(be, convolve):
    np, logsumexp = be.np, be.logsumexp

    def pool(x):  # examples/convnet.py:112-119
        n, c, h, w = x.shape
        return np.max(np.max(x.reshape((n, c, h // 2, 2, w // 2, 2)), axis=3), axis=4)

    def predict(p, X):
        h = pool(convolve(X, p["c1"], axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode="valid") + p["b1"])
        h = pool(convolve(h, p["c2"], axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode="valid") + p["b2"])
        h = h.reshape((h.shape[0], 256))
        h = np.tanh(np.dot(h, p["w3"]) + p["b3"])
        h = np.tanh(np.dot(h, p["w4"]) + p["b4"])
        out = np.dot(h, p["w5"]) + p["b5"]
        return out - logsumexp(out, axis=1, keepdims=True)

    def loss(p, X, T):
        return -np.sum(predict(p, X) * T)

    return {"loss": loss, "grad": be.grad(loss)}


# --------------------------------------------------------------------------------------
# uniform runner: name -> {output name -> host array tree}
# --------------------------------------------------------------------------------------
def run_config(name, be, inputs):
    """Run workload ``name`` with backend ``be`` on host ``inputs``; return host results."""
    dev = tree_map(be.put, inputs)
    if name == "tanh":
        prog = tanh_program(be)
        out = {k: prog[k](dev["x"]) for k in ("d1", "d2", "d3")}
    elif name == "bcast":
        prog = bcast_program(be)
        dA, db, dc = prog["grad"](dev["A"], dev["b"], dev["c"])
        out = {"dA": dA, "db": db, "dc": dc}
    elif name == "mlp":
        prog = mlp_program(be)
        out = {"grad": prog["grad"](dev["params"], dev["X"], dev["T"])}
    elif name == "rnn":
        prog = rnn_program(be)
        out = {"grad": prog["grad"](dev["params"], dev["inputs"], dev["targets"])}
    elif name == "rosen":
        prog = rosen_program(be)
        out = {
            "grad": prog["grad"](dev["x"]),
            "hvp_rev": prog["hvp_rev"](dev["x"], dev["v"]),
            "hvp_fwd": prog["hvp_fwd"](dev["x"], dev["v"]),
        }
    else:
        raise KeyError(name)
    return tree_map(be.get, out)


CONFIG_INPUTS = {
    "tanh": tanh_inputs,
    "bcast": bcast_inputs,
    "mlp": mlp_inputs,
    "rnn": rnn_inputs,
    "rosen": rosen_inputs,
}
