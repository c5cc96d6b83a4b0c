"""Answers that come from no tracer: textbook derivatives and brute force, in NumPy.

Used to pin the oracle's restatement (and, transitively, the device path) where
the reference's tests hold no vectors.  Everything is computed in float64
whatever the workload's dtype, so it also serves as the accuracy yardstick for
float32 results.  TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

import numpy as np
from scipy.special import logsumexp as _lse


# config 1: f = tanh, derivatives in terms of t = tanh(x)
def tanh_derivatives(x):
    t = np.tanh(np.asarray(x, np.float64))
    s = 1.0 - t * t
    return {"d1": s, "d2": -2.0 * t * s, "d3": -2.0 * s * (1.0 - 3.0 * t * t)}


# config 2: L = sum_i logsumexp_j(A_ij b_j + c_i); S = row softmax of the argument
def bcast_grads(A, b, c):
    A, b, c = (np.asarray(v, np.float64) for v in (A, b, c))
    Z = A * b[None, :] + c[:, None]
    S = np.exp(Z - _lse(Z, axis=1, keepdims=True))
    return {"dA": S * b[None, :], "db": np.sum(A * S, axis=0), "dc": np.sum(S, axis=1)}


# config 3: hand-written backprop of the tanh MLP with log-softmax loss
def mlp_grads(params, X, T):
    params = [(np.asarray(W, np.float64), np.asarray(b, np.float64)) for W, b in params]
    X, T = np.asarray(X, np.float64), np.asarray(T, np.float64)
    acts, pre = [X], []
    for W, b in params:
        pre.append(acts[-1] @ W + b)
        acts.append(np.tanh(pre[-1]))
    out = pre[-1]
    softmax = np.exp(out - _lse(out, axis=1, keepdims=True))
    # loss = -sum((out - lse(out)) * T)  ->  d/d out = -(T - softmax * sum_k T_k)
    delta = -(T - softmax * T.sum(axis=1, keepdims=True))
    grads = []
    for layer in range(len(params) - 1, -1, -1):
        W, _ = params[layer]
        grads.append((acts[layer].T @ delta, delta.sum(axis=0)))
        if layer:
            delta = (delta @ W.T) * (1.0 - np.tanh(pre[layer - 1]) ** 2)
    return grads[::-1]


# config 4: hand-written backprop through time of the tanh RNN
def rnn_grads(params, inputs, targets):
    p = {k: np.asarray(v, np.float64) for k, v in params.items()}
    inputs, targets = np.asarray(inputs, np.float64), np.asarray(targets, np.float64)
    Tn, B, _ = inputs.shape
    ones = np.ones((B, 1))
    h = [np.repeat(p["init hiddens"], B, axis=0)]
    cats = []
    for t in range(Tn):
        cats.append(np.hstack((inputs[t], h[-1], ones)))
        h.append(np.tanh(cats[-1] @ p["change"]))
    scale = -1.0 / (Tn * B)
    dchange, dpredict = np.zeros_like(p["change"]), np.zeros_like(p["predict"])
    dh_next = np.zeros_like(h[0])
    n_in = inputs.shape[2]
    # outputs 0..Tn-1 enter the loss (output k is produced from hidden state k)
    for k in range(Tn, -1, -1):
        dh = dh_next
        if k < Tn:
            hc = np.hstack((h[k], ones))
            out = hc @ p["predict"]
            sm = np.exp(out - _lse(out, axis=1, keepdims=True))
            dout = scale * (targets[k] - sm * targets[k].sum(axis=1, keepdims=True))
            dpredict += hc.T @ dout
            dh = dh + (dout @ p["predict"].T)[:, :-1]
        if k == 0:
            dinit = dh.sum(axis=0, keepdims=True)
            break
        dpre = dh * (1.0 - h[k] ** 2)
        dchange += cats[k - 1].T @ dpre
        dh_next = (dpre @ p["change"].T)[:, n_in:-1]
    return {"init hiddens": dinit, "change": dchange, "predict": dpredict}


# config 5: Rosenbrock chain, gradient and tridiagonal Hessian times v
def rosen_grad(x):
    x = np.asarray(x, np.float64)
    g = np.zeros_like(x)
    d = x[1:] - x[:-1] ** 2
    g[1:] += 200.0 * d
    g[:-1] += -400.0 * x[:-1] * d - 2.0 * (1.0 - x[:-1])
    return g


def rosen_hvp(x, v):
    x, v = np.asarray(x, np.float64), np.asarray(v, np.float64)
    diag = np.zeros_like(x)
    diag[1:] += 200.0
    diag[:-1] += 1200.0 * x[:-1] ** 2 - 400.0 * x[1:] + 2.0
    off = -400.0 * x[:-1]
    out = diag * v
    out[:-1] += off * v[1:]
    out[1:] += off * v[:-1]
    return out


def numerical_grad(f, x, eps=1e-6):
    """Central differences, element by element (tiny inputs only)."""
    x = np.array(x, np.float64)
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        old = x[i]
        x[i] = old + eps
        hi = f(x)
        x[i] = old - eps
        lo = f(x)
        x[i] = old
        g[i] = (hi - lo) / (2 * eps)
    return g
