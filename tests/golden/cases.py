"""Cases shared by the fixture generator and the tests that replay them.

``SMALL`` are the reduced sizes of the five workloads; ``extra_cases`` are small
graphs whose exact value depends on accumulation order, on NumPy-2 dtype
promotion inside reduction rules, or on the rank/axes handling of the
contraction adjoints.  Written against a ``configs.Backend`` so the same code
runs on the reference (when writing fixtures), the CPU oracle and the device.
"""

import numpy as onp

SMALL = {
    "tanh": dict(n=257),
    "bcast": dict(rows=37, cols=29),
    "mlp": dict(batch=16, layer_sizes=(12, 9, 7, 5)),
    "rnn": dict(seq_len=5, batch=6, input_size=7, state_size=8, output_size=7),
    "rosen": dict(n=33),
}


def flatten(prefix, tree, out):
    if isinstance(tree, (list, tuple)):
        for i, t in enumerate(tree):
            flatten(f"{prefix}/{i}", t, out)
    elif isinstance(tree, dict):
        for k, t in tree.items():
            flatten(f"{prefix}/{k}", t, out)
    else:
        out[prefix] = onp.asarray(tree)


def extra_cases(be):
    """Small graphs whose exact value depends on accumulation order or promotion."""
    np, grad, P = be.np, be.grad, be.put
    rs = onp.random.RandomState(7)
    out = {}
    x = P(rs.randn(6))
    # repeated-index gather: cotangent scattered with sequential accumulation
    out["dup_index_010"] = grad(lambda x: np.sum(np.sin(x[[0, 1, 0]]) * P(onp.array([1.0, 2.0, 3.0]))))(x)
    out["dup_index_00"] = grad(lambda x: np.sum(x[[0, 0]] ** 2))(x)
    # dense + sparse contributions to the same node
    out["mix_dense_sparse"] = grad(lambda x: np.sum(x * x) + x[2] * 3.0 + np.sum(x[1:4]) + x[2] ** 2)(x)
    # fan-out with three dense contributions (vs.add then mut_add)
    out["fanout3"] = grad(lambda x: np.sum(np.exp(x) + np.sin(x) * x + x / 3.0))(x)
    # reduction rules and their dtypes under NumPy-2 promotion
    x32h = rs.randn(4, 5).astype(onp.float32)
    x32 = P(x32h)
    out["mean_f32_all"] = grad(lambda x: np.mean(x))(x32)
    out["mean_f32_axis0"] = grad(lambda x: np.sum(np.mean(x, axis=0) ** 2))(x32)
    out["sum_f32_axis1"] = grad(lambda x: np.sum(np.sum(x, axis=1, keepdims=True) ** 2))(x32)
    out["var_f32"] = grad(lambda x: np.var(x))(x32)
    out["std_f64_axis1"] = grad(lambda x: np.sum(np.std(x, axis=1)))(P(x32h.astype(onp.float64)))
    out["max_axis0"] = grad(lambda x: np.sum(np.max(x, axis=0)))(P(x32h.astype(onp.float64)))
    # binary rules over broadcasting shapes (unbroadcast over every axis pattern)
    a, b = rs.randn(3, 4), rs.randn(1, 4) + 3.0
    for opname in ("add", "subtract", "multiply", "true_divide", "power", "maximum"):
        op = getattr(np, opname)
        base = onp.abs(a) + 0.5 if opname == "power" else a
        ga, gb = grad(lambda a, b: np.sum(np.sin(op(a, b))), (0, 1))(P(base), P(b))
        out[f"bin_{opname}_34_14/a"], out[f"bin_{opname}_34_14/b"] = ga, gb
        ga, gb = grad(lambda a, b: np.sum(np.sin(op(a, b))), (0, 1))(P(base[0]), P(b[0, 0]))
        out[f"bin_{opname}_4_s/a"], out[f"bin_{opname}_4_s/b"] = ga, gb
    # logsumexp rules, every axis form
    m = P(rs.randn(5, 4))
    for axis in (None, 0, 1):
        for keepdims in (False, True):
            key = f"lse_axis{axis}_keep{int(keepdims)}"
            out[key] = grad(lambda m: np.sum(np.cos(be.logsumexp(m, axis=axis, keepdims=keepdims))))(m)
    # dot in its rank combinations
    Ah, Bh, vh = rs.randn(3, 4), rs.randn(4, 5), rs.randn(4)
    A, B, v = P(Ah), P(Bh), P(vh)
    gA, gB = grad(lambda A, B: np.sum(np.sin(np.dot(A, B))), (0, 1))(A, B)
    out["dot_mm/A"], out["dot_mm/B"] = gA, gB
    gA, gv = grad(lambda A, v: np.sum(np.sin(np.dot(A, v))), (0, 1))(A, v)
    out["dot_mv/A"], out["dot_mv/v"] = gA, gv
    gv, gB = grad(lambda v, B: np.sum(np.sin(np.dot(v, B))), (0, 1))(v, B)
    out["dot_vm/v"], out["dot_vm/B"] = gv, gB
    gu, gv = grad(lambda u, v: np.sin(np.dot(u, v)), (0, 1))(P(vh[::-1].copy()), v)
    out["dot_vv/u"], out["dot_vv/v"] = gu, gv
    # tensordot with list axes, second order through the adjoint primitives
    T1h, T2h = rs.randn(2, 3, 4), rs.randn(4, 3, 5)
    T1, T2 = P(T1h), P(T2h)
    f = lambda T1, T2: np.sum(np.sin(np.tensordot(T1, T2, axes=[[1, 2], [1, 0]])))
    g1, g2 = grad(f, (0, 1))(T1, T2)
    out["tensordot/T1"], out["tensordot/T2"] = g1, g2
    out["tensordot_2nd"] = grad(lambda T1: np.sum(np.cos(grad(f, 1)(T1, T2))))(T1)
    out["dot_2nd"] = grad(lambda A: np.sum(np.cos(grad(lambda A, B: np.sum(np.sin(np.dot(A, B))), 1)(A, B))))(A)
    return {k: be.get(val) for k, val in out.items()}


