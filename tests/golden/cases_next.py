"""Small seeded cases for the components either side of the hot path: container flattening,
optimizers, Jacobians/Hessians, and the rest of the elementwise rule table.

``next_cases(be, ext)`` is written against a ``configs.Backend`` plus a namespace ``ext`` with
``flatten, sgd, rmsprop, adam, jacobian, hessian, convolve`` so the same code runs on the reference (when
writing fixtures), the CPU oracle and the device.
"""

import numpy as onp


def _params(rs, P):
    return {
        "layers": [(P((0.3 * rs.randn(4, 3)).astype(onp.float32)), P(onp.zeros(3, onp.float32))),
                   (P((0.3 * rs.randn(3, 2)).astype(onp.float32)), P((0.1 * rs.randn(2)).astype(onp.float32)))],
        "scale": P(onp.asarray(1.5)),
    }


def next_cases(be, ext):
    np, grad, P = be.np, be.grad, be.put
    rs = onp.random.RandomState(11)
    out = {}

    # ---- flatten / unflatten (misc/flatten.py:11-35) ------------------------------------------
    params = _params(rs, P)
    flat, unflatten = ext.flatten(params)
    out["flatten/flat"] = flat
    out["flatten/roundtrip"] = unflatten(flat * 2.0)
    out["flatten/grad"] = grad(lambda p: np.sum(ext.flatten(p)[0] ** 2))(params)
    f32 = [P(rs.randn(3).astype(onp.float32)), (P(rs.randn(2, 2).astype(onp.float32)),)]
    flat32, un32 = ext.flatten(f32)
    out["flatten/f32_flat"] = flat32
    out["flatten/f32_roundtrip"] = un32(flat32)

    # ---- optimizers (misc/optimizers.py:33-75) on a small two-layer regression ---------------------
    X = P(rs.randn(5, 4).astype(onp.float32))
    Y = P(rs.randn(5, 2).astype(onp.float32))

    def loss(p, i):
        h = np.tanh(np.dot(X, p["layers"][0][0]) + p["layers"][0][1])
        y = np.dot(h, p["layers"][1][0]) + p["layers"][1][1]
        return np.sum((y * p["scale"] - Y) ** 2) * (1.0 + 0.1 * i)

    seen = {}

    def callback(x, i, g):
        if i == 2:
            seen["x"], seen["g"] = x, g

    out["opt/sgd"] = ext.sgd(grad(loss), params, num_iters=4, step_size=0.05, mass=0.8)
    out["opt/rmsprop"] = ext.rmsprop(grad(loss), params, num_iters=4, step_size=0.02)
    out["opt/adam"] = ext.adam(grad(loss), params, callback=callback, num_iters=5, step_size=0.01)
    out["opt/adam_callback_x"] = seen["x"]
    out["opt/adam_callback_g"] = seen["g"]
    # float64 parameters from the start
    p64 = [P(rs.randn(6)), P(rs.randn(2, 3))]
    q = lambda p, i: np.sum(np.sin(p[0]) * np.sum(p[1] ** 2)) + np.sum(p[1])  # noqa: E731
    out["opt/adam_f64"] = ext.adam(grad(q), p64, num_iters=3)
    out["opt/sgd_f64"] = ext.sgd(grad(q), p64, num_iters=3)
    out["opt/rmsprop_f64"] = ext.rmsprop(grad(q), p64, num_iters=3)

    # ---- jacobian / hessian (differential_operators.py:57-91) -------------------------------------
    A = P(rs.randn(3, 4))
    x = P(rs.randn(4))
    out["jac/matvec"] = ext.jacobian(lambda v: np.tanh(np.dot(A, v)))(x)
    out["jac/matrix_in"] = ext.jacobian(lambda M: np.dot(M, x) ** 2)(A)
    out["hess/quartic"] = ext.hessian(lambda v: np.sum(np.dot(A, v) ** 4) + np.sum(np.sin(v) * v))(x)

    # ---- the other differential operators (differential_operators.py:95-200), through ``ext.ag`` -------------
    ag = ext.ag
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        M, xv, vv = P(rs.randn(3, 4).astype(dtype)), P(rs.randn(4).astype(dtype)), P(rs.randn(4).astype(dtype))
        tv = P(rs.randn(3).astype(dtype))
        f = lambda z: np.sum(np.tanh(np.dot(M, z)) ** 2)  # noqa: E731,B023
        h = lambda z: np.tanh(np.dot(M, z))  # noqa: E731,B023
        out[f"operators/value_and_grad_{tag}"] = ag.value_and_grad(f)(xv)
        out[f"operators/grad_and_aux_{tag}"] = ag.grad_and_aux(lambda z: (f(z), np.sin(z)))(xv)  # noqa: B023
        out[f"operators/elementwise_grad_{tag}"] = ag.elementwise_grad(lambda z: np.sin(z) * z)(xv)
        out[f"operators/hessian_vector_product_{tag}"] = ag.hessian_vector_product(f)(xv, vv)
        out[f"operators/hessian_tensor_product_{tag}"] = ag.hessian_tensor_product(
            lambda Z: np.sum(np.tanh(Z) ** 2 * Z))(M, M * 0.5)
        out[f"operators/make_hvp_{tag}"] = ag.make_hvp(f)(xv)[0](vv)
        out[f"operators/vector_jacobian_product_{tag}"] = ag.vector_jacobian_product(h)(xv, tv)
        out[f"operators/tensor_jacobian_product_{tag}"] = ag.tensor_jacobian_product(lambda Z: np.sin(Z) * xv)(M, M * 2.0)  # noqa: B023
        out[f"operators/make_jvp_reversemode_{tag}"] = ext.make_jvp_reversemode(h)(xv)(vv)
        out[f"operators/make_jvp_{tag}"] = ag.make_jvp(h)(xv)(vv)
        out[f"operators/make_vjp_{tag}"] = ag.make_vjp(h)(xv)[0](tv)
        out[f"operators/make_ggnvp_{tag}"] = ag.make_ggnvp(h)(xv)(vv)
        out[f"operators/checkpoint_{tag}"] = grad(lambda z: np.sum(ag.checkpoint(h)(z) * tv))(xv)  # noqa: B023
        out[f"operators/grad_named_{tag}"] = ag.grad_named(lambda a, b: np.sum(np.dot(a, b) ** 2), "b")(M, xv)
        out[f"operators/jacobian_matrix_out_{tag}"] = ext.jacobian(lambda z: np.outer(np.sin(z), z))(xv)
        out[f"operators/grad_argnum_tuple_{tag}"] = grad(lambda a, b: np.sum(np.dot(a, b) ** 2), (1, 0))(M, xv)

    # ---- the rest of the elementwise rule table (numpy_vjps.py:104-135, 160-185, 215) ------------------
    u = rs.uniform(0.1, 0.9, (3, 4))          # inside every domain below
    w = rs.uniform(1.1, 3.0, (3, 4))
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        U, W = P(u.astype(dtype)), P(w.astype(dtype))
        for name in "exp2 log2 log10 tan arcsin arccos arctan arcsinh arctanh fabs rad2deg deg2rad".split():
            f = getattr(np, name)
            out[f"ufunc/{name}_{tag}/value"] = f(U)
            out[f"ufunc/{name}_{tag}/grad"] = grad(lambda z: np.sum(f(z) * W))(U)
        out[f"ufunc/arccosh_{tag}/grad"] = grad(lambda z: np.sum(np.arccosh(z) * U))(W)
        row = P(rs.uniform(0.2, 2.0, (1, 4)).astype(dtype))
        for name in "fmax fmin arctan2 hypot logaddexp".split():
            f = getattr(np, name)
            out[f"ufunc/{name}_{tag}/value"] = f(U, row)
            out[f"ufunc/{name}_{tag}/grad"] = grad(lambda a, b: np.sum(f(a, b) * W), (0, 1))(U, row)
        out[f"ufunc/clip_{tag}/grad"] = grad(lambda z: np.sum(np.clip(z, 0.3, 0.6) * W))(U)
        # single-argument grads keep the dtype the rule produces (no container accumulation casts it back)
        out[f"ufunc/maximum_{tag}/grad_single"] = grad(lambda z: np.sum(np.maximum(z, 0.5) * W))(U)
        out[f"ufunc/fmin_{tag}/grad_single"] = grad(lambda z: np.sum(np.fmin(z, row) * W))(U)
    # where: the rule's zeros are float64, so a float32 operand's cotangent is promoted (numpy_vjps.py:226-230)
    W32 = P(u.astype(onp.float32))
    out["ufunc/where_f32/grad_single"] = grad(lambda z: np.sum(np.where(z > 0.5, z, 2.0 * z) * z))(W32)
    out["ufunc/where_f64/grad_single"] = grad(lambda z: np.sum(np.where(z > 0.5, z, 2.0 * z) * z))(P(u))
    second = P(rs.uniform(0.2, 0.8, 5))
    out["ufunc/second_order"] = grad(lambda z: np.sum(grad(lambda t: np.sum(np.arctan(t) * np.log2(t) + np.tan(t)))(z)))(second)
    tie = P(onp.array([1.0, 2.0, 2.0, onp.nan, 3.0]))
    other = P(onp.array([1.0, 1.0, 3.0, 2.0, onp.nan]))
    out["ufunc/fmax_ties_nan"] = grad(lambda a, b: np.sum(np.fmax(a, b) * P(onp.arange(1.0, 6.0))), (0, 1))(tie, other)

    # ---- max / min over axes with ties (numpy_vjps.py:515-530; float64 results whatever the operand) ------
    tied = rs.randint(-2, 3, (4, 3, 5)).astype(onp.float64)
    tied[0] += rs.randn(3, 5)
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        Z = P(tied.astype(dtype))
        for fname in ("max", "min"):
            f = getattr(np, fname)
            for axis, keepdims in ((None, False), (0, False), (1, True), (2, False), ((0, 2), True)):
                value = f(Z, axis=axis, keepdims=keepdims)
                wts = P(onp.asarray(rs.randn(*onp.shape(be.get(value)))).astype(dtype))
                out[f"extremum/{fname}_{tag}_{axis}_{keepdims}/grad"] = grad(
                    lambda z: np.sum(f(z, axis=axis, keepdims=keepdims) * wts))(Z)  # noqa: B023

    # ---- dtype and value of every rule on a float32 operand: reverse, forward and second order ------------
    # (NumPy-2 promotion inside the reference's rule bodies decides the dtype: bool masks, integer counts,
    # float64 zeros and Python scalars all behave differently)
    xs = rs.uniform(0.2, 0.9, (3, 4)).astype(onp.float32)
    ys = rs.uniform(0.2, 0.9, (3, 4)).astype(onp.float32)
    ts = rs.randn(3, 4).astype(onp.float32)
    X32, Y32, T32 = P(xs), P(ys), P(ts)
    sweep = {}
    for name in ("exp log tanh sinh cosh sin cos sqrt square abs reciprocal log1p expm1 exp2 log2 log10 tan arcsin "
                 "arccos arctan arcsinh arctanh fabs negative sign rad2deg deg2rad").split():
        sweep[name] = lambda a, n=name: np.sum(getattr(np, n)(a))
    for name in "sum mean prod max min var std".split():
        for axis in (None, 0, 1):
            sweep[f"{name}_ax{axis}"] = lambda a, n=name, ax=axis: np.sum(getattr(np, n)(a, axis=ax))
    sweep["var_ddof1"] = lambda a: np.sum(np.var(a, axis=0, ddof=1))
    sweep["std_keepdims"] = lambda a: np.sum(np.std(a, axis=1, keepdims=True))
    for name in "add subtract multiply divide power maximum minimum fmax fmin arctan2 hypot logaddexp".split():
        sweep[f"{name}_array"] = lambda a, n=name: np.sum(getattr(np, n)(a, Y32))
        sweep[f"{name}_scalar"] = lambda a, n=name: np.sum(getattr(np, n)(a, 0.5))
        sweep[f"{name}_second_arg"] = lambda a, n=name: np.sum(getattr(np, n)(Y32, a))
    sweep["clip"] = lambda a: np.sum(np.clip(a, 0.3, 0.6))
    sweep["where"] = lambda a: np.sum(np.where(a > 0.5, a, 2.0 * a))
    sweep["reshape_T"] = lambda a: np.sum(np.reshape(a, (4, 3)).T * 2.0)
    sweep["getitem"] = lambda a: np.sum(a[1:, ::2] ** 2)
    sweep["dot"] = lambda a: np.sum(np.dot(a, Y32.T))
    sweep["int_power"] = lambda a: np.sum(a ** 3)
    sweep["divide_by_int"] = lambda a: np.sum(a / 3)
    sweep["mean_times_two"] = lambda a: np.mean(a) * 2
    sweep["concatenate"] = lambda a: np.sum(np.concatenate([a, a * 2], axis=0))
    sweep["repeat"] = lambda a: np.sum(np.repeat(a, 2, axis=1))
    sweep["expand_squeeze"] = lambda a: np.sum(np.squeeze(np.expand_dims(a, 0)))
    sweep["logsumexp_rows"] = lambda a: np.sum(be.logsumexp(a, axis=1))
    sweep["power_scalar_base"] = lambda a: np.sum(2.0 ** a)  # log(2.0) is a numpy.float64 inside the rule: float64 out
    for name in "subtract divide arctan2 hypot logaddexp maximum fmin".split():
        sweep[f"{name}_scalar_first"] = lambda a, n=name: np.sum(getattr(np, n)(0.5, a))
        sweep[f"{name}_numpy_scalar"] = lambda a, n=name: np.sum(getattr(np, n)(a, onp.float64(0.5)))
    for name, f in sweep.items():
        out[f"sweep/{name}/grad"] = grad(f)(X32)
        if not name.startswith("hypot"):  # the reference defines no forward rule for hypot
            value, tangent = be.make_jvp(f)(X32)(T32)
            out[f"sweep/{name}/jvp_value"], out[f"sweep/{name}/jvp_tangent"] = value, tangent
        out[f"sweep/{name}/second"] = grad(lambda a: np.sum(grad(f)(a) * T32))(X32)  # noqa: B023

    # ---- the namespace's other forms on (3,4) operands, both precisions: stacking, indexing, contractions of every
    # rank, methods and operators, multi-axis statistics, mixed operand types; reverse, forward, second order ----
    hA, hB, hv, hT = rs.uniform(0.2, 0.9, (3, 4)), rs.randn(4, 5), rs.randn(4), rs.randn(2, 3, 4)
    ramp = onp.arange(16.0).reshape(4, 4)
    rows = onp.array([2, 0, 2, 1])
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        A_, B_, v_, T_ = P(hA.astype(dtype)), P(hB.astype(dtype)), P(hv.astype(dtype)), P(hT.astype(dtype))
        R_, A64, I_ = P(ramp.astype(dtype)), P(hA), P(onp.arange(12).reshape(3, 4))
        forms = {
            "stack": lambda a: np.sum(np.stack([a, a * 2.0, np.sin(a)], axis=1) ** 2),
            "vstack": lambda a: np.sum(np.vstack([a, a * 3.0]) ** 2),
            "hstack": lambda a: np.sum(np.hstack([a, a * a]) * 1.5),
            "array_of_rows": lambda a: np.sum(np.array([a[0], a[1] * 2.0, a[2]]) ** 2),
            "array_of_scalars": lambda a: np.sum(np.array([a[0, 0], a[1, 1] * 2.0, 3.0]) ** 2),
            "moveaxis": lambda a: np.sum(np.moveaxis(np.expand_dims(a, 0), 0, 2) * 2.0),
            "swapaxes": lambda a: np.sum(np.dot(np.swapaxes(a, 0, 1), a)),
            "ravel": lambda a: np.sum(np.ravel(a)[::2] ** 2),
            "outer": lambda a: np.sum(np.outer(a[0], v_) * np.outer(a[0], v_)),
            "matmul_2d": lambda a: np.sum(np.matmul(a, B_) ** 2),
            "matmul_vec": lambda a: np.sum(np.matmul(a, v_) ** 2),
            "matmul_vec_left": lambda a: np.sum(np.matmul(v_[:3], a) ** 2),
            "matmul_batched": lambda a: np.sum(np.matmul(T_, a.T) ** 2),
            "dot_vec_vec": lambda a: np.dot(a[0], v_) * 2.0,
            "dot_mat_vec": lambda a: np.sum(np.dot(a, v_)),
            "dot_nd": lambda a: np.sum(np.dot(T_, a.T) * 0.5),
            "tensordot_2": lambda a: np.tensordot(a, a, axes=2) * 1.0,
            "tensordot_axes": lambda a: np.sum(np.tensordot(T_, a, axes=([2], [1])) ** 2),
            "tensordot_0": lambda a: np.sum(np.tensordot(a[0], v_, axes=0)),
            "take_rows": lambda a: np.sum(a[rows] * R_),
            "take_negative_slices": lambda a: np.sum(a[-2:, 1:-1] ** 3),
            "take_int": lambda a: np.sum(a[1] * a[-1]),
            "take_newaxis": lambda a: np.sum(a[:, None, :] * a[None, :, :]),
            "take_ellipsis": lambda a: np.sum(a[..., 1] ** 2),
            "broadcast_to": lambda a: np.sum(np.broadcast_to(a[:1], (5, 4)) * R_[0]),
            "atleast_2d": lambda a: np.sum(np.atleast_2d(a[0]) * 2.0),
            "var_two_axes": lambda a: np.sum(np.var(np.expand_dims(a, 0) * T_[:1], axis=(0, 2))),
            "mean_two_axes_keepdims": lambda a: np.sum(np.mean(a, axis=(0, 1), keepdims=True) * 3.0),
            "sum_negative_axis": lambda a: np.sum(np.sum(a, axis=-1) ** 2),
            "astype_float64": lambda a: np.sum(a.astype(onp.float64) ** 2),
            "astype_float32": lambda a: np.sum(a.astype(onp.float32) ** 2),
            "methods": lambda a: ((a.T.sum(axis=1) * a.mean(axis=0)).sum() + a.reshape(2, 6).max() + a.ravel().min()
                                  + np.dot(a, v_).prod()),
            "operators": lambda a: np.sum((-a) ** 2 / (a + 2.0) - (1.0 - a) * (2 - a) + 3 / (a * a + 1)),
            "powers": lambda a: np.sum(2.0 ** a + a ** 2.0 + a ** 0.5 + a ** -1),
            "where_and_mask": lambda a: np.sum(np.where(a > 0.5, np.exp(a), -a) * (a < 0.8)),
            "logical": lambda a: np.sum(a * np.logical_and(a > 0.3, a < 0.7) + a * np.logical_or(a > 0.8, a < 0.25) * 2.0),
            "abs_sign": lambda a: np.sum(np.abs(a - 0.5) * np.sign(a - 0.5)),
            "std_var_all": lambda a: np.std(a) + np.var(a, ddof=1),
            "times_float64_array": lambda a: np.sum(a * A64),
            "times_integer_array": lambda a: np.sum(a * I_),
            "squeeze_axis": lambda a: np.sum(np.squeeze(a[:, :1], axis=1) * v_[:3]),
            "repeat_axis0": lambda a: np.sum(np.repeat(a, 3, axis=0) * 0.5),
            "concatenate_axis1": lambda a: np.sum(np.concatenate((a, a[:, :2]), axis=1) ** 2),
            "prod_axis": lambda a: np.sum(np.prod(a, axis=1)),
            "softmax_shift": lambda a: np.sum(np.exp(a - np.max(a, axis=1, keepdims=True))),
        }
        tangent_in, weights2 = P((hA * 0.3).astype(dtype)), P(hA[::-1].copy().astype(dtype))
        for name, f in forms.items():
            out[f"forms/{name}_{tag}/grad"] = grad(f)(A_)
            if name not in ("astype_float64", "astype_float32", "var_two_axes"):  # no forward rule / a NameError there
                out[f"forms/{name}_{tag}/jvp_tangent"] = be.make_jvp(f)(A_)(tangent_in)[1]
            out[f"forms/{name}_{tag}/second"] = grad(lambda a: np.sum(grad(f)(a) * weights2))(A_)  # noqa: B023

    # ---- einsum (numpy_vjps.py:815-848): contraction, batch, summed-out, three operands, ellipsis ------
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        E = {k: P(rs.randn(*shp).astype(dtype)) for k, shp in
             dict(a=(3, 4), b=(4, 5), c=(5, 2), t=(2, 3, 4), u=(2, 4, 5), v=(6, 4), w=(1, 4, 5)).items()}
        cases = [
            ("mm", "ij,jk->ik", ("a", "b")), ("implicit", "ij,jk", ("a", "b")), ("batched", "bij,bjk->bik", ("t", "u")),
            ("summed_out", "ij,kj->i", ("a", "v")), ("three", "ij,jk,kl->il", ("a", "b", "c")),
            ("transpose", "ij->ji", ("a",)), ("total", "ij->", ("a",)), ("outer", "ij,kl->ijkl", ("a", "c")),
            ("ellipsis", "...ij,...jk->...ik", ("t", "w")), ("inner_batch", "bij,bij->b", ("t", "t")),
        ]
        for name, spec, ops in cases:
            args = tuple(E[o] for o in ops)
            out[f"einsum/{name}_{tag}/value"] = np.einsum(spec, *args)
            weights = P(onp.asarray(rs.randn(*onp.shape(be.get(out[f"einsum/{name}_{tag}/value"])))).astype(dtype))
            f = lambda *xs: np.sum(np.einsum(spec, *xs) * weights)  # noqa: E731,B023
            out[f"einsum/{name}_{tag}/grad"] = grad(f, tuple(range(len(args))))(*args)

    # ---- scipy.signal.convolve (scipy/signal.py:10-217): modes, operand orders, free / contracted axes ----
    conv = ext.convolve
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        C = {k: P(rs.randn(*shp).astype(dtype)) for k, shp in
             dict(v5=(5,), v3=(3,), v4=(4,), img=(2, 3, 6, 5), filt=(3, 4, 3, 2), m45=(4, 5), m23=(2, 3), m62=(6, 2),
                  m33=(3, 3), vol=(3, 4, 3), cube=(2, 2, 2), bat=(2, 5, 4), bank=(3, 2, 2)).items()}
        specs = []
        for mode in ("full", "valid", "same"):
            specs += [(f"1d_{mode}", ("v5", "v3"), dict(mode=mode)), (f"1d_swapped_{mode}", ("v3", "v5"), dict(mode=mode)),
                      (f"1d_even_{mode}", ("v5", "v4"), dict(mode=mode)),
                      (f"2d_{mode}", ("m45", "m23"), dict(mode=mode)), (f"2d_swapped_{mode}", ("m23", "m45"), dict(mode=mode)),
                      (f"3d_{mode}", ("vol", "cube"), dict(mode=mode)),
                      (f"free_axes_{mode}", ("bat", "bank"), dict(axes=([1, 2], [1, 2]), mode=mode)),
                      (f"convnet_{mode}", ("img", "filt"), dict(axes=([2, 3], [2, 3]), dot_axes=([1], [0]), mode=mode))]
        specs += [("2d_mixed_full", ("m45", "m62"), dict(mode="full")), ("2d_mixed_same", ("m45", "m62"), dict(mode="same")),
                  ("2d_equal_full", ("m33", "m33"), dict(mode="full")), ("2d_equal_valid", ("m33", "m33"), dict(mode="valid")),
                  ("one_axis_of_two", ("m45", "m23"), dict(axes=([1], [1]), mode="full")),
                  ("dot_first", ("m45", "m45"), dict(axes=([1], [1]), dot_axes=([0], [0]), mode="full"))]
        for name, ops, kw in specs:
            a, b = C[ops[0]], C[ops[1]]
            value = conv(a, b, **kw)
            out[f"conv/{name}_{tag}/value"] = value
            weights = P(rs.randn(*onp.shape(be.get(value))).astype(dtype))
            f = lambda x, y: np.sum(conv(x, y, **kw) * weights)  # noqa: E731,B023
            out[f"conv/{name}_{tag}/grad"] = grad(f, (0, 1))(a, b)
    # second order: the cotangent rules differentiated again (every flip of operands and result occurs)
    for mode in ("full", "valid", "same"):
        for name, ops, kw in [("1d", ("v5", "v4"), {}), ("1d_swapped", ("v3", "v5"), {}),
                              ("convnet", ("img", "filt"), dict(axes=([2, 3], [2, 3]), dot_axes=([1], [0])))]:
            a, b = C[ops[0]], C[ops[1]]
            first = lambda x, y: np.sum(np.sin(conv(x, y, mode=mode, **kw)))  # noqa: E731,B023
            second = lambda x, y: sum(np.sum(np.tanh(d)) for d in grad(first, (0, 1))(x, y))  # noqa: E731,B023
            out[f"conv/second_{name}_{mode}"] = grad(second, (0, 1))(a, b)
    

    # ---- the rest of the array-function table (numpy_vjps.py:128-137, 193-216, 352-405, 552-566, 863-870): remainder,
    # nan_to_num, roll, diagonals and triangles, tile, kron, inner; reverse, forward, second order, both precisions ----
    tA, tQ, tV, tT = rs.uniform(-0.9, 0.9, (3, 4)), rs.randn(4, 4), rs.randn(4), rs.randn(2, 3, 4)
    tB, tY = rs.randn(2, 3), rs.uniform(0.2, 0.6, (3, 4)) * rs.choice([-1.0, 1.0], (3, 4))
    tS = rs.randn(2, 3, 3)
    special = tA.copy()
    special[0, 1], special[1, 2], special[2, 0] = onp.nan, onp.inf, -onp.inf
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        A_, Q_, v_, T_, B_, Y_ = (P(h.astype(dtype)) for h in (tA, tQ, tV, tT, tB, tY))
        S_, C_ = P(special.astype(dtype)), P(tS.astype(dtype))
        W34, W44, W55 = (P(rs.randn(n, m).astype(dtype)) for n, m in ((3, 4), (4, 4), (5, 5)))
        table = {
            "remainder_array": (lambda a: np.sum(np.remainder(a, Y_) * W34), A_),
            "mod_scalar": (lambda a: np.sum(np.mod(a, 0.3) * W34), A_),
            "mod_negative_scalar": (lambda a: np.sum(np.mod(a, -0.4) * W34), A_),
            "mod_second_arg": (lambda a: np.sum(np.mod(Q_[:3] * 3.0, a) * W34), Y_),
            "mod_operator": (lambda a: np.sum((a % Y_) * W34), A_),
            "nan_to_num": (lambda a: np.sum(np.nan_to_num(a * 2.0) * 1e-30 * W34), S_),
            "roll_axis0": (lambda a: np.sum(np.roll(a, 1, axis=0) * W34), A_),
            "roll_axis1_negative": (lambda a: np.sum(np.roll(a, -2, axis=1) * W34), A_),
            "roll_flat": (lambda a: np.sum(np.roll(a, 5) * W34), A_),
            "roll_wraps": (lambda a: np.sum(np.roll(a, 9, axis=-1) * W34), A_),
            "diag_of_matrix": (lambda q: np.sum(np.diag(q, 1) ** 2), Q_),
            "diag_of_vector": (lambda q: np.sum(np.diag(q[0], -1) ** 2 * W55), Q_),
            "diag_twice": (lambda q: np.sum(np.diag(np.diag(q)) * W44), Q_),
            "diagonal_last_axes": (lambda t: np.sum(np.diagonal(t, 0, -1, -2) ** 2), C_),
            "make_diagonal": (lambda a: np.sum(np.make_diagonal(a, 0, -1, -2) * W44[None, :, :] * 2.0), A_),
            "trace": (lambda q: np.trace(q) * 2.0, Q_),
            "trace_offset": (lambda q: np.trace(q, offset=1) ** 2, Q_),
            "trace_rectangle": (lambda a: np.trace(a, offset=-1) * 3.0, A_),
            "trace_of_stack": (lambda t: np.sum(np.trace(t) * v_), T_),
            "tril": (lambda q: np.sum(np.tril(q) * W44), Q_),
            "triu_offset": (lambda q: np.sum(np.triu(q, 1) ** 2), Q_),
            "tril_rectangle": (lambda a: np.sum(np.tril(a, -1) * W34), A_),
            "triu_batched": (lambda t: np.sum(np.triu(t, -1) ** 2), T_),
            "tile_2d": (lambda a: np.sum(np.tile(a, (2, 3)) ** 2), A_),
            "tile_more_reps": (lambda a: np.sum(np.tile(a, (2, 1, 2)) * T_[:, :, :1] * 0.5), A_),
            "tile_vector_scalar_reps": (lambda q: np.sum(np.tile(q[1], 3) ** 3), Q_),
            "kron_2d": (lambda a: np.sum(np.kron(a, B_) ** 2), A_),
            "kron_2d_second": (lambda a: np.sum(np.kron(B_, a) ** 2), A_),
            "kron_1d": (lambda q: np.sum(np.kron(q[0], v_) ** 2), Q_),
            "kron_2d_1d": (lambda a: np.sum(np.kron(a, v_) ** 2), A_),
            "kron_both": (lambda a: np.sum(np.kron(a, a.T) * 0.5), A_),
            "inner_matrices": (lambda a: np.sum(np.inner(a, Q_) ** 2), A_),
            "inner_vectors": (lambda q: np.inner(q[0], v_) ** 2, Q_),
            "inner_stack_vector": (lambda t: np.sum(np.inner(t, v_) ** 2), T_),
            "inner_second": (lambda a: np.sum(np.inner(T_, a) ** 2), A_),
            "flipud": (lambda a: np.sum(np.flipud(a) * W34), A_),
            "fliplr": (lambda a: np.sum(np.fliplr(a) ** 2 * W34), A_),
            "fliplr_of_stack": (lambda t: np.sum(np.fliplr(t) * W34), T_),
            "rot90": (lambda q: np.sum(np.rot90(q) * W44), Q_),
            "rot90_half_turn": (lambda q: np.sum(np.rot90(q, 2) ** 2 * W44), Q_),
            "rot90_back": (lambda a: np.sum(np.rot90(a, -1) * W34.T), A_),
            "reversed_rows": (lambda a: np.sum(a[::-1] * W34), A_),
            "reversed_strided_columns": (lambda a: np.sum(a[:, ::-2] ** 2 * W34[:, :2]), A_),
            "reversed_both_partial": (lambda a: np.sum(a[2:0:-1, ::-1] * W34[:2]), A_),
            "reversed_after_ellipsis": (lambda t: np.sum(t[..., ::-1] ** 2 * W34), T_),
            "reversed_with_newaxis_and_int": (lambda t: np.sum(t[1, None, ::-1] * W34), T_),
            "cumsum_flat": (lambda a: np.sum(np.cumsum(a) ** 2), A_),
            "cumsum_axis0": (lambda a: np.sum(np.cumsum(a, axis=0) * W34), A_),
            "cumsum_axis1": (lambda a: np.sum(np.cumsum(a, axis=1) ** 2), A_),
            "cumsum_middle_axis": (lambda t: np.sum(np.cumsum(t, axis=1) * W34), T_),
            "cumsum_last_axis_of_stack": (lambda t: np.sum(np.cumsum(t, axis=-1) ** 2), T_),
            "split_even": (lambda a: np.sum(np.split(a, 2, axis=1)[0] * np.split(a, 2, axis=1)[1]), A_),
            "split_at_indices": (lambda a: np.sum(np.split(a, [1, 3], axis=1)[1] ** 2) + np.sum(np.split(a, [1, 3], 1)[2]), A_),
            "array_split_uneven": (lambda a: np.sum(np.array_split(a, 3, axis=1)[0] ** 2) + np.sum(np.array_split(a, 3, 1)[2] ** 3), A_),
            "vsplit": (lambda q: np.sum(np.vsplit(q, 2)[1] * W44[:2]), Q_),
            "hsplit": (lambda q: np.sum(np.hsplit(q, 2)[0] ** 2), Q_),
            "dsplit": (lambda t: np.sum(np.dsplit(t, 2)[1] ** 2 * W34[:, :2]), T_),
            "rollaxis": (lambda t: np.sum(np.rollaxis(t, 2) * W34.T[:, None, :]), T_),
            "rollaxis_to_end": (lambda t: np.sum(np.rollaxis(t, 0, 3) ** 2 * W34[:, :, None]), T_),
            "diff": (lambda a: np.sum(np.diff(a) ** 2), A_),
            "diff_twice_axis0": (lambda q: np.sum(np.diff(q, n=2, axis=0) * W44[:2]), Q_),
            "diff_vector_thrice": (lambda q: np.sum(np.diff(q[0], 3) ** 2), Q_),
            "cross_first": (lambda t: np.sum(np.cross(t[0].T, C_[0][:1] * 2.0) ** 2), T_),
            "cross_second": (lambda t: np.sum(np.cross(C_[1][None, :, :], t[:, :, :3]) ** 2), T_),
            "cross_axis": (lambda a: np.sum(np.cross(a, W34, axis=0) * Y_), A_),
            "sinc": (lambda a: np.sum(np.sinc(a) * W34), A_),
            "logaddexp2_array": (lambda a: np.sum(np.logaddexp2(a, Y_) * W34), A_),
            "logaddexp2_scalar": (lambda a: np.sum(np.logaddexp2(a, 0.5) ** 2), A_),
            "logaddexp2_second_arg": (lambda a: np.sum(np.logaddexp2(Y_ * 3.0, a) * W34), A_),
            "sort": (lambda q: np.sum(np.sort(q[1] * q[2]) * v_ ** 2), Q_),
            "sort_through_take": (lambda a: np.sum(np.sort(np.ravel(a))[::3] ** 2), A_),
            # (which of the two smallest comes first is the selection algorithm's business: weigh them alike)
            "partition": (lambda q: np.sum(np.partition(q[0] * q[3], 2)[:2]) * 2.0 + np.partition(q[0] * q[3], 2)[2] ** 2, Q_),
            "real_conj": (lambda a: np.sum(np.real(a) * np.conj(a) * 2.0), A_),
        }
        for name, (f, x) in table.items():
            out[f"table/{name}_{tag}/value"] = f(x)
            out[f"table/{name}_{tag}/grad"] = grad(f)(x)
            tangent_in = P(rs.randn(*onp.shape(be.get(x))).astype(dtype))
            out[f"table/{name}_{tag}/jvp_tangent"] = be.make_jvp(f)(x)(tangent_in)[1]
            if not name.startswith(("mod", "remainder_array", "nan_to_num")):  # piecewise linear in x: no second order
                weights2 = P(rs.randn(*onp.shape(be.get(x))).astype(dtype))
                out[f"table/{name}_{tag}/second"] = grad(lambda a: np.sum(grad(f)(a) * weights2))(x)  # noqa: B023
    # ---- rules that nothing above exercises: degrees/radians (numpy_vjps.py:112-115, numpy_jvps.py:78-81), full
    # (88-89; 33), array(ndmin=) (665-670), the pad and arccosh tangents (numpy_jvps.py:303, 105), einsum in the
    # sublist convention and with repeated subscripts (numpy_vjps.py:790-854), linspace (240-244) and gradient
    # (297-342).  A generator of their own, so that the draws above stay what they were. ----
    rs2 = onp.random.RandomState(23)
    hA, hQ, hv = rs2.randn(3, 4), rs2.randn(4, 4), rs2.randn(4)
    hT, hC = rs2.randn(2, 3, 4), rs2.uniform(1.2, 3.0, (3, 4))
    hG = rs2.randn(6, 5)
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        A_, Q_, v_, T_, C_, G_ = (P(h.astype(dtype)) for h in (hA, hQ, hv, hT, hC, hG))
        W34, W44 = P(rs2.randn(3, 4).astype(dtype)), P(rs2.randn(4, 4).astype(dtype))
        s0, s1 = P(onp.asarray(0.7, dtype)), P(onp.asarray(-1.9, dtype))
        lin_w = P(rs2.randn(7).astype(dtype))
        more = {
            "degrees": (lambda a: np.sum(np.degrees(a) ** 2 * W34), A_),
            "radians": (lambda a: np.sum(np.sin(np.radians(a * 50.0)) * W34), A_),
            "rad2deg": (lambda a: np.sum(np.rad2deg(a) * W34), A_),
            "deg2rad": (lambda a: np.sum(np.deg2rad(a) ** 3 * W34), A_),
            "full": (lambda f: np.sum(np.full((3, 4), f) ** 2 * W34), s0),
            "full_with_dtype": (lambda f: np.sum(np.full(4, np.sin(f), dtype=dtype) * v_), s1),  # noqa: B023
            "array_ndmin": (lambda a: np.sum(np.array(a, ndmin=4)[0, 0] ** 2 * W34), A_),
            "array_ndmin_of_scalar": (lambda f: np.sum(np.array(f, ndmin=2) ** 3), s0),
            "pad_constant": (lambda a: np.sum(np.pad(a, ((1, 2), (0, 1)), "constant") ** 2), A_),
            "pad_one_width": (lambda q: np.sum(np.pad(q, 1, "constant")[1:, :-1] * W44[0, 0] * np.pad(q, 1, "constant")[:-1, 1:]), Q_),
            "arccosh": (lambda c: np.sum(np.arccosh(c) * W34), C_),
            "arccosh_composed": (lambda c: np.sum(np.arccosh(c * c) ** 2), C_),
            "einsum_sublist": (lambda a: np.sum(np.einsum(a, [0, 1], Q_, [1, 2], [0, 2]) ** 2 * W34), A_),
            "einsum_sublist_second": (lambda q: np.sum(np.einsum(A_, [0, 1], q, [1, 2], [0, 2]) * W34), Q_),
            "einsum_sublist_ellipsis": (lambda t: np.sum(np.einsum(t, [Ellipsis, 0, 1], Q_, [1, 2], [Ellipsis, 0, 2]) ** 2), T_),
            # (the reference's rule cannot differentiate the operand that carries a repeated subscript; the others it can)
            "einsum_repeated_other_operand": (lambda w: np.sum(np.einsum("ii,ij->j", Q_, w) ** 2), W44),
            "einsum_repeated_other_operand_first": (lambda a: np.sum(np.einsum("ij,jj->i", a, Q_) ** 2), A_),
            "einsum_repeated_three_operands": (lambda a: np.sum(np.einsum("ij,jj,j->i", a, Q_, v_) * a[:, 0]), A_),
            "linspace_start": (lambda f: np.sum(np.linspace(f, 2.5, 7) ** 2 * lin_w), s0),  # noqa: B023
            "linspace_stop": (lambda f: np.sum(np.sin(np.linspace(-0.5, f, 7)) * lin_w), s1),  # noqa: B023
            "linspace_both": (lambda f: np.sum(np.linspace(f, f * f, 7) ** 2), s0),
            # (the reference's cotangent needs at least four samples along each differentiated axis)
            "gradient_vector": (lambda q: np.sum(np.gradient(q[0]) ** 2), Q_),
            "gradient_axis0": (lambda m: np.sum(np.gradient(m, axis=0) * np.sin(m)), G_),
            "gradient_axis1": (lambda a: np.sum(np.gradient(a, axis=1) ** 2 * W34), A_),
            "gradient_last_axis_of_stack": (lambda t: np.sum(np.gradient(t, axis=-1) ** 2), T_),
            "gradient_all_axes": (lambda m: np.sum(np.gradient(m)[0] * np.gradient(m)[1]), G_),
            "gradient_axis_pair": (lambda m: np.sum(np.gradient(m, axis=(1, 0))[0] ** 2) + np.sum(np.gradient(m, axis=(1, 0))[1]), G_),
        }
        for name, (f, x) in more.items():
            out[f"more/{name}_{tag}/value"] = f(x)
            out[f"more/{name}_{tag}/grad"] = grad(f)(x)
            tangent_in = P(onp.asarray(rs2.randn(*onp.shape(be.get(x)))).astype(dtype))
            out[f"more/{name}_{tag}/jvp_tangent"] = be.make_jvp(f)(x)(tangent_in)[1]
            weights2 = P(onp.asarray(rs2.randn(*onp.shape(be.get(x)))).astype(dtype))
            out[f"more/{name}_{tag}/second"] = grad(lambda a: np.sum(grad(f)(a) * weights2))(x)  # noqa: B023
    # ---- joins written with the index tricks and the list-taking helpers of numpy_wrapper.py:58-60, 73-80, 139-169
    # (r_, c_, append, column_stack, select).  A generator of their own again. ----
    rs3 = onp.random.RandomState(31)
    h32, h32b, h3 = rs3.randn(3, 2), rs3.randn(3, 2), rs3.randn(3)
    hsel = rs3.randn(3, 4)
    c1, c2 = rs3.randn(3, 4) > 0.2, rs3.randn(3, 4) > -0.3
    for dtype in (onp.float64, onp.float32):
        tag = "f32" if dtype == onp.float32 else "f64"
        X_, K_, V_, S_ = (P(h.astype(dtype)) for h in (h32, h32b, h3, hsel))
        W62, W36, W34b = (P(rs3.randn(*shape).astype(dtype)) for shape in ((6, 2), (3, 6), (3, 4)))
        w9, w8 = P(rs3.randn(9).astype(dtype)), P(rs3.randn(8).astype(dtype))
        M1, M2 = P(c1), P(c2)
        joins = {
            "r_double": (lambda x: np.sum(np.r_[x, x] ** 2 * W62), X_),
            "r_mixed": (lambda x: np.sum(np.sin(np.r_[x, K_]) * W62), X_),
            "r_vector_and_range": (lambda v: np.sum(np.r_[v, V_, 1:4] ** 2 * w9), V_),
            "c_mixed": (lambda x: np.sum(np.c_[x, K_, x] ** 3 * W36), X_),
            "c_vectors": (lambda v: np.sum(np.c_[v, V_ * v] ** 2), V_),
            "append_flat": (lambda x: np.sum(np.append(x, K_[0]) ** 2 * w8), X_),
            "append_axis": (lambda x: np.sum(np.tanh(np.append(x, K_, axis=0)) * W62), X_),
            "column_stack": (lambda v: np.sum(np.column_stack((v, K_, v * v)) ** 2), V_),
            "select": (lambda a: np.sum(np.select([M1, M2], [a * a, np.sin(a)], default=0.5) * W34b), S_),
        }
        for name, (f, x) in joins.items():
            out[f"joins/{name}_{tag}/value"] = f(x)
            out[f"joins/{name}_{tag}/grad"] = grad(f)(x)
            tangent_in = P(onp.asarray(rs3.randn(*onp.shape(be.get(x)))).astype(dtype))
            out[f"joins/{name}_{tag}/jvp_tangent"] = be.make_jvp(f)(x)(tangent_in)[1]
            weights2 = P(onp.asarray(rs3.randn(*onp.shape(be.get(x)))).astype(dtype))
            out[f"joins/{name}_{tag}/second"] = grad(lambda a: np.sum(grad(f)(a) * weights2))(x)  # noqa: B023
    return out
