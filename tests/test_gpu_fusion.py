"""Elementwise chains evaluated as one launch (``agmi_program``, ``autograd_amd/numpy/fusion.py``).

The fused evaluation must give, bit for bit, what the same steps give when every rule is launched on its own
(``fusion.ENABLED = False``): each instruction of a program is the one-rule kernel's functor, rounded on its own.
Checked here on the workloads the chains come from (config 1: tanh to third order, reference
examples/tanh.py:22-23; config 5: Rosenbrock Hessian-vector products through ``x[1:]`` / ``x[:-1]`` and their scattered
cotangents, autograd/numpy/numpy_vjps.py:919-950), on seeded random programs, and at the C ABI (argument checking,
shifted leaves, range masks, row layouts, ragged extents).
"""

import numpy as onp
import pytest

pytestmark = pytest.mark.gpu

from cases_random import make_program  # noqa: E402  (tests/golden is on sys.path, see conftest.py)

F32, F64 = onp.dtype("float32"), onp.dtype("float64")


@pytest.fixture()
def dnp():
    import autograd_amd.numpy as dnp

    return dnp


class unfused:
    """``with unfused(): ...``: every elementwise step is launched on its own, as before chains were deferred."""

    def __enter__(self):
        from autograd_amd.numpy import fusion

        self.was, fusion.ENABLED = fusion.ENABLED, False

    def __exit__(self, *exc):
        from autograd_amd.numpy import fusion

        fusion.ENABLED = self.was


def _both_ways(fn):
    from autograd_amd.numpy import fusion

    assert fusion.ENABLED
    before = dict(fusion.COUNTS)
    fused = fn()
    ran = {k: fusion.COUNTS[k] - before[k] for k in before}
    with unfused():
        plain = fn()
    return fused, plain, ran


def _same_bits(a, b):
    a, b = onp.asarray(a), onp.asarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and onp.array_equal(a, b, equal_nan=True)


# ---- the workloads ---------------------------------------------------------------------------------
@pytest.mark.parametrize("order", ["d1", "d2", "d3"])
@pytest.mark.parametrize("n", [4099, 1 << 20])
def test_tanh_orders_fused_equal_unfused(order, n):
    from autograd_amd import configs

    be = configs.device_backend()
    x = be.put(configs.tanh_inputs(n=n)["x"])
    f = configs.tanh_program(be)[order]
    fused, plain, ran = _both_ways(lambda: be.get(f(x)))
    assert _same_bits(fused, plain)
    # launches: one program for the first two orders, a handful for the third
    assert ran["programs"] <= {"d1": 1, "d2": 1, "d3": 6}[order] and ran["single"] == 0 and ran["unfused"] == 0


@pytest.mark.parametrize("which", ["grad", "hvp_rev", "hvp_fwd"])
@pytest.mark.parametrize("n", [4097, 1 << 20])
def test_rosenbrock_fused_equals_unfused(which, n):
    from autograd_amd import configs

    be = configs.device_backend()
    inp = configs.rosen_inputs(n=n)
    x, v = be.put(inp["x"]), be.put(inp["v"])
    p = configs.rosen_program(be)
    call = (lambda: be.get(p["grad"](x))) if which == "grad" else (lambda: be.get(p[which](x, v)))
    fused, plain, ran = _both_ways(call)
    assert _same_bits(fused, plain)
    # slices of x and the cotangents scattered back through them stay inside ONE program
    assert ran["programs"] == 1 and ran["single"] == 0 and ran["unfused"] == 0


def test_mlp_gradient_fused_equals_unfused():
    """Dense layers: bias + tanh in the forward contraction's epilogue, the tanh rule in the cotangent contraction's."""
    from autograd_amd import configs
    from autograd_amd.numpy import fusion

    be = configs.device_backend()
    inp = configs.mlp_inputs(batch=192, layer_sizes=(100, 256, 128, 10), seed=3)
    rs = onp.random.RandomState(0)
    params = [(be.put(W), be.put((0.1 * rs.randn(*b.shape)).astype(b.dtype))) for W, b in inp["params"]]
    X, T = be.put(inp["X"]), be.put(inp["T"])
    g = configs.mlp_program(be)["grad"]

    def run():
        return [tuple(be.get(a) for a in layer) for layer in g(params, X, T)]

    fused, plain, ran = _both_ways(run)
    assert ran["layers"] == 4  # two hidden layers forward, two backward
    for lf, lp in zip(fused, plain):
        for a, b in zip(lf, lp):
            assert _same_bits(a, b)


@pytest.mark.parametrize("dtype", [F64, F32])
def test_random_programs_fused_equal_unfused(dtype, dnp):
    import autograd_amd as ag
    from autograd_amd.scipy.special import logsumexp as dlse

    checked = 0
    for seed in range(300, 380):
        program, inputs = make_program(seed)
        dev = [dnp.asarray(a.astype(dtype)) for a in inputs]
        argnums = tuple(range(len(dev)))
        call = lambda: [g.numpy() for g in ag.grad(lambda *xs: program(dnp, dlse, *xs), argnums)(*dev)]  # noqa: E731
        fused, plain, _ = _both_ways(call)
        for k, (a, b) in enumerate(zip(fused, plain)):
            assert _same_bits(a, b), (seed, k)
        checked += 1
    assert checked == 80


def test_forward_values_fused_equal_unfused(dnp):
    """Values, not only cotangents: pending chains read by reductions, contractions, slices and the host."""
    rs = onp.random.RandomState(5)
    a, b = rs.randn(257, 130), rs.rand(130) + 0.5
    A, B = dnp.asarray(a), dnp.asarray(b)

    def run():
        y = dnp.exp(-A * A) / (1.0 + dnp.sqrt(dnp.abs(A) + B))   # a chain with a broadcast row
        z = dnp.tanh(y) * y - dnp.log1p(y * y)
        return [z.numpy(), dnp.sum(z, axis=0).numpy(), dnp.dot(z, z.T)[:3].numpy(), (z[10:20] + 1.0).numpy(),
                float(dnp.max(z)), dnp.where(z > 0.1, z, -z).numpy()]

    fused, plain, ran = _both_ways(run)
    assert ran["programs"] >= 1
    for f, p in zip(fused, plain):
        assert _same_bits(f, p)


def test_a_long_chain_is_cut_into_programs(dnp):
    from autograd_amd.numpy import fusion

    x = dnp.asarray(onp.linspace(0.1, 1.0, 5000))

    def run():
        y = x
        for k in range(400):  # more steps than one program holds
            y = y * 1.01 + dnp.sin(y) if k % 7 == 0 else y * 0.99 + 0.001
        return y.numpy()

    fused, plain, ran = _both_ways(run)
    assert _same_bits(fused, plain)
    assert 2 <= ran["programs"] <= 40 and ran["instructions"] >= 400


def test_leaves_are_not_written_while_an_expression_reads_them(dnp):
    """A pending expression reads its operands when it is evaluated: item assignment into one of them in between
    goes to a buffer of its own (NumPy semantics: ``y`` was computed before the write)."""
    x = dnp.asarray(onp.arange(8.0))
    y = dnp.exp(x) + x          # pending
    x[0] = 100.0                # must not reach y
    assert onp.array_equal(y.numpy(), onp.exp(onp.arange(8.0)) + onp.arange(8.0))
    assert float(x[0]) == 100.0


# ---- the entry point ---------------------------------------------------------------------------------
def W(op, dst, a=0, b=0, c=0, d=0):
    return op | dst << 8 | a << 12 | b << 16 | c << 20 | d << 24


def test_the_sum_of_a_whole_array_runs_when_its_value_is_read(dnp):
    """The last step of most losses is the sum of a whole array.  `grad` never reads its value, so no kernel runs for
    it; `value_and_grad`, arithmetic on the scalar or a host read run it then, on the values the array had when the sum
    was taken (a later item assignment goes to a buffer of its own)."""
    import autograd_amd as ag
    from autograd_amd import _lib

    rs = onp.random.RandomState(9)
    x = rs.randn(300, 70)
    X = dnp.asarray(x)
    calls = []
    real = _lib.map_reduce
    _lib.map_reduce = lambda *a, **k: (calls.append(a[0]), real(*a, **k))[1]
    try:
        g = ag.grad(lambda a: dnp.sum(dnp.tanh(a) * a))(X).numpy()
        assert calls == []  # nothing was reduced: the cotangent of a sum is a broadcast of g
        v, g2 = ag.value_and_grad(lambda a: dnp.sum(dnp.tanh(a) * a))(X)
        assert len(calls) == 1 and onp.allclose(float(v), onp.sum(onp.tanh(x) * x), rtol=1e-12)
        assert onp.array_equal(g2.numpy(), g)
        s = dnp.sum(X)
        n = len(calls)
        X[0, 0] = 1000.0           # after the sum was taken
        assert len(calls) == n and onp.allclose(float(s), onp.sum(x), rtol=1e-12) and len(calls) == n + 1
        assert onp.allclose(float(dnp.sum(X)), onp.sum(x) - x[0, 0] + 1000.0, rtol=1e-12)
        assert onp.allclose((dnp.sum(X) * 2.0 + 1.0).numpy(), 2.0 * (onp.sum(x) - x[0, 0] + 1000.0) + 1.0, rtol=1e-12)
    finally:
        _lib.map_reduce = real


def test_kept_programs_are_found_by_structure_and_bound_to_new_tensors(dnp):
    """A loop evaluates the same expression again and again: its program is emitted once and found again by the
    structure of the expression; what differs between two expressions of one structure (which arrays, which of them
    are one and the same array, scalar values, the sign of a zero) either is bound anew or gives another program."""
    from autograd_amd.numpy import fusion

    rs = onp.random.RandomState(5)
    n = 10007
    fusion._PROGRAMS.clear()

    def f(x, y, c):
        return dnp.tanh(x * y + c) / (dnp.exp(x) + 2.0) - y

    def ref(x, y, c):
        return onp.tanh(x * y + c) / (onp.exp(x) + 2.0) - y

    for k in range(6):
        x, y = rs.randn(n), rs.randn(n)
        got = f(dnp.asarray(x), dnp.asarray(y), 0.5).numpy()
        with unfused():
            want = f(dnp.asarray(x), dnp.asarray(y), 0.5).numpy()
        assert onp.array_equal(got, want) and onp.allclose(got, ref(x, y, 0.5), rtol=1e-10, atol=1e-12)
        assert len(fusion._PROGRAMS) == 1, k
    # the same array in both places is another structure (one leaf, not two), and so is another scalar
    x = rs.randn(n)
    X = dnp.asarray(x)
    assert onp.allclose(f(X, X, 0.5).numpy(), ref(x, x, 0.5), rtol=1e-10, atol=1e-12)
    assert len(fusion._PROGRAMS) == 2
    y = rs.randn(n)
    got = f(X, dnp.asarray(y), -0.25).numpy()
    with unfused():
        assert onp.array_equal(got, f(X, dnp.asarray(y), -0.25).numpy())
    assert len(fusion._PROGRAMS) == 3
    # 0.0 and -0.0 are different immediates: 1 / (x * 0.0) against 1 / (x * -0.0)
    pos = (1.0 / (dnp.abs(X) * 0.0 + 0.0)).numpy()
    neg = (1.0 / (dnp.abs(X) * -0.0 + -0.0)).numpy()
    assert onp.all(pos == onp.inf) and onp.all(neg == -onp.inf)
    # views of one array at different offsets (the Rosenbrock pattern) against two separate arrays of the same sizes
    fusion._PROGRAMS.clear()
    g = lambda a, b: (a * 3.0 + b * b).numpy()  # noqa: E731
    z = rs.randn(n + 1)
    Z = dnp.asarray(z)
    assert onp.array_equal(g(Z[1:], Z[:-1]), z[1:] * 3.0 + z[:-1] * z[:-1])
    u, v = rs.randn(n), rs.randn(n)
    assert onp.array_equal(g(dnp.asarray(u), dnp.asarray(v)), u * 3.0 + v * v)
    assert onp.array_equal(g(Z[1:], Z[:-1]), z[1:] * 3.0 + z[:-1] * z[:-1])
    # with the cache off the same programs come out
    was, fusion.CACHE = fusion.CACHE, False
    try:
        assert onp.array_equal(g(Z[1:], Z[:-1]), z[1:] * 3.0 + z[:-1] * z[:-1])
    finally:
        fusion.CACHE = was


@pytest.mark.parametrize("dtype", [F64, F32])
@pytest.mark.parametrize("shape", [(1,), (3, 7), (1000003,), (1024, 1000), (5, 3, 130), (513, 2)])
def test_program_equals_the_one_rule_kernels(dtype, shape):
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    n = int(onp.prod(shape))
    x = D.from_numpy(onp.linspace(-3, 3, n).astype(dtype).reshape(shape))
    y = D.from_numpy(onp.random.RandomState(1).rand(*shape).astype(dtype) + 0.5)
    nreg = 8 if dtype == F64 else 16
    two, one = nreg - 1, nreg - 2
    # r2 = exp(x * 2) ; r3 = (1 - r2) / y ; r2 = -1 * r3 * x / y**2 (div rule) ; out0 = r3 + r2, out1 = tanh(r3)
    words = [W(Op.MUL, 2, 0, two), W(Op.EXP, 2, 2), W(Op.SUB, 3, one, 2), W(Op.DIV, 3, 3, 1), W(Op.DIV_VJP1, 2, one, 3, 1),
             W(Op.ADD, 2, 3, 2), W(Op.TANH, 3, 3), W(_lib.PROGRAM_STORE, 2, 2, 0), W(_lib.PROGRAM_STORE, 3, 3, 1)]
    out0, out1 = _lib.empty(shape, dtype), _lib.empty(shape, dtype)
    assert _lib.program(_lib.DTYPE_CODE[dtype], shape, (out0, out1), (x._t, y._t), [2.0, 1.0], words, nreg)
    from autograd_amd.numpy import fusion

    with unfused():
        m = lambda op, *xs: D.map_op(op, dtype, *xs)  # noqa: E731
        r2 = m(Op.EXP, m(Op.MUL, x, D.full((), 2.0, dtype)))
        r3 = m(Op.DIV, m(Op.SUB, D.full((), 1.0, dtype), r2), y)
        want0 = m(Op.ADD, r3, m(Op.DIV_VJP1, D.full((), 1.0, dtype), r3, y)).numpy()
        want1 = m(Op.TANH, r3).numpy()
    assert fusion.ENABLED
    assert onp.array_equal(out0.cpu().numpy(), want0) and onp.array_equal(out1.cpu().numpy(), want1)


@pytest.mark.parametrize("dtype", [F64, F32])
def test_program_row_and_column_broadcasts(dtype):
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    for rows, cols in ((512, 1024), (37, 1001), (4, 5), (1, 300), (300, 1)):
        rs = onp.random.RandomState(rows + cols)
        A = D.from_numpy(rs.randn(rows, cols).astype(dtype))
        b = D.from_numpy(rs.randn(cols).astype(dtype))
        c = D.from_numpy(rs.randn(rows, 1).astype(dtype))
        with unfused():
            want = D.map_op(Op.TANH, dtype, D.map_op(Op.ADD, dtype, D.map_op(Op.MUL, dtype, A, b), c)).numpy()
        out = _lib.empty((rows, cols), dtype)
        words = [W(Op.MUL, 0, 0, 1), W(Op.ADD, 0, 0, 2), W(Op.TANH, 0, 0), W(_lib.PROGRAM_STORE, 0, 0, 0)]
        ok = _lib.program(_lib.DTYPE_CODE[dtype], (rows, cols), (out,), (A._t, b._t.expand(rows, cols), c._t.expand(rows, cols)), [],
                          words, 8)
        assert ok and onp.array_equal(out.cpu().numpy(), want)
        # a transposed leaf has no unit stride along the rows: reported, nothing launched
        At = D.from_numpy(rs.randn(cols, rows).astype(dtype))._t.t()
        if rows > 1 and cols > 1:
            assert not _lib.program(_lib.DTYPE_CODE[dtype], (rows, cols), (out,), (At, b._t.expand(rows, cols), c._t.expand(rows, cols)),
                                    [], words, 8)


@pytest.mark.parametrize("dtype", [F64, F32])
@pytest.mark.parametrize("n", [5, 515, 4096, 100003])
def test_program_shifted_leaves_and_masks(dtype, n):
    """out[i] = x[i-1] * x[i+1] inside [1, n-1), and -x[i] outside: leaves read at moved addresses, one select."""
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    xh = onp.random.RandomState(n).randn(n).astype(dtype)
    x = D.from_numpy(xh)
    want = -xh.copy()
    want[1:n - 1] = xh[:n - 2] * xh[2:]
    words = [W(Op.MUL, 3, 0, 1), W(Op.NEG, 4, 2), W(_lib.PROGRAM_MASK, 3, 3, 0, 4), W(_lib.PROGRAM_STORE, 3, 3, 0)]
    out = _lib.empty((n,), dtype)
    t = x._t
    shifted = [(-1, 1, n + 1), (1, -1, n - 1), (0, 0, n)]   # (shift, first readable index, one past the last)
    assert _lib.program(_lib.DTYPE_CODE[dtype], (n,), (out,), (t, t, t), [], words, 8, shifted, [(1, n - 1)])
    assert onp.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("dtype", [F64, F32])
def test_chained_instructions_equal_their_two_rules(dtype, dnp):
    """``(a * b) * c``, ``a * b - c``, ``c - a * b``, ``(a + b) * c``, ``(a - b) * c`` as ONE instruction each give what the
    two one-rule kernels give, and the emitter forms them (and ``a * b + c``) where a product, sum or difference is read
    once, by a sum, difference or product: fewer interpreted instructions, same bits."""
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D
    from autograd_amd.numpy import fusion

    rs = onp.random.RandomState(21)
    n = 70001
    a, b, c = (rs.randn(n).astype(dtype) for _ in range(3))
    A, B, C = (D.from_numpy(v) for v in (a, b, c))
    code = _lib.DTYPE_CODE[dtype]
    two = {Op.MUL_MUL: (Op.MUL, Op.MUL, False), Op.MUL_SUB: (Op.MUL, Op.SUB, False), Op.MUL_RSUB: (Op.MUL, Op.SUB, True),
           Op.ADD_MUL: (Op.ADD, Op.MUL, False), Op.SUB_MUL: (Op.SUB, Op.MUL, False), Op.MUL_ADD: (Op.MUL, Op.ADD, False)}
    for both, (first, second, swapped) in two.items():
        out = _lib.empty((n,), dtype)
        assert _lib.program(code, (n,), (out,), (A._t, B._t, C._t), [], [W(both, 3, 0, 1, 2), W(_lib.PROGRAM_STORE, 3, 3, 0)], 8)
        with unfused():
            t = D.map_op(first, dtype, A, B)
            want = (D.map_op(second, dtype, C, t) if swapped else D.map_op(second, dtype, t, C)).numpy()
        assert onp.array_equal(out.cpu().numpy(), want), both
    # through the emitter: seven rules, four instructions
    X, Y, Z = (dnp.asarray(v) for v in (a, b, c))
    seen = []
    real = _lib.program
    _lib.program = lambda *args, **k: (seen.append([w & 255 for w in args[5]]), real(*args, **k))[1]
    try:
        fusion._PROGRAMS.clear()
        f = lambda: ((X * Y) * Z - (X - Y) * Z + (Z - X * X) * (Y + Z)).numpy()  # noqa: E731
        got = f()
    finally:
        _lib.program = real
    with unfused():
        want = f()
    assert onp.array_equal(got, want)
    assert len(seen) == 1 and len(seen[0]) < 9 and any(op in two for op in seen[0]), seen
    was, fusion.CHAINED = fusion.CHAINED, False
    try:
        fusion._PROGRAMS.clear()
        assert onp.array_equal(f(), want)
    finally:
        fusion.CHAINED = was
        fusion._PROGRAMS.clear()


# ---- recurring programs get a kernel of their own -------------------------------------------------------
class specializing:
    """``with specializing(n): ...``: programs seen ``n`` times are compiled (0: never)."""

    def __init__(self, after):
        self.after = after

    def __enter__(self):
        from autograd_amd import _lib

        self.was = _lib.specialize_after(self.after)

    def __exit__(self, *exc):
        from autograd_amd import _lib

        _lib.specialize_after(self.was)


@pytest.fixture()
def compiler(dnp):
    """Skips when the run-time compiler cannot be used on this machine (the library then keeps every program with the
    interpreter, which the rest of the suite covers): a probe program is handed over under ``specializing(1)`` and must
    come back compiled."""
    from autograd_amd import _lib

    before = _lib.specialized_programs()[1]
    with specializing(1):
        x = dnp.asarray(onp.linspace(0.0, 1.0, 257))
        (x * 1.234567 + dnp.sin(x) * 0.7654321).numpy()
    if _lib.specialized_programs()[1] == before:  # (launches served by compiled kernels: none was added)
        pytest.skip("the run-time compiler did not produce a kernel here: " + _lib.lib().agmi_last_error().decode()[:200])


@pytest.mark.parametrize("dtype", [F64, F32])
def test_a_specialised_kernel_gives_the_interpreters_bits(dtype, dnp, compiler):
    """The same expression by the interpreter, by the kernel compiled for it, and rule by rule: the same bits, on
    flat arrays with ragged ends, on row / column broadcasts, with shifted vectors and masks, and with a row sum
    inside the chain; functions from every family of the functor table."""
    from autograd_amd import _lib
    from autograd_amd.numpy import fusion

    rs = onp.random.RandomState(31)

    def cases():
        n = 100003
        x, y = (rs.randn(n).astype(dtype) for _ in range(2))
        X, Y = dnp.asarray(x), dnp.asarray(y)
        yield lambda: (dnp.tanh(X * Y + 0.5) / (dnp.exp(X) + 2.0) - Y).numpy()
        yield lambda: (dnp.sin(X) * dnp.log1p(dnp.abs(Y)) + dnp.sqrt(dnp.abs(X)) ** 1.5 - dnp.arctan2(X, Y)).numpy()
        yield lambda: (X[1:] * X[:-1] - Y[1:] * 3.0 + (X[1:] - Y[:-1]) * Y[1:]).numpy()
        a, b, c = rs.randn(300, 130).astype(dtype), rs.randn(130).astype(dtype), rs.randn(300, 1).astype(dtype)
        A, B, C = dnp.asarray(a), dnp.asarray(b), dnp.asarray(c)
        yield lambda: (dnp.tanh(A * B + C) * A - dnp.exp(C) * B).numpy()
        yield lambda: ((A * B) - dnp.exp(A - C) * dnp.sum(A * B, axis=1, keepdims=True)).numpy()

    for f in cases():
        before = _lib.specialized_programs()
        with specializing(0):
            fusion._PROGRAMS.clear()
            interpreted = f()
        assert _lib.specialized_programs() == before
        with specializing(1):
            compiled = f()
            again = f()
        after = _lib.specialized_programs()
        assert after[1] >= before[1] + 2, (before, after)      # both evaluations ran on the compiled kernel
        with unfused():
            plain = f()
        assert _same_bits(compiled, interpreted) and _same_bits(again, interpreted) and _same_bits(interpreted, plain)


@pytest.mark.parametrize("dtype", [F64, F32])
def test_a_specialised_kernel_treats_special_values_as_the_interpreter_does(dtype, dnp, compiler):
    """Infinities, NaNs, signed zeros, subnormals and values at the edge of overflow through the long functors and the
    two-rule instructions: interpreted, compiled and rule by rule give the same bits (the compiled kernel is built with
    the library's floating-point flags: no contraction, no flushing of subnormals, no packed float32 forms)."""
    from autograd_amd.numpy import fusion

    tiny = onp.finfo(dtype).tiny
    big = onp.finfo(dtype).max
    special = onp.array([0.0, -0.0, onp.inf, -onp.inf, onp.nan, tiny, -tiny, tiny / 8, -tiny / 16, big, -big, big / 3, 1.0, -1.0,
                         88.7, -87.3, 709.7, -745.1, 1e-30, 3.0e38, 0.5, 2.0], dtype=dtype)
    a = onp.repeat(special, len(special))
    b = onp.tile(special, len(special))
    A, B = dnp.asarray(a), dnp.asarray(b)
    chains = [
        lambda: dnp.exp(A) * B - dnp.tanh(B) / (A + B),
        lambda: dnp.sqrt(dnp.abs(A)) * B + dnp.log(dnp.abs(B) + dnp.abs(A)),
        lambda: (A * B) * A - (A - B) * B + (A + B) * (B - A * A),
        lambda: dnp.maximum(A, B) / dnp.minimum(A, B) + dnp.where(A > B, A, B) * 0.5,
        lambda: dnp.power(dnp.abs(A), 0.3) * dnp.sin(B) + dnp.arctan2(A, B) - dnp.log1p(dnp.abs(B)) * dnp.expm1(A * 1e-3),
    ]
    for k, f in enumerate(chains):
        with onp.errstate(all="ignore"):
            with specializing(0):
                fusion._PROGRAMS.clear()
                interpreted = f().numpy()
            with specializing(1):
                compiled = f().numpy()
            with unfused():
                plain = f().numpy()
        assert _same_bits(compiled, interpreted), k
        assert _same_bits(interpreted, plain), k


def test_programs_are_specialised_after_a_few_sightings_and_never_while_a_graph_records(dnp, compiler):
    import autograd_amd as ag
    from autograd_amd import _lib, graphs

    rs = onp.random.RandomState(8)
    n = 50021
    X = dnp.asarray(rs.randn(n))
    f = lambda x: dnp.exp(x * 0.37) * x - dnp.cos(x) / (x * x + 1.25)  # noqa: E731  (an expression no other test uses)
    with specializing(3):
        c0, l0 = _lib.specialized_programs()
        first = f(X).numpy()
        second = f(X).numpy()
        assert _lib.specialized_programs() == (c0, l0)                  # two sightings: the interpreter
        third = f(X).numpy()
        assert _lib.specialized_programs() == (c0 + 1, l0 + 1)          # compiled and used
        assert onp.array_equal(first, second) and onp.array_equal(first, third)
        # a function about to be recorded compiles its programs during the eager warm-up run, and replays them
        g = lambda x: dnp.sinh(x * 0.21) - x / (dnp.exp(x) + 3.5)  # noqa: E731
        eager = g(X).numpy()
        c1, l1 = _lib.specialized_programs()
        replayed = graphs.capture(g, X)
        c2, l2 = _lib.specialized_programs()
        assert c2 == c1 + 1 and l2 >= l1 + 2                             # warm-up and recording both ran it
        for _ in range(3):
            Z = dnp.asarray(rs.randn(n))
            assert onp.array_equal(replayed(Z).numpy(), g(Z).numpy())
        assert onp.array_equal(replayed(X).numpy(), eager)
        assert _lib.specialize_after(-1) == 3                            # the recording put the setting back


ROW_SUM_SHAPES = [(256, 128), (64, 512), (70, 256), (1000, 65), (100, 64), (1, 40), (7, 5), (3, 2), (300, 257)]


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("shape", ROW_SUM_SHAPES)
def test_row_sums_read_back_by_the_chain_are_formed_inside_it(dtype, shape, dnp):
    """``g - exp(x - lse) * sum(g, axis=1, keepdims=True)`` (the cotangent of a log-softmax, reference
    examples/rnn.py:50-52 under autograd/numpy/numpy_vjps.py:76-93 and autograd/scipy/special.py:127-144): the row sums
    of the pending ``g`` are formed by the program that reads them back, in the order the reduction kernel adds a row
    of that length, so the chain is one launch and gives the separate launches' bits.  Shapes the reduction kernel
    treats otherwise (rows longer than a wave's tile; long rows with few of them) keep the separate reduction."""
    from autograd_amd import _lib
    from autograd_amd._lib import Op, Red
    from autograd_amd.numpy import devarray as D
    from autograd_amd.numpy import fusion

    rows, cols = shape
    if dtype == F64 and cols > 256:
        pytest.skip("wider than a float64 tile: covered by the float32 case of the same width")
    rs = onp.random.RandomState(rows * 1000 + cols)
    a, t = rs.randn(*shape).astype(dtype), rs.rand(*shape).astype(dtype)
    x = (rs.randn(*shape) * 3).astype(dtype)
    lse = onp.log(onp.sum(onp.exp(x.astype(F64)), axis=1, keepdims=True)).astype(dtype)
    A, T, X, L = (dnp.asarray(v) for v in (a, t, x, lse))
    reduced = []
    real = _lib.map_reduce
    _lib.map_reduce = lambda *args, **k: (reduced.append(args[0]), real(*args, **k))[1]

    def chain(negated):
        g = A * T
        if negated:  # the unbroadcast of a subtraction's second cotangent negates inside the reduction
            s = D.map_reduce(Op.NEG, Red.SUM, dtype, (g,), (1,), True)
            return (g + dnp.exp(X - L) * s).numpy()
        s = dnp.sum(g, axis=1, keepdims=True)
        return (g - dnp.exp(X - L) * s).numpy()

    try:
        for negated in (False, True):
            del reduced[:]
            before = dict(fusion.COUNTS)
            got = chain(negated)
            inside = cols <= fusion.ROWSUM_WIDEST[dtype] and cols >= 2 and (cols <= 64 or rows >= 64)
            assert len(reduced) == (0 if inside else 1), (reduced, inside)
            assert fusion.COUNTS["programs"] - before["programs"] == 1 and fusion.COUNTS["unfused"] == before["unfused"]
            with unfused():
                want = chain(negated)
            assert _same_bits(got, want)
            g64 = a.astype(F64) * t
            ref = g64 - onp.exp(x.astype(F64) - lse) * g64.sum(axis=1, keepdims=True)
            assert onp.allclose(got, ref, rtol=1e-4 if dtype == F32 else 1e-11, atol=(1e-4 if dtype == F32 else 1e-11) * cols)
    finally:
        _lib.map_reduce = real


def test_row_sums_of_special_values_and_of_an_array_in_memory(dnp):
    """The in-chain row sum follows the reduction kernel on rows with infinities and NaNs, sums an operand that already
    lies in memory just the same, and still gives the reduction's own result when that is read as well."""
    rs = onp.random.RandomState(12)
    g = rs.randn(128, 96)
    g[3, 5], g[7, 0], g[9, 95] = onp.inf, onp.nan, -onp.inf
    g[11, 2], g[11, 3] = onp.inf, -onp.inf
    G, Y = dnp.asarray(g), dnp.asarray(rs.randn(128, 96))

    def both():
        s = dnp.sum(G, axis=1, keepdims=True)
        return (Y * s + G).numpy(), s.numpy()

    got, sums = both()
    with unfused():
        want, want_sums = both()
    assert _same_bits(got, want) and _same_bits(sums, want_sums)
    with onp.errstate(invalid="ignore"):
        assert onp.allclose(sums, g.sum(axis=1, keepdims=True), equal_nan=True)


def test_log_softmax_gradient_is_the_same_with_row_sums_inside_the_chain(dnp):
    """The whole pattern through the tracer: gradient of ``-sum(log_softmax(x) * t)`` (reference examples/rnn.py:50-61,
    examples/neural_net.py:24-28), fused against unfused bit for bit and against the closed form."""
    import autograd_amd as ag
    from autograd_amd.scipy.special import logsumexp

    rs = onp.random.RandomState(3)
    for dtype, shape in ((F32, (256, 128)), (F64, (100, 10)), (F32, (64, 300))):
        x = rs.randn(*shape).astype(dtype)
        t = onp.eye(shape[1], dtype=dtype)[rs.randint(0, shape[1], shape[0])]
        X, T = dnp.asarray(x), dnp.asarray(t)

        def loss(z):
            return -dnp.sum((z - logsumexp(z, axis=1, keepdims=True)) * T)

        fused, plain, ran = _both_ways(lambda: ag.grad(loss)(X).numpy())
        assert _same_bits(fused, plain) and ran["unfused"] == 0
        x64 = x.astype(F64)
        soft = onp.exp(x64 - x64.max(axis=1, keepdims=True))
        soft /= soft.sum(axis=1, keepdims=True)
        assert onp.allclose(fused, soft - t, rtol=0, atol=2e-6 if dtype == F32 else 1e-14)


@pytest.mark.parametrize("dtype", [F32, F64])
@pytest.mark.parametrize("shape", ROW_SUM_SHAPES)
def test_the_logsumexp_of_short_rows_is_formed_by_the_chain_that_reads_it(dtype, shape, dnp):
    """``x - logsumexp(x, axis=1, keepdims=True)`` (reference examples/rnn.py:50-52, examples/neural_net.py:24-28 over
    autograd/scipy/special.py:119-147): for rows that fit a wave's tile nothing runs when the logsumexp is taken; the
    log-softmax is one program that forms it (in the reduction kernel's order: the same bits as the separate
    reduction, infinities, NaNs and all -inf rows included), and a reader of the value itself gets the reduction's."""
    from autograd_amd import _lib
    from autograd_amd.numpy import fusion
    from autograd_amd.scipy.special import logsumexp

    rows, cols = shape
    if dtype == F64 and cols > 256:
        pytest.skip("wider than a float64 tile: covered by the float32 case of the same width")
    rs = onp.random.RandomState(rows + 7 * cols)
    x = (rs.randn(*shape) * 4).astype(dtype)
    x[0, 0] = onp.inf
    if rows > 2:
        x[1, :] = -onp.inf
        x[2, cols - 1] = onp.nan
    if rows > 4:
        x[3, 0], x[3, 1] = 700.0, -700.0
        x[4, :] = 3.25
    X = dnp.asarray(x)
    reduced = []
    real = _lib.map_reduce
    _lib.map_reduce = lambda *args, **k: (reduced.append(args[1]), real(*args, **k))[1]
    try:
        inside = fusion.rows_fit_a_wave(shape, dtype)
        lse = logsumexp(X, axis=1, keepdims=True)
        assert (reduced == []) == inside
        got = (X - lse).numpy()
        assert (reduced == []) == inside            # the chain formed it: still no reduction launched
        value = lse.numpy()                         # a reader of the value itself
        assert len(reduced) == 1
    finally:
        _lib.map_reduce = real
    with unfused():
        want_value = logsumexp(X, axis=1, keepdims=True).numpy()
        want = (X - logsumexp(X, axis=1, keepdims=True)).numpy()
    assert _same_bits(value, want_value) and _same_bits(got, want)
    from scipy.special import logsumexp as host_lse

    with onp.errstate(all="ignore"):
        ref = host_lse(x.astype(F64), axis=1, keepdims=True)
    ok = onp.isfinite(ref[:, 0])
    assert onp.allclose(value[ok], ref[ok], rtol=2e-6 if dtype == F32 else 1e-13)
    assert onp.array_equal(onp.isnan(value), onp.isnan(ref)) and onp.array_equal(onp.isinf(value), onp.isinf(ref))


def test_a_row_sum_outside_the_kernels_shapes_is_refused_at_the_library():
    from autograd_amd import _lib
    from autograd_amd._lib import Op
    from autograd_amd.numpy import devarray as D

    code = _lib.DTYPE_CODE[F32]
    words = [W(_lib.PROGRAM_ROWSUM, 1, 0), W(Op.ADD, 2, 0, 1), W(_lib.PROGRAM_STORE, 2, 2, 0)]
    for shape, fits in (((64, 512), True), ((64, 513), False), ((8, 100), False), ((8, 64), True)):
        x = D.from_numpy(onp.ones(shape, F32))
        out = _lib.empty(shape, F32)
        assert _lib.program(code, shape, (out,), (x._t,), [], words, 16) == fits
        if fits:
            assert onp.array_equal(out.cpu().numpy(), onp.full(shape, shape[1] + 1.0, F32))
    x = D.from_numpy(onp.ones((64, 64), F32))
    out = _lib.empty((64, 64), F32)
    assert not _lib.program(code, (64, 64), (out,), (x._t,), [], words, 8)  # the row-sum variant has 16 registers


def test_program_arguments_are_checked():
    from autograd_amd import _lib
    from autograd_amd._lib import AgmiError, Op
    from autograd_amd.numpy import devarray as D

    x = D.from_numpy(onp.ones(64))
    out = _lib.empty((64,), F64)
    code = _lib.DTYPE_CODE[F64]
    store = W(_lib.PROGRAM_STORE, 1, 1, 0)
    with pytest.raises(AgmiError, match="holds nothing"):      # reads a register nothing wrote
        _lib.program(code, (64,), (out,), (x._t,), [], [W(Op.ADD, 1, 0, 5), store], 8)
    with pytest.raises(AgmiError, match="unknown op"):
        _lib.program(code, (64,), (out,), (x._t,), [], [W(200, 1, 0, 0), store], 8)
    with pytest.raises(AgmiError, match="not every output"):
        _lib.program(code, (64,), (out,), (x._t,), [], [W(Op.NEG, 1, 0)], 8)
    with pytest.raises(AgmiError, match="range"):              # a mask that was not passed
        _lib.program(code, (64,), (out,), (x._t,), [], [W(_lib.PROGRAM_MASK, 1, 0, 2, 0), store], 8)
    with pytest.raises(AgmiError, match="registers"):          # more leaves and immediates than registers
        _lib.program(code, (64,), (out,), (x._t,) * 5, [1.0] * 4, [W(Op.NEG, 1, 0), store], 8)
    # what the checks let through runs
    assert _lib.program(code, (64,), (out,), (x._t,), [], [W(Op.NEG, 1, 0), store], 8)
    assert onp.array_equal(out.cpu().numpy(), -onp.ones(64))
