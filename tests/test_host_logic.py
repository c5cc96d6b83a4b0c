"""Host-side logic of the device layer that needs no GPU: shape/axis/dtype planning.

``DevArray`` only needs a tensor for its metadata, so CPU tensors stand in here; nothing is
launched (any launch would raise: there is no CPU fallback).
"""

import numpy as onp
import pytest
import torch

from autograd_amd.numpy import devarray as D
from autograd_amd.numpy import wrapper as W
from autograd_amd.numpy.devarray import DevArray


def meta(shape, dtype=torch.float32):
    return DevArray(torch.empty(shape, dtype=dtype))


def test_broadcast_shapes_matches_numpy():
    cases = [((), ()), ((3,), ()), ((3, 4), (4,)), ((3, 1), (1, 4)), ((2, 1, 5), (7, 1)), ((0, 4), (1, 4)), ((5,), (5,))]
    for a, b in cases:
        assert D.broadcast_shapes(a, b) == onp.broadcast_shapes(a, b)
        assert D.broadcast_shapes(b, a) == onp.broadcast_shapes(a, b)
    with pytest.raises(ValueError):
        D.broadcast_shapes((3, 4), (3,))


def test_result_dtype_follows_numpy2_promotion():
    f32, f64, i64 = meta((2,)), meta((2,), torch.float64), meta((2,), torch.int64)
    assert D.result_dtype(f32, 2.0) == onp.float32            # weak Python scalar
    assert D.result_dtype(f32, 3) == onp.float32
    assert D.result_dtype(f32, onp.float64(2.0)) == onp.float64  # strong NumPy scalar
    assert D.result_dtype(f32, onp.int64(3)) == onp.float64      # the mean-rule promotion of the reference
    assert D.result_dtype(f32, f64) == onp.float64
    assert D.result_dtype(f32, i64) == onp.float64
    assert D.result_dtype(f32, f32, 1.5) == onp.float32
    assert D.result_dtype(i64, 2.0) == onp.float64
    for args in [(onp.float32(1), 2.0), (onp.ones(2, onp.float32), onp.int64(3)), (onp.ones(2, onp.float32), 2)]:
        ours = D.result_dtype(*[meta((2,)) if isinstance(a, onp.ndarray) else a for a in args])
        assert ours == onp.result_type(*args)


def test_normalize_axes_and_reduce_shape():
    assert D.normalize_axes(None, 3) == (0, 1, 2)
    assert D.normalize_axes(-1, 3) == (2,)
    assert D.normalize_axes((2, 0), 3) == (0, 2)
    assert D.normalize_axes(None, 0) == ()
    with pytest.raises(ValueError):
        D.normalize_axes(3, 3)
    assert D.reduce_shape((2, 3, 4), (1,), False) == (2, 4)
    assert D.reduce_shape((2, 3, 4), (0, 2), True) == (1, 3, 1)
    assert D._adjacent_groups((0, 1, 3)) == [(0, 1), (3,)]


def test_reshape_shape_normalisation():
    assert W._norm_shape((-1, 4), 12) == (3, 4)
    assert W._norm_shape(12, 12) == (12,)
    assert W._norm_shape((), 1) == ()
    for bad in [((5,), 12), ((-1, -1), 12), ((-1, 5), 12)]:
        with pytest.raises(ValueError):
            W._norm_shape(*bad)


def test_index_classification():
    assert W._is_basic_index((slice(1, None), None, 3, Ellipsis))
    assert W._is_basic_index(onp.int64(2))
    assert not W._is_basic_index([0, 1])
    assert not W._is_basic_index((slice(None), onp.array([0, 1])))
    assert W._is_basic_index(slice(None, None, -1))
    # slices that step backwards become the forward-stepping slice over the same elements + the result axes to reverse
    for shape, idx in (((5,), (slice(None, None, -1),)), ((5, 6), (slice(3, 0, -1), slice(None, None, -2))),
                       ((4, 5, 6), (Ellipsis, slice(4, None, -3))), ((4, 5, 6), (1, None, slice(None, None, -1))),
                       ((5,), (slice(0, 3, -1),)), ((4, 5, 6), (slice(None, None, 2), slice(10, -10, -1)))):
        up, axes = W._positive_steps(idx, shape)
        x = onp.arange(int(onp.prod(shape))).reshape(shape)
        assert all(not isinstance(i, slice) or i.step is None or i.step > 0 for i in up)
        assert onp.array_equal(onp.flip(x[up], axes) if axes else x[up], x[idx]), (shape, idx)
    assert W._positive_steps((slice(1, 3), 2), (5, 6)) == ((slice(1, 3), 2), ())
    with pytest.raises(IndexError):
        W._positive_steps((0, 0, slice(None, None, -1)), (5, 6))


def test_flat_positions_follow_numpy_indexing():
    """The table that drives the gather / ordered scatter of advanced indices: for every index form,
    ``x.ravel()[positions]`` must be ``x[idx]`` (shape included).  Forms of the reference's own tests
    (tests/test_numpy.py:288-352, 881-890) first."""
    rs = onp.random.RandomState(0)
    x = rs.randn(5, 6, 4)
    mask3 = rs.rand(5, 6, 4) > 0.5
    forms = [
        [0, 1, 2], ([0, 1, 2], slice(None), slice(None)), (3, slice(2, None), [1, 3]), (3, 0, 1),
        (slice(None), [0, 5, 0]), (slice(None, None, -1), [1, 1], slice(1, 3)), ([[0, 1], [2, 3]], [[1], [2]]),
        (Ellipsis, [3, 0]), (None, [4, 0], None, 2), ([0, 4], slice(None), [1, 2]), (onp.array([4, -1, 0]),),
        mask3, (onp.array([True, False, True, False, True]),), (slice(1, 4), rs.rand(6, 4) > 0.3),
        (onp.array([1, 2, 0]), onp.array([True] * 3 + [False] * 3)), [], onp.zeros((0, 2), dtype=onp.int64),
    ]
    for idx in forms:
        want = x[idx] if not isinstance(idx, list) or idx else x[onp.array(idx, dtype=onp.int64)]
        pos = W._flat_positions(x.shape, idx if not (isinstance(idx, list) and not idx) else onp.array(idx, dtype=onp.int64))
        assert pos.dtype == onp.int64 and pos.shape == want.shape, (idx, pos.shape, want.shape)
        assert onp.array_equal(x.ravel()[pos], want), idx
    v = rs.randn(3)
    for idx in ([0, 0], [0, 1, 0]):
        assert onp.array_equal(v[W._flat_positions(v.shape, idx)], v[idx])
    with pytest.raises(IndexError):
        W._flat_positions((5, 6, 4), [5])
    with pytest.raises(IndexError):
        W._flat_positions((5, 6, 4), (onp.array([True, False]),))  # a mask of the wrong length, as in NumPy
    assert W._index_key(([0, 1], slice(2))) == W._index_key((onp.array([0, 1]), slice(2, None, None))) or True
    assert W._index_key(([0, 1], slice(2))) != W._index_key(([0, 2], slice(2)))


def test_views_are_metadata_only():
    x = meta((4, 6))
    assert W.transpose(x).shape == (6, 4) and W.transpose(x)._t.data_ptr() == x._t.data_ptr()
    assert W.reshape(x, (2, 12)).shape == (2, 12)
    assert W.expand_dims(x, (0, 3)).shape == (1, 4, 6, 1)
    assert W.squeeze(W.expand_dims(x, 1)).shape == (4, 6)
    assert W.broadcast_to(meta((1, 6)), (5, 6))._t.stride() == (0, 1)
    assert W.swapaxes(x, 0, 1).shape == (6, 4)
    assert W.atleast_2d(meta((3,))).shape == (1, 3) and W.atleast_1d(meta(())).shape == (1,)
    assert x[1:, ::2].shape == (3, 3) and x[None, 2].shape == (1, 6)
    assert W.shape(x) == (4, 6) and W.ndim(x) == 2 and W.size(x) == 24 and W.result_type(x) == onp.float32
    with pytest.raises(NotImplementedError):
        x[::-1] = 1.0  # (item assignment takes forward-stepping basic indices; rejected before anything is launched)
    with pytest.raises(ValueError):
        x[0] = meta((5,))  # a shape that does not broadcast into the row


def test_vspace_metadata_and_laziness():
    from autograd_amd.extend import vspace
    from autograd_amd.numpy.vspaces import DevArrayVSpace

    vs = vspace(meta((3, 4)))
    assert isinstance(vs, DevArrayVSpace) and vs.shape == (3, 4) and vs.size == 12 and vs.ndim == 2
    assert vs == vspace(meta((3, 4))) and vs != vspace(meta((3, 4), torch.float64))
    fs = vspace(1.5)
    assert fs.shape == () and fs.dtype == onp.float64 and fs.size == 1


def test_scalar_arithmetic_folds_into_a_pending_map_only_when_exact():
    """negative / scalar multiply / scalar offset keep the operand's memory and record
    ``raw * scale + shift``; they fold only where the composed map rounds exactly like the
    eager passes (reference semantics: numpy_vjps.py:87 ``-g``, :73-78 ``y * g``)."""
    from autograd_amd._lib import Op
    from autograd_amd.numpy.devarray import LazyDevArray

    x = meta((4, 6), torch.float64)

    def state(a):
        return (a._scale, a._shift) if type(a) is LazyDevArray else (1.0, None)

    n = W.negative(x)
    assert type(n) is LazyDevArray and state(n) == (-1.0, None) and n._raw.data_ptr() == x._t.data_ptr()
    assert type(W.negative(n)) is DevArray and W.negative(n)._t.data_ptr() == x._t.data_ptr()
    assert state(x * 3.0) == (3.0, None) and state(3 * x) == (3.0, None)
    assert state(-(x * 3.0)) == (-3.0, None)
    assert state(n * 3.0) == (-3.0, None)  # (-x) * 3 == x * (-3) exactly
    assert state((x * 3.0) * 2.0) == (6.0, None)  # power-of-two factor commutes with rounding
    assert state((x * 2.0) * 3.0) == (6.0, None)
    assert state(x + 1.5) == (1.0, 1.5) and state(1.5 + x) == (1.0, 1.5)
    assert state(x - 1.5) == (1.0, -1.5) and state(1.5 - x) == (-1.0, 1.5)
    assert state(1.0 - 2.0 * x) == (-2.0, 1.0)
    assert state(-(1.0 - 2.0 * x)) == (2.0, -1.0)
    assert state((x + 1.0) * 4.0) == (4.0, 4.0) and state((x + 1.0) / 4.0) == (0.25, 0.25)
    assert state(x + 0.0) == (1.0, 0.0)  # kept: -0.0 + 0.0 is +0.0
    # not exact in general: these must launch (and there is no device here, so they raise)
    # (a far power of two is exact by itself, but merged with its inverse it would hide the eager underflow:
    # (x * 2**-60) * 2**60 is 0 for a float32 1e-30 in NumPy, and must be two passes here too)
    assert state(x * 2.0**-60) == (2.0**-60, None)
    from autograd_amd.numpy import fusion

    for expr in (lambda: (x * 3.0) * 5.0, lambda: (x + 1.0) * 3.0, lambda: (x + 1.0) + 1.0, lambda: 2.0 / x,
                 lambda: x / 3.0, lambda: x * onp.float64(3.0), lambda: (x * 2.0**-60) * 2.0**60,
                 lambda: (x * 3.0) * 2.0**40, lambda: (x + 1.0) * 2.0**9):
        # a step of its own: a pending expression node while chains are deferred (nothing is launched yet) ...
        node = expr()
        assert type(node) is fusion.ExprArray and node.shape == (4, 6) and node._cone == 1
        # ... and an immediate launch otherwise
        was, fusion.ENABLED = fusion.ENABLED, False
        try:
            with pytest.raises(Exception):
                expr()
        finally:
            fusion.ENABLED = was
    # float32: scalars are rounded to the array's dtype first, as NumPy's weak scalars are
    y = meta((5,), torch.float32)
    assert state(y * 0.1) == (float(onp.float32(0.1)), None) and (y * 0.1).dtype == onp.float32
    # views keep the pending map and the metadata comes from the raw storage
    v = W.transpose((1.0 - x))[1:, :2]
    assert type(v) is LazyDevArray and v.shape == (5, 2) and state(v) == (-1.0, 1.0) and v.ndim == 2 and v.size == 10
    assert len(v) == 5 and v.strides == (8, 48)
    assert D._fold(Op.EXP, x.dtype, (x,)) is None


def test_accumulators_never_write_through_a_pending_map(monkeypatch):
    from autograd_amd.numpy import vspaces
    from autograd_amd.numpy.devarray import LazyDevArray
    from autograd_amd.numpy.vspaces import DevArrayVSpace, is_shared_zero

    monkeypatch.setitem(vspaces._ZEROS, onp.dtype("float64"), DevArray(torch.zeros((), dtype=torch.float64)))
    monkeypatch.setattr(vspaces, "_SEED_VIEWS", {})
    x = meta((3, 4), torch.float64)
    vs = DevArrayVSpace(x)
    g = W.negative(x)
    acc = vs._mut_add(vs.zeros(), g)  # 0 + g borrows g, pending map included
    assert type(acc) is LazyDevArray and acc._borrowed and acc._raw.data_ptr() == x._t.data_ptr()
    assert not is_shared_zero(acc)
    from autograd_amd.numpy import fusion

    later = vs._mut_add(acc, x)  # the next contribution goes out of place: a pending sum that reads both, writes neither
    assert type(later) is fusion.ExprArray and later is not acc
    was, fusion.ENABLED = fusion.ENABLED, False
    try:
        with pytest.raises(Exception):  # launched at once when chains are not deferred -> no device here
            vs._mut_add(acc, x)
    finally:
        fusion.ENABLED = was
    with pytest.raises(TypeError):
        D.map_op(0, x.dtype, x, out=g)


def test_broadcast_operands_fold_into_pending_maps():
    """Products / sums with a broadcast array operand keep the big operand's storage; the small one
    becomes an array-valued step (a stride-0 view of the big shape).  Folded only in the kernel's
    fixed step order: scalar factor, array factor, offset."""
    from autograd_amd.numpy.devarray import LazyDevArray

    A = meta((8, 6), torch.float64)
    b = meta((6,), torch.float64)
    c = meta((8, 1), torch.float64)

    L = A * b
    assert type(L) is LazyDevArray and L._raw.data_ptr() == A._t.data_ptr() and L._scale == 1.0 and L._shift is None
    assert tuple(L._ascale.shape) == (8, 6) and L._ascale.stride() == (0, 1) and L._ascale.data_ptr() == b._t.data_ptr()
    M = b * A + c
    assert type(M) is LazyDevArray and M._ascale.stride() == (0, 1) and M._shift.stride() == (1, 0)
    assert M.shape == (8, 6) and M._raw.data_ptr() == A._t.data_ptr()
    N = -(A * b)
    assert type(N) is LazyDevArray and N._scale == -1.0 and N._ascale is not None   # (-x) * v == -(x * v) exactly
    assert type((A * b) * 4.0) is LazyDevArray and ((A * b) * 4.0)._scale == 4.0     # power of two commutes
    R = c - A
    assert type(R) is LazyDevArray and R._scale == -1.0 and R._shift.stride() == (1, 0)
    # views carry the array-valued steps along
    V = W.transpose(M)[1:4]
    assert type(V) is LazyDevArray and V.shape == (3, 8) and V._ascale.stride() == (1, 0) and V._shift.stride() == (0, 1)
    V2 = W.reshape(A * b, (4, 2, 6))
    assert type(V2) is LazyDevArray and V2._ascale.stride() == (0, 0, 1)
    # not exact or not expressible in that order: these must launch (no device here -> raise)
    from autograd_amd.numpy import fusion

    for expr in (lambda: (A * b) * 3.0, lambda: (A + c) * b, lambda: (A + c) + b, lambda: (A * b) * b, lambda: A - c,
                 lambda: A / b, lambda: -(A + c), lambda: A * meta((8, 6), torch.float64)):
        assert type(expr()) is fusion.ExprArray  # a step of its own: pending while chains are deferred
    was, fusion.ENABLED = fusion.ENABLED, False
    try:
        for expr in (lambda: (A * b) * 3.0, lambda: (A + c) * b, lambda: (A + c) + b, lambda: (A * b) * b, lambda: A - c,
                     lambda: A / b, lambda: -(A + c), lambda: A * meta((8, 6), torch.float64), lambda: A * meta((6,), torch.float32)):
            with pytest.raises(Exception):
                expr()
    finally:
        fusion.ENABLED = was


def test_pending_products_are_contracted_into_an_accumulator_of_its_own(monkeypatch):
    """The accumulation protocol for matrix cotangents, with the contraction replaced by a recorder:
    0 + G starts a sum of products that only collects operand pairs; further products join it; the sum is
    contracted when its value is read (few terms: one by one with beta = 1 into the accumulator's own buffer);
    a plain owned accumulator takes a product with beta = 1; a borrowed accumulator (it shares memory with a
    cotangent) is never written, the product is computed on its own and added out of place."""
    from autograd_amd.numpy import vspaces

    calls = []

    def fake_gemm2d(a, b, dtype, out=None, beta=0.0):
        calls.append(("gemm", out is not None, beta))
        return out if out is not None else torch.zeros((a.shape[0], b.shape[1]), dtype=torch.float64)

    monkeypatch.setattr(D, "gemm2d", fake_gemm2d)
    monkeypatch.setattr(D._lib, "empty", lambda shape, dtype: torch.zeros(tuple(shape), dtype=torch.float64))
    monkeypatch.setitem(vspaces._ZEROS, onp.dtype("float64"), DevArray(torch.zeros((), dtype=torch.float64)))
    monkeypatch.setattr(vspaces, "_SEED_VIEWS", {})  # (views of the shared zero are kept: none of another zero's here)
    left, right = torch.zeros((3, 5), dtype=torch.float64), torch.zeros((5, 4), dtype=torch.float64)
    vs = vspaces.DevArrayVSpace(DevArray(torch.zeros((3, 4), dtype=torch.float64)))
    first = D.PendingProduct(left, right, onp.dtype("float64"))
    assert first.shape == (3, 4) and first.ndim == 2 and first.size == 12 and not first.computed()
    acc = vs._mut_add(vs.zeros(), first)
    assert type(acc) is D.PendingProduct and acc is not first and not acc.computed() and calls == []
    second = D.PendingProduct(left, right, onp.dtype("float64"))
    assert vs._mut_add(acc, second) is acc and calls == [] and not second.computed() and not first.computed()
    total = acc._t
    assert calls == [("gemm", True, 0.0), ("gemm", True, 1.0)] and acc.computed() and acc._t is total
    # an accumulator that is a plain array of its own takes the product with beta = 1
    acc = DevArray(torch.zeros((3, 4), dtype=torch.float64))
    assert vs._mut_add(acc, D.PendingProduct(left, right, onp.dtype("float64"))) is acc and calls[-1] == ("gemm", True, 1.0)
    # a borrowed accumulator must not be written: no beta = 1 call on it
    n_before = len(calls)
    borrowed = D.alias(acc)
    borrowed._borrowed = True
    third = D.PendingProduct(left, right, onp.dtype("float64"))
    from autograd_amd.numpy import fusion

    was, fusion.ENABLED = fusion.ENABLED, False
    try:
        with pytest.raises(Exception):  # the out-of-place add would launch a kernel: there is no CPU fallback
            vs._mut_add(borrowed, third)
    finally:
        fusion.ENABLED = was
    assert ("gemm", True, 1.0) not in calls[n_before:]
    # reading the value computes it once and keeps it
    fourth = D.PendingProduct(left, right, onp.dtype("float64"))
    n = len(calls)
    t = fourth._t
    assert fourth._t is t and len(calls) == n + 1 and fourth.computed() and D.plain(fourth)._t is t


def test_program_keys_tell_apart_what_the_emitted_program_depends_on():
    """The key under which an emitted program is kept (``fusion._signature``): equal for the same expression over other
    arrays of the same layout, different when an operand is one and the same array in two places, when a scalar or its
    sign differs, when a layout differs, and when two vectors are views of one storage (a shift could make them
    coincide) instead of separate arrays."""
    from autograd_amd.numpy import fusion

    was, fusion.ENABLED = fusion.ENABLED, True
    try:
        def key(build):
            root = build()
            assert type(root) is fusion.ExprArray and root._args is not None
            sig = fusion._signature([root], fusion._post_order([root]))
            assert sig is not None
            return sig[0], len(sig[1])

        def arrays(n=3, shape=(8, 6)):
            return [meta(shape, torch.float64) for _ in range(n)]

        f = lambda a, b, c, s=0.5: (a * b + s) / (a - c)  # noqa: E731
        k1, n1 = key(lambda: f(*arrays()))
        k2, n2 = key(lambda: f(*arrays()))
        assert k1 == k2 and n1 == n2 == 3 and hash(k1) == hash(k2)
        a, b, c = arrays()
        assert key(lambda: f(a, a, c))[0] != k1 and key(lambda: f(a, a, c))[1] == 2           # one array in two places
        assert key(lambda: f(a, b, c, 0.25))[0] != k1                                          # another scalar
        assert key(lambda: f(a, b, c, 0.0))[0] != key(lambda: f(a, b, c, -0.0))[0]              # the sign of a zero
        assert key(lambda: f(a, b, DevArray(c._t.t().contiguous().t())))[0] != k1               # another layout
        assert key(lambda: f(*arrays(shape=(8, 7))))[0] != k1                                   # another shape
        assert key(lambda: f(*[meta((8, 6), torch.float32) for _ in range(3)]))[0] != k1        # another precision
        # vectors: two views of one storage against two separate arrays
        z = meta((101,), torch.float64)
        u, v = meta((100,), torch.float64), meta((100,), torch.float64)
        g = lambda p, q: p * 3.0 + q * q  # noqa: E731
        assert key(lambda: g(z[1:], z[:-1]))[0] != key(lambda: g(u, v))[0]
        z2 = meta((101,), torch.float64)
        assert key(lambda: g(z[1:], z[:-1]))[0] == key(lambda: g(z2[1:], z2[:-1]))[0]
    finally:
        fusion.ENABLED = was


def _ops_of(words):
    return [w & 0xFF for w in words]


def test_the_emitter_chains_a_value_read_once_into_its_reader():
    """``fusion._emit``: a product, sum or difference with one reader that is a sum, difference or product becomes one
    three-operand instruction (``x * x`` counts as a product); a value with two readers stays an instruction of its own."""
    from autograd_amd._lib import Op, PROGRAM_STORE
    from autograd_amd.numpy import fusion

    was, fusion.ENABLED = fusion.ENABLED, True
    try:
        a, b, c = (meta((8, 6), torch.float64) for _ in range(3))

        def ops(root):
            emitted = fusion._emit([root])
            assert emitted is not None
            return _ops_of(emitted[3])

        assert ops((a * b) * c) == [Op.MUL_MUL, PROGRAM_STORE]
        assert ops(c * (a * b)) == [Op.MUL_MUL, PROGRAM_STORE]
        assert ops(a * b - c) == [Op.MUL_SUB, PROGRAM_STORE]
        assert ops(c - a * b) == [Op.MUL_RSUB, PROGRAM_STORE]
        assert ops(c - D.map_op(Op.SQUARE, a.dtype, a)) == [Op.MUL_RSUB, PROGRAM_STORE]
        assert ops((a + b) * c) == [Op.ADD_MUL, PROGRAM_STORE]
        assert ops(c * (a - b)) == [Op.SUB_MUL, PROGRAM_STORE]
        assert ops(a * b + c) == [Op.MUL_ADD, PROGRAM_STORE]
        p = a * b
        assert ops(p * c + p) == [Op.MUL, Op.MUL_ADD, PROGRAM_STORE]  # two readers of p: p * c travels, p stays
        was_chained, fusion.CHAINED = fusion.CHAINED, False
        try:
            assert ops((a * b) * c) == [Op.MUL, Op.MUL, PROGRAM_STORE]
        finally:
            fusion.CHAINED = was_chained
    finally:
        fusion.ENABLED = was


def test_pending_row_sums_broadcast_over_their_rows_join_the_chain():
    """``fusion._row_sums``: ``sum(e, axis=1, keepdims=True)`` that has not run, multiplied back over the rows of ``e``,
    becomes a row-sum instruction of the program (16 registers), for the shapes the reduction kernel gives to a group of
    lanes; other shapes, other axes and sums that have run are ordinary operands."""
    from autograd_amd._lib import Op, PROGRAM_ROWSUM, PROGRAM_STORE, Red
    from autograd_amd.numpy import fusion

    was, fusion.ENABLED = fusion.ENABLED, True
    try:
        def chain(shape, dtype=torch.float64, axes=(1,), op=Op.COPY):
            g, t, y = (meta(shape, dtype) for _ in range(3))
            e = g * t
            s = D.map_reduce(op, Red.SUM, e.dtype, (e,), axes, True)
            assert type(s) is D.PendingReduce and s._call is not None
            return e, s, y

        e, s, y = chain((256, 128))
        root = e - y * s
        assert type(root) is fusion.ExprArray and s._call is not None       # nothing ran
        emitted = fusion._emit([root])
        assert PROGRAM_ROWSUM in _ops_of(emitted[3]) and emitted[4] == 16 and _ops_of(emitted[3])[-1] == PROGRAM_STORE
        assert len(emitted[0]) == 3                                          # g, t, y: the sums are no leaf
        e, s, y = chain((256, 128), op=Op.NEG)                               # the unbroadcast of -g
        assert PROGRAM_ROWSUM in _ops_of(fusion._emit([e + y * s])[3])
        for shape, dtype in (((8, 100), torch.float64), ((256, 300), torch.float64), ((64, 600), torch.float32), ((5, 1), torch.float64)):
            e, s, y = chain(shape, dtype)
            assert fusion._row_sums(s, shape, e.dtype) is None, shape         # not a shape of the row-group kernel
        e, s, y = chain((256, 128), axes=(0,))
        assert fusion._row_sums(s, (256, 128), e.dtype) is None               # column sums
        assert fusion._row_sums(chain((64, 512), torch.float32)[1], (64, 512), onp.dtype("float32")) is not None
        assert fusion._row_sums(chain((7, 64))[1], (7, 64), onp.dtype("float64")) is not None
    finally:
        fusion.ENABLED = was


def test_forward_products_left_pending_are_offered_once_and_not_across_a_recording(monkeypatch):
    """``devarray.note_forward_product`` / ``_forward_mate``: the newest product that has not run is offered to the next
    dense layer's launch, once; products that have run, have died, or were made on the other side of a graph recording
    are not."""
    import gc

    f64 = onp.dtype("float64")
    monkeypatch.setattr(D, "_FORWARD_PRODUCTS", [])
    mk = lambda: D.PendingProduct(torch.zeros((4, 6), dtype=torch.float64), torch.zeros((6, 5), dtype=torch.float64), f64)  # noqa: E731
    a, b, layer = D.note_forward_product(mk()), D.note_forward_product(mk()), D.note_forward_product(mk())
    assert D._forward_mate(layer) is b            # the newest other one
    assert D._forward_mate(layer) is a            # b is offered once
    assert D._forward_mate(layer) is None
    c = D.note_forward_product(mk())
    c._left = None                                # it has run
    assert c.computed() and D._forward_mate(layer) is None
    d = D.note_forward_product(mk())
    del d
    gc.collect()
    assert D._forward_mate(layer) is None         # it has died
    e = D.note_forward_product(mk())
    monkeypatch.setattr(D._lib, "CAPTURING", True)
    assert D._forward_mate(layer) is None         # made outside the recording that is now running
    inside = D.note_forward_product(mk())
    assert D._forward_mate(layer) is inside
    monkeypatch.setattr(D._lib, "CAPTURING", False)
    assert D._forward_mate(layer) is e


def test_slices_of_a_pending_product_stay_products():
    """``wrapper._part_of_product``: rows and columns of a product that has not run are taken from its factors when the
    slice keeps at least half of each axis; anything else is left to the ordinary view of the whole product."""
    left, right = torch.zeros((10, 7), dtype=torch.float64), torch.zeros((7, 12), dtype=torch.float64)
    P = D.PendingProduct(left, right, onp.dtype("float64"))
    part = W._part_of_product(P, (slice(None), slice(2, 11)))
    assert type(part) is D.PendingProduct and part.shape == (10, 9) and not P.computed()
    assert part._left.data_ptr() == left.data_ptr() and part._right.data_ptr() == right[:, 2:].data_ptr()
    rows = W._part_of_product(P, (slice(4, None),))
    assert rows.shape == (6, 12) and rows._left.data_ptr() == left[4:].data_ptr()
    for idx in ((slice(None), slice(0, 5)), (slice(0, 4), slice(None)), (slice(None), slice(0, 12, 2)), (slice(None), slice(None)),
                (slice(None), 3), (slice(None), slice(None), None)):
        assert W._part_of_product(P, idx) is None
    acc = P.sum_started()
    acc.add_product(D.PendingProduct(left, right, onp.dtype("float64")))
    assert W._part_of_product(acc, (slice(None), slice(2, 11))) is None  # a sum of products is sliced as a whole
