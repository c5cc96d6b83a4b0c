"""N-d ``convolve`` on device arrays, with its reverse- and forward-mode rules.

Counterpart of the reference's autograd/scipy/signal.py:10-217.  There the forward is an
``as_strided`` window view of the explicitly zero-padded larger operand contracted with the
flipped smaller one by ``numpy.einsum`` (45-65), and each cotangent is another ``convolve`` of
the incoming cotangent with the other operand, flipped (153-214).  Here one kernel
(``agmi_correlate``) does the window contraction directly: padding is a bounds test, flips are
negative strides, the transposes that bring axes into (free, contracted, convolved) order are
stride permutations.  No operand is copied unless a group of its free or contracted axes cannot
be walked with a single stride.

``convolve`` takes one keyword beyond the reference's, ``flip=(a, b, out)``: operand ``A`` / ``B``
is read reversed along its convolved axes, and the result is written reversed along its own.
The cotangent rules use it in place of the reference's ``Y[flipped_idxs]`` views (a device array
has no negative strides to offer), which keeps them closed under further differentiation.
"""

import numpy as onp

from .. import _lib
from ..extend import defjvp, defvjp, primitive
from ..numpy import devarray as D
from ..numpy import wrapper as np
from ..numpy.devarray import DevArray

_MODES = ("valid", "full", "same")
_NO_FLIP = (False, False, False)


def _check_mode(mode):
    assert mode in _MODES, f"Mode {mode} undefined, it can be one of 'valid', 'full', and 'same'"


def _out_extent(n_A, n_B, mode):
    """Length of the result along a convolved axis (scipy/signal.py:135-143)."""
    return {"full": n_A + n_B - 1, "same": n_A, "valid": abs(n_A - n_B) + 1}[mode]


def _axis_roles(A_shape, B_shape, conv_axes, dot_axes, mode):
    """(roles, shapes): for "A" and "B" the convolved ("conv"), contracted ("dot") and free
    ("ignore") axes with their extents, and for "out" where A's free axes, B's free axes and the
    convolved axes sit in the result, which is laid out in that order (scipy/signal.py:91-132)."""
    if conv_axes is None:
        conv_axes = (range(len(A_shape)),) * 2
    roles, shapes = {}, {}
    for k, (name, shape) in enumerate((("A", A_shape), ("B", B_shape))):
        conv, dot = tuple(conv_axes[k]), tuple(dot_axes[k])
        free = tuple(ax for ax in range(len(shape)) if ax not in conv and ax not in dot)
        roles[name] = {"conv": conv, "dot": dot, "ignore": free}
        shapes[name] = {role: tuple(shape[ax] for ax in axs) for role, axs in roles[name].items()}
    assert len(roles["A"]["dot"]) == len(roles["B"]["dot"])
    assert len(roles["A"]["conv"]) == len(roles["B"]["conv"])
    bounds = onp.cumsum([0, len(roles["A"]["ignore"]), len(roles["B"]["ignore"]), len(roles["A"]["conv"])])
    spans = [tuple(range(lo, hi)) for lo, hi in zip(bounds, bounds[1:])]
    roles["out"] = dict(zip(("ignore_A", "ignore_B", "conv"), spans))
    shapes["out"] = {"ignore_A": shapes["A"]["ignore"], "ignore_B": shapes["B"]["ignore"],
                     "conv": tuple(_out_extent(a, b, mode) for a, b in zip(shapes["A"]["conv"], shapes["B"]["conv"]))}
    return roles, shapes


def _merged_stride(sizes, strides):
    """Single element stride that walks a group of axes in row-major order, or None."""
    dims = [(n, s) for n, s in zip(sizes, strides) if n != 1]
    if not dims:
        return 0
    for (_, s_outer), (n_inner, s_inner) in zip(dims, dims[1:]):
        if s_outer != s_inner * n_inner:
            return None
    return dims[-1][1]


def _window_operand(field, t, roles, flipped):
    """Fill the C block's ``filter`` / ``signal`` member for tensor ``t`` whose axes have the given
    roles.  Returns the tensor that owns the memory (``t`` or a contiguous transposed copy)."""
    n_free, n_dot = len(roles["ignore"]), len(roles["dot"])
    view = t.permute(roles["ignore"] + roles["dot"] + roles["conv"])
    sizes, strides = tuple(view.shape), view.stride()
    batch = _merged_stride(sizes[:n_free], strides[:n_free])
    dot = _merged_stride(sizes[n_free:n_free + n_dot], strides[n_free:n_free + n_dot])
    if batch is None or dot is None:
        view = D.copy(DevArray(view))._t
        strides = view.stride()
        batch = _merged_stride(sizes[:n_free], strides[:n_free])
        dot = _merged_stride(sizes[n_free:n_free + n_dot], strides[n_free:n_free + n_dot])
    first = 0
    for d, (n, s) in enumerate(zip(sizes[n_free + n_dot:], strides[n_free + n_dot:])):
        if flipped:
            first += (n - 1) * s
            s = -s
        field.strides[d] = s
    field.data = view.data_ptr() + first * view.element_size()
    field.batch_stride, field.dot_stride = batch, dot
    return view


def _prod(xs):
    p = 1
    for x in xs:
        p *= x
    return p


@primitive
def convolve(A, B, axes=None, dot_axes=None, mode="full", flip=_NO_FLIP):
    if dot_axes is None:
        dot_axes = [(), ()]
    _check_mode(mode)
    A, B = D.asarray(A), D.asarray(B)
    if axes is None:
        axes = [list(range(A.ndim)), list(range(A.ndim))]
    dtype = D.result_dtype(A, B)
    if dtype not in D._FLOATS:
        raise TypeError(f"convolve: {dtype} operands are not supported on the device")
    roles, shapes = _axis_roles(A.shape, B.shape, axes, dot_axes, mode)
    n_conv = len(roles["A"]["conv"])
    if n_conv == 0:
        # nothing slides: what is left is the contraction over dot_axes, free axes of A before those of B
        from ..numpy.wrapper import _tensordot_raw

        return _tensordot_raw(D.asarray(A, dtype), D.asarray(B, dtype), axes=(list(dot_axes[0]), list(dot_axes[1])))
    if not 1 <= n_conv <= 3:
        raise NotImplementedError(f"convolve over {n_conv} axes (1 to 3 are supported on the device)")
    if shapes["A"]["dot"] != shapes["B"]["dot"]:
        raise ValueError(f"contracted axes differ: {shapes['A']['dot']} vs {shapes['B']['dot']}")

    # which operand is the window that slides over the other (scipy/signal.py:19-44)
    sizes = list(zip(shapes["A"]["conv"], shapes["B"]["conv"]))
    if mode == "same":
        window_is_A = False
    else:
        window_is_A = True
        if any(b < a for a, b in sizes):
            if mode == "valid" and not all(b <= a for a, b in sizes):
                raise ValueError("One array must be larger than the other along all convolved dimensions")
            if mode == "valid" or B.size <= A.size:
                window_is_A = False
    W, S = ("A", "B") if window_is_A else ("B", "A")

    out_shape = shapes["out"]["ignore_A"] + shapes["out"]["ignore_B"] + shapes["out"]["conv"]
    out = D.empty(out_shape, dtype)
    if out.size == 0:
        return out

    c = _lib.AgmiCorrelation()
    c.n_conv = n_conv
    c.filter_batch, c.signal_batch = _prod(shapes[W]["ignore"]), _prod(shapes[S]["ignore"])
    c.dot = _prod(shapes["A"]["dot"])
    for d in range(n_conv):
        K, N = shapes[W]["conv"][d], shapes[S]["conv"][d]
        c.window[d], c.extent[d] = K, N
        c.pad_before[d] = {"valid": 0, "full": K - 1, "same": K - 1 - (K - 1) // 2}[mode]
        c.out_extent[d] = shapes["out"]["conv"][d]
    operands = {"A": A, "B": B}
    tensors = {k: D.asarray(v, dtype)._t for k, v in operands.items()}
    reversed_ = {"A": bool(flip[0]), "B": bool(flip[1])}
    # convolution proper reads the window back to front; a window that is itself to be read flipped goes forward
    keep_w = _window_operand(c.filter, tensors[W], roles[W], not reversed_[W])
    keep_s = _window_operand(c.signal, tensors[S], roles[S], reversed_[S])
    n_positions = _prod(shapes["out"]["conv"])
    free_B = _prod(shapes["out"]["ignore_B"])
    stride_A, stride_B = free_B * n_positions, n_positions
    c.out_filter_stride, c.out_signal_stride = (stride_A, stride_B) if window_is_A else (stride_B, stride_A)
    first, step = 0, 1
    for d in reversed(range(n_conv)):
        n = shapes["out"]["conv"][d]
        if flip[2]:
            first += (n - 1) * step
            c.out_strides[d] = -step
        else:
            c.out_strides[d] = step
        step *= n
    c.out = out._t.data_ptr() + first * out._t.element_size()
    taps = c.dot * _prod(shapes[W]["conv"])
    _lib.correlate(_lib.DTYPE_CODE[dtype], c, (keep_w.numel() + keep_s.numel() + out.size) * dtype.itemsize,
                   2.0 * out.size * taps)
    return out


def _grad_convolve(argnum, ans, A, B, axes=None, dot_axes=None, mode="full", flip=_NO_FLIP):
    """scipy/signal.py:153-214, with the flips carried as flags: the cotangent w.r.t. X is the
    convolution of g (read reversed if the result was written reversed) with Y read the other
    way round than the forward pass read it, written reversed if the forward pass read X reversed."""
    if dot_axes is None:
        dot_axes = [(), ()]
    _check_mode(mode)
    A_shape, B_shape = np.shape(A), np.shape(B)
    axes, shapes = _axis_roles(A_shape, B_shape, axes, dot_axes, mode)
    if argnum == 0:
        Y, _X_, _Y_, ignore_Y = B, "A", "B", "ignore_B"
        flip_X, flip_Y = flip[0], flip[1]
    elif argnum == 1:
        Y, _X_, _Y_, ignore_Y = A, "B", "A", "ignore_A"
        flip_X, flip_Y = flip[1], flip[0]
    else:
        raise NotImplementedError(f"Can't take grad of convolve w.r.t. arg {argnum}")

    if mode == "full":
        new_mode = "valid"
    elif mode == "valid":
        if any(x_size > y_size for x_size, y_size in zip(shapes[_X_]["conv"], shapes[_Y_]["conv"])):
            new_mode = "full"
        else:
            new_mode = "valid"
    else:
        new_mode = "valid"
    new_flip = (bool(flip[2]), not flip_Y, bool(flip_X))
    new_order = tuple(int(i) for i in onp.argsort(axes[_X_]["ignore"] + axes[_X_]["dot"] + axes[_X_]["conv"]))

    def vjp(g):
        if mode == "same":
            g_pad = [(0, 0)] * np.ndim(g)
            for ax, ax_B in zip(axes["out"]["conv"], axes["B"]["conv"]):
                left_bound = (B_shape[ax_B] - 1) // 2
                widths = (left_bound, B_shape[ax_B] - 1 - left_bound)
                # g is read reversed when the result was written reversed: pad what it will be read as
                g_pad[ax] = widths[::-1] if flip[2] else widths
            g = np.pad(g, g_pad, mode="constant")
        result = convolve(g, Y, axes=[axes["out"]["conv"], axes[_Y_]["conv"]],
                          dot_axes=[axes["out"][ignore_Y], axes[_Y_]["ignore"]], mode=new_mode, flip=new_flip)
        return np.transpose(result, new_order)

    return vjp


defvjp(convolve, lambda *a, **k: _grad_convolve(0, *a, **k), lambda *a, **k: _grad_convolve(1, *a, **k))
# bilinear: the tangent in either slot goes through the same contraction (the reference defines no forward rule)
defjvp(convolve, "same", "same")
