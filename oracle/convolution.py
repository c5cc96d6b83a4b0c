"""N-d convolution for the oracle's NumPy value type.

Restates the reference's autograd/scipy/signal.py: the forward (10-65) pads the operand that is
slid over, takes a strided window view of it and contracts that view with the reversed other
operand by ``numpy.einsum`` with integer axis labels (68-76); each cotangent (153-214) is a
convolution of the incoming cotangent with the reversed other operand in the complementary
mode.  The views and the einsum call are formed exactly as there, so results agree bit for bit.
TEST INFRASTRUCTURE: see ``oracle/__init__.py``.
"""

import numpy as onp
from numpy.lib.stride_tricks import as_strided

from autograd_amd.extend import defvjp, primitive

from . import np_namespace as np

_MODES = ("valid", "full", "same")


def _mode_ok(mode):
    assert mode in _MODES, f"Mode {mode} undefined, it can be one of 'valid', 'full', and 'same'"


def _out_size(a, b, mode):  # signal.py:135-143
    if mode == "full":
        return a + b - 1
    if mode == "same":
        return a
    if mode == "valid":
        return abs(a - b) + 1
    raise ValueError(f"Mode {mode} not recognized")


def _roles(A_shape, B_shape, conv_axes, dot_axes, mode):
    """signal.py:91-132"""
    if conv_axes is None:
        conv_axes = (tuple(range(len(A_shape))), tuple(range(len(A_shape))))
    ax = {}
    for name, shape, n in (("A", A_shape, 0), ("B", B_shape, 1)):
        ax[name] = {"conv": tuple(conv_axes[n]), "dot": tuple(dot_axes[n]),
                    "ignore": tuple(i for i in range(len(shape)) if i not in conv_axes[n] and i not in dot_axes[n])}
    assert len(ax["A"]["dot"]) == len(ax["B"]["dot"])
    assert len(ax["A"]["conv"]) == len(ax["B"]["conv"])
    a, b, c = len(ax["A"]["ignore"]), len(ax["B"]["ignore"]), len(ax["A"]["conv"])
    ax["out"] = {"ignore_A": tuple(range(a)), "ignore_B": tuple(range(a, a + b)), "conv": tuple(range(a + b, a + b + c))}
    sh = {"A": {k: tuple(A_shape[i] for i in v) for k, v in ax["A"].items()},
          "B": {k: tuple(B_shape[i] for i in v) for k, v in ax["B"].items()}}
    return ax, sh


def _reversed(ndim, axes):
    idx = [slice(None)] * ndim
    for a in axes:
        idx[a] = slice(None, None, -1)
    return tuple(idx)


def _zero_pad(S, W, axes, mode):
    """Pad the slid-over operand S for window W.  signal.py:79-88 (axes = (S axes, W axes))"""
    widths = [(0, 0)] * S.ndim
    for a_s, a_w in zip(*axes):
        k = W.shape[a_w]
        if mode == "full":
            widths[a_s] = (k - 1, k - 1)
        elif mode == "same":
            after = (k - 1) // 2
            widths[a_s] = (k - 1 - after, after)
    return onp.pad(S, widths, mode="constant")


def _labelled_contraction(X, Y, paired_axes):
    """einsum with integer labels: axis k of X is label k, of Y label X.ndim + k, and each
    (x_axis, y_axis) pair shares a label beyond those, so it is summed.  signal.py:68-76"""
    x_labels = list(range(X.ndim))
    y_labels = list(range(X.ndim, X.ndim + Y.ndim))
    shared = X.ndim + Y.ndim
    for n, (ax, ay) in enumerate(zip(*paired_axes)):
        x_labels[ax] = y_labels[ay] = shared + n
    return onp.einsum(X, x_labels, Y, y_labels)


@primitive
def convolve(A, B, axes=None, dot_axes=None, mode="full"):
    if dot_axes is None:
        dot_axes = [(), ()]
    _mode_ok(mode)
    if axes is None:
        axes = [list(range(A.ndim)), list(range(A.ndim))]
    pairs = list(zip(*axes))
    if any(B.shape[b] < A.shape[a] for a, b in pairs):  # signal.py:19-32
        if mode == "valid" and not all(B.shape[b] <= A.shape[a] for a, b in pairs):
            raise ValueError("One array must be larger than the other along all convolved dimensions")
        elif mode == "valid" or (mode == "full" and B.size <= A.size):
            n_free_B = B.ndim - len(dot_axes[1]) - len(axes[1])
            n_free_A = A.ndim - len(dot_axes[0]) - len(axes[0])
            free_B = list(range(n_free_B))
            free_A = list(range(n_free_B, n_free_B + n_free_A))
            conv = list(range(n_free_B + n_free_A, n_free_B + n_free_A + len(axes[0])))
            swapped = convolve(B, A, axes=axes[::-1], dot_axes=dot_axes[::-1], mode=mode)
            return swapped.transpose(free_A + free_B + conv)

    if mode == "same":  # the roles are not symmetric: A is slid over, B is the window (signal.py:34-42)
        B, A = A, B
        axes = axes[::-1]
        dot_axes = dot_axes[::-1]
    if mode != "valid":
        B = _zero_pad(B, A, axes[::-1], mode)
    view_shape, view_strides = list(B.shape), list(B.strides)
    reverse = [slice(None)] * A.ndim
    for a, b in zip(*axes):  # signal.py:45-54
        view_shape.append(abs(B.shape[b] - A.shape[a]) + 1)
        view_strides.append(B.strides[b])
        view_shape[b] = A.shape[a]
        reverse[a] = slice(None, None, -1)
    windows = as_strided(B, view_shape, view_strides)
    window = A[tuple(reverse)]
    paired = [list(axes[n]) + list(dot_axes[n]) for n in (0, 1)]
    if mode == "same":  # signal.py:56-63
        n_free_S = B.ndim - len(dot_axes[1]) - len(axes[1])
        n_conv = len(axes[0])
        n_free_W = A.ndim - len(dot_axes[0]) - len(axes[0])
        free_S = list(range(n_free_S))
        conv = list(range(n_free_S, n_free_S + n_conv))
        free_W = list(range(n_free_S + n_conv, n_free_S + n_conv + n_free_W))
        return _labelled_contraction(windows, window, paired[::-1]).transpose(free_S + free_W + conv)
    return _labelled_contraction(window, windows, paired)


def _grad_convolve(argnum, ans, A, B, axes=None, dot_axes=None, mode="full"):
    """signal.py:153-214"""
    if dot_axes is None:
        dot_axes = [(), ()]
    _mode_ok(mode)
    axes, shapes = _roles(A.shape, B.shape, axes, dot_axes, mode)
    if argnum == 0:
        Y, x, y, free_y = B, "A", "B", "ignore_B"
    elif argnum == 1:
        Y, x, y, free_y = A, "B", "A", "ignore_A"
    else:
        raise NotImplementedError(f"Can't take grad of convolve w.r.t. arg {argnum}")
    if mode == "full":
        new_mode = "valid"
    elif mode == "valid":
        grows = any(nx > ny for nx, ny in zip(shapes[x]["conv"], shapes[y]["conv"]))
        new_mode = "full" if grows else "valid"
    else:
        new_mode = "valid"
    B_shape = B.shape

    def vjp(g):
        if mode == "same":
            widths = [(0, 0)] * g.ndim
            for a_out, a_B in zip(axes["out"]["conv"], axes["B"]["conv"]):
                before = (B_shape[a_B] - 1) // 2
                widths[a_out] = (before, B_shape[a_B] - 1 - before)
            g = np.pad(g, widths, mode="constant")
        result = convolve(g, Y[_reversed(Y.ndim, axes[y]["conv"])],
                          axes=[axes["out"]["conv"], axes[y]["conv"]],
                          dot_axes=[axes["out"][free_y], axes[y]["ignore"]], mode=new_mode)
        order = onp.argsort(axes[x]["ignore"] + axes[x]["dot"] + axes[x]["conv"])
        return np.transpose(result, order)

    return vjp


defvjp(convolve, lambda *a, **k: _grad_convolve(0, *a, **k), lambda *a, **k: _grad_convolve(1, *a, **k))
