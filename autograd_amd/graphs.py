"""Record a differentiated function once, replay it as one HIP graph.

A gradient evaluation on fixed shapes launches the same kernels with the same arguments every
time; what changes is the contents of the input buffers.  For launch-bound programs (the tanh
RNN tapes a few thousand small kernels per evaluation, reference examples/rnn.py:20-61) the
Python tracer and the per-launch host cost then bound the rate, not the GPU.  ``capture`` runs
the function once under HIP stream capture, so that every kernel the tracer's forward and
backward passes launch (``core.backward_pass``, core.py:26-33 of the reference, included) lands
in one graph, and returns a callable that copies new input values into the recorded input
buffers and replays the graph: one host call per evaluation, results bit-identical to the
eager path because the very same kernels run in the very same order.

Only kernel launches can be recorded.  A function that moves data between host and device
while it runs (``.numpy()``, ``float(x)``, integer-array indexing, uploading a NumPy constant)
or whose control flow depends on array *values* cannot be captured; ``capture`` raises for the
former, and replays the branch taken at capture time for the latter.
"""

import numbers

import numpy as onp
import torch

from . import _lib
from ._lib import Op
from .numpy import devarray as D
from .numpy.devarray import DevArray


def _flatten(tree, leaves):
    """Structure of a nest of tuples/lists/dicts with its leaves appended to ``leaves``."""
    if isinstance(tree, (list, tuple)):
        return (type(tree), [_flatten(t, leaves) for t in tree])
    if isinstance(tree, dict):
        return (dict, [(k, _flatten(v, leaves)) for k, v in tree.items()])
    leaves.append(tree)
    return None


def _unflatten(struct, it):
    if struct is None:
        return next(it)
    kind, items = struct
    if kind is dict:
        return {k: _unflatten(s, it) for k, s in items}
    return kind(_unflatten(s, it) for s in items)


def _static_copy(x):
    out = D.empty(x.shape, x.dtype)
    _copy_into(out, x)
    return out


def _copy_into(dst, src):
    if dst.dtype in D._FLOATS:
        D.map_op(Op.COPY, dst.dtype, src, out=dst)
    else:
        code = _lib.DTYPE_CODE[dst.dtype]
        _lib.cast(code, code, dst.shape, dst._t, src._t)


class CapturedFunction:
    """``fun`` recorded on the shapes and dtypes of ``example_args`` (see :func:`capture`)."""

    def __init__(self, fun, example_args, warmup=1):
        _lib.device()
        leaves = []
        self._in_struct = _flatten(tuple(example_args), leaves)
        self._static_in = []  # DevArray for array leaves, the constant itself otherwise
        for leaf in leaves:
            if isinstance(leaf, onp.ndarray):
                leaf = D.from_numpy(leaf)
            self._static_in.append(_static_copy(leaf) if isinstance(leaf, DevArray) else leaf)
        self._last = [None] * len(leaves)  # the array object last copied into each input buffer
        self._writes_seen = D.ITEM_WRITES  # value of the item-assignment counter at the last call
        args = _unflatten(self._in_struct, iter(self._static_in))
        # eager runs first: one-time allocations (shared zeros, the reduction workspace) happen outside the graph's
        # memory pool, unsupported programs fail here plainly, and the elementwise programs of a function that is
        # about to be replayed many times get their specialised kernels now (none can be compiled while recording)
        sightings = _lib.specialize_after(-1)
        if sightings > 0:
            _lib.specialize_after(1)
        try:
            for _ in range(max(int(warmup), 1)):
                warm = []
                _flatten(fun(*args), warm)
                for o in warm:
                    if isinstance(o, DevArray):
                        D.plain(o)  # (results still pending are written out, as the recording will)
        finally:
            _lib.specialize_after(sightings)
        _lib.synchronize()
        self._graph = torch.cuda.CUDAGraph()
        timer, _lib._TIMER = _lib._TIMER, None
        _lib.CAPTURING = True
        try:
            with torch.cuda.graph(self._graph):
                out = fun(*args)
                out_leaves = []
                self._out_struct = _flatten(out, out_leaves)
                # pending maps are written out inside the graph; outputs that alias an input
                # buffer are copied so that the next call's input copy cannot change them
                in_ptrs = {a._t.data_ptr() for a in self._static_in if isinstance(a, DevArray)}
                self._static_out = [self._own(o, in_ptrs) for o in out_leaves]
        finally:
            _lib.CAPTURING = False
            _lib._TIMER = timer
        _lib.synchronize()

    @staticmethod
    def _own(o, in_ptrs):
        if not isinstance(o, DevArray):
            return o
        o = D.plain(o)
        return _static_copy(o) if o._t.data_ptr() in in_ptrs else o

    @property
    def static_inputs(self):
        """The recorded input buffers, in the nesting of the arguments.  A caller that writes new
        values into them itself (an optimizer step) can then call :meth:`replay` directly."""
        return _unflatten(self._in_struct, iter(self._static_in))

    def replay(self):
        """Run the recorded kernels on whatever the input buffers hold now."""
        self._graph.replay()
        return _unflatten(self._out_struct, iter(self._static_out))

    def __call__(self, *args):
        """Evaluate on ``args`` (same nesting, shapes and dtypes as at capture).

        Returns the recorded output arrays: the next call overwrites them, so copy what must
        outlive it.  An argument array that is the same object as in the previous call is not
        copied again, unless some array has been written by item assignment since (``D.ITEM_WRITES``)."""
        leaves = []
        struct = _flatten(tuple(args), leaves)
        if struct != self._in_struct:
            raise TypeError("captured function called with a different argument structure than it was captured on")
        last = self._last
        unwritten = self._writes_seen == D.ITEM_WRITES  # no item assignment anywhere since the last call
        self._writes_seen = D.ITEM_WRITES
        for k, (leaf, static) in enumerate(zip(leaves, self._static_in)):
            if isinstance(static, DevArray):
                if leaf is last[k] and unwritten and isinstance(leaf, DevArray):
                    continue
                src = D.from_numpy(leaf) if isinstance(leaf, onp.ndarray) else leaf
                if not isinstance(src, DevArray) or src.shape != static.shape or src.dtype != static.dtype:
                    raise TypeError(
                        f"captured function: argument leaf {k} must be a {static.dtype} array of shape {static.shape}"
                    )
                if src._h().data_ptr() != static._t.data_ptr() or type(src) is not DevArray:
                    _copy_into(static, src)
                last[k] = leaf
            elif isinstance(static, numbers.Number):
                if not (isinstance(leaf, numbers.Number) and leaf == static):
                    raise ValueError(
                        f"captured function: non-array argument leaf {k} is a constant of the recording "
                        f"({static!r}); got {leaf!r}"
                    )
            elif leaf is not static and leaf != static:
                raise ValueError(f"captured function: non-array argument leaf {k} differs from the recording")
        return self.replay()


def capture(fun, *example_args, warmup=1):
    """Record ``fun(*example_args)`` into a HIP graph and return the replaying callable.

    ``fun`` is typically ``grad(f)``, ``elementwise_grad(f)`` or a whole training step; its
    arguments and results are device arrays or nests (tuple / list / dict) of them.  Non-array
    argument leaves are constants of the recording.
    """
    return CapturedFunction(fun, example_args, warmup=warmup)
