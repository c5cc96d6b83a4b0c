"""Small helpers shared by the tracer and the rule tables.

Behavioural counterpart of the reference's autograd/util.py:4-40 (tuple
substitution helpers and the reverse topological ordering used by the backward
replay).
"""

import gc
from operator import attrgetter

__all__ = ["subvals", "subval", "func", "toposort", "collector_paused"]


class collector_paused:
    """``with collector_paused(): ...`` switches Python's cyclic garbage collector off for the block
    (re-entrant; the previous state comes back when the outermost block ends).

    A tape is acyclic: a node's closure holds its parents' boxes and the forward values, never the
    node itself, so reference counting alone frees it.  The cyclic collector, triggered by the tens
    of objects every traced call allocates, only adds scans of a heap that keeps growing while the
    tape is alive: about a quarter of the host time of a 2 600-node evaluation."""

    _depth = 0
    _was_enabled = False

    def __enter__(self):
        cls = collector_paused
        if cls._depth == 0:
            cls._was_enabled = gc.isenabled()
            if cls._was_enabled:
                gc.disable()
        cls._depth += 1

    def __exit__(self, *exc):
        cls = collector_paused
        cls._depth -= 1
        if cls._depth == 0 and cls._was_enabled:
            gc.enable()
        return False


def subvals(seq, index_value_pairs):
    """Return ``tuple(seq)`` with ``seq[i]`` replaced by ``v`` for each ``(i, v)``."""
    out = list(seq)
    for i, v in index_value_pairs:
        out[i] = v
    return tuple(out)


def subval(seq, index, value):
    """Single-position form of :func:`subvals`."""
    out = list(seq)
    out[index] = value
    return tuple(out)


def func(f):
    """Identity; lets ``func(Class.method)`` read the same for bound primitives."""
    return f


_get_parents = attrgetter("parents")


def toposort(end_node, parents=_get_parents):
    """Yield the nodes reachable from ``end_node``, every node after all of its children.

    The visiting order is part of the contract (reference autograd/util.py:21-40):
    the order in which cotangent contributions reach a node fixes the floating
    point order of their accumulation.  Phase one counts, by a depth-first walk
    with an explicit LIFO stack, how many times each node is reached as a
    parent.  Phase two keeps a LIFO stack of nodes whose children have all been
    emitted; a parent is pushed when its last child is emitted, so for a node
    with several parents the subtree of the last-listed parent that became
    ready is replayed first.
    """
    pending_children = {}
    work = [end_node]
    while work:
        node = work.pop()
        seen = pending_children.get(node)
        if seen is None:
            pending_children[node] = 1
            work.extend(parents(node))
        else:
            pending_children[node] = seen + 1

    ready = [end_node]
    while ready:
        node = ready.pop()
        yield node
        for parent in parents(node):
            remaining = pending_children[parent]
            if remaining == 1:
                ready.append(parent)
            else:
                pending_children[parent] = remaining - 1


def quick_grad_check(fun, arg0, extra_args=(), kwargs=None, verbose=True, eps=1e-4, rtol=1e-4, atol=1e-6, rs=None):
    """The retired name of a reverse-mode, first-order ``check_grads`` with respect to the first argument
    (reference util.py:45-61); warns and delegates.  The tolerance arguments are accepted and ignored, as there."""
    import warnings

    warnings.warn("The quick_grad_check function is deprecated. See the update guide:\n"
                  "https://github.com/HIPS/autograd/blob/master/docs/updateguide.md")
    from .test_util import check_grads

    check_grads(lambda first: fun(first, *extra_args, **(kwargs or {})), modes=["rev"], order=1)(arg0)
