"""Function tracing: boxes, trace levels and the ``primitive`` wrapper.

This is the value-type-agnostic recording layer.  It has the same contract as
the reference's autograd/tracer.py:14-195 so that rule tables and value types
written for that API (``primitive``, ``Box.register``, ``register_notrace``)
work unchanged; it contains no arithmetic.

Terminology: a *box* wraps a value taking part in a trace; ``_trace`` is the
nesting level of the trace that created it (inner differentiation = higher
level) and ``_node`` the tape node that produced it.  A primitive called with
boxed arguments strips only the boxes of the highest level present, calls
itself on the remaining values (which may still be boxes of outer traces, so
the call is recorded there as well), and re-boxes the result with a new node.
"""

import warnings
from collections import defaultdict

from .util import subvals, toposort  # noqa: F401  (toposort re-exported as in the reference)
from .wrap_util import wraps

__all__ = [
    "trace",
    "Node",
    "primitive",
    "register_notrace",
    "notrace_primitive",
    "find_top_boxed_args",
    "Box",
    "new_box",
    "isbox",
    "getval",
    "trace_primitives_map",
    "trace_stack",
]


class Node:
    """Base class of tape nodes.  Subclasses define what is recorded per call.

    Constructor protocol (reference autograd/tracer.py:25-38):
    ``NodeType(value, fun, args, kwargs, parent_argnums, parents)`` for an
    interior node, ``NodeType.new_root(*a, **k)`` -> ``initialize_root`` for the
    node attached to the traced function's input.
    """

    __slots__ = []

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        raise AssertionError("Node subclasses must define __init__")

    def initialize_root(self, *args, **kwargs):
        raise AssertionError("Node subclasses must define initialize_root")

    @classmethod
    def new_root(cls, *args, **kwargs):
        root = cls.__new__(cls)
        root.initialize_root(*args, **kwargs)
        return root


class _OpenTrace:
    """``with trace_stack.new_trace() as level``: one more nesting level for the duration of the block."""

    __slots__ = ("stack",)

    def __init__(self, stack):
        self.stack = stack

    def __enter__(self):
        self.stack.top += 1
        return self.stack.top

    def __exit__(self, *exc):
        self.stack.top -= 1
        return False


class TraceStack:
    """Process-global counter of nested traces (single-threaded by contract)."""

    def __init__(self):
        self.top = -1

    def new_trace(self):
        return _OpenTrace(self)


trace_stack = TraceStack()


def trace(start_node, fun, x):
    """Run ``fun`` on a boxed ``x``; return ``(end_value, end_node)``.

    ``end_node`` is None (with a warning) when the output does not depend on the
    input through this trace (reference autograd/tracer.py:14-22).
    """
    with trace_stack.new_trace() as level:
        start_box = new_box(x, level, start_node)
        end_box = fun(start_box)
        if isbox(end_box) and end_box._trace == start_box._trace:
            return end_box._value, end_box._node
        warnings.warn("Output seems independent of input.")
        return end_box, None


class Box:
    """Wrapper for a value that takes part in a trace.

    ``Box.register(value_type)`` on a subclass declares that values of
    ``value_type`` are boxed with that subclass (reference
    autograd/tracer.py:157-180).
    """

    type_mappings = {}
    types = set()

    __slots__ = ["_value", "_trace", "_node"]

    def __init__(self, value, trace, node):
        self._value = value
        self._trace = trace
        self._node = node

    def __bool__(self):
        return bool(self._value)

    __nonzero__ = __bool__

    def __str__(self):
        return f"Autograd {type(self).__name__} with value {self._value!s}"

    @classmethod
    def register(cls, value_type):
        Box.types.add(cls)
        Box.type_mappings[value_type] = cls
        Box.type_mappings[cls] = cls


box_type_mappings = Box.type_mappings
box_types = Box.types


def new_box(value, trace, node):
    try:
        box_cls = box_type_mappings[type(value)]
    except KeyError:
        raise TypeError(f"Can't differentiate w.r.t. type {type(value)}") from None
    return box_cls(value, trace, node)


def isbox(x):
    return type(x) in box_types


def getval(x):
    while type(x) in box_types:
        x = x._value
    return x


def find_top_boxed_args(args):
    """Return ``(boxes, level, node_type)`` for the boxes of the highest trace level.

    ``boxes`` is a list of ``(argnum, box)``; ``level`` is -1 when no positional
    argument is a box (reference autograd/tracer.py:119-140; keyword arguments
    are never differentiated).
    """
    top_level = -1
    top_boxes = []
    top_node_type = None
    for argnum, arg in enumerate(args):
        if type(arg) in box_types:
            level = arg._trace
            if level > top_level:
                top_boxes = [(argnum, arg)]
                top_level = level
                top_node_type = type(arg._node)
            elif level == top_level:
                top_boxes.append((argnum, arg))
    return top_boxes, top_level, top_node_type


trace_primitives_map = {}
notrace_primitives = defaultdict(set)


def primitive(f_raw):
    """Wrap ``f_raw`` so that calls with boxed arguments are recorded on the tape.

    The wrapper carries ``.fun`` (the raw function) and
    ``._is_autograd_primitive``; derivative rules are attached to the wrapper
    with ``defvjp`` / ``defjvp`` (reference autograd/tracer.py:44-99).
    """

    @wraps(f_raw)
    def f_wrapped(*args, **kwargs):
        # this wrapper runs for every array operation of a traced program, so it scans the arguments itself:
        # first for the highest trace level present, then to unbox the arguments of that level
        top = -1
        for arg in args:
            if type(arg) in box_types and arg._trace > top:
                top = arg._trace
        if top < 0:
            return f_raw(*args, **kwargs)
        argvals, argnums, parents = list(args), [], []
        nested = False  # a box of an outer trace remains among the values: they go through the wrapper again
        for argnum, arg in enumerate(args):
            if type(arg) in box_types:
                if arg._trace == top:
                    value = argvals[argnum] = arg._value
                    argnums.append(argnum)
                    parents.append(arg._node)
                    if type(value) in box_types:
                        nested = True
                else:
                    nested = True
        argvals = tuple(argvals)
        node_constructor = type(parents[0])
        if f_wrapped in notrace_primitives[node_constructor]:
            return f_wrapped(*argvals, **kwargs)
        ans = f_wrapped(*argvals, **kwargs) if nested else f_raw(*argvals, **kwargs)
        node = node_constructor(ans, f_wrapped, argvals, kwargs, tuple(argnums), tuple(parents))
        box_cls = box_type_mappings.get(type(ans))
        if box_cls is None:
            return new_box(ans, top, node)  # raises the type error
        return box_cls(ans, top, node)

    f_wrapped.fun = f_raw
    f_wrapped._is_autograd_primitive = True
    try:
        trace_primitives_map[f_raw] = f_wrapped
    except TypeError:  # unhashable callables cannot be looked up by identity
        pass
    return f_wrapped


def register_notrace(trace_type, primitive_fun):
    """Declare that ``primitive_fun`` is constant for traces using ``trace_type`` nodes."""
    notrace_primitives[trace_type].add(primitive_fun)


def notrace_primitive(f_raw):
    """Wrap a function that never participates in a trace: unbox everything, call."""

    @wraps(f_raw)
    def f_wrapped(*args, **kwargs):
        return f_raw(*[getval(a) for a in args], **kwargs)

    f_wrapped._is_primitive = True
    return f_wrapped
