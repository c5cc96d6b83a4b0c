"""Two tracers that record something other than derivative rules.

``const_graph`` (reference autograd/misc/tracers.py:25-57) evaluates a function once under a recording tracer and
from then on replays the recorded primitive calls only: Python control flow, and every call that did not depend
on the traced arguments, run once.  ``full_graph`` (59-75) returns the final node of a trace in which each node
keeps its value and how it was made.  Both are ordinary ``Node`` subclasses handed to ``trace``, the mechanism of
autograd/tracer.py:14-38, so device arrays pass through them like any other value.

The recording is kept as a flat program: one step per primitive call, whose traced operands are slot numbers
into a list of values, so a replay is one loop over the steps.
"""

from functools import partial

from ..tracer import Node, trace
from ..util import toposort
from ..wrap_util import wraps


class RecordedCall(Node):
    """One primitive call: the function, its arguments as given (traced ones are overwritten on replay), which
    positions were traced and the nodes they came from."""

    __slots__ = ["parents", "call", "operands", "options", "traced_positions"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        self.parents = list(parents)
        self.call, self.options = fun, kwargs
        self.traced_positions = tuple(parent_argnums)
        held = list(args)
        for position in self.traced_positions:
            held[position] = None  # (the value of the first evaluation is not kept alive)
        self.operands = held

    def initialize_root(self):
        self.parents, self.call, self.operands, self.options, self.traced_positions = [], None, [], {}, ()


def _program(last):
    """Steps ``(call, operands, options, traced_positions, source_slots)`` from the input (slot 0) to ``last``."""
    order = list(toposort(last))[::-1]  # parents before children; the root first
    slot_of = {id(node): slot for slot, node in enumerate(order)}
    steps = []
    for node in order[1:]:
        steps.append((node.call, node.operands, node.options, node.traced_positions,
                      tuple(slot_of[id(p)] for p in node.parents)))
    return steps


def const_graph_unary(fun):
    """``fun`` of one argument; the first call records, later calls replay."""
    recorded = []
    pending = [fun]  # dropped after recording: it may hold bound arguments

    def evaluate(x):
        if not recorded:
            value, last = trace(RecordedCall.new_root(), pending.pop(), x)
            if last is None:
                raise ValueError("Output is independent of input")
            recorded.append(_program(last))
            return value
        values = [x]
        for call, operands, options, positions, sources in recorded[0]:
            actual = list(operands)
            for position, source in zip(positions, sources):
                actual[position] = values[source]
            values.append(call(*actual, **options))
        return values[-1]

    return evaluate


def const_graph(fun, *args, **kwargs):
    """``fun`` with ``args`` / ``kwargs`` bound; the returned function takes the remaining positional arguments."""
    bound = partial(fun, *args, **kwargs)
    evaluate = const_graph_unary(lambda rest: bound(*rest))

    @wraps(fun)
    def replaying(*rest):
        return evaluate(rest)

    return replaying


class FullGraphNode(Node):
    """Keeps the value and the recipe ``(fun, args, kwargs, (argnum, parent) pairs)`` of every call."""

    __slots__ = ["value", "recipe"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        self.value = value
        self.recipe = (fun, args, kwargs, list(zip(parent_argnums, parents)))

    def initialize_root(self):
        self.value = None
        self.recipe = (lambda x: x, (), {}, [])


def full_graph(fun, *args, **kwargs):
    """The last node of the trace of ``fun(*args, **kwargs)`` with all positional arguments traced together."""
    _, last = trace(FullGraphNode.new_root(), lambda packed: fun(*packed, **kwargs), args)
    return last
