"""Reverse and forward mode on top of the tracer, and the vector-space layer.

Same contract as the reference's autograd/core.py:11-345 (same public names, argument meaning and
error behaviour).  The functions in this file are the host side of the hot path: ``backward_pass``
replays the tape and ``add_outgrads`` accumulates cotangents; the arithmetic they trigger lives in
the value type's rules and ``VSpace`` (for device arrays: HIP kernels).

Accumulation protocol (reference autograd/core.py:185-205), kept exactly because it decides both
aliasing and floating-point order: a node's cotangent is stored as ``(value, owned)``.  The first
dense contribution is kept by reference and is NOT owned (it may alias a tape value or another
node's cotangent); the second goes through ``vs.add`` which produces a fresh, owned buffer; later
ones are added in place with ``vs.mut_add``.  Sparse contributions (``SparseObject``) are always
scattered into an owned dense buffer, which is zero-filled on first use or copied from a
predecessor that was not owned.
"""

import warnings
from itertools import count

from .tracer import Box, Node, box_type_mappings, getval, isbox, new_box, primitive, toposort, trace, trace_stack
from .util import collector_paused, func, subval


def _undefined(mode, fun, argnums):
    """Message of the error raised when a primitive has no rule of kind ``mode`` (core.py:43-45, 133-135)."""
    return f"{mode} of {getattr(fun, '__name__', fun)} wrt argnums {argnums} not defined"


def _bad_rule(mode, rule, fun):
    return TypeError(f"Bad {mode} '{rule}' for '{fun.__name__}'")


def settle(value):
    """A derivative as it is handed to the caller: value types whose arithmetic may be deferred
    (they define ``_settled``) complete it here, inside whatever is timing the evaluation;
    containers are walked, boxes and everything else pass through."""
    kind = type(value)
    finish = getattr(kind, "_settled", None)
    if finish is not None:
        return finish(value)
    if kind is tuple or kind is list:
        _settle_together(value)
        return kind(settle(item) for item in value)
    if kind is dict:
        _settle_together(value.values())
        return {key: settle(item) for key, item in value.items()}
    return value


def _settle_together(items):
    """Items of one container whose type can complete several values in one go (``_settle_group``:
    the cotangents of several arguments usually share most of their arithmetic) are handed over together."""
    groups = None
    for item in items:
        together = getattr(type(item), "_settle_group", None)
        if together is not None:
            if groups is None:
                groups = {}
            groups.setdefault(together, []).append(item)
    if groups is not None:
        for together, members in groups.items():
            if len(members) > 1:
                together(members)


# ----------------------------------------------------------------------------------------------
# reverse mode (reference core.py:11-108)
# ----------------------------------------------------------------------------------------------
primitive_vjps = {}


def make_vjp(fun, x):
    """Trace ``fun`` at ``x``; return ``(vjp, fun(x))``.  A result that does not depend on ``x``
    (nothing was traced) has the zero cotangent."""
    if (type(x) is tuple and x and getattr(fun, "unpacks_its_tuple", False)
            and all(type(element) in box_type_mappings for element in x)):
        return _make_vjp_by_element(fun, x)
    value, last = trace(VJPNode.new_root(), fun, x)
    if last is None:
        return (lambda g: vspace(x).zeros()), value
    return (lambda g: settle(backward_pass(g, last))), value


def _make_vjp_by_element(fun, xs):
    """``make_vjp`` for the tuple of arguments that several ``argnum`` s select, every element traced from a root
    of its own.  Only for a ``fun`` that declares ``unpacks_its_tuple`` (``wrap_util.unary_to_nary`` sets it on the
    function it builds for several ``argnum`` s: that function does nothing with the tuple but unpack it).  A
    tuple that a caller passes as ONE argument is boxed as a container, as in the reference: user code may hand it
    to a primitive or return a slice of it, which needs the box.

    The reference boxes the tuple itself (autograd/builtins.py:37-96): each element then reaches ``fun`` through a
    ``container_take`` node whose cotangent is scattered back into a tuple of zeros (builtins.py:24-34,
    core.py:185-215).  Here ``fun`` receives a plain tuple of boxes, so those nodes, the sparse cotangents and the
    tuple-level accumulation never exist; what they did to the values is applied once at the end: element ``i`` of
    the result is ``vspace(xs[i]).mut_add(zeros, cotangent of root i)``, which is what gives a cotangent the dtype of
    its argument (a float64 cotangent of a float32 argument comes back float32, unlike with a single ``argnum``) and
    turns a ``-0.0`` into ``0.0``, exactly as the scattered form does."""
    with trace_stack.new_trace() as level:
        roots = [VJPNode.new_root() for _ in xs]
        end_box = fun(tuple(new_box(x, level, root) for x, root in zip(xs, roots)))
        traced = isbox(end_box) and end_box._trace == level
    if not traced:
        warnings.warn("Output seems independent of input.")
        return (lambda g: vspace(xs).zeros()), end_box
    end_node = end_box._node
    position = {root: i for i, root in enumerate(roots)}

    def pull_back(g):
        table = {end_node: (g, False)}
        found = {}
        with collector_paused():
            for node in toposort(end_node):
                cotangent = table.pop(node)[0]
                if node in position:
                    found[position[node]] = cotangent
                    continue
                for parent, share in zip(node.parents, node.vjp(cotangent)):
                    table[parent] = add_outgrads(table.get(parent), share)
        out = []
        for i, x in enumerate(xs):
            space = vspace(x)
            if i not in found:
                out.append(space.zeros())
            elif isbox(found[i]):  # this pull-back is itself being traced: through the primitive
                out.append(space.mut_add(None, found[i]))
            else:
                out.append(space._mut_add(space.zeros(), found[i]))  # (what the primitive would run)
        return settle(tuple(out))

    return pull_back, end_box._value


def make_vjp_and_batched(fun, x):
    """One trace, two pull-backs: ``(vjp, batched_vjp, fun(x))``.  ``batched_vjp(G, n, unstack, stack)`` replays
    the tape once for ``n`` cotangents stacked along axis 0 of ``G`` (see ``batched_backward_pass``); it is
    None when nothing was traced."""
    value, last = trace(VJPNode.new_root(), fun, x)
    if last is None:
        return (lambda g: vspace(x).zeros()), None, value
    return ((lambda g: settle(backward_pass(g, last))),
            (lambda G, n, unstack, stack: settle(batched_backward_pass(G, last, n, unstack, stack))), value)


def backward_pass(g, end_node):
    """Replay the tape from ``end_node`` and return the root's cotangent.

    Nodes come in ``toposort`` order, so a node's cotangent is complete when its turn comes: it is
    taken out of the table, handed to the closure its rule built at trace time (``node.vjp``), and
    what comes back is folded into the parents' entries."""
    table = {end_node: (g, False)}
    cotangent = g
    with collector_paused():
        for node in toposort(end_node):
            cotangent = table.pop(node)[0]
            for parent, share in zip(node.parents, node.vjp(cotangent)):
                table[parent] = add_outgrads(table.get(parent), share)
    return cotangent


def _no_cotangents(g):
    return ()


# ---- one backward pass for a whole batch of cotangents -----------------------------------------
# `jacobian` (reference differential_operators.py:57-73) replays the tape once per element of the
# output, each time with a standard basis vector as the cotangent.  Here the basis vectors are
# stacked along a new leading axis and go through the tape together: rules registered with
# `batch_safe` accept cotangents with that extra axis (the value type's rule table says how, see
# `BatchMode`); any other node's rule is applied to the slices one by one and the results are
# stacked again, so every tape can be replayed this way and the number of kernel launches no longer
# grows with the output size when all its rules are batch-safe.
batch_safe_vjps = set()


def batch_safe(*funs):
    """Declare that the reverse rules of ``funs`` accept cotangents with a leading batch axis while
    ``BatchMode.active`` is set (they raise ``NotBatchable`` for argument forms they do not cover)."""
    batch_safe_vjps.update(funs)


class NotBatchable(Exception):
    """Raised by a batch-safe rule for a call it cannot treat with the batch axis in place."""


class BatchMode:
    """Dynamic state of a batched replay: ``active`` is 1 while a rule runs on stacked cotangents."""

    active = 0


def batched_backward_pass(G, end_node, n, unstack, stack):
    """``backward_pass`` for ``n`` cotangents stacked along axis 0 of ``G``.  ``unstack(value, i)``
    gives the i-th cotangent of a stacked value, ``stack(list)`` puts rule results back together (both
    come from the value type's namespace); raises ``NotBatchable`` when a result is not stackable."""
    table = {end_node: (G, False)}
    cotangent = G
    with collector_paused():
        for node in toposort(end_node):
            cotangent = table.pop(node)[0]
            if not node.parents:
                continue
            shares = None
            if getattr(node, "fun", None) in batch_safe_vjps:
                BatchMode.active = 1
                try:
                    shares = tuple(node.vjp(cotangent))
                except NotBatchable:
                    shares = None
                finally:
                    BatchMode.active = 0
            if shares is None:
                per_slice = [tuple(node.vjp(unstack(cotangent, i))) for i in range(n)]
                shares = tuple(stack([dense(row[k]) for row in per_slice]) for k in range(len(node.parents)))
            for parent, share in zip(node.parents, shares):
                table[parent] = add_outgrads(table.get(parent), share)
    return cotangent


def dense(share):
    """A rule's result as a dense value (sparse scatter objects are added into zeros)."""
    if type(share) in sparse_object_types:
        return sparse_add(vspace(share), None, share)
    return share


class VJPNode(Node):
    """Tape node of reverse mode: its parents and the closure mapping its cotangent to theirs."""

    __slots__ = ["parents", "vjp", "fun"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        maker = primitive_vjps.get(fun)
        if maker is None:
            raise NotImplementedError(_undefined("VJP", fun, parent_argnums))
        self.parents = parents
        self.fun = fun  # which rule table entry made `vjp` (a batched replay asks whether it is batch-safe)
        self.vjp = maker(parent_argnums, value, args, kwargs)

    def initialize_root(self):
        self.parents, self.vjp, self.fun = [], _no_cotangents, None


def defvjp_argnums(fun, vjpmaker):
    """Most general form: ``vjpmaker(argnums, ans, args, kwargs) -> (g -> cotangents, one per argnum)``."""
    primitive_vjps[fun] = vjpmaker


def defvjp_argnum(fun, vjpmaker):
    """``vjpmaker(argnum, ans, args, kwargs) -> (g -> cotangent)``, asked once per traced argument."""

    def for_all(argnums, *call):
        closures = [vjpmaker(n, *call) for n in argnums]
        return lambda g: (c(g) for c in closures)

    defvjp_argnums(fun, for_all)


def translate_vjp(vjpfun, fun, argnum):
    """A per-argument rule as given to ``defvjp`` -> maker; ``None`` stands for a zero cotangent."""
    if vjpfun is None:
        return lambda ans, *args, **kwargs: lambda g: vspace(args[argnum]).zeros()
    if not callable(vjpfun):
        raise _bad_rule("VJP", vjpfun, fun)
    return vjpfun


def defvjp(fun, *vjpmakers, **kwargs):
    """One maker per positional argument: ``maker(ans, *args, **kw) -> (g -> cotangent)``.

    ``argnums=`` names the positions the makers refer to (default 0, 1, ...).  Calls with one or two
    traced arguments, nearly all of them, get closures without a loop."""
    makers = {n: translate_vjp(m, fun, n) for n, m in zip(kwargs.get("argnums", count()), vjpmakers)}

    def undefined(n):
        listed = "argnum 0" if n == 1 else "argnums 0, 1"
        return NotImplementedError(f"VJP of {fun.__name__} wrt {listed} not defined")

    def for_all(argnums, ans, args, kwargs):
        n = len(argnums)
        if n == 1:
            only = makers.get(argnums[0])
            if only is None:
                raise undefined(1)
            closure = only(ans, *args, **kwargs)
            return lambda g: (closure(g),)
        if n == 2:
            first, second = makers.get(argnums[0]), makers.get(argnums[1])
            if first is None or second is None:
                raise undefined(2)
            first, second = first(ans, *args, **kwargs), second(ans, *args, **kwargs)
            return lambda g: (first(g), second(g))
        closures = [makers[k](ans, *args, **kwargs) for k in argnums]
        return lambda g: (c(g) for c in closures)

    defvjp_argnums(fun, for_all)


# ----------------------------------------------------------------------------------------------
# forward mode (reference core.py:114-179)
# ----------------------------------------------------------------------------------------------
primitive_jvps = {}


def make_jvp(fun, x):
    """``jvp(g) -> (fun(x), tangent of fun at x along g)``; tangents are pushed as the trace runs."""

    def jvp(g):
        value, last = trace(JVPNode.new_root(g), fun, x)
        tangent = vspace(value).zeros() if last is None else settle(last.g)
        return value, tangent

    return jvp


class JVPNode(Node):
    """Forward-mode node: holds the tangent of its value, computed when the node is made."""

    __slots__ = ["g"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        rule = primitive_jvps.get(fun)
        if rule is None:
            raise NotImplementedError(_undefined("JVP", fun, parent_argnums))
        self.g = rule(parent_argnums, [p.g for p in parents], value, args, kwargs)

    def initialize_root(self, g):
        self.g = g


def defjvp_argnums(fun, jvpmaker):
    """Most general form: ``jvpmaker(argnums, tangents, ans, args, kwargs) -> tangent``."""
    primitive_jvps[fun] = jvpmaker


def defjvp_argnum(fun, jvpmaker):
    """``jvpmaker(argnum, g, ans, args, kwargs) -> tangent``; the contributions of all traced arguments add up."""

    def for_all(argnums, gs, ans, args, kwargs):
        return sum_outgrads(jvpmaker(n, g, ans, args, kwargs) for n, g in zip(argnums, gs))

    defjvp_argnums(fun, for_all)


def translate_jvp(jvpfun, fun, argnum):
    """A per-argument rule as given to ``defjvp``: a callable, ``None`` (zero tangent) or ``"same"``
    (``fun`` is linear in that argument, so it is applied to the tangent in the argument's place)."""
    if jvpfun is None:
        return lambda g, ans, *args, **kwargs: vspace(ans).zeros()
    if jvpfun == "same" and isinstance(jvpfun, str):
        return lambda g, ans, *args, **kwargs: fun(*subval(args, argnum, g), **kwargs)
    if isinstance(jvpfun, str) or not callable(jvpfun):
        raise _bad_rule("JVP", jvpfun, fun)
    return jvpfun


def defjvp(fun, *jvpfuns, **kwargs):
    """One rule per positional argument: ``rule(g, ans, *args, **kw) -> tangent`` (see ``translate_jvp``)."""
    rules = {n: translate_jvp(r, fun, n) for n, r in zip(kwargs.get("argnums", count()), jvpfuns)}

    def for_all(argnums, gs, ans, args, kwargs):
        return sum_outgrads(rules[n](g, ans, *args, **kwargs) for n, g in zip(argnums, gs))

    defjvp_argnums(fun, for_all)


def def_linear(fun):
    """``fun`` is linear in each positional argument: its tangent is ``fun`` with the tangent put in place."""
    defjvp_argnum(fun, lambda argnum, g, ans, args, kwargs: fun(*subval(args, argnum, g), **kwargs))


# ----------------------------------------------------------------------------------------------
# cotangent accumulation (reference core.py:185-215)
# ----------------------------------------------------------------------------------------------
def add_outgrads(prev_g_flagged, g):
    """Fold one more contribution ``g`` into ``(value, owned)``, or start one (module docstring)."""
    scattered = type(g) in sparse_object_types
    if not prev_g_flagged:
        if scattered:
            return sparse_add(vspace(g), None, g), True
        return g, False
    acc, owned = prev_g_flagged
    vs = vspace(g)
    if scattered:
        if not owned:
            acc = vs.mut_add(None, acc)  # zeros += acc: a buffer of this entry's own
        return sparse_add(vs, acc, g), True
    if owned:
        return vs.mut_add(acc, g), True
    return vs.add(acc, g), True


def sum_outgrads(gs):
    total = None
    for g in gs:
        total = add_outgrads(total, g)
    return total[0]


@primitive
def sparse_add(vs, x_prev, x_new):
    """``x_new`` (a ``SparseObject``) scattered into ``x_prev``, or into zeros when there is none yet."""
    return x_new.mut_add(vs.zeros() if x_prev is None else x_prev)


# ----------------------------------------------------------------------------------------------
# vector spaces (reference core.py:218-315)
# ----------------------------------------------------------------------------------------------
def _required(name):
    def missing(self, *args):
        raise AssertionError(f"{name} is not defined for {self!r}")

    missing.__name__ = name
    return missing


class VSpace:
    """Vector space of a value type: what cotangents of such values look like.

    A subclass provides ``zeros, ones, standard_basis, randn, _inner_prod`` and may override
    ``_add, _mut_add, _scalar_mul, _covector``.  The public operations are primitives, so that a
    backward pass run under the tracer can itself be differentiated.  Two vspaces are equal when
    their types and attributes are.
    """

    __slots__ = []
    mappings = {}  # value type -> callable giving the vspace of a value
    iscomplex = False

    def __init__(self, value):
        pass

    zeros = _required("zeros")
    ones = _required("ones")
    standard_basis = _required("standard_basis")
    randn = _required("randn")
    _inner_prod = _required("_inner_prod")

    # overridable arithmetic, here for value types with Python operators
    def _add(self, x, y):
        return x + y

    def _mut_add(self, x, y):
        x += y
        return x

    def _scalar_mul(self, x, a):
        return x * a

    def _covector(self, x):
        return x

    @primitive
    def add(self, x_prev, x_new):
        return self._add(x_prev, x_new)

    @primitive
    def mut_add(self, x_prev, x_new):
        return self._mut_add(self.zeros() if x_prev is None else x_prev, x_new)

    @primitive
    def scalar_mul(self, x, a):
        return self._scalar_mul(x, a)

    @primitive
    def inner_prod(self, x, y):
        return self._inner_prod(x, y)

    @primitive
    def covector(self, x):
        return self._covector(x)

    def __eq__(self, other):
        return type(self) == type(other) and self.__dict__ == other.__dict__

    __hash__ = None

    def __repr__(self):
        return f"{type(self).__name__}_{self.__dict__}"

    @classmethod
    def register(cls, value_type, vspace_maker=None):
        VSpace.mappings[value_type] = vspace_maker or cls


def vspace(value):
    """The vector space ``value`` lives in (of the value inside, for a box)."""
    maker = VSpace.mappings.get(type(value))
    if maker is not None:
        return maker(value)
    if isbox(value):
        return vspace(getval(value))
    raise TypeError(
        f"Can't find vector space for value {value} of type {type(value)}. "
        f"Valid types are {VSpace.mappings.keys()}"
    )


class SparseObject:
    """A cotangent given as "how to add me into a dense buffer" (scatter form): ``mut_add(buffer)``
    returns the buffer with this contribution added; ``vs`` is the dense buffer's vector space."""

    __slots__ = ["vs", "mut_add"]

    def __init__(self, vs, mut_add):
        self.vs, self.mut_add = vs, mut_add


class SparseBox(Box):
    __slots__ = []


SparseBox.register(SparseObject)
VSpace.register(SparseObject, lambda sparse: sparse.vs)
sparse_object_types = {SparseObject, SparseBox}


# ----------------------------------------------------------------------------------------------
# rules of the accumulation primitives themselves, so that a traced backward pass stays
# differentiable (reference core.py:319-345).  Argument 0 is the vector space: no rule.
# ----------------------------------------------------------------------------------------------
def identity_vjp(argnums, *args):
    return lambda g: g


def identity_jvp(g, *args, **kwargs):
    return g


for _sum in (sparse_add, func(VSpace.add), func(VSpace.mut_add)):
    defvjp(_sum, None, identity_vjp, identity_vjp)
    defjvp(_sum, None, identity_jvp, identity_jvp)

defvjp(
    func(VSpace.scalar_mul),
    None,
    lambda ans, vs, x, a: lambda g: vs.covector(vs.scalar_mul(vs.covector(g), a)),
    lambda ans, vs, x, a: lambda g: vs.inner_prod(g, vs.covector(x)),
)
defvjp(
    func(VSpace.inner_prod),
    None,
    lambda ans, vs, x, y: lambda g: vs.covector(vs.scalar_mul(y, g)),
    lambda ans, vs, x, y: lambda g: vs.covector(vs.scalar_mul(x, g)),
)
defvjp(func(VSpace.covector), None, lambda ans, vs, x: lambda g: vs.covector(g))
for _bilinear in (func(VSpace.scalar_mul), func(VSpace.inner_prod)):
    defjvp(_bilinear, None, "same", "same")
defjvp(func(VSpace.covector), None, "same")


# ----------------------------------------------------------------------------------------------
# The pre-1.2 way of attaching reverse rules, kept as warning shims (reference core.py:347-415):
# a primitive obtained from THIS module, or from the package's top level (autograd/__init__.py:1), carries
# ``defgrad`` / ``defvjp`` / ``defvjp_is_zero`` methods that translate to ``defvjp`` above.
# ``extend.primitive`` is the plain one.
# ----------------------------------------------------------------------------------------------
_OLD_STYLE = ("The {} method is deprecated. See the update guide and tutorial:\n"
              "https://github.com/HIPS/autograd/blob/master/docs/updateguide.md\n"
              "https://github.com/HIPS/autograd/blob/master/docs/tutorial.md")
_plain_primitive = primitive


def _old_style_rules(wrapped):
    """The three legacy registration methods of ``wrapped``; each call re-registers every rule given so far."""
    import warnings

    makers = {}  # argnum -> maker in today's form, or None for a zero cotangent

    def register(method):
        warnings.warn(_OLD_STYLE.format(method))
        positions = sorted(makers)
        defvjp(wrapped, *(makers[n] for n in positions), argnums=positions)

    def defgrad(gradfun, argnum=0):  # already (ans, *args) -> (g -> cotangent)
        makers[argnum] = gradfun
        register("defgrad")

    def defvjp_unstaged(rule, argnum=0):  # rule(g, ans, vs, gvs, *args): everything at once
        makers[argnum] = lambda ans, *args, **kwargs: lambda g: rule(g, ans, vspace(args[argnum]), vspace(g), *args, **kwargs)
        register("defvjp")

    def defvjp_is_zero(argnums=(0,)):
        makers.update((n, None) for n in argnums)
        register("defvjp_is_zero")

    return defgrad, defvjp_unstaged, defvjp_is_zero


def primitive_with_deprecation_warnings(f_raw):
    wrapped = _plain_primitive(f_raw)
    wrapped.defgrad, wrapped.defvjp, wrapped.defvjp_is_zero = _old_style_rules(wrapped)
    return wrapped


primitive = primitive_with_deprecation_warnings  # (shadows the import on purpose, as reference core.py:415 does)
