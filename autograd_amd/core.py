"""Reverse and forward mode on top of the tracer, and the vector-space layer.

Same contract as the reference's autograd/core.py:11-345.  The functions in
this file are the host side of the hot path: ``backward_pass`` replays the tape
and ``add_outgrads`` accumulates cotangents; the arithmetic they trigger lives
in the value type's rules and ``VSpace`` (for device arrays: HIP kernels).

Accumulation protocol (reference autograd/core.py:185-205), kept exactly
because it decides both aliasing and floating-point order: a node's cotangent
is stored as ``(value, mutable)``.  The first dense contribution is kept by
reference and is NOT mutable (it may alias a tape value or another node's
cotangent); the second goes through ``vs.add`` which produces a fresh, mutable
buffer; later ones are added in place with ``vs.mut_add``.  Sparse
contributions (``SparseObject``) are always scattered into a mutable dense
buffer, which is zero-filled on first use or copied from a non-mutable
predecessor.
"""

from functools import reduce
from itertools import count

from .tracer import Box, Node, getval, isbox, primitive, toposort, trace
from .util import func, subval

# ----------------------------------------------------------------------------
# reverse mode
# ----------------------------------------------------------------------------


def make_vjp(fun, x):
    """Trace ``fun`` at ``x``; return ``(vjp, fun(x))`` (reference core.py:11-23)."""
    start_node = VJPNode.new_root()
    end_value, end_node = trace(start_node, fun, x)
    if end_node is None:

        def vjp(g):
            return vspace(x).zeros()

    else:

        def vjp(g):
            return settle(backward_pass(g, end_node))

    return vjp, end_value


def settle(value):
    """A derivative as it is handed to the caller: value types whose arithmetic may be deferred
    (they define ``_settled``) complete it here, inside whatever is timing the evaluation;
    containers are walked, boxes and everything else pass through."""
    t = type(value)
    done = getattr(t, "_settled", None)
    if done is not None:
        return done(value)
    if t is tuple or t is list:
        return t(settle(v) for v in value)
    if t is dict:
        return {k: settle(v) for k, v in value.items()}
    return value


def backward_pass(g, end_node):
    """Replay the tape from ``end_node``; return the root's cotangent.

    One iteration per tape node in ``toposort`` order (reference
    core.py:26-33).  ``node.vjp`` is the closure built at trace time by the
    primitive's rule.
    """
    outgrads = {end_node: (g, False)}
    outgrad = (g, False)
    for node in toposort(end_node):
        outgrad = outgrads.pop(node)
        ingrads = node.vjp(outgrad[0])
        for parent, ingrad in zip(node.parents, ingrads):
            outgrads[parent] = add_outgrads(outgrads.get(parent), ingrad)
    return outgrad[0]


class VJPNode(Node):
    __slots__ = ["parents", "vjp"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        self.parents = parents
        try:
            vjpmaker = primitive_vjps[fun]
        except KeyError:
            fun_name = getattr(fun, "__name__", fun)
            raise NotImplementedError(
                f"VJP of {fun_name} wrt argnums {parent_argnums} not defined"
            ) from None
        self.vjp = vjpmaker(parent_argnums, value, args, kwargs)

    def initialize_root(self):
        self.parents = []
        self.vjp = lambda g: ()


primitive_vjps = {}


def defvjp_argnums(fun, vjpmaker):
    """``vjpmaker(argnums, ans, args, kwargs) -> (g -> tuple of cotangents)``."""
    primitive_vjps[fun] = vjpmaker


def defvjp_argnum(fun, vjpmaker):
    """``vjpmaker(argnum, ans, args, kwargs) -> (g -> cotangent)``."""

    def vjp_argnums(argnums, *args):
        vjps = [vjpmaker(argnum, *args) for argnum in argnums]
        return lambda g: (vjp(g) for vjp in vjps)

    defvjp_argnums(fun, vjp_argnums)


def defvjp(fun, *vjpmakers, **kwargs):
    """One maker per positional argument: ``maker(ans, *args, **kw) -> (g -> cotangent)``.

    ``None`` means "cotangent is zero"; ``argnums=`` selects which positions the
    makers refer to (reference core.py:68-108).
    """
    maker_argnums = kwargs.get("argnums", count())
    makers = {
        argnum: translate_vjp(maker, fun, argnum) for argnum, maker in zip(maker_argnums, vjpmakers)
    }

    def vjp_argnums(argnums, ans, args, kwargs):
        n = len(argnums)
        if n == 1:
            (argnum,) = argnums
            try:
                maker = makers[argnum]
            except KeyError:
                raise NotImplementedError(
                    f"VJP of {fun.__name__} wrt argnum 0 not defined"
                ) from None
            vjp = maker(ans, *args, **kwargs)
            return lambda g: (vjp(g),)
        if n == 2:
            a0, a1 = argnums
            try:
                maker0, maker1 = makers[a0], makers[a1]
            except KeyError:
                raise NotImplementedError(
                    f"VJP of {fun.__name__} wrt argnums 0, 1 not defined"
                ) from None
            vjp0 = maker0(ans, *args, **kwargs)
            vjp1 = maker1(ans, *args, **kwargs)
            return lambda g: (vjp0(g), vjp1(g))
        vjps = [makers[argnum](ans, *args, **kwargs) for argnum in argnums]
        return lambda g: (vjp(g) for vjp in vjps)

    defvjp_argnums(fun, vjp_argnums)


def translate_vjp(vjpfun, fun, argnum):
    if vjpfun is None:
        return lambda ans, *args, **kwargs: lambda g: vspace(args[argnum]).zeros()
    if callable(vjpfun):
        return vjpfun
    raise TypeError(f"Bad VJP '{vjpfun}' for '{fun.__name__}'")


# ----------------------------------------------------------------------------
# forward mode
# ----------------------------------------------------------------------------


def make_jvp(fun, x):
    """Return ``jvp(g) -> (fun(x), tangent)`` (reference core.py:114-123)."""

    def jvp(g):
        start_node = JVPNode.new_root(g)
        end_value, end_node = trace(start_node, fun, x)
        if end_node is None:
            return end_value, vspace(end_value).zeros()
        return end_value, settle(end_node.g)

    return jvp


class JVPNode(Node):
    __slots__ = ["g"]

    def __init__(self, value, fun, args, kwargs, parent_argnums, parents):
        parent_gs = [parent.g for parent in parents]
        try:
            jvpmaker = primitive_jvps[fun]
        except KeyError:
            name = getattr(fun, "__name__", fun)
            raise NotImplementedError(
                f"JVP of {name} wrt argnums {parent_argnums} not defined"
            ) from None
        self.g = jvpmaker(parent_argnums, parent_gs, value, args, kwargs)

    def initialize_root(self, g):
        self.g = g


primitive_jvps = {}


def defjvp_argnums(fun, jvpmaker):
    """``jvpmaker(argnums, gs, ans, args, kwargs) -> tangent``."""
    primitive_jvps[fun] = jvpmaker


def defjvp_argnum(fun, jvpmaker):
    """``jvpmaker(argnum, g, ans, args, kwargs) -> tangent`` summed over boxed args."""

    def jvp_argnums(argnums, gs, ans, args, kwargs):
        return sum_outgrads(jvpmaker(argnum, g, ans, args, kwargs) for argnum, g in zip(argnums, gs))

    defjvp_argnums(fun, jvp_argnums)


def defjvp(fun, *jvpfuns, **kwargs):
    """One rule per positional argument: ``rule(g, ans, *args, **kw) -> tangent``.

    ``"same"`` applies ``fun`` itself to the tangent (linear in that argument);
    ``None`` is a zero tangent (reference core.py:156-174).
    """
    rule_argnums = kwargs.get("argnums", count())
    rules = {argnum: translate_jvp(rule, fun, argnum) for argnum, rule in zip(rule_argnums, jvpfuns)}

    def jvp_argnums(argnums, gs, ans, args, kwargs):
        return sum_outgrads(rules[argnum](g, ans, *args, **kwargs) for argnum, g in zip(argnums, gs))

    defjvp_argnums(fun, jvp_argnums)


def translate_jvp(jvpfun, fun, argnum):
    if jvpfun is None:
        return lambda g, ans, *a, **k: vspace(ans).zeros()
    if isinstance(jvpfun, str):
        if jvpfun == "same":
            return lambda g, ans, *args, **kwargs: fun(*subval(args, argnum, g), **kwargs)
        raise TypeError(f"Bad JVP '{jvpfun}' for '{fun.__name__}'")
    if callable(jvpfun):
        return jvpfun
    raise TypeError(f"Bad JVP '{jvpfun}' for '{fun.__name__}'")


def def_linear(fun):
    """Declare ``fun`` linear in every positional argument (reference core.py:177-179)."""
    defjvp_argnum(fun, lambda argnum, g, ans, args, kwargs: fun(*subval(args, argnum, g), **kwargs))


# ----------------------------------------------------------------------------
# cotangent accumulation and vector spaces
# ----------------------------------------------------------------------------


def add_outgrads(prev_g_flagged, g):
    """Fold one more contribution ``g`` into ``(value, mutable)`` (see module docstring)."""
    sparse = type(g) in sparse_object_types
    if prev_g_flagged:
        vs = vspace(g)
        prev_g, mutable = prev_g_flagged
        if mutable:
            if sparse:
                return sparse_add(vs, prev_g, g), True
            return vs.mut_add(prev_g, g), True
        if sparse:
            prev_g_mutable = vs.mut_add(None, prev_g)
            return sparse_add(vs, prev_g_mutable, g), True
        return vs.add(prev_g, g), True
    if sparse:
        return sparse_add(vspace(g), None, g), True
    return g, False


def sum_outgrads(gs):
    return reduce(add_outgrads, gs, None)[0]


@primitive
def sparse_add(vs, x_prev, x_new):
    x_prev = x_prev if x_prev is not None else vs.zeros()
    return x_new.mut_add(x_prev)


class VSpace:
    """Vector space of a value type: what cotangents of such values look like.

    A subclass provides ``zeros, ones, standard_basis, randn, _inner_prod`` and
    may override ``_add, _mut_add, _scalar_mul, _covector`` (reference
    core.py:218-286).  Two vspaces are equal when type and attributes are.
    """

    __slots__ = []
    mappings = {}
    iscomplex = False

    def __init__(self, value):
        pass

    def zeros(self):
        raise AssertionError(repr(self))

    def ones(self):
        raise AssertionError(repr(self))

    def standard_basis(self):
        raise AssertionError(repr(self))

    def randn(self):
        raise AssertionError(repr(self))

    @primitive
    def mut_add(self, x_prev, x_new):
        x_prev = x_prev if x_prev is not None else self.zeros()
        return self._mut_add(x_prev, x_new)

    @primitive
    def add(self, x_prev, x_new):
        return self._add(x_prev, x_new)

    @primitive
    def scalar_mul(self, x, a):
        return self._scalar_mul(x, a)

    @primitive
    def inner_prod(self, x, y):
        return self._inner_prod(x, y)

    @primitive
    def covector(self, x):
        return self._covector(x)

    def _add(self, x, y):
        return x + y

    def _mut_add(self, x, y):
        x += y
        return x

    def _scalar_mul(self, x, a):
        return x * a

    def _inner_prod(self, x, y):
        raise AssertionError(repr(self))

    def _covector(self, x):
        return x

    def __eq__(self, other):
        return type(self) == type(other) and self.__dict__ == other.__dict__

    __hash__ = None

    def __repr__(self):
        return f"{type(self).__name__}_{self.__dict__}"

    @classmethod
    def register(cls, value_type, vspace_maker=None):
        VSpace.mappings[value_type] = vspace_maker if vspace_maker else cls


def vspace(value):
    try:
        return VSpace.mappings[type(value)](value)
    except KeyError:
        if isbox(value):
            return vspace(getval(value))
        raise TypeError(
            f"Can't find vector space for value {value} of type {type(value)}. "
            f"Valid types are {VSpace.mappings.keys()}"
        ) from None


class SparseBox(Box):
    __slots__ = []


class SparseObject:
    """A cotangent given as "how to add me into a dense buffer" (scatter form)."""

    __slots__ = ["vs", "mut_add"]

    def __init__(self, vs, mut_add):
        self.vs = vs
        self.mut_add = mut_add


VSpace.register(SparseObject, lambda x: x.vs)
SparseBox.register(SparseObject)
sparse_object_types = {SparseObject, SparseBox}

# ----------------------------------------------------------------------------
# rules for the accumulation primitives themselves, so that a traced backward
# pass stays differentiable (reference core.py:319-345)
# ----------------------------------------------------------------------------


def identity_vjp(argnums, *args):
    return lambda g: g


defvjp(sparse_add, None, identity_vjp, identity_vjp)
defvjp(func(VSpace.add), None, identity_vjp, identity_vjp)
defvjp(func(VSpace.mut_add), None, identity_vjp, identity_vjp)
defvjp(
    func(VSpace.inner_prod),
    None,
    lambda ans, vs, x, y: lambda g: vs.covector(vs.scalar_mul(y, g)),
    lambda ans, vs, x, y: lambda g: vs.covector(vs.scalar_mul(x, g)),
)
defvjp(func(VSpace.covector), None, lambda ans, vs, x: lambda g: vs.covector(g))
defvjp(
    func(VSpace.scalar_mul),
    None,
    lambda ans, vs, x, a: lambda g: vs.covector(vs.scalar_mul(vs.covector(g), a)),
    lambda ans, vs, x, a: lambda g: vs.inner_prod(g, vs.covector(x)),
)


def identity_jvp(g, *args, **kwargs):
    return g


defjvp(sparse_add, None, identity_jvp, identity_jvp)
defjvp(func(VSpace.mut_add), None, identity_jvp, identity_jvp)
defjvp(func(VSpace.add), None, identity_jvp, identity_jvp)
defjvp(func(VSpace.scalar_mul), None, "same", "same")
defjvp(func(VSpace.inner_prod), None, "same", "same")
defjvp(func(VSpace.covector), None, "same")
