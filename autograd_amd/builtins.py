"""Differentiable tuples, lists and dicts.

Contract of the reference's autograd/builtins.py:24-286 (same names and behaviour): containers are
boxed (``SequenceBox``, ``DictBox``); indexing a boxed container is the primitive
``container_take``, whose cotangent is the scatter-form object built by ``container_untake``;
container vector spaces apply the leaves' vector spaces across the structure.  Pure host-side
bookkeeping: the leaves do the arithmetic.
"""

from .extend import Box, SparseObject, VSpace, defjvp, defjvp_argnum, defvjp, defvjp_argnum, notrace_primitive, primitive
from .extend import vspace
from .util import subvals

# the Python builtins this module shadows with traceable versions
isinstance_, type_, tuple_, list_, dict_ = isinstance, type, tuple, list, dict

# type queries see through boxes and are never traced (builtins.py:18-22)
isinstance = notrace_primitive(isinstance_)
type = notrace_primitive(type_)


# ---- taking an element out of a container, and its cotangent (builtins.py:24-34, 99-109) ---------
@primitive
def container_take(A, idx, space=None):
    """``A[idx]``.  ``space``: None, or a callable giving ``vspace(A)`` (boxes pass one that computes it once for all
    the items taken from the same container, see ``_ContainerBox.__getitem__``); the value does not depend on it."""
    return A[idx]


@primitive
def container_untake(x, idx, vs):
    """Cotangent of ``container_take``: a zero container with ``x`` added at ``idx``, in scatter form.

    ``idx`` is a key / position, or a slice of a sequence (then ``x`` is the matching run of
    elements).  The addition happens leaf by leaf with the leaf vspaces' ``_mut_add``; the container
    itself is rebuilt with the entry replaced."""
    leaf_spaces = vs.shape[idx]
    if isinstance_(idx, slice):
        merged = lambda old: [s._mut_add(o, new) for s, o, new in zip(leaf_spaces, old, x)]  # noqa: E731
    else:
        merged = lambda old: leaf_spaces._mut_add(old, x)  # noqa: E731
    return SparseObject(vs, lambda A: vs._subval(A, idx, merged(A[idx])))


defvjp(container_take,
       lambda ans, A, idx, space=None: lambda g: container_untake(g, idx, vspace(A) if space is None else space()))
defvjp(container_untake, lambda ans, x, idx, _: lambda g: container_take(g, idx))
for _linear in (container_take, container_untake):
    defjvp(_linear, "same")


# ---- boxes (builtins.py:37-96) -------------------------------------------------------------------
class _SpaceOnce:
    """``vspace(value)``, computed at the first call: the cotangent rules of all the items taken from one container
    need the container's vector space, which is as large as the container."""

    __slots__ = ("value", "space")

    def __init__(self, value):
        self.value, self.space = value, None

    def __call__(self):
        if self.space is None:
            self.space, self.value = vspace(self.value), None
        return self.space


_SPACE = object()  # key of the shared `_SpaceOnce` among a box's taken items (no index compares equal to it)


class _ContainerBox(Box):
    """What tuples, lists and dicts share when boxed: traced item access, untraced size and membership."""

    __slots__ = ["_taken"]

    def __getitem__(self, idx):
        """Traced item access (builtins.py:37-40).  An item taken before is handed out again as the same box, so a
        loop that reads ``params["W"]`` at every step leaves one ``container_take`` node on the tape instead of one
        per step: the uses then share that node the way they would had the program kept the item in a variable,
        and its cotangents are accumulated there (core.py:185-205) before ONE scattered add into the container."""
        try:
            taken = self._taken
        except AttributeError:
            taken = self._taken = {_SPACE: _SpaceOnce(self._value)}
        try:
            return taken[idx]
        except KeyError:
            item = taken[idx] = container_take(self, idx, space=taken[_SPACE])
            return item
        except TypeError:  # an index that cannot be a key (a slice)
            return container_take(self, idx, space=taken[_SPACE])

    def __len__(self):
        return len(self._value)

    def __contains__(self, item):
        return item in self._value


class SequenceBox(_ContainerBox):
    __slots__ = []

    def __add__(self, other):
        return sequence_extend_right(self, *other)

    def __radd__(self, other):
        return sequence_extend_left(self, *other)

    def index(self, item):
        return self._value.index(item)


class DictBox(_ContainerBox):
    """Keys are plain values; every way of reaching a value goes through the traced item access."""

    __slots__ = []

    def __iter__(self):
        return iter(self._value)

    iterkeys = __iter__

    def itervalues(self):
        return (self[key] for key in self._value)

    def iteritems(self):
        return ((key, self[key]) for key in self._value)

    def keys(self):
        return list_(self._value)

    def values(self):
        return list_(self.itervalues())

    def items(self):
        return list_(self.iteritems())

    def get(self, k, d=None):
        return self[k] if k in self._value else d


for _seq in (tuple_, list_):
    SequenceBox.register(_seq)
DictBox.register(dict_)


# ---- building containers out of (possibly boxed) elements (builtins.py:112-195) -------------------
@primitive
def sequence_extend_right(seq, *elts):
    return seq + type_(seq)(elts)


@primitive
def sequence_extend_left(seq, *elts):
    return type_(seq)(elts) + seq


@primitive
def make_sequence(seq_type, *args):
    return seq_type(args)


@primitive
def _make_dict(keys, vals):
    return dict_(zip(keys, vals))


def _cotangent_of_extend_right(argnum, ans, args, kwargs):
    # argument 0 is the sequence (the head of the result), argument k > 0 its k-th appended element
    head = len(args[0])
    if argnum == 0:
        return lambda g: g[:head]
    return lambda g: g[head + argnum - 1]


def _cotangent_of_extend_left(argnum, ans, args, kwargs):
    # the new elements come first, the sequence (argument 0) is the tail
    n_new = len(args) - 1
    if argnum == 0:
        return lambda g: g[n_new:]
    return lambda g: g[argnum - 1]


defvjp_argnum(sequence_extend_right, _cotangent_of_extend_right)
defvjp_argnum(sequence_extend_left, _cotangent_of_extend_left)
defvjp_argnum(make_sequence, lambda argnum, *args: lambda g: g[argnum - 1])
defjvp_argnum(make_sequence, lambda argnum, g, ans, args, kwargs: container_untake(g, argnum - 1, vspace(ans)))
defvjp(_make_dict, lambda ans, keys, vals: lambda g: list(g[key] for key in keys), argnums=(1,))


def _looks_like(builtin):
    """Metaclass making ``isinstance(x, traced_type)`` answer for the builtin it stands in for."""

    class Meta(type_(builtin)):
        def __instancecheck__(cls, instance):
            return isinstance_(instance, builtin)

    return Meta


class tuple(tuple_, metaclass=_looks_like(tuple_)):
    """``tuple(xs)`` that keeps boxed elements traceable."""

    def __new__(cls, xs):
        return make_sequence(tuple_, *xs)


class list(list_, metaclass=_looks_like(list_)):
    """``list(xs)`` that keeps boxed elements traceable."""

    def __new__(cls, xs):
        return make_sequence(list_, *xs)


class dict(dict_, metaclass=_looks_like(dict_)):
    """``dict(...)`` that keeps boxed values traceable."""

    def __new__(cls, *args, **kwargs):
        plain = dict_(*args, **kwargs)
        return _make_dict(plain.keys(), list(plain.values())) if plain else plain


# ---- vector spaces (builtins.py:198-286) ----------------------------------------------------------
class ContainerVSpace(VSpace):
    """Vspace of a container: ``self.shape`` is the same container holding the leaves' vspaces.

    Subclasses say how to walk and rebuild their kind of container: ``_values``, ``_kv_pairs``,
    ``_map(f, *containers)`` (``f`` gets the leaf vspace first) and ``_subval(xs, key, x)``."""

    def __init__(self, value):
        self.shape = value  # _map walks self.shape: first the values themselves, then their vspaces
        self.shape = self._map(vspace)

    def _leafwise(self, method, *containers, extra=()):
        return self._map(lambda leaf_vs, *leaves: getattr(leaf_vs, method)(*leaves, *extra), *containers)

    def _total(self, per_leaf):
        return sum(self._values(per_leaf))

    @property
    def size(self):
        return self._total(self._map(lambda leaf_vs: leaf_vs.size))

    def zeros(self):
        return self._leafwise("zeros")

    def ones(self):
        return self._leafwise("ones")

    def randn(self):
        return self._leafwise("randn")

    def standard_basis(self):
        origin = self.zeros()
        for key, leaf_vs in self._kv_pairs(self.shape):
            for unit in leaf_vs.standard_basis():
                yield self._subval(origin, key, unit)

    def _add(self, xs, ys):
        return self._leafwise("_add", xs, ys)

    def _mut_add(self, xs, ys):
        return self._leafwise("_mut_add", xs, ys)

    def _scalar_mul(self, xs, a):
        return self._leafwise("_scalar_mul", xs, extra=(a,))

    def _covector(self, xs):
        return self._leafwise("_covector", xs)

    def _inner_prod(self, xs, ys):
        return self._total(self._leafwise("_inner_prod", xs, ys))


class SequenceVSpace(ContainerVSpace):
    seq_type = None  # set by the concrete classes

    def _values(self, x):
        return x

    def _kv_pairs(self, x):
        return enumerate(x)

    def _build(self, items):
        return self.seq_type(items)

    def _map(self, f, *args):
        return self._build(map(f, self.shape, *args))

    def _subval(self, xs, idx, x):
        return self._build(subvals(xs, [(idx, x)]))


class ListVSpace(SequenceVSpace):
    seq_type = list_


class TupleVSpace(SequenceVSpace):
    seq_type = tuple_


class NamedTupleVSpace(SequenceVSpace):
    """For namedtuple types (a subclass sets ``seq_type``): built from positional fields."""

    def _build(self, items):
        return self.seq_type(*items)


class DictVSpace(ContainerVSpace):
    def _values(self, x):
        return x.values()

    def _kv_pairs(self, x):
        return x.items()

    def _map(self, f, *args):
        return {key: f(leaf_vs, *(x[key] for x in args)) for key, leaf_vs in self.shape.items()}

    def _subval(self, xs, idx, x):
        out = dict_(xs)
        out[idx] = x
        return out


ListVSpace.register(list_)
TupleVSpace.register(tuple_)
DictVSpace.register(dict_)
