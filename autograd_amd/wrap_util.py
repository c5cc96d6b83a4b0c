"""Argument-number plumbing for the differential operators.

Counterpart of the reference's autograd/wrap_util.py:6-52: ``unary_to_nary``
turns an operator defined on one-argument functions (``op(fun, x)``) into the
user-facing ``op(fun, argnum=0)(*args, **kwargs)`` form, where ``argnum`` may be
an int or a tuple/list of ints (then the differentiated value is the tuple of
those arguments).
"""

from contextlib import suppress

from .util import collector_paused, subvals

__all__ = ["unary_to_nary", "wraps", "wrap_nary_f", "get_name", "get_doc"]


def get_name(f):
    return getattr(f, "__name__", "[unknown name]")


def get_doc(f):
    return getattr(f, "__doc__", "")


def wraps(fun, namestr="{fun}", docstr="{doc}", **fmt):
    """Decorator copying a (formatted) name and docstring from ``fun``."""

    def decorate(f):
        if namestr == "{fun}" and docstr == "{doc}":  # a plain copy (made on every call of a differential operator)
            try:
                f.__name__, f.__doc__ = get_name(fun), get_doc(fun)
            except AttributeError:
                pass
            return f
        with suppress(AttributeError, KeyError, ValueError):
            f.__name__ = namestr.format(fun=get_name(fun), **fmt)
            f.__doc__ = docstr.format(fun=get_name(fun), doc=get_doc(fun), **fmt)
        return f

    return decorate


def wrap_nary_f(fun, op, argnum):
    name = "{op}_of_{fun}_wrt_argnum_{argnum}"
    doc = (
        "    {op} of function {fun} with respect to argument number {argnum}. Takes the\n"
        "    same arguments as {fun} but returns the {op}.\n    "
    )
    return wraps(fun, name, doc, op=get_name(op), argnum=argnum)


def unary_to_nary(unary_operator):
    @wraps(unary_operator)
    def nary_operator(fun, argnum=0, *op_args, **op_kwargs):
        assert type(argnum) in (int, tuple, list), argnum
        single = isinstance(argnum, int)

        @wrap_nary_f(fun, unary_operator, argnum)
        def nary_f(*args, **kwargs):
            @wraps(fun)
            def unary_f(x):
                pairs = [(argnum, x)] if single else zip(argnum, x)
                return fun(*subvals(args, pairs), **kwargs)

            unary_f.unpacks_its_tuple = not single  # (lets make_vjp trace the picked arguments one by one)
            x0 = args[argnum] if single else tuple(args[i] for i in argnum)
            with collector_paused():  # see util.collector_paused: tapes hold no cycles
                return unary_operator(unary_f, x0, *op_args, **op_kwargs)

        return nary_f

    return nary_operator
