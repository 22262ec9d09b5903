"""Cache keys (python/parpy/key.py:3-37 of the reference).

Two keys: the name of a code object on disk is a digest of the generated code and the flags it is built with; the
in-memory key of a specialisation is the parsed function, a description of the arguments (shapes and element types
of arrays, values of scalars) and the settings of the options object.
"""
import hashlib


def _generate_function_key(code, opts):
    h = hashlib.sha256()
    for part in (code, opts.includes, opts.libs, opts.extra_flags):
        h.update(str(part).encode("utf-8"))
        h.update(b"\x00")
    return h.hexdigest()


def _describe_argument(arg):
    """Hashable description of what a specialisation depends on in one argument."""
    from .buffer import Buffer
    if isinstance(arg, dict):
        return tuple((k, _describe_argument(arg[k])) for k in sorted(arg))
    if isinstance(arg, Buffer):
        if arg.shape == ():
            v = arg.numpy()
            return ("scalar", str(v.dtype), v.item())
        return ("array", arg.shape, str(arg.dtype))
    return (type(arg).__name__, arg)


_printed = {}


def _ast_key(ir_ast):
    """Printed form of a parsed function; it never changes after parsing, so it is printed once."""
    hit = _printed.get(id(ir_ast))
    if hit is None or hit[0] is not ir_ast:
        from .compiler import print_ast
        hit = _printed[id(ir_ast)] = (ir_ast, print_ast(ir_ast))
    return hit[1]


def _generate_fast_cache_key(ir_ast, args, opts):
    # a tuple: the (long) printed function keeps its cached hash from one call to the next
    return (_ast_key(ir_ast), tuple(_describe_argument(a) for a in args), opts._fast_key())
