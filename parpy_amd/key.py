"""Cache keys (python/parpy/key.py:3-37 of the reference)."""
import hashlib


def _generate_function_key(code, opts):
    s = f"{code}+{opts.includes}+{opts.libs}+{opts.extra_flags}"
    h = hashlib.new("sha256")
    h.update(s.encode("utf-8"))
    return h.hexdigest()


def _print_argument_key(arg):
    from .buffer import Buffer
    if isinstance(arg, dict):
        s = [f"{k}: {_print_argument_key(v)}" for k, v in sorted(arg.items())]
        return "{" + ", ".join(s) + "}"
    if isinstance(arg, Buffer):
        if len(arg.shape) == 0:
            v = arg.numpy()
            return f"{v};{v.dtype}"
        shape_strs = [f"{s}" for s in arg.shape]
        return f"[{','.join(shape_strs)};{arg.dtype}]"
    return f"{arg!r}"


def _print_arguments_key(args):
    return "-".join(_print_argument_key(arg) for arg in args)


_ast_keys = {}


def _ast_key(ir_ast):
    """Printed form of a parsed function; it never changes after parsing, so it is printed once."""
    k = _ast_keys.get(id(ir_ast))
    if k is None or k[0] is not ir_ast:
        from .compiler import print_ast
        k = _ast_keys[id(ir_ast)] = (ir_ast, print_ast(ir_ast))
    return k[1]


def _generate_fast_cache_key(ir_ast, args, opts):
    extra = [getattr(opts, n, None) for n in ("opt_vectorize", "opt_lds_rows", "opt_reg_cache",
                                              "opt_hoist_invariant", "opt_narrow_index", "opt_mfma_sddmm",
                                              "opt_unswitch", "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_noalias_scopes", "assume_aligned", "reg_budget")]
    # a tuple: the (long) printed function keeps its cached hash from one call to the next
    return (_ast_key(ir_ast), _print_arguments_key(args), str(opts), tuple(extra))
