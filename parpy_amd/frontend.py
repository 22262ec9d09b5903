"""Python `ast` -> S-expression serialiser for the C++ compiler core.

The reference walks CPython's `ast` nodes from Rust through pyo3
(src/py/from_py.rs:332-720).  The C++ core has no CPython dependency, so this
module performs that walk in Python and hands over a text form; everything
after it (symbol binding, label association, call inlining, specialisation,
lowering, code generation) happens in C++.

What is accepted is what the reference accepts: `for` over `range` with 1-3
arguments and a literal step, `while`, `if`, single-target assignment and
augmented assignment, `with parpy.gpu:`, `parpy.label("x")` statements,
statement calls to other jitted functions, `return expr`; expressions made
of names, literals, unary / binary / boolean operators, single comparisons,
conditional expressions, subscripts with step-free slices, tuples and calls
to the operators of `parpy_amd.operators`.  Operators are recognised the way
the reference does it (src/py/from_py.rs:148-218): by *evaluating* the name in
the decorated function's globals/locals and comparing the object with the
members of the operators module, so any import alias works.

Grammar (every node carries its source span as `@l0:c0:l1:c1`):

  (fun "name" @i (params (p "x" TYPE|none @i) ...) (body S ...))
  S ::= (for @i "v" LO HI STEP (body S ...)) | (while @i C (body ...))
      | (if @i C (then ...) (else ...)) | (assign @i DST E) | (withgpu @i (body ...))
      | (callstmt @i "f" E ...) | (label @i "l") | (return @i E)
  E ::= (var @i "x") | (int @i n) | (float @i x) | (bool @i true|false) | (str @i "s")
      | (unop @i OP E) | (binop @i OP E E) | (ifexp @i C A B)
      | (sub @i E IDX) | (slice @i LO|none HI|none) | (tuple @i E ...)
      | (builtin @i NAME AXIS|none E ...) | (call @i "f" E ...)
"""
import ast as pyast
import builtins
import math

from . import operators as _ops
from . import types as _types
from .options import ElemSize

_UNOPS = {pyast.USub: "sub", pyast.Not: "not", pyast.Invert: "bitneg"}
_BINOPS = {
    pyast.Add: "add", pyast.Sub: "sub", pyast.Mult: "mul", pyast.Div: "div",
    pyast.FloorDiv: "floordiv", pyast.Mod: "rem", pyast.Pow: "pow",
    pyast.BitAnd: "bitand", pyast.BitOr: "bitor", pyast.BitXor: "bitxor",
    pyast.LShift: "shl", pyast.RShift: "shr", pyast.Eq: "eq", pyast.NotEq: "neq",
    pyast.LtE: "leq", pyast.GtE: "geq", pyast.Lt: "lt", pyast.Gt: "gt",
}
_BOOLOPS = {pyast.And: "and", pyast.Or: "or"}

_BUILTIN_NAMES = ["exp", "inf", "log", "min", "max", "abs", "cos", "sin", "sqrt",
                  "tanh", "atan2", "sum", "prod", "label", "gpu"]
_CONVERTS = {"float16": "f16", "float32": "f32", "float64": "f64", "int8": "i8",
             "int16": "i16", "int32": "i32", "int64": "i64", "uint8": "u8",
             "uint16": "u16", "uint32": "u32", "uint64": "u64"}


class FrontendError(RuntimeError):
    pass


def _quote(s):
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"').replace("\n", "\\n") + '"'


def _fmt_float(v):
    if math.isinf(v):
        return "inf" if v > 0 else "-inf"
    if math.isnan(v):
        return "nan"
    return repr(float(v))


class _Converter:
    def __init__(self, filepath, line_ofs, col_ofs, tops, globs, locs):
        self.filepath = filepath
        self.line_ofs = line_ofs
        self.col_ofs = col_ofs
        self.tops = tops
        self.globs = globs
        self.locs = locs

    # -- helpers ----------------------------------------------------------
    def info(self, node):
        l0 = getattr(node, "lineno", 0) + self.line_ofs
        l1 = (getattr(node, "end_lineno", None) or getattr(node, "lineno", 0)) + self.line_ofs
        c0 = getattr(node, "col_offset", 0) + self.col_ofs
        c1 = (getattr(node, "end_col_offset", None) or 0) + self.col_ofs
        return f"@{l0}:{c0}:{l1}:{c1}"

    def err(self, node, msg):
        """Report `msg` with the source lines of `node`, the way the reference does
        (src/utils/info.rs:90-121): 'On line(s) a-b of file f:' followed by the lines."""
        import linecache
        l0 = getattr(node, "lineno", 0) + self.line_ofs
        l1 = (getattr(node, "end_lineno", None) or getattr(node, "lineno", 0)) + self.line_ofs
        where = f"line {l0}" if l0 == l1 else f"lines {l0}-{l1}"
        lines = [linecache.getline(self.filepath, n).rstrip("\n") for n in range(l0, l1 + 1)]
        excerpt = "\n".join(f"{n:4d} | {t}" for n, t in zip(range(l0, l1 + 1), lines) if t)
        raise FrontendError(f"{msg}\n\nOn {where} of file {self.filepath}:\n{excerpt}")

    def eval_name(self, src):
        return eval(src, self.globs, self.locs)

    def lookup_builtin(self, node):
        """Name of the operator `node` evaluates to, or None (src/py/from_py.rs:148-218)."""
        try:
            obj = self.eval_name(pyast.unparse(node))
        except Exception:
            return None
        if isinstance(obj, float):
            # `inf` is a plain float: identify it by value like the reference's `==` does.
            return "inf" if math.isinf(obj) and obj > 0 else None
        for n in _BUILTIN_NAMES:
            if obj is getattr(_ops, n):
                return n
        for n, tag in _CONVERTS.items():
            if obj is getattr(_ops, n):
                return "convert_" + tag
        return None

    # -- expressions ------------------------------------------------------
    def expr(self, e):
        i = self.info(e)
        if isinstance(e, pyast.Name):
            b = self.lookup_builtin(e)
            if b is not None:
                return f"(builtin {i} {b} none)"
            return f"(var {i} {_quote(e.id)})"
        if isinstance(e, pyast.Constant):
            v = e.value
            if isinstance(v, bool):
                return f"(bool {i} {'true' if v else 'false'})"
            if isinstance(v, int):
                return f"(int {i} {v})"
            if isinstance(v, float):
                return f"(float {i} {_fmt_float(v)})"
            if isinstance(v, str):
                return f"(str {i} {_quote(v)})"
            self.err(e, f"Unsupported literal value {v!r}")
        if isinstance(e, pyast.UnaryOp):
            op = _UNOPS.get(type(e.op))
            if op is None:
                self.err(e, f"Unsupported unary expression {pyast.dump(e.op)}")
            return f"(unop {i} {op} {self.expr(e.operand)})"
        if isinstance(e, pyast.BinOp):
            op = _BINOPS.get(type(e.op))
            if op is None:
                self.err(e, f"Unsupported binary operation: {pyast.dump(e.op)}")
            return f"(binop {i} {op} {self.expr(e.left)} {self.expr(e.right)})"
        if isinstance(e, pyast.BoolOp):
            op = _BOOLOPS[type(e.op)]
            acc = self.expr(e.values[0])
            for v in e.values[1:]:
                acc = f"(binop {i} {op} {acc} {self.expr(v)})"
            return acc
        if isinstance(e, pyast.Compare):
            if len(e.ops) != 1 or len(e.comparators) != 1:
                self.err(e, "Sequences of comparisons are not supported")
            op = _BINOPS.get(type(e.ops[0]))
            if op is None:
                self.err(e, f"Unsupported binary operation: {pyast.dump(e.ops[0])}")
            return f"(binop {i} {op} {self.expr(e.left)} {self.expr(e.comparators[0])})"
        if isinstance(e, pyast.IfExp):
            return f"(ifexp {i} {self.expr(e.test)} {self.expr(e.body)} {self.expr(e.orelse)})"
        if isinstance(e, pyast.Subscript):
            return f"(sub {i} {self.expr(e.value)} {self.expr(e.slice)})"
        if isinstance(e, pyast.Slice):
            if e.step is not None:
                self.err(e, "Slices with a step size are not supported")
            lo = self.expr(e.lower) if e.lower is not None else "none"
            hi = self.expr(e.upper) if e.upper is not None else "none"
            return f"(slice {i} {lo} {hi})"
        if isinstance(e, pyast.Attribute):
            b = self.lookup_builtin(e)
            if b is None:
                self.err(e, f"Unknown built-in operator {pyast.unparse(e)}")
            return f"(builtin {i} {b} none)"
        if isinstance(e, pyast.Tuple):
            return f"(tuple {i} {' '.join(self.expr(x) for x in e.elts)})"
        if isinstance(e, pyast.Call):
            return self.call(e, i)
        self.err(e, f"Unsupported expression: {pyast.unparse(e)}")

    def call(self, e, i):
        axis = None
        for kw in e.keywords:
            if kw.arg != "axis" or axis is not None:
                self.err(e, f"Unsupported keyword argument in call: {kw.arg}")
            v = kw.value
            if isinstance(v, pyast.Constant) and isinstance(v.value, int) and not isinstance(v.value, bool):
                axis = v.value
            elif isinstance(v, pyast.UnaryOp) and isinstance(v.op, pyast.USub) and \
                    isinstance(v.operand, pyast.Constant) and isinstance(v.operand.value, int):
                axis = -v.operand.value
            else:
                self.err(e, "Expected integer literal value for 'axis' keyword argument")
        args = " ".join(self.expr(a) for a in e.args)
        b = self.lookup_builtin(e.func) if isinstance(e.func, (pyast.Name, pyast.Attribute)) else None
        if b is not None:
            ax = "none" if axis is None else str(axis)
            return f"(builtin {i} {b} {ax}{' ' if args else ''}{args})"
        if isinstance(e.func, pyast.Name):
            if e.func.id in self.tops:
                if axis is not None:
                    self.err(e, "Unsupported keyword argument in call: axis")
                return f"(call {i} {_quote(e.func.id)}{' ' if args else ''}{args})"
            self.err(e, f"Call to unknown function {e.func.id}")
        self.err(e, "Unsupported call target type")

    # -- statements -------------------------------------------------------
    def stmts(self, body):
        return " ".join(self.stmt(s) for s in body)

    def stmt(self, s):
        i = self.info(s)
        if isinstance(s, pyast.For):
            if not isinstance(s.target, pyast.Name):
                self.err(s, "For-loops must assign to a single variable")
            it = s.iter
            ok = isinstance(it, pyast.Call) and isinstance(it.func, pyast.Name)
            if ok:
                try:
                    ok = self.eval_name(it.func.id) is builtins.range
                except Exception:
                    ok = False
            if not ok:
                self.err(s, "For-loop must iterate using the range builtin")
            a = it.args
            if len(a) == 1:
                lo, hi, step = f"(int {i} 0)", self.expr(a[0]), 1
            elif len(a) == 2:
                lo, hi, step = self.expr(a[0]), self.expr(a[1]), 1
            elif len(a) == 3:
                lo, hi = self.expr(a[0]), self.expr(a[1])
                step = self.literal_step(a[2])
            else:
                self.err(s, "Invalid number of arguments passed to range")
            if s.orelse:
                self.err(s, "For-loops with an else-clause are not supported")
            return f"(for {i} {_quote(s.target.id)} {lo} {hi} {step} (body {self.stmts(s.body)}))"
        if isinstance(s, pyast.If):
            return f"(if {i} {self.expr(s.test)} (then {self.stmts(s.body)}) (else {self.stmts(s.orelse)}))"
        if isinstance(s, pyast.Assign):
            if len(s.targets) > 1:
                self.err(s, "Cannot have more than one target of assignment")
            t = s.targets[0]
            if not isinstance(t, (pyast.Name, pyast.Subscript)):
                self.err(s, "Unsupported form of assignment")
            return f"(assign {i} {self.expr(t)} {self.expr(s.value)})"
        if isinstance(s, pyast.AugAssign):
            op = _BINOPS.get(type(s.op))
            if op is None:
                self.err(s, f"Unsupported binary operation: {pyast.dump(s.op)}")
            dst = self.expr(s.target)
            return f"(assign {i} {dst} (binop {i} {op} {dst} {self.expr(s.value)}))"
        if isinstance(s, pyast.While):
            if s.orelse:
                self.err(s, "While-loops with an else-clause are not supported")
            return f"(while {i} {self.expr(s.test)} (body {self.stmts(s.body)}))"
        if isinstance(s, pyast.Expr):
            v = s.value
            if isinstance(v, pyast.Call):
                b = self.lookup_builtin(v.func) if isinstance(v.func, (pyast.Name, pyast.Attribute)) else None
                if b == "label":
                    if len(v.args) != 1:
                        self.err(s, "Label statement expects one argument")
                    a = v.args[0]
                    if not (isinstance(a, pyast.Constant) and isinstance(a.value, str)):
                        self.err(s, "First argument of parpy.label should be a string literal "
                                    "representing the label name")
                    return f"(label {i} {_quote(a.value)})"
                if b is None and isinstance(v.func, pyast.Name):
                    if v.func.id not in self.tops:
                        self.err(s, f"Call to unknown function {v.func.id}")
                    if v.keywords:
                        self.err(s, f"Unsupported keyword argument in call: {v.keywords[0].arg}")
                    args = " ".join(self.expr(a) for a in v.args)
                    return f"(callstmt {i} {_quote(v.func.id)}{' ' if args else ''}{args})"
            self.err(s, "Unsupported expression statement")
        if isinstance(s, pyast.With):
            if len(s.items) != 1:
                self.err(s, "With statements using multiple items is not supported")
            item = s.items[0]
            if item.optional_vars is not None:
                self.err(s, "With statements using the 'as' keyword are not supported")
            if self.lookup_builtin(item.context_expr) != "gpu":
                self.err(s, "With statements are only supported for 'parpy.gpu'")
            return f"(withgpu {i} (body {self.stmts(s.body)}))"
        if isinstance(s, pyast.Return):
            if s.value is None:
                self.err(s, "Empty return statements are not supported")
            return f"(return {i} {self.expr(s.value)})"
        self.err(s, f"Unsupported statement: {pyast.unparse(s)}")

    def literal_step(self, e):
        v = None
        if isinstance(e, pyast.Constant) and isinstance(e.value, int) and not isinstance(e.value, bool):
            v = e.value
        elif isinstance(e, pyast.UnaryOp) and isinstance(e.op, pyast.USub) and \
                isinstance(e.operand, pyast.Constant) and isinstance(e.operand.value, int):
            v = -e.operand.value
        if v is None:
            self.err(e, "Range step size must be an integer literal")
        if v == 0:
            self.err(e, "Range step size must be non-zero")
        return v

    # -- function ---------------------------------------------------------
    def annotation(self, a, node):
        if a is None:
            return "none"
        try:
            ty = self.eval_name(pyast.unparse(a))
        except Exception:
            self.err(node, "Unsupported parameter type annotation")
        if isinstance(ty, ElemSize):
            return f"(scalar {ty.value})"
        if isinstance(ty, _types.ExtType):
            return f"(pointer {ty.sz.value})"
        self.err(node, "Unsupported parameter type annotation")

    def fundef(self, tree):
        fn = tree.body[0]
        if not isinstance(fn, pyast.FunctionDef):
            raise FrontendError("Expected a function definition")
        params = " ".join(
            f"(p {_quote(a.arg)} {self.annotation(a.annotation, a)} {self.info(a)})"
            for a in fn.args.args)
        stmts = fn.body
        if stmts and isinstance(stmts[0], pyast.Expr) and isinstance(stmts[0].value, pyast.Constant) \
                and isinstance(stmts[0].value.value, str):
            stmts = stmts[1:]   # documentation string
        body = self.stmts(stmts)
        ret = self.annotation(fn.returns, fn) if fn.returns is not None else "none"
        return f"(fun {_quote(fn.name)} {self.info(fn)} {ret} (params {params}) (body {body}))"


def external_to_sexpr(tree, info, vars, ext_name, header, backend_code, nthreads):
    """Serialise the declaration of an external: only the signature of the decorated function is used."""
    filepath, line_ofs, col_ofs = info
    globs, locs = vars
    c = _Converter(filepath, line_ofs, col_ofs, {}, globs, locs)
    fn = tree.body[0]
    if not isinstance(fn, pyast.FunctionDef):
        raise FrontendError("Expected a function definition")
    params = []
    for a in fn.args.args:
        if a.annotation is None:
            c.err(a, "Unsupported parameter type annotation")
        params.append(f"(p {_quote(a.arg)} {c.annotation(a.annotation, a)} {c.info(a)})")
    if fn.returns is None:
        c.err(fn, "Unsupported return type annotation on external function")
    try:
        ret = c.annotation(fn.returns, fn)
    except FrontendError:
        c.err(fn, "Unsupported return type annotation on external function")
    if not ret.startswith("(scalar"):
        c.err(fn, "Unsupported return type annotation on external function")
    return (f"(ext {_quote(fn.name)} {_quote(ext_name)} {ret} (params {' '.join(params)}) {_quote(header or '')} "
            f"{backend_code} {int(nthreads or 0)} {c.info(fn)})")


def to_sexpr(tree, info, tops, vars):
    """Serialise a parsed function definition.  `info` = (file, line_ofs, col_ofs),
    `tops` = names of previously jitted functions / externals, `vars` = (globals, locals)."""
    filepath, line_ofs, col_ofs = info
    globs, locs = vars
    return _Converter(filepath, line_ofs, col_ofs, tops, globs, locs).fundef(tree)
