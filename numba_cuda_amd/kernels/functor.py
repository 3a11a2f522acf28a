"""From a Python binary functor to the body of a device function.

The reference hands the functor of `Reduce` to its JIT (kernels/reduction.py:15-20,
:175-192), which types it and compiles it.  Here the functor is RUN on two recording
stand-ins: arithmetic, comparisons, conditionals and `math` calls build an expression
tree (`trace`), the tree is typed for one element type with the JIT's rules, and written
out as C++ with every conversion spelled as a cast (`body_for`).  The HIP run-time
compiler turns that into kernels (csrc/reduce_custom.hip).

What a functor may do: + - * / // % ** (integer powers: constant exponent), & | ^ << >> ~,
unary minus, abs(), comparisons, `x if cond else y`, if / else statements, and / or / not
on conditions, min() / max(), numeric constants (also from globals and closures), the
functions of `math` listed in _MATH (also as numpy functions of the same name), and
`.real`, `.imag`, `.conjugate()`.  Anything else - loops over data, int(), float(), other
attributes, calls to other functions with side effects - raises NotImplementedError with
the reason.

Complex elements (complex64 / complex128) and complex constants: + - * / and unary minus
as the JIT lowers them (numba/cuda/cpython/numbers.py:1091-1196: the product is
(ac - bd) + (ad + bc)i, the quotient CPython's algorithm), == and !=, abs() (hypot),
z ** 2 (a product, :1062-1078; other powers are not translated), .real / .imag /
.conjugate() (:1003-1024).  What Python refuses for complex numbers is refused here with
the same TypeError: ordering comparisons, // and %, bitwise operators, `math` functions.

Typing rules restated from the reference's JIT (numba's integer typing: operations on
integers are carried out in 64 bits, signed unless both operands are unsigned; a boolean
in arithmetic is an int64; true division gives float64 for integers; float32 stays
float32 among float32 operands and becomes float64 with Python floats or integers;
math.floor / math.ceil return int64; complex64 stays complex64 with float32 and complex64
operands and becomes complex128 with anything wider, Python complex constants are
complex128; the result is converted to the element type - except complex to real, which the
JIT refuses too).
"""

import math
import types

import numpy as np

_MAX_CONDITIONS = 12
_MAX_RUNS = 512


class Untranslatable(NotImplementedError):
    pass


class Expr:
    """Node of the expression tree: op in {"a", "b", "const", <operator>, "ite", "call"}."""

    __slots__ = ("op", "args", "value")

    def __init__(self, op, args=(), value=None):
        self.op, self.args, self.value = op, tuple(args), value

    def key(self):
        if self.op == "const":
            v = self.value
            return ("const", type(v).__name__, v.hex() if isinstance(v, float) else repr(v))
        return (self.op, self.value) + tuple(x.key() for x in self.args)

    def __repr__(self):
        if self.op in ("a", "b"):
            return self.op
        if self.op == "const":
            return repr(self.value)
        return "%s(%s)" % (self.op if self.op != "call" else self.value, ", ".join(map(repr, self.args)))


_A, _B = Expr("a"), Expr("b")

_BINARY = {"add": "__add__", "sub": "__sub__", "mul": "__mul__", "truediv": "__truediv__",
           "floordiv": "__floordiv__", "mod": "__mod__", "pow": "__pow__", "and": "__and__", "or": "__or__",
           "xor": "__xor__", "lshift": "__lshift__", "rshift": "__rshift__"}
_COMPARE = {"lt": "__lt__", "le": "__le__", "gt": "__gt__", "ge": "__ge__", "eq": "__eq__", "ne": "__ne__"}
_UNARY = {"neg": "__neg__", "pos": "__pos__", "abs": "__abs__", "invert": "__invert__"}
_PARTS = ("real", "imag", "conj")           # .real, .imag, .conjugate(): unary nodes too

# math function -> (C name for double, arity, result): "f" float like the argument,
# "i" int64 (floor / ceil / trunc), "b" boolean
_MATH = {
    "sqrt": ("sqrt", 1, "f"), "exp": ("exp", 1, "f"), "exp2": ("exp2", 1, "f"), "expm1": ("expm1", 1, "f"),
    "log": ("log", 1, "f"), "log2": ("log2", 1, "f"), "log10": ("log10", 1, "f"), "log1p": ("log1p", 1, "f"),
    "sin": ("sin", 1, "f"), "cos": ("cos", 1, "f"), "tan": ("tan", 1, "f"), "asin": ("asin", 1, "f"),
    "acos": ("acos", 1, "f"), "atan": ("atan", 1, "f"), "sinh": ("sinh", 1, "f"), "cosh": ("cosh", 1, "f"),
    "tanh": ("tanh", 1, "f"), "asinh": ("asinh", 1, "f"), "acosh": ("acosh", 1, "f"), "atanh": ("atanh", 1, "f"),
    "erf": ("erf", 1, "f"), "erfc": ("erfc", 1, "f"), "gamma": ("tgamma", 1, "f"), "lgamma": ("lgamma", 1, "f"),
    "fabs": ("fabs", 1, "f"), "floor": ("floor", 1, "i"), "ceil": ("ceil", 1, "i"), "trunc": ("trunc", 1, "i"),
    "atan2": ("atan2", 2, "f"), "hypot": ("hypot", 2, "f"), "pow": ("pow", 2, "f"), "fmod": ("fmod", 2, "f"),
    "copysign": ("copysign", 2, "f"),
    "isnan": ("isnan", 1, "b"), "isinf": ("isinf", 1, "b"), "isfinite": ("isfinite", 1, "b"),
}
# numpy spells some of them differently
_NUMPY_NAMES = {"arcsin": "asin", "arccos": "acos", "arctan": "atan", "arcsinh": "asinh", "arccosh": "acosh",
                "arctanh": "atanh", "arctan2": "atan2"}


# numpy function -> (operator, which inputs in which order)
_UFUNC_OPERATOR = {
    "add": ("add", (0, 1)), "subtract": ("sub", (0, 1)), "multiply": ("mul", (0, 1)),
    "true_divide": ("truediv", (0, 1)), "divide": ("truediv", (0, 1)), "floor_divide": ("floordiv", (0, 1)),
    "remainder": ("mod", (0, 1)), "mod": ("mod", (0, 1)), "power": ("pow", (0, 1)),
    "bitwise_and": ("and", (0, 1)), "bitwise_or": ("or", (0, 1)), "bitwise_xor": ("xor", (0, 1)),
    "left_shift": ("lshift", (0, 1)), "right_shift": ("rshift", (0, 1)),
    "less": ("lt", (0, 1)), "less_equal": ("le", (0, 1)), "greater": ("gt", (0, 1)),
    "greater_equal": ("ge", (0, 1)), "equal": ("eq", (0, 1)), "not_equal": ("ne", (0, 1)),
    "negative": ("neg", (0,)), "positive": ("pos", (0,)), "absolute": ("abs", (0,)), "fabs": ("abs", (0,)),
    "invert": ("invert", (0,)), "bitwise_not": ("invert", (0,)),
    "conjugate": ("conj", (0,)),
}


def _lift(x):
    if isinstance(x, _Value):
        return x.expr
    if isinstance(x, (bool, np.bool_)):
        return Expr("const", value=bool(x))
    if isinstance(x, (int, float, complex, np.integer, np.floating, np.complexfloating)):
        return Expr("const", value=x)
    raise Untranslatable("an operand of type %s is mixed into the computation" % type(x).__name__)


class _Script:
    """Answers to the conditions a run meets: the given ones first, True afterwards."""

    def __init__(self, answers):
        self.answers = answers
        self.conditions = []
        self.decided = {}

    def decide(self, expr):
        key = expr.key()
        if key in self.decided:            # the same question again on this path
            return self.decided[key]
        self.decided[key] = answer = self._fresh(expr)
        return answer

    def _fresh(self, expr):
        k = len(self.conditions)
        if k >= _MAX_CONDITIONS:
            raise Untranslatable("more than %d conditions on one path (a loop over the data?)" % _MAX_CONDITIONS)
        self.conditions.append(expr)
        return self.answers[k] if k < len(self.answers) else True


class _Value:
    """Stand-in for an operand or an intermediate value."""

    __slots__ = ("expr", "script")

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        """numpy functions applied to stand-ins (np.sqrt(a), np.float32(2) * a, ...)."""
        name = ufunc.__name__
        if method != "__call__" or kwargs:
            raise Untranslatable("numpy.%s.%s on an operand" % (name, method))
        if name in _UFUNC_OPERATOR and len(inputs) == len(_UFUNC_OPERATOR[name][1]):
            op, order = _UFUNC_OPERATOR[name]
            return _Value(Expr(op, [_lift(inputs[k]) for k in order]), self.script)
        if name in ("maximum", "minimum", "fmax", "fmin") and len(inputs) == 2:
            x, y = _lift(inputs[0]), _lift(inputs[1])
            cond = Expr("ge" if name in ("maximum", "fmax") else "le", (x, y))
            return _Value(Expr("ite", (cond, x, y)), self.script)
        name = _NUMPY_NAMES.get(name, name)
        if name in _MATH:
            return _math_call(name, *inputs)
        raise Untranslatable("numpy.%s is not among the translated functions" % ufunc.__name__)

    def __init__(self, expr, script):
        self.expr, self.script = expr, script

    def __bool__(self):
        e = self.expr
        if e.op == "const":
            return bool(e.value)
        if e.op not in _COMPARE and not (e.op == "call" and _MATH[e.value][2] == "b"):
            e = Expr("ne", (e, Expr("const", value=0)))
        return self.script.decide(e)

    def __hash__(self):
        return id(self)

    def _refuse(self, what):
        raise Untranslatable("%s of an operand cannot be translated" % what)

    def __int__(self):
        self._refuse("int()")

    def __float__(self):
        self._refuse("float()")

    def __index__(self):
        self._refuse("use as an index")

    def __iter__(self):
        self._refuse("iteration")

    def __getitem__(self, _):
        self._refuse("indexing")

    def __round__(self, *_):
        self._refuse("round()")

    def __complex__(self):
        self._refuse("complex()")

    @property
    def real(self):
        return _Value(Expr("real", (self.expr,)), self.script)

    @property
    def imag(self):
        return _Value(Expr("imag", (self.expr,)), self.script)

    def conjugate(self):
        return _Value(Expr("conj", (self.expr,)), self.script)


def _install_operators():
    def binary(op, swapped):
        def method(self, other):
            try:
                o = _lift(other)
            except Untranslatable:
                return NotImplemented
            args = (o, self.expr) if swapped else (self.expr, o)
            return _Value(Expr(op, args), self.script)
        return method

    def unary(op):
        def method(self):
            return _Value(Expr(op, (self.expr,)), self.script)
        return method

    for op, dunder in _BINARY.items():
        setattr(_Value, dunder, binary(op, False))
        setattr(_Value, "__r" + dunder[2:], binary(op, True))
    for op, dunder in _COMPARE.items():
        setattr(_Value, dunder, binary(op, False))
    for op, dunder in _UNARY.items():
        setattr(_Value, dunder, unary(op))


def _math_call(name, *args):
    """math.<name> on stand-ins builds a node; on plain numbers it is the real function."""
    script = next((x.script for x in args if isinstance(x, _Value)), None)
    if script is None:
        return getattr(math, name)(*args)
    cname, arity, _ = _MATH[name]
    if len(args) != arity:
        raise Untranslatable("math.%s takes %d argument(s)" % (name, arity))
    return _Value(Expr("call", [_lift(x) for x in args], value=name), script)


_install_operators()


class _MathProxy:
    """Stands in for the `math` module inside the functor while it is traced."""

    def __getattr__(self, name):
        if name in _MATH:
            return lambda *args: _math_call(name, *args)
        value = getattr(math, name)
        if callable(value):
            def refuse(*args):
                if any(isinstance(x, _Value) for x in args):
                    raise Untranslatable("math.%s is not among the translated functions" % name)
                return value(*args)
            return refuse
        return value            # pi, e, inf, ...


_MATH_PROXY = _MathProxy()
_MATH_FUNCTIONS = {getattr(math, name): name for name in _MATH if hasattr(math, name)}


def _swap_math(value):
    if value is math:
        return _MATH_PROXY
    try:
        name = _MATH_FUNCTIONS.get(value)
    except TypeError:
        return value
    if name is not None:
        return lambda *args: _math_call(name, *args)
    return value


def _rebound(functor):
    """The functor with `math` (and functions imported from it) replaced, in its globals
    and its closure, by versions that accept the stand-ins."""
    if not isinstance(functor, types.FunctionType):
        return functor
    code = functor.__code__
    new_globals = None
    for name in code.co_names:
        if name in functor.__globals__:
            old = functor.__globals__[name]
            new = _swap_math(old)
            if new is not old:
                if new_globals is None:
                    new_globals = dict(functor.__globals__)
                new_globals[name] = new
    closure = functor.__closure__
    if closure:
        cells = []
        for cell in closure:
            try:
                old = cell.cell_contents
            except ValueError:
                cells.append(cell)
                continue
            new = _swap_math(old)
            cells.append(cell if new is old else types.CellType(new))
        closure = tuple(cells)
    if new_globals is None and closure == functor.__closure__:
        return functor
    clone = types.FunctionType(code, new_globals if new_globals is not None else functor.__globals__,
                               functor.__name__, functor.__defaults__, closure)
    clone.__kwdefaults__ = functor.__kwdefaults__
    return clone


def trace(functor):
    """Expression tree of functor(a, b); Untranslatable (a NotImplementedError) if the
    functor does something that cannot be expressed."""
    fn = _rebound(functor)
    runs = [0]

    def run(answers):
        runs[0] += 1
        if runs[0] > _MAX_RUNS:
            raise Untranslatable("too many paths through the functor")
        script = _Script(answers)
        try:
            out = fn(_Value(_A, script), _Value(_B, script))
        except Untranslatable:
            raise
        except RecursionError:
            raise Untranslatable("unbounded recursion on the operands")
        except Exception as e:     # the functor tripped over the stand-ins
            raise Untranslatable("%s: %s" % (type(e).__name__, e))
        try:
            expr = _lift(out)
        except Untranslatable:
            raise Untranslatable("the functor returned %r, not a number" % (out,))
        return expr, script.conditions

    def paths(answers):
        expr, conditions = run(answers)
        if len(conditions) > len(answers):
            cond = conditions[len(answers)]
            yes = paths(answers + (True,))
            no = paths(answers + (False,))
            if yes.key() == no.key():
                return yes
            return Expr("ite", (cond, yes, no))
        return expr

    return paths(())


# ---- typing and C++ ---------------------------------------------------------------------

_B1, _I64, _U64 = np.dtype(np.bool_), np.dtype(np.int64), np.dtype(np.uint64)
_F16, _F32, _F64 = np.dtype(np.float16), np.dtype(np.float32), np.dtype(np.float64)
_C64, _C128 = np.dtype(np.complex64), np.dtype(np.complex128)
_CTYPE = {np.dtype(np.int8): "signed char", np.dtype(np.int16): "short", np.dtype(np.int32): "int",
          _I64: "nbh_i64", np.dtype(np.uint8): "unsigned char", np.dtype(np.uint16): "unsigned short",
          np.dtype(np.uint32): "unsigned int", _U64: "nbh_u64", _F16: "_Float16", _F32: "float", _F64: "double",
          _B1: "bool", _C64: "nbh_c64", _C128: "nbh_c128"}


def _machine(t):
    """Type an operand takes part in arithmetic with."""
    if t.kind in "bi":
        return _I64
    if t.kind == "u":
        return _U64
    return t


def _part(t):
    """Type of the real and imaginary parts of a complex type."""
    return _F32 if t == _C64 else _F64


def _common(t1, t2):
    t1, t2 = _machine(t1), _machine(t2)
    if t1.kind == "c" or t2.kind == "c":
        # the complex type whose parts hold both: float32 parts only among complex64,
        # float32 and float16
        r1 = _part(t1) if t1.kind == "c" else t1
        r2 = _part(t2) if t2.kind == "c" else t2
        return _C64 if _common(r1, r2) in (_F16, _F32) else _C128
    if t1.kind in "iu" and t2.kind in "iu":
        return _U64 if (t1 == _U64 and t2 == _U64) else _I64
    if t1.kind == "f" and t2.kind == "f":
        return t1 if t1.itemsize >= t2.itemsize else t2
    # integer with float: the float type if it holds the integers that can occur - in this
    # translator integers in arithmetic are 64 bits wide, so float64
    return _F64


def _convert(code, src, dst):
    if src == dst:
        return code
    if src.kind == "c" and dst.kind != "c" and dst != _B1:
        raise TypeError("cannot convert %s to %s" % (src, dst))          # the JIT has no such cast either
    if dst.kind == "c":
        if src == _F16:
            code = "(float)(%s)" % code
        return "nbh_cplx_from<%s>(%s)" % (_CTYPE[_part(dst)], code)
    if dst == _B1 and src.kind == "c":
        return "((%s) != nbh_cplx_from<%s>(0))" % (code, _CTYPE[_part(src)])
    if dst == _B1:
        return "((%s) != 0)" % code
    if src == _F16 and dst.kind in "iub":
        code = "(float)(%s)" % code
    if dst == _F16 and src.kind in "iu":
        code = "(double)(%s)" % code
    return "(%s)(%s)" % (_CTYPE[dst], code)


def _float_literal(v):
    v = float(v)
    if v != v:
        return "__builtin_nan(\"\")"
    if v in (math.inf, -math.inf):
        return "(-__builtin_inf())" if v < 0 else "__builtin_inf()"
    return "(%s)" % v.hex()


class _Writer:
    def __init__(self, elem):
        self.elem = elem

    def emit(self, e):
        """-> (C++ expression, dtype)."""
        op = e.op
        if op in ("a", "b"):
            if self.elem == _B1:
                return "(%s != 0)" % op, _B1
            return op, self.elem
        if op == "const":
            return self.constant(e.value)
        if op == "ite":
            c, tc = self.emit(e.args[0])
            x, tx = self.emit(e.args[1])
            y, ty = self.emit(e.args[2])
            t = tx if tx == ty else _common(tx, ty)
            return "(%s ? %s : %s)" % (_convert(c, tc, _B1), _convert(x, tx, t), _convert(y, ty, t)), t
        if op == "call":
            return self.call(e)
        if op in _UNARY:
            return self.unary(op, *self.emit(e.args[0]))
        if op in _PARTS:
            return self.part(op, *self.emit(e.args[0]))
        x, tx = self.emit(e.args[0])
        y, ty = self.emit(e.args[1])
        if op in _COMPARE:
            return self.compare(op, x, tx, y, ty), _B1
        return self.binary(op, x, tx, y, ty, e)

    def constant(self, v):
        if isinstance(v, (bool, np.bool_)):
            return ("true" if v else "false"), _B1
        if isinstance(v, np.floating):
            t = np.dtype(type(v))
            if t not in (_F16, _F32, _F64):
                raise Untranslatable("constant of type %s" % t)
            return _convert(_float_literal(v), _F64, t), t
        if isinstance(v, float):
            return _float_literal(v), _F64
        if isinstance(v, (complex, np.complexfloating)):
            t = np.dtype(type(v)) if isinstance(v, np.complexfloating) else _C128
            if t not in (_C64, _C128):
                raise Untranslatable("constant of type %s" % t)
            r = _CTYPE[_part(t)]
            return "%s{(%s)%s, (%s)%s}" % (_CTYPE[t], r, _float_literal(v.real), r, _float_literal(v.imag)), t
        if isinstance(v, np.integer):
            t = _machine(np.dtype(type(v)))
            v = int(v)
        else:
            t = _I64 if v < 2**63 else _U64
        if v < -2**63 or v >= 2**64:
            raise Untranslatable("the integer constant %d does not fit 64 bits" % v)
        if t == _U64:
            return "%dULL" % v, _U64
        if v == -2**63:
            return "(-9223372036854775807LL - 1LL)", _I64
        return "(%dLL)" % v, _I64

    def part(self, op, x, tx):
        """.real / .imag / .conjugate(): parts of a complex number; a real number is its own
        real part and conjugate, its imaginary part a zero of its type
        (numba/cuda/cpython/numbers.py:1003-1046)."""
        if tx.kind == "c":
            if op == "conj":
                return "nbh_conj(%s)" % x, tx
            return "(%s).%s" % (x, "re" if op == "real" else "im"), _part(tx)
        if op == "imag":
            return _convert("0", _I64, tx), tx
        return x, tx

    def unary(self, op, x, tx):
        t = _machine(tx)
        x = _convert(x, tx, t)
        if op == "pos":
            return x, t
        if t.kind == "c":
            if op == "neg":
                return "(-%s)" % x, t
            if op == "abs":
                return "nbh_cabs(%s)" % x, _part(t)
            raise TypeError("bad operand type for unary ~: %s" % t)
        if t.kind in "iu":
            if op == "neg":
                return "(%s)(0ULL - (nbh_u64)%s)" % (_CTYPE[t], x), t
            if op == "invert":
                return "(~%s)" % x, t
            if t == _U64:
                return x, t
            return "(%s < 0 ? (nbh_i64)(0ULL - (nbh_u64)%s) : %s)" % (x, x, x), t
        if op == "invert":
            raise TypeError("~ is not defined for %s" % t)
        if op == "neg":
            return "(-%s)" % x, t
        if t == _F64:
            return "fabs(%s)" % x, t
        return _convert("fabsf(%s)" % _convert(x, t, _F32), _F32, t), t

    def compare(self, op, x, tx, y, ty):
        sign = {"lt": "<", "le": "<=", "gt": ">", "ge": ">=", "eq": "==", "ne": "!="}[op]
        mx, my = _machine(tx), _machine(ty)
        if (mx.kind == "c" or my.kind == "c") and op not in ("eq", "ne"):
            raise TypeError("'%s' not supported between %s and %s" % (sign, tx, ty))
        if {mx, my} == {_I64, _U64}:
            # value comparison of a signed with an unsigned number
            if mx == _U64:
                flipped = {"lt": "gt", "le": "ge", "gt": "lt", "ge": "le", "eq": "eq", "ne": "ne"}[op]
                return self.compare(flipped, y, ty, x, tx)
            s, u = _convert(x, tx, _I64), _convert(y, ty, _U64)
            negative = {"lt": "true", "le": "true", "gt": "false", "ge": "false", "eq": "false", "ne": "true"}[op]
            return "(%s < 0 ? %s : ((nbh_u64)%s %s %s))" % (s, negative, s, sign, u)
        t = _common(tx, ty)
        return "(%s %s %s)" % (_convert(x, tx, t), sign, _convert(y, ty, t))

    def binary(self, op, x, tx, y, ty, e):
        if op in ("and", "or", "xor"):
            sign = {"and": "&", "or": "|", "xor": "^"}[op]
            if tx == _B1 and ty == _B1:
                return "(bool)(%s %s %s)" % (x, sign, y), _B1
            if _machine(tx).kind not in "iu" or _machine(ty).kind not in "iu":
                raise TypeError("bitwise %s is not defined for %s and %s" % (op, tx, ty))
            t = _common(tx, ty)
            return "(%s %s %s)" % (_convert(x, tx, t), sign, _convert(y, ty, t)), t
        if op in ("lshift", "rshift"):
            if _machine(tx).kind not in "iu" or _machine(ty).kind not in "iu":
                raise TypeError("shifts are not defined for %s and %s" % (tx, ty))
            t = _machine(tx)
            amount = "((int)%s & 63)" % _convert(y, ty, _machine(ty))
            if op == "lshift":
                return "(%s)((nbh_u64)%s << %s)" % (_CTYPE[t], _convert(x, tx, t), amount), t
            return "(%s >> %s)" % (_convert(x, tx, t), amount), t
        t = _common(tx, ty)
        if t.kind == "c":
            if op == "pow":
                exponent = e.args[1]
                if exponent.op != "const" or exponent.value != 2:
                    raise Untranslatable("complex ** is translated for the exponent 2 only")
                base = _convert(x, tx, t)
                return "(%s * %s)" % (base, base), t
            if op in ("floordiv", "mod"):
                raise TypeError("can't take floor or mod of complex number")       # Python's words
            sign = {"add": "+", "sub": "-", "mul": "*", "truediv": "/"}[op]
            return "(%s %s %s)" % (_convert(x, tx, t), sign, _convert(y, ty, t)), t
        if op == "truediv":
            if t.kind in "iu":
                t = _F64
            return "(%s / %s)" % (_convert(x, tx, t), _convert(y, ty, t)), t
        if op == "pow":
            if t.kind in "iu":
                exponent = e.args[1]
                if exponent.op != "const" or isinstance(exponent.value, (float, np.floating)) or int(exponent.value) < 0:
                    raise Untranslatable("integer ** needs a constant, non-negative integer exponent")
                r = "nbh_ipow(%s, %s)" % (_convert(x, tx, _I64), _convert(y, ty, _I64))
                return _convert(r, _I64, t), t
            if t == _F64:
                return "pow(%s, %s)" % (_convert(x, tx, t), _convert(y, ty, t)), t
            r = "powf(%s, %s)" % (_convert(x, tx, _F32), _convert(y, ty, _F32))
            return _convert(r, _F32, t), t
        if op in ("floordiv", "mod"):
            helper = "nbh_floordiv" if op == "floordiv" else "nbh_mod"
            w = _F32 if t == _F16 else t
            r = "%s(%s, %s)" % (helper, _convert(x, tx, w), _convert(y, ty, w))
            return _convert(r, w, t), t
        sign = {"add": "+", "sub": "-", "mul": "*"}[op]
        if t.kind in "iu":
            # wrap-around arithmetic: carried out on unsigned words
            return "(%s)((nbh_u64)%s %s (nbh_u64)%s)" % (_CTYPE[t], _convert(x, tx, t), sign, _convert(y, ty, t)), t
        return "(%s %s %s)" % (_convert(x, tx, t), sign, _convert(y, ty, t)), t

    def call(self, e):
        name = e.value
        cname, _, result = _MATH[name]
        args = [self.emit(x) for x in e.args]
        # float32 arguments keep the function in float32; anything else computes in float64
        kinds = [_machine(t) for _, t in args]
        if any(t.kind == "c" for t in kinds):
            raise TypeError("can't convert complex to float (math.%s)" % name)      # Python's words
        if all(t in (_F32, _F16) for t in kinds):
            w, cname = _F32, (cname if result == "b" else cname + "f")
        else:
            w = _F64
        code = "%s(%s)" % (cname, ", ".join(_convert(c, t, w) for c, t in args))
        if result == "i":
            return "(nbh_i64)%s" % code, _I64
        if result == "b":
            return "(bool)%s" % code, _B1
        return code, w


def body_for(expr, dtype):
    """C++ body of `T nbh_op(T a, T b)` for elements of `dtype` (booleans travel as bytes
    holding 0 or 1)."""
    dtype = np.dtype(dtype)
    if dtype not in _CTYPE:
        raise NotImplementedError("Reduce with a general functor does not support dtype %s" % dtype)
    code, t = _Writer(dtype).emit(expr)
    if dtype == _B1:
        return "    return (T)(%s ? 1 : 0);" % _convert(code, t, _B1)
    return "    return %s;" % _convert(code, t, dtype)
