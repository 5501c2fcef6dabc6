"""Python functions of ``(t, x)`` turned into kernel code by tracing them.

The reference translates the *source* of a node / connection function into OpenCL
with an AST visitor (``nengo_ocl/ast_conversion.py``: ``OclFunction`` :863-931,
function tables :63-226) and falls back to a host callback when that fails
(``simulator.py:910-966``).  This module reaches the same goal another way: it
*calls* the function once (or a few times) with symbolic arguments and records the
arithmetic that happens.  Closures, helper functions, loops over fixed ranges, list
comprehensions, numpy reductions and indexing then need no special support: Python
itself executes them; only the leaves (arithmetic on an input, a math function of
an input, a comparison) are intercepted.

* ``t`` is a scalar `Expr`, ``x`` a numpy object array of `Expr` (so ``x[0]``,
  ``x[1:]``, ``len(x)``, ``x.mean()``, ``np.dot(w, x)`` behave as on a float array).
* numpy ufuncs reach `Expr.__array_ufunc__` (scalars), `ExprArray.__array_ufunc__`
  (the input vector and what is computed from it) or the same-named methods (elements
  of plain object arrays); functions of the ``math`` module, which insist on real
  floats, are swapped for tracing stand-ins in a copy of the function's globals and
  closure cells.
* A condition on a traced value (``if x[0] > 0``, ``max(a, b)``, ``all(x > 2)``, a
  conditional expression) cannot be answered once and for all: the function is run
  again for the other answer and the results are joined by a select, for every such
  condition met (bounded number of runs).
* Whatever cannot be traced (``float(x[0])``, an unknown C extension function, data
  dependent loops) raises `TraceError`, a NotImplementedError, on which the
  Simulator keeps the function on the host like the reference.  A function whose two
  traces differ (random numbers, internal state) or whose code stores to attributes,
  subscripts, globals or closure cells is refused as well.

`trace` returns the outputs as expression graphs; `generate` writes them as the
``code`` text ``plan_direct`` takes (statements assigning ``OUTPUT__[i]``);
`evaluate` interprets them on the host (used by tests to check a trace against the
function it came from).
"""

import dis
import inspect
import math
import types

import numpy as np

OUTPUT_NAME = "OUTPUT__"
MAX_RUNS = 256  # paths through the conditions of one function


class TraceError(NotImplementedError):
    pass


# op -> (C spelling, host implementation); unary float functions
_UNARY = {
    "sin": ("sinf", math.sin), "cos": ("cosf", math.cos), "tan": ("tanf", math.tan),
    "arcsin": ("asinf", math.asin), "arccos": ("acosf", math.acos),
    "arctan": ("atanf", math.atan), "sinh": ("sinhf", math.sinh), "cosh": ("coshf", math.cosh),
    "tanh": ("tanhf", math.tanh), "arcsinh": ("asinhf", math.asinh),
    "arccosh": ("acoshf", math.acosh), "arctanh": ("atanhf", math.atanh),
    "exp": ("expf", math.exp), "exp2": ("exp2f", lambda a: 2.0 ** a),
    "expm1": ("expm1f", math.expm1), "log": ("logf", math.log), "log2": ("log2f", math.log2),
    "log10": ("log10f", math.log10), "log1p": ("log1pf", math.log1p),
    "sqrt": ("sqrtf", math.sqrt), "cbrt": ("cbrtf", lambda a: math.copysign(abs(a) ** (1 / 3), a)),
    "fabs": ("fabsf", abs), "floor": ("floorf", math.floor), "ceil": ("ceilf", math.ceil),
    "trunc": ("truncf", math.trunc), "rint": ("rintf", lambda a: float(np.rint(a))),
    "erf": ("erff", math.erf), "erfc": ("erfcf", math.erfc), "gamma": ("tgammaf", math.gamma),
    "lgamma": ("lgammaf", math.lgamma), "neg": ("-", lambda a: -a),
}
_BINARY_FN = {
    "arctan2": ("atan2f", math.atan2), "hypot": ("hypotf", math.hypot),
    "fmod": ("fmodf", math.fmod), "copysign": ("copysignf", math.copysign),
    "pow": ("powf", lambda a, b: a ** b), "maximum": ("fmaxf", max), "minimum": ("fminf", min),
}
_INFIX = {
    "add": ("+", lambda a, b: a + b), "sub": ("-", lambda a, b: a - b),
    "mul": ("*", lambda a, b: a * b), "div": ("/", lambda a, b: a / b),
}
_COMPARE = {
    "lt": ("<", lambda a, b: a < b), "le": ("<=", lambda a, b: a <= b),
    "gt": (">", lambda a, b: a > b), "ge": (">=", lambda a, b: a >= b),
    "eq": ("==", lambda a, b: a == b), "ne": ("!=", lambda a, b: a != b),
}
_LOGIC = {"and": ("&&", lambda a, b: bool(a) and bool(b)), "or": ("||", lambda a, b: bool(a) or bool(b))}


class _Tracer:
    """State of one run of the traced function: interned nodes, decisions taken."""

    def __init__(self):
        self.nodes = {}
        self.forced = []      # answers to give to the first conditions met
        self.conditions = []  # conditions met in this run, in order
        self.answers = []
        self.seen = {}

    def decide(self, cond):
        if cond in self.seen:  # asked again within the run: same answer
            return self.seen[cond]
        k = len(self.conditions)
        answer = self.forced[k] if k < len(self.forced) else True
        self.conditions.append(cond)
        self.answers.append(answer)
        self.seen[cond] = answer
        return answer


_ACTIVE = None


def _node(op, *args, value=None):
    tracer = _ACTIVE
    if tracer is None:
        raise TraceError("expression used outside of a trace")
    # constants are told apart by type and sign too (True is not 1.0, -0.0 is not 0.0)
    key = (op, type(value).__name__, repr(value)) + tuple(id(a) for a in args)
    node = tracer.nodes.get(key)
    if node is None:
        node = Expr.__new__(Expr)
        node.op, node.args, node.value = op, args, value
        node.is_bool = op in _COMPARE or op in _LOGIC or op == "not" or (
            op == "const" and isinstance(value, bool)) or (
            op == "select" and args[1].is_bool and args[2].is_bool)
        tracer.nodes[key] = node
    return node


def _const(value):
    if isinstance(value, (bool, np.bool_)):
        return _node("const", value=bool(value))
    return _node("const", value=float(value))


def _wrap(value):
    if isinstance(value, Expr):
        return value
    if isinstance(value, (bool, int, float, np.integer, np.floating, np.bool_)):
        return _const(value)
    if isinstance(value, np.ndarray) and value.ndim == 0:
        return _wrap(value.item())
    raise TraceError("cannot use a %s in traced arithmetic" % type(value).__name__)


def _apply(op, *args):
    """Node for ``op(args)``; constants are folded with the host implementation."""
    args = tuple(_wrap(a) for a in args)
    if all(a.op == "const" for a in args):
        impl = (_UNARY.get(op) or _BINARY_FN.get(op) or _INFIX.get(op) or _COMPARE.get(op)
                or _LOGIC.get(op))
        if impl is not None:
            try:
                return _const(impl[1](*[a.value for a in args]))
            except (ValueError, ZeroDivisionError, OverflowError):
                pass  # left to the device's float arithmetic (inf / nan)
    return _node(op, *args)


def _select(cond, a, b):
    cond, a, b = _wrap(cond), _wrap(a), _wrap(b)
    if a is b:
        return a
    if cond.op == "const":
        return a if cond.value else b
    return _node("select", cond, a, b)


def _pow(a, b):
    a, b = _wrap(a), _wrap(b)
    if (b.op == "const" and not b.is_bool and math.isfinite(b.value) and b.value == int(b.value)
            and 0 <= b.value <= 4):
        n = int(b.value)
        if n == 0:
            return _const(1.0)
        out = a
        for _ in range(n - 1):
            out = _apply("mul", out, a)
        return out
    if b.op == "const" and b.value == 0.5:
        return _apply("sqrt", a)
    return _apply("pow", a, b)


def _floordiv(a, b):
    return _apply("floor", _apply("div", a, b))


def _mod(a, b):  # Python's sign convention: the result has the sign of b
    return _apply("sub", a, _apply("mul", _floordiv(a, b), b))


def _sign(a):
    return _select(_apply("gt", a, 0.0), 1.0, _select(_apply("lt", a, 0.0), -1.0, 0.0))


def _not(a):
    a = _wrap(a)
    if a.op == "const":
        return _const(not a.value)
    return _node("not", a if a.is_bool else _apply("ne", a, 0.0))


def _isnan(a):
    return _apply("ne", a, a)


def _isinf(a):
    return _apply("eq", _apply("fabs", a), math.inf)


def _isfinite(a):
    return _apply("lt", _apply("fabs", a), math.inf)


def _signbit(a):  # true for -0.0 as well
    return _apply("lt", _apply("copysign", 1.0, a), 0.0)


def _ldexp(a, b):
    return _apply("mul", a, _apply("exp2", b))


def _logaddexp(a, b):  # log(exp(a) + exp(b)) without overflow
    return _apply("add", _apply("maximum", a, b),
                  _apply("log1p", _apply("exp", _apply("neg", _apply("fabs", _apply("sub", a, b))))))


def _logaddexp2(a, b):
    return _apply("add", _apply("maximum", a, b),
                  _apply("log2", _apply("add", 1.0, _apply("exp2", _apply("neg", _apply("fabs", _apply("sub", a, b)))))))


def _logic(op):
    def fn(a, b):
        a, b = _wrap(a), _wrap(b)
        a = a if a.is_bool else _apply("ne", a, 0.0)
        b = b if b.is_bool else _apply("ne", b, 0.0)
        return _apply(op, a, b)
    return fn


# numpy ufunc name -> implementation on Exprs / numbers
_UFUNCS = {name: (lambda a, _op=name: _apply(_op, a)) for name in _UNARY if name != "neg"}
_UFUNCS.update({name: (lambda a, b, _op=name: _apply(_op, a, b))
                for name in ("arctan2", "hypot", "fmod", "copysign", "maximum", "minimum")})
_UFUNCS.update({
    "add": lambda a, b: _apply("add", a, b), "subtract": lambda a, b: _apply("sub", a, b),
    "multiply": lambda a, b: _apply("mul", a, b), "divide": lambda a, b: _apply("div", a, b),
    "true_divide": lambda a, b: _apply("div", a, b), "floor_divide": _floordiv,
    "remainder": _mod, "mod": _mod, "power": _pow, "float_power": _pow,
    "negative": lambda a: _apply("neg", a), "positive": lambda a: _wrap(a),
    "absolute": lambda a: _apply("fabs", a), "abs": lambda a: _apply("fabs", a),
    "square": lambda a: _apply("mul", a, a), "reciprocal": lambda a: _apply("div", 1.0, a),
    "sign": _sign, "fmax": lambda a, b: _apply("maximum", a, b),
    "fmin": lambda a, b: _apply("minimum", a, b),
    "deg2rad": lambda a: _apply("mul", a, math.pi / 180), "radians": lambda a: _apply("mul", a, math.pi / 180),
    "rad2deg": lambda a: _apply("mul", a, 180 / math.pi), "degrees": lambda a: _apply("mul", a, 180 / math.pi),
    "less": lambda a, b: _apply("lt", a, b), "less_equal": lambda a, b: _apply("le", a, b),
    "greater": lambda a, b: _apply("gt", a, b), "greater_equal": lambda a, b: _apply("ge", a, b),
    "equal": lambda a, b: _apply("eq", a, b), "not_equal": lambda a, b: _apply("ne", a, b),
    "logical_and": _logic("and"), "logical_or": _logic("or"), "logical_not": _not,
    "conjugate": lambda a: _wrap(a),
    "asin": lambda a: _apply("arcsin", a), "acos": lambda a: _apply("arccos", a),
    "atan": lambda a: _apply("arctan", a), "asinh": lambda a: _apply("arcsinh", a),
    "acosh": lambda a: _apply("arccosh", a), "atanh": lambda a: _apply("arctanh", a),
    "atan2": lambda a, b: _apply("arctan2", a, b), "pow": _pow,
    "isnan": _isnan, "isinf": _isinf, "isfinite": _isfinite, "signbit": _signbit,
    "ldexp": _ldexp, "logaddexp": _logaddexp, "logaddexp2": _logaddexp2,
})


class Expr:
    """A node of a traced expression: ``op`` applied to ``args`` (or a constant / input)."""

    __slots__ = ("op", "args", "value", "is_bool", "__weakref__")
    __array_priority__ = 1e9
    __hash__ = object.__hash__

    def __init__(self, *args, **kwargs):
        raise TypeError("expressions are made by tracing")

    # numpy hands ufunc calls with an Expr among the arguments over to this
    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        impl = _UFUNCS.get(ufunc.__name__)
        if method != "__call__" or impl is None or kwargs.get("out") is not None:
            raise TraceError("numpy.%s (%s) of a traced value" % (ufunc.__name__, method))
        if any(isinstance(i, np.ndarray) for i in inputs):
            return np.frompyfunc(impl, len(inputs), 1)(*inputs)
        return impl(*inputs)

    def __add__(self, o): return _UFUNCS["add"](self, o)
    def __radd__(self, o): return _UFUNCS["add"](o, self)
    def __sub__(self, o): return _UFUNCS["subtract"](self, o)
    def __rsub__(self, o): return _UFUNCS["subtract"](o, self)
    def __mul__(self, o): return _UFUNCS["multiply"](self, o)
    def __rmul__(self, o): return _UFUNCS["multiply"](o, self)
    def __truediv__(self, o): return _UFUNCS["divide"](self, o)
    def __rtruediv__(self, o): return _UFUNCS["divide"](o, self)
    def __floordiv__(self, o): return _floordiv(self, o)
    def __rfloordiv__(self, o): return _floordiv(o, self)
    def __mod__(self, o): return _mod(self, o)
    def __rmod__(self, o): return _mod(o, self)
    def __pow__(self, o): return _pow(self, o)
    def __rpow__(self, o): return _pow(o, self)
    def __neg__(self): return _apply("neg", self)
    def __pos__(self): return self
    def __abs__(self): return _apply("fabs", self)
    def __round__(self, ndigits=None):
        if ndigits:
            raise TraceError("round() to digits")
        return _apply("rint", self)
    def __floor__(self): return _apply("floor", self)
    def __ceil__(self): return _apply("ceil", self)
    def __trunc__(self): return _apply("trunc", self)
    def __lt__(self, o): return _apply("lt", self, o)
    def __le__(self, o): return _apply("le", self, o)
    def __gt__(self, o): return _apply("gt", self, o)
    def __ge__(self, o): return _apply("ge", self, o)
    def __eq__(self, o): return _apply("eq", self, o)
    def __ne__(self, o): return _apply("ne", self, o)
    def __and__(self, o): return _logic("and")(self, o)
    def __rand__(self, o): return _logic("and")(o, self)
    def __or__(self, o): return _logic("or")(self, o)
    def __ror__(self, o): return _logic("or")(o, self)
    def __invert__(self): return _not(self)

    def __bool__(self):
        if self.op == "const":
            return bool(self.value)
        if _ACTIVE is None:
            raise TraceError("truth value of a traced expression outside of a trace")
        return _ACTIVE.decide(self if self.is_bool else _apply("ne", self, 0.0))

    def _concrete(self, *a):
        if self.op == "const":
            return self.value
        raise TraceError("a traced value was converted to a Python number")

    def __float__(self): return float(self._concrete())
    def __int__(self): return int(self._concrete())
    __index__ = __int__

    real = property(lambda self: self)
    imag = property(lambda self: _const(0.0))

    def __repr__(self):
        if self.op == "const":
            return repr(self.value)
        if self.op == "in":
            return "%s[%d]" % self.value
        return "%s(%s)" % (self.op, ", ".join(repr(a) for a in self.args))


# numpy's loops over object arrays call a method named like the ufunc on every element
for _name, _impl in _UFUNCS.items():
    if not hasattr(Expr, _name):
        setattr(Expr, _name, (lambda self, *a, _f=_impl: _f(self, *a)))


_UFUNCS["clip"] = lambda a, lo, hi: _apply("minimum", _apply("maximum", a, lo), hi)


class ExprArray(np.ndarray):
    """The traced input vector: an object array whose ufunc calls build expressions
    directly (``np.maximum(x, 0)`` becomes one fmaxf per element instead of a condition
    to explore, ``np.sign`` / ``np.abs`` work), whatever numpy's own loops over object
    arrays would do; everything else (indexing, slicing, reductions by + and *, dot
    products) is numpy's."""

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        plain = [i.view(np.ndarray) if isinstance(i, ExprArray) else i for i in inputs]
        impl = _UFUNCS.get(ufunc.__name__)
        if "out" in kwargs:
            raise TraceError("ufuncs writing into an existing array")
        if impl is not None and method == "__call__" and not kwargs:
            out = np.frompyfunc(impl, ufunc.nin, 1)(*plain)
        elif (impl is not None and method == "reduce" and plain[0].ndim == 1
              and kwargs.get("axis", 0) in (0, None) and not kwargs.get("keepdims")
              and len(plain[0]) > 0):
            out = plain[0][0]
            for v in plain[0][1:]:
                out = impl(out, v)
        else:
            out = getattr(ufunc, method)(*plain, **kwargs)
        if isinstance(out, np.ndarray) and out.dtype == object:
            return out.view(ExprArray)
        return out


# ----------------------------------------------------------------- math stand-ins
class _MathShim:
    """Looks like the ``math`` module; functions accept traced values."""

    _NAMES = {"sin": "sin", "cos": "cos", "tan": "tan", "asin": "asin", "acos": "acos",
              "atan": "atan", "atan2": "atan2", "sinh": "sinh", "cosh": "cosh", "tanh": "tanh",
              "asinh": "asinh", "acosh": "acosh", "atanh": "atanh", "exp": "exp",
              "expm1": "expm1", "log2": "log2", "log10": "log10", "log1p": "log1p",
              "sqrt": "sqrt", "pow": "pow", "fabs": "fabs", "floor": "floor", "ceil": "ceil",
              "trunc": "trunc", "fmod": "fmod", "hypot": "hypot", "copysign": "copysign",
              "degrees": "degrees", "radians": "radians", "erf": "erf", "erfc": "erfc",
              "gamma": "gamma", "lgamma": "lgamma", "isnan": "isnan", "isinf": "isinf",
              "isfinite": "isfinite", "ldexp": "ldexp"}

    def __getattr__(self, name):
        real = getattr(math, name)
        if not callable(real):
            return real
        return self.function(name, real)

    @classmethod
    def function(cls, name, real):
        def traced(*args):
            if not any(isinstance(a, Expr) for a in args):
                return real(*args)
            if name == "log":
                if len(args) == 2:
                    return _apply("div", _apply("log", args[0]), _apply("log", args[1]))
                return _apply("log", args[0])
            if name not in cls._NAMES:
                raise TraceError("math.%s of a traced value" % name)
            return _UFUNCS[cls._NAMES[name]](*args)
        traced.__name__ = name
        return traced


_MATH = _MathShim()
_STORE_OPS = {"STORE_ATTR", "STORE_SUBSCR", "STORE_GLOBAL", "STORE_DEREF", "DELETE_ATTR",
              "DELETE_SUBSCR", "DELETE_GLOBAL", "DELETE_DEREF"}


def _swap(value):
    if value is math:
        return _MATH
    if isinstance(value, types.BuiltinFunctionType) and getattr(value, "__module__", None) == "math":
        return _MathShim.function(value.__name__, value)
    return value


def _check_code(code):
    for ins in dis.get_instructions(code):
        if ins.opname in _STORE_OPS:
            raise TraceError("the function stores to an attribute, item, global or closure "
                             "variable (%s): it may keep state between calls" % ins.opname)
    for const in code.co_consts:
        if isinstance(const, types.CodeType):
            _check_code(const)


def _for_tracing(fn):
    """`fn` with the math module (and functions imported from it) replaced by stand-ins."""
    if isinstance(fn, np.ufunc):
        return fn
    if not inspect.isfunction(fn):
        call = getattr(type(fn), "__call__", None)
        if inspect.isfunction(call):
            _check_code(call.__code__)
        return fn
    _check_code(fn.__code__)
    names = set(fn.__code__.co_names)
    globs = fn.__globals__
    swapped = {k: _swap(globs[k]) for k in names if k in globs and _swap(globs[k]) is not globs[k]}
    closure = fn.__closure__
    if closure is not None:
        cells = []
        for cell in closure:
            try:
                cells.append(types.CellType(_swap(cell.cell_contents)))
            except ValueError:  # empty cell
                cells.append(cell)
        closure = tuple(cells)
    if not swapped and closure == fn.__closure__:
        return fn
    new_globals = dict(globs)
    new_globals.update(swapped)
    new = types.FunctionType(fn.__code__, new_globals, fn.__name__, fn.__defaults__, closure)
    new.__kwdefaults__ = fn.__kwdefaults__
    return new


# ----------------------------------------------------------------- tracing
def _run(fn, tracer, t_in, x_dim, out_dim):
    global _ACTIVE
    previous, _ACTIVE = _ACTIVE, tracer
    try:
        args = []
        if t_in:
            args.append(_node("in", value=("t", 0)))
        if x_dim is not None:
            x = np.empty(x_dim, dtype=object)
            for i in range(x_dim):
                x[i] = _node("in", value=("x", i))
            args.append(x.view(ExprArray))
        try:
            result = fn(*args)
        except TraceError:
            raise
        except Exception as e:  # noqa: BLE001 -- anything the function does with symbols
            raise TraceError("tracing failed with %s: %s" % (type(e).__name__, e))
        try:
            flat = np.asarray(result, dtype=object).ravel()
            outputs = [_wrap(v) for v in flat]
        except TraceError:
            raise
        except Exception as e:  # noqa: BLE001
            raise TraceError("unusable return value: %s" % (e,))
        if len(outputs) != out_dim:
            raise TraceError("the function returned %d values, %d expected" % (len(outputs), out_dim))
        return outputs
    finally:
        _ACTIVE = previous


def _explore(fn, tracer, prefix, t_in, x_dim, out_dim, budget):
    """Outputs of `fn` as a tree of selects over the conditions it asks about."""
    global _ACTIVE
    if budget[0] <= 0:
        raise TraceError("more than %d paths through the function's conditions" % MAX_RUNS)
    budget[0] -= 1
    tracer.forced, tracer.conditions, tracer.answers, tracer.seen = list(prefix), [], [], {}
    outputs = _run(fn, tracer, t_in, x_dim, out_dim)
    conditions, answers = list(tracer.conditions), list(tracer.answers)
    for k in reversed(range(len(prefix), len(conditions))):
        other = _explore(fn, tracer, answers[:k] + [False], t_in, x_dim, out_dim, budget)
        previous, _ACTIVE = _ACTIVE, tracer
        try:
            outputs = [_select(conditions[k], a, b) for a, b in zip(outputs, other)]
        finally:
            _ACTIVE = previous
    return outputs


class Traced:
    """Result of `trace`: ``outputs`` (one expression per output element), the input
    layout, and ``code`` for ``plan_direct``."""

    def __init__(self, outputs, t_in, x_dim):
        self.outputs, self.t_in, self.x_dim = outputs, t_in, x_dim
        self.input_names = (["t"] if t_in else []) + (["x"] if x_dim is not None else [])
        self.init = ""
        self.code = generate(outputs)

    def __call__(self, t=None, x=None):
        return evaluate(self.outputs, t, x)


def trace(fn, t_in, x_dim, out_dim):
    """Trace ``fn(t, x)`` (``t`` passed if `t_in`, ``x`` of length `x_dim` unless None)
    returning `out_dim` values."""
    target = _for_tracing(fn)
    budget = [MAX_RUNS]
    first = Traced(_explore(target, _Tracer(), [], t_in, x_dim, out_dim, budget), t_in, x_dim)
    again = Traced(_explore(target, _Tracer(), [], t_in, x_dim, out_dim, [MAX_RUNS]), t_in, x_dim)
    if first.code != again.code:
        raise TraceError("two traces of the function differ (random numbers or internal state)")
    return first


# ----------------------------------------------------------------- code, evaluation
def _order(outputs):
    """Nodes reachable from `outputs`, arguments before users."""
    order, seen, stack = [], set(), [(o, False) for o in reversed(outputs)]
    while stack:
        node, done = stack.pop()
        if done:
            order.append(node)
            continue
        if id(node) in seen:
            continue
        seen.add(id(node))
        stack.append((node, True))
        for a in reversed(node.args):
            if id(a) not in seen:
                stack.append((a, False))
    return order


def _literal(value):
    if isinstance(value, bool):
        return "true" if value else "false"
    if math.isnan(value):
        return "NAN"
    if math.isinf(value):
        return "INFINITY" if value > 0 else "-INFINITY"
    if abs(value) > float(np.finfo(np.float32).max):  # beyond float32
        return "INFINITY" if value > 0 else "-INFINITY"
    text = repr(float(np.float32(value)))
    if "e" not in text and "." not in text:
        text += ".0"
    return text + "f"


def generate(outputs):
    """Statements computing ``OUTPUT__[i]`` from ``t[0]`` / ``x[i]`` in float32."""
    names, lines = {}, []

    def as_float(node):
        name = names[id(node)]
        return "(%s ? 1.0f : 0.0f)" % name if node.is_bool else name

    def as_bool(node):
        name = names[id(node)]
        return name if node.is_bool else "(%s != 0.0f)" % name

    for node in _order(outputs):
        op, args = node.op, node.args
        if op == "const":
            names[id(node)] = _literal(node.value)
            continue
        if op == "in":
            expr = "%s[%d]" % node.value
        elif op == "neg":
            expr = "-%s" % as_float(args[0])
        elif op in _UNARY:
            expr = "%s(%s)" % (_UNARY[op][0], as_float(args[0]))
        elif op in _BINARY_FN:
            expr = "%s(%s, %s)" % (_BINARY_FN[op][0], as_float(args[0]), as_float(args[1]))
        elif op in _INFIX:
            expr = "%s %s %s" % (as_float(args[0]), _INFIX[op][0], as_float(args[1]))
        elif op in _COMPARE:
            expr = "%s %s %s" % (as_float(args[0]), _COMPARE[op][0], as_float(args[1]))
        elif op in _LOGIC:
            expr = "%s %s %s" % (as_bool(args[0]), _LOGIC[op][0], as_bool(args[1]))
        elif op == "not":
            expr = "!%s" % as_bool(args[0])
        elif op == "select":
            conv = as_bool if node.is_bool else as_float
            expr = "%s ? %s : %s" % (as_bool(args[0]), conv(args[1]), conv(args[2]))
        else:
            raise TraceError("no code for %r" % op)
        name = "v%d" % len(lines)
        lines.append("const %s %s = %s;" % ("bool" if node.is_bool else "float", name, expr))
        names[id(node)] = name
    for i, out in enumerate(outputs):
        lines.append("%s[%d] = %s;" % (OUTPUT_NAME, i, as_float(out)))
    return "\n".join(lines)


def evaluate(outputs, t=None, x=None):
    """The traced outputs for concrete inputs, in double precision on the host."""
    values = {}
    for node in _order(outputs):
        op = node.op
        a = [values[id(arg)] for arg in node.args]
        try:
            if op == "const":
                v = node.value
            elif op == "in":
                v = float(t) if node.value[0] == "t" else float(x[node.value[1]])
            elif op == "select":
                v = a[1] if a[0] else a[2]
            elif op == "not":
                v = not a[0]
            else:
                impl = (_UNARY.get(op) or _BINARY_FN.get(op) or _INFIX.get(op)
                        or _COMPARE.get(op) or _LOGIC.get(op))[1]
                v = impl(*a) if op in _LOGIC else impl(*[float(q) for q in a])
        except (ValueError, ZeroDivisionError, OverflowError):
            v = float("nan")
        values[id(node)] = v
    return np.array([float(values[id(o)]) for o in outputs])
