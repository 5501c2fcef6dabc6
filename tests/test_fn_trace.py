"""Python functions traced into kernel code (`nengo_ocl_amd.fn_trace`): the traced
expression graph, evaluated on the host in double precision, must reproduce the function
it came from on random inputs; what cannot be traced must be refused, not mistranslated;
the generated kernels must compile for gfx950.  The function families follow the
reference's translator tests (nengo_ocl/tests/test_ast_conversion.py: slices :28-36,
nested calls :39-47, closures :95-104, lambdas :114-145, the math / numpy function tables
:207-296, vector functions :299-328 and the constructs of `print_various_ocl` :331-503)."""

import math
from math import sin as imported_sin

import numpy as np
import pytest

from nengo_ocl_amd import fn_trace as ft

SCALE = 3.0
W = np.array([0.5, -1.0, 2.0])


def _helper(v):
    return v ** 2 + 1


def closures(t, x):
    local = 0.25
    return SCALE * x[0] + t * local


def loops(x):
    acc = 0
    for i in range(len(x)):
        acc = acc + (i + 1) * x[i]
    return [acc, acc / len(x)]


def branches(x):
    if x[0] > 1:
        y = x[0] * 2
    elif x[0] < -1:
        y = -x[0]
    else:
        y = x[1]
    return y + 1


class Scaler:
    def __init__(self, k):
        self.k = k

    def __call__(self, t, x):
        return self.k * x[0] ** 2


CASES = [
    # function, takes t, size of x (None: no x), number of outputs
    (lambda t: t, True, None, 1),
    (lambda t, x: x, True, 3, 3),
    (closures, True, 1, 1),
    (loops, False, 4, 2),
    (branches, False, 2, 1),
    (Scaler(2.5), True, 1, 1),
    (lambda t, x: x[0] * x[1], True, 2, 1),
    (lambda x: [math.sin(x[0]) * 2, np.cos(x[1]) + math.pi, imported_sin(x[0])], False, 2, 3),
    (lambda x: x + 3 if all(x > 2) else x - 1, False, 3, 3),
    (lambda x: [np.maximum(0.1, np.sin(2)) * x[4 - i] for i in range(5)], False, 5, 5),
    (lambda x: x[len(x) // 2:], False, 4, 2),
    (lambda x: x[1:3], False, 4, 2),
    (lambda x: np.sum(x), False, 3, 1),
    (lambda x: np.mean(x), False, 3, 1),
    (lambda x: x.min(), False, 4, 1),
    (lambda x: x.max() - np.min(x), False, 4, 1),
    (lambda x: np.sqrt((x ** 2).mean()), False, 5, 1),
    (lambda x: np.dot(W, x), False, 3, 1),
    (lambda x: _helper(x[0]) / _helper(x[1]), False, 2, 1),
    (lambda x: max(x[0], x[1], 0.3) + min(x[0], 0.0), False, 2, 1),
    (lambda x: abs(x[0]) % 0.7 + x[1] // 0.3 + (-x[0]) % 1.5, False, 2, 1),
    (lambda x: 1.0 if x[0] > 0 and x[1] > 0 else (-1.0 if x[0] < -0.5 or x[1] > 3 else 0.0), False, 2, 1),
    (lambda x: np.where(x > 0, x, 0.1 * x), False, 3, 3),
    (lambda t: np.sin(2 * np.pi * t) * np.exp(-t), True, None, 1),
    (np.sin, True, None, 1),
    (lambda t, x: [t > 0.5, x[0] >= x[1], not (x[0] > 0)], True, 2, 3),
    (lambda x: np.prod(x) + np.linalg.norm(x), False, 3, 1),
    (lambda x: np.clip(x, -0.5, 0.5), False, 3, 3),
    (lambda x: sorted(x)[1], False, 3, 1),
    (lambda x: np.sign(x) * np.abs(x) ** 1.5, False, 2, 2),
    (lambda x: (x[0] ** 3, x[0] ** 0.5 if x[0] > 0 else 0.0, 2 ** x[1], x[1] ** -2), False, 2, 4),
    (lambda x: round(x[0]) + math.floor(x[1]) + math.ceil(x[0]) + np.trunc(x[1]), False, 2, 1),
    (lambda t: [1.0, 2.0], True, None, 2),
    # (appended: the GPU test names earlier cases by position)
    (lambda x: [np.logaddexp(x[0], x[1]), np.ldexp(x[0], 2), 1.0 if np.isfinite(x[1]) else 0.0,
                2.0 if np.isnan(x[0]) else x[0], -1.0 if np.signbit(x[1]) else 1.0], False, 2, 5),
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_trace_reproduces_the_function(case):
    fn, t_in, x_dim, out_dim = CASES[case]
    traced = ft.trace(fn, t_in, x_dim, out_dim)
    assert traced.input_names == (["t"] if t_in else []) + (["x"] if x_dim else [])
    rng = np.random.RandomState(case)
    for _ in range(300):
        t = rng.uniform(0, 2)
        x = rng.uniform(-3, 4, size=x_dim) if x_dim else None
        args = ([t] if t_in else []) + ([x] if x_dim else [])
        want = np.asarray(fn(*args), dtype=np.float64).ravel()
        np.testing.assert_allclose(traced(t, x), want, rtol=1e-13, atol=1e-13)


UNARY_DOMAINS = {"arccos": (-1, 1), "arcsin": (-1, 1), "arctanh": (-1, 1), "arccosh": (1, 10),
                 "log": (0.01, 10), "log2": (0.01, 10), "log10": (0.01, 10), "log1p": (-0.9, 10),
                 "sqrt": (0, 10), "gamma": (0.1, 10), "lgamma": (0.1, 10)}


@pytest.mark.parametrize("module", ["numpy", "math"])
def test_function_tables(module):
    """Every one-argument function of the numpy / math tables, traced and evaluated."""
    np_names = ["sin", "cos", "tan", "arcsin", "arccos", "arctan", "sinh", "cosh", "tanh",
                "arcsinh", "arccosh", "arctanh", "exp", "exp2", "expm1", "log", "log2", "log10",
                "log1p", "sqrt", "cbrt", "fabs", "floor", "ceil", "trunc", "rint", "square",
                "reciprocal", "negative", "absolute", "sign", "deg2rad", "rad2deg", "degrees",
                "radians"]
    math_names = ["sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "asinh",
                  "acosh", "atanh", "exp", "expm1", "log", "log2", "log10", "log1p", "sqrt", "fabs",
                  "floor", "ceil", "trunc", "degrees", "radians", "erf", "erfc", "gamma", "lgamma"]
    alias = {"asin": "arcsin", "acos": "arccos", "atanh": "arctanh", "acosh": "arccosh"}
    rng = np.random.RandomState(1)
    for name in (np_names if module == "numpy" else math_names):
        real = getattr(np if module == "numpy" else math, name)
        fn = (lambda x, f=real: f(x[0]))
        if module == "math":  # the stand-in is found through the function's globals
            fn = eval("lambda x: math.%s(x[0])" % name, {"math": math})
        traced = ft.trace(fn, False, 1, 1)
        lo, hi = UNARY_DOMAINS.get(alias.get(name, name), (-3, 3))
        for v in rng.uniform(lo, hi, size=50):
            want = float(real(v))
            assert traced(None, [v])[0] == pytest.approx(want, rel=1e-12, abs=1e-12), name
    two = {"numpy": [np.arctan2, np.hypot, np.fmod, np.copysign, np.power, np.maximum, np.minimum,
                     np.fmax, np.fmin, np.add, np.subtract, np.multiply, np.divide,
                     np.floor_divide, np.remainder],
           "math": [math.atan2, math.hypot, math.fmod, math.copysign, math.pow, math.log]}
    for real in two[module]:
        if module == "math":
            fn = eval("lambda x: math.%s(x[0], x[1])" % real.__name__, {"math": math})
        else:
            fn = (lambda x, f=real: f(x[0], x[1]))
        traced = ft.trace(fn, False, 2, 1)
        for a, b in rng.uniform(0.1, 5, size=(50, 2)):
            assert traced(None, [a, b])[0] == pytest.approx(float(real(a, b)), rel=1e-12), real


def _stateful_factory():
    calls = []

    def fn(t):
        calls.append(t)
        return len(calls)

    return fn


class Counter:
    def __init__(self):
        self.n = 0

    def __call__(self, t):
        self.n += 1
        return self.n


def _store_item(x):
    y = np.zeros(2)
    y[0] = x[0]
    return y


REFUSED = [
    (lambda x: float(x[0]), False, 1, 1),                 # needs a real number
    (lambda x: int(x[0]) + 1, False, 1, 1),
    (lambda x: np.random.rand() * x[0], False, 1, 1),    # another value on every call
    (lambda t: np.random.normal(), True, None, 1),
    (lambda x: [x[0], x[1]], False, 2, 3),                # wrong number of outputs
    (lambda x: x[0] if x[0] > 0 else [x[0], x[1]], False, 2, 1),
    (lambda x: np.fft.fft(x).real, False, 4, 4),          # a library that wants floats
    (lambda x: "text", False, 1, 1),
    (_stateful_factory(), True, None, 1),
    (Counter(), True, None, 1),
    (_store_item, False, 1, 2),
    (lambda x: [v for v in range(int(abs(x[0])))], False, 1, 1),
]


@pytest.mark.parametrize("case", range(len(REFUSED)))
def test_untraceable_functions_are_refused(case):
    fn, t_in, x_dim, out_dim = REFUSED[case]
    with pytest.raises(NotImplementedError):
        ft.trace(fn, t_in, x_dim, out_dim)


def test_too_many_paths_are_refused():
    fn = lambda x: sum(1.0 if v > 0 else 0.0 for v in x)  # 2^12 sign patterns
    with pytest.raises(ft.TraceError, match="paths"):
        ft.trace(fn, False, 12, 1)
    assert ft.trace(fn, False, 5, 1)(None, [1, -1, 2, -2, 3])[0] == 3


def test_constants_keep_type_and_sign():
    traced = ft.trace(lambda x: [True, 1.0, -0.0, 0.0, np.inf, 1e300, x[0] * 0], False, 1, 7)
    assert "true ? 1.0f : 0.0f" in traced.code.replace("(", "").replace(")", "")
    assert "-0.0f" in traced.code and "INFINITY" in traced.code
    out = traced(None, [2.0])
    assert out[0] == 1 and out[1] == 1 and np.signbit(out[2]) and not np.signbit(out[3])


def test_generated_kernels_compile_for_gfx950():
    """Every traced case through the run-time compiler (needs no device); a source that does
    not compile is reported with the compiler's message."""
    from nengo_ocl_amd import _lib
    from nengo_ocl_amd import hipra_nonlinearities as nl

    lib = _lib.lib()
    for fn, t_in, x_dim, out_dim in CASES:
        traced = ft.trace(fn, t_in, x_dim, out_dim)
        source = nl.direct_kernel_source(traced.code, traced.init, traced.input_names)
        assert nl.compile_direct(lib, source)
    with pytest.raises(NotImplementedError, match="nosuch"):
        nl.compile_direct(lib, nl.direct_kernel_source("OUTPUT__[0] = nosuch(t[0]);", "", ["t"]))
    with pytest.raises(NotImplementedError):
        nl.direct_kernel_source("", "", ["a", "b", "c"])


def test_classification_and_scaling_functions():
    """isnan / isinf / isfinite / signbit, ldexp, logaddexp / logaddexp2 (the rest of the
    reference translator's table, ast_conversion.py:103-105, 137, 164-171, 194): traced from
    numpy and from math, against the functions themselves, special values included."""
    special = [0.0, -0.0, 1.5, -2.25, np.inf, -np.inf, np.nan, 1e-40, 3e38]
    for name in ("isnan", "isinf", "isfinite", "signbit"):
        traced = ft.trace(lambda x, f=getattr(np, name): f(x[0]), False, 1, 1)
        for v in special:
            assert bool(traced(None, [v])[0]) == bool(getattr(np, name)(v)), (name, v)
    for name in ("isnan", "isinf", "isfinite"):
        traced = ft.trace(eval("lambda x: 1.0 if math.%s(x[0]) else 0.0" % name, {"math": math}),
                          False, 1, 1)
        for v in special:
            assert bool(traced(None, [v])[0]) == bool(getattr(math, name)(v)), (name, v)
    rng = np.random.RandomState(3)
    two = {"ldexp": lambda a, b: np.ldexp(a, int(b)), "logaddexp": np.logaddexp,
           "logaddexp2": np.logaddexp2}
    for name, real in two.items():
        fn = (lambda x: np.ldexp(x[0], 3)) if name == "ldexp" else (lambda x, f=real: f(x[0], x[1]))
        traced = ft.trace(fn, False, 2, 1)
        for a, b in rng.uniform(-30, 30, size=(50, 2)):
            want = float(np.ldexp(a, 3)) if name == "ldexp" else float(real(a, b))
            assert traced(None, [a, b])[0] == pytest.approx(want, rel=1e-12, abs=1e-12), name
    big = ft.trace(lambda x: np.logaddexp(x[0], x[1]), False, 2, 1)
    assert big(None, [1000.0, 999.0])[0] == pytest.approx(float(np.logaddexp(1000.0, 999.0)))
    assert ft.trace(lambda x: math.ldexp(x[0], 2), False, 1, 1)(None, [1.5])[0] == 6.0
