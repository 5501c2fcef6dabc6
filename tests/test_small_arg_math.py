"""The small-argument expm1 / log1p of the neuron kernels (csrc/small_arg_math.h), built for
the host by g++ from the same header the device code includes, against the host's math
library in extended precision: errors in units of the last place of a double, and what
the neuron update keeps of them (the value rounded to float32).  Fused multiply-adds are
IEEE operations on both sides, so the host build computes the device's bits."""

import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "nengo-ocl_amd", "csrc")

WRAPPER = r"""
#include "small_arg_math.h"
extern "C" void both(const double* x, long n, double* em, double* lp, double* em_any, double* lp_any) {
    for (long i = 0; i < n; ++i) {
        em[i] = nhip_expm1_small(x[i]);
        lp[i] = nhip_log1p_small(x[i]);
        em_any[i] = nhip_expm1(x[i]);
        lp_any[i] = nhip_log1p(x[i]);
    }
}
"""


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    d = tmp_path_factory.mktemp("small_arg_math")
    src = d / "wrapper.cpp"
    src.write_text(WRAPPER)
    so = d / "libsmallarg.so"
    subprocess.check_call(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-I", CSRC,
                           str(src), "-o", str(so), "-lm"])
    lib = ctypes.CDLL(str(so))
    P = ctypes.c_void_p
    lib.both.argtypes = [P, ctypes.c_long, P, P, P, P]
    lib.both.restype = None
    return lib


def run(lib, x):
    x = np.ascontiguousarray(x, dtype=np.float64)
    outs = [np.empty_like(x) for _ in range(4)]
    lib.both(x.ctypes.data, x.size, *[o.ctypes.data for o in outs])
    return outs


def ulps(got, want_ld):
    """|got - want| in units of the last place of the double nearest to want."""
    want = want_ld.astype(np.float64)
    spacing = np.spacing(np.abs(want))
    err = np.abs(got.astype(np.longdouble) - want_ld) / spacing.astype(np.longdouble)
    return np.where(want == 0, (got != want).astype(np.longdouble), err)


def samples(rng, n):
    # float32 values, as the callers pass them: uniform in the interval, logarithmically
    # spread towards zero, the ends of the interval, zeros of both signs, denormals
    uniform = rng.uniform(-0.0625, 0.0625, size=n).astype(np.float32)
    small = (-(10.0 ** rng.uniform(-12, -1.21, size=n))).astype(np.float32)
    edge = np.array([0.0, -0.0, 0.0625, -0.0625, 0.05, -0.05, -0.04877058, 1e-45, -1e-45,
                     1e-38, -1e-38, np.float32(-0.001) / np.float32(0.02)], dtype=np.float32)
    return np.concatenate([uniform, small, edge]).astype(np.float64)


def test_small_argument_series_against_extended_precision(lib):
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("no extended-precision long double on this host")
    rng = np.random.RandomState(5)
    x = samples(rng, 1_000_000)
    em, lp, _, _ = run(lib, x)
    xl = x.astype(np.longdouble)
    for name, got, want in (("expm1", em, np.expm1(xl)), ("log1p", lp, np.log1p(xl))):
        e = ulps(got, want)
        print("%s: largest error %.3f units in the last place of a double" % (name, float(e.max())))
        assert float(e.max()) <= 0.75, name
        # what the neuron update keeps: the value rounded to float32
        as_float = got.astype(np.float32)
        want_float = want.astype(np.float32)  # one rounding from extended precision
        differ = int((as_float.view(np.uint32) != want_float.view(np.uint32)).sum())
        print("%s: %d of %d float32 results differ from the correctly rounded value" % (
            name, differ, x.size))
        assert differ <= 2, name
        # signs of zero
        z = x == 0
        assert np.array_equal(np.signbit(got[z]), np.signbit(x[z]))


def test_other_arguments_take_the_library_routine(lib):
    x = np.array([-0.0626, 0.07, -0.5, 1.0, -0.999, 30.0, -30.0, np.inf, np.nan], dtype=np.float64)
    _, _, em, lp = run(lib, x)
    with np.errstate(all="ignore"):
        want_em, want_lp = np.expm1(x), np.log1p(x)
    for got, want in ((em, want_em), (lp, want_lp)):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isinf(got), np.isinf(want))
        ok = np.isfinite(want)
        # the host library here, numpy possibly with a routine of its own: 2 ulp apart at most
        assert np.all(np.abs(got[ok] - want[ok]) <= 2 * np.spacing(np.abs(want[ok])))
    # and inside the interval the two entry points are the same function
    inner = np.array([-0.05, 0.03, -0.0625], dtype=np.float64)
    a, b, c, d = run(lib, inner)
    assert np.array_equal(a, c) and np.array_equal(b, d)
