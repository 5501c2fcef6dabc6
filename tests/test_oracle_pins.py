"""Pins for the CPU oracle: each restated kernel is checked against something that
does not share its code -- literal vectors held by the reference's own tests,
closed forms, float64 brute force, library routines (numpy / scipy).

The reference itself cannot be imported here (nengo, pyopencl and mako are not
installed), so these are what fix the oracle's behaviour; the GPU tests then
compare the HIP kernels with the oracle.
"""

import numpy as np
import pytest

from helpers import PHILOX_KNOWN_ANSWERS, RA, clone
from oracle import oracle as orc


# ------------------------------------------------------------------ GEMV
def golden(name):
    import json
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                        "reference_test_vectors.json")
    with open(path) as f:
        return json.load(f)[name]


def test_gemv_literal_vectors():
    """nengo_ocl/tests/test_clra_gemv.py:60-93 (fixture gemv_basic): Y0 = 4.5, Y1 = [3.3, 5.9]."""
    g = golden("gemv_basic")
    A, X, Y = RA(g["A"]), RA(g["X"]), RA(g["Y"])
    A_js = RA(g["A_js"], dtype=np.int32)
    X_js = RA(g["X_js"], dtype=np.int32)
    orc.plan_block_gemv(None, g["alpha"], A, A_js, X, X_js, g["beta"], Y).plans[0]()
    for i, want in enumerate(g["expected_Y"]):
        np.testing.assert_allclose(Y[i].ravel(), want, rtol=1e-6)


@pytest.mark.parametrize("k,p,m,n", [(4, 1, 10, 10), (10, 1, 550, 550), (4, 4, 10, 10),
                                     (4, 4, 500, 300)])
def test_gemv_seeded_random_against_float64(k, p, m, n):
    """The seeded sweep of test_clra_gemv.py:96-145 (RandomState(3294), alpha 0.5, beta 0.1)."""
    rng = np.random.RandomState(3294)
    aa = [rng.normal(size=(m, n)) for _ in range(k)]
    xx = [rng.normal(size=n) for _ in range(k)]
    yy = [rng.normal(size=m) for _ in range(k)]
    ajs = [rng.randint(k, size=p) for _ in range(k)]
    xjs = [rng.randint(k, size=p) for _ in range(k)]
    A, X, Y = RA(aa), RA(xx), RA(yy)
    Y0 = clone(Y)
    orc.plan_block_gemv(None, 0.5, A, RA(ajs, dtype=np.int32), X, RA(xjs, dtype=np.int32), 0.1, Y).plans[0]()
    for i in range(k):
        ref = 0.1 * Y0[i].astype(np.float64)
        for aj, xj in zip(ajs[i], xjs[i]):
            ref += 0.5 * (A[aj].astype(np.float64) @ X[xj].astype(np.float64))
        np.testing.assert_allclose(Y[i], ref, rtol=1e-4, atol=1e-4)


def test_gemv_gamma_yin_and_strides():
    """gamma, a Y_in different from Y, a transposed-stride X and a row-strided A: a dropped
    term, a swapped operand or a wrong stride changes the result."""
    from nengo_ocl_amd.raggedarray import RaggedArray

    rng = np.random.RandomState(1234)
    base = RA([rng.rand(6, 10), rng.rand(40), rng.rand(6), rng.rand(6)])
    s = base.starts
    base.add_views([s[0] + 2, s[1] + 1], [6, 7], [7, 1], [10, 5], [1, 1])  # A = M[:, 2:9], x = v[1::5][:7]
    Y = RaggedArray.from_buffer(base.buf, [s[2]], [6], [1], [1], [1])
    Yin = RaggedArray.from_buffer(base.buf, [s[3]], [6], [1], [1], [1])
    expect = 0.7 + 0.6 * base[3][:, 0].astype(np.float64) + 0.5 * (
        base[0][:, 2:9].astype(np.float64) @ base[1][1::5][:7, 0].astype(np.float64))
    orc.plan_block_gemv(None, 0.5, base, [np.array([4])], base, [np.array([5])], 0.6, Y, Y_in=Yin,
                        gamma=0.7).plans[0]()
    np.testing.assert_allclose(Y[0][:, 0], expect, rtol=1e-6)


def test_gemv_block_order_is_the_reference_order():
    """The four strided partial sums per 128-column tile (fused multiply-add per
    element), (s0+s2)+(s1+s3), tiles in order (clra_gemv.py:1043-1058, :1148-1153),
    replayed step by step in numpy."""
    rng = np.random.RandomState(5)
    n = 300  # three tiles: 128, 128, 44
    a = rng.normal(size=(1, n)).astype(np.float32)
    x = rng.normal(size=n).astype(np.float32)
    y0 = np.float32(0.25)
    Y = RA([[y0]])
    orc.plan_block_gemv(None, 1.0, RA([a]), [np.array([0])], RA([x]), [np.array([0])], 1.0, Y).plans[0]()
    total = y0
    for c0 in range(0, n, 128):
        s = np.zeros(4, dtype=np.float32)
        for jj in range(min(128, n - c0)):  # fused multiply-add: exact product, one rounding
            s[jj % 4] = np.float32(np.longdouble(a[0, c0 + jj]) * np.longdouble(x[c0 + jj])
                                   + np.longdouble(s[jj % 4]))
        total = np.float32(total + np.float32(np.float32(s[0] + s[2]) + np.float32(s[1] + s[3])))
    assert Y[0][0, 0] == total


@pytest.mark.parametrize("coefs", [(0.1, 0.3, 0.7), ([0.1, 0.1], [0.3, 0.25], [0.7, 0.7])],
                         ids=["literals", "beta-per-item"])
def test_gemv_coefficients_are_double_literals_or_float_arrays(coefs):
    """`float_cl_clra` (clra_gemv.py:17-32): a coefficient that is the same for every item is
    written into the kernel text as a double literal, so `alpha * (s0 + s1)` (:1058),
    `beta * yin` (:1148) and `sum + gamma` (:1153) are double operations rounded to float32
    once each; coefficients that differ between items are float32 arrays and the operations
    float32.  Replayed in numpy with values float32 does not hold (0.1, 0.3, 0.7)."""
    rng = np.random.RandomState(8)
    n = 200  # two tiles
    m = 40
    A = [rng.normal(size=(m, n)).astype(np.float32) for _ in range(2)]
    x = rng.normal(size=n).astype(np.float32)
    y0 = [rng.normal(size=m).astype(np.float32) for _ in range(2)]
    Y = RA(y0)
    alpha, beta, gamma = coefs
    orc.plan_block_gemv(None, alpha, RA(A), [np.array([0]), np.array([1])], RA([x]),
                        [np.array([0]), np.array([0])], beta, Y, gamma=gamma).plans[0]()

    def typed(c, b):  # the operand as the kernel sees it: double literal or float32 element
        c = np.asarray(c, dtype=np.float64)
        if c.ndim == 0 or len(set(c.tolist())) == 1:
            return np.float64(c.ravel()[0])
        return np.float32(c[b])

    changed = False
    for b in range(2):
        al, be, ga = typed(alpha, b), typed(beta, b), typed(gamma, b)
        for r in range(m):
            total = np.float32(be * y0[b][r])  # numpy promotes float32 * float64 to float64
            plain = np.float32(np.float32(be) * y0[b][r])
            for c0 in range(0, n, 128):
                s = np.zeros(4, dtype=np.float32)
                for jj in range(min(128, n - c0)):
                    s[jj % 4] = np.float32(np.longdouble(A[b][r, c0 + jj]) * np.longdouble(x[c0 + jj])
                                           + np.longdouble(s[jj % 4]))
                tile = np.float32(np.float32(s[0] + s[2]) + np.float32(s[1] + s[3]))
                total = np.float32(total + np.float32(al * tile))
                plain = np.float32(plain + np.float32(np.float32(al) * tile))
            want = np.float32(total + ga)
            changed |= want != np.float32(plain + np.float32(ga))
            assert Y[b][r, 0] == want, (b, r)
    assert changed  # float32 coefficients would have given other bits somewhere


# ------------------------------------------------------------------- LIF
def lif_step_float64(dt, J, V, W, tau_rc, tau_ref, amplitude=1.0):
    """nengo's LIF.step as the reference's test_lif_step (:35-91) runs it on the host:
    refractory countdown, exponential integration over the non-refractory part of the
    step, spike with interpolated spike time."""
    W = W - dt
    delta_t = np.clip(dt - W, 0, dt)
    V = V - (J - V) * np.expm1(-delta_t / tau_rc)
    spiked = V > 1
    out = spiked * (amplitude / dt)
    t_spike = dt + tau_rc * np.log1p(-(V[spiked] - 1) / (J[spiked] - 1))
    V[V < 0] = 0
    V[spiked] = 0
    W[spiked] = tau_ref + t_spike
    return V, W, out


def test_lif_step_against_float64():
    rng = np.random.RandomState(8)
    dt, ref, amp = 1e-3, 2e-3, 1.0
    n_neurons = [12345, 23456, 34567]
    taus = rng.uniform(15e-3, 80e-3, size=3)
    J = RA([rng.normal(scale=1.2, size=n) for n in n_neurons])
    V = RA([rng.uniform(0, 1, size=n) for n in n_neurons])
    W = RA([rng.uniform(-5 * dt, 5 * dt, size=n) for n in n_neurons])
    S = RA([np.zeros(n) for n in n_neurons])
    V0, W0 = clone(V), clone(W)
    orc.plan_lif(None, dt, J, V, W, S, ref, RA([t * np.ones(n) for t, n in zip(taus, n_neurons)]), amp)()
    n_spikes = 0
    for i in range(3):
        v, w, s = lif_step_float64(dt, J[i][:, 0].astype(np.float64), V0[i][:, 0].astype(np.float64),
                                   W0[i][:, 0].astype(np.float64), taus[i], ref, amp)
        agree = (S[i][:, 0] > 0) == (s > 0)
        assert agree.mean() > 0.9999  # a float32 voltage within rounding of the threshold may differ
        np.testing.assert_allclose(V[i][agree, 0], v[agree], atol=1e-5)
        np.testing.assert_allclose(W[i][agree, 0], w[agree], atol=1e-6)
        np.testing.assert_allclose(S[i][agree, 0], s[agree])
        n_spikes += int((s > 0).sum())
    assert n_spikes > 50  # the spike branch is exercised


def test_lif_constant_input_rate_and_bounds():
    """Constant J: the spike count over 1 s is rate(J) within one spike, where
    rate = 1/(tau_ref + tau_rc*log1p(1/(J-1))); J <= 1 never spikes and V -> J;
    V stays in [0, 1] and S takes two values."""
    dt, tau_rc, tau_ref, amp = 1e-3, 0.02, 0.002, 1.0
    Jv = np.array([0.5, 0.99, 1.0, 1.05, 1.5, 2.0, 5.0, 10.0, 40.0], dtype=np.float32)
    J, V, W, S = RA([Jv]), RA([np.zeros(Jv.size)]), RA([np.zeros(Jv.size)]), RA([np.zeros(Jv.size)])
    plan = orc.plan_lif(None, dt, J, V, W, S, tau_ref, tau_rc, amp)
    counts = np.zeros(Jv.size)
    for _ in range(1000):
        plan()
        counts += S[0][:, 0] * dt
        assert np.all(V[0] >= 0) and np.all(V[0] <= 1)
        assert set(np.unique(S[0])) <= {0.0, np.float32(1000.0)}
    rate = np.zeros(Jv.size)
    m = Jv > 1
    rate[m] = 1.0 / (tau_ref + tau_rc * np.log1p(1.0 / (Jv[m].astype(np.float64) - 1)))
    assert np.all(counts[~m] == 0)
    assert np.all(np.abs(counts - rate) <= 1.0 + 1e-9)
    np.testing.assert_allclose(V[0][:2, 0], Jv[:2], rtol=1e-4)  # subthreshold voltage settles at J


def test_lif_upsample_equals_substeps():
    rng = np.random.RandomState(2)
    dt = 1e-3
    J = RA([rng.normal(1.5, 1.0, size=500)])
    V = RA([rng.uniform(0, 1, size=500)])
    W = RA([rng.uniform(-2 * dt, 2 * dt, size=500)])
    S = RA([np.zeros(500)])
    V2, W2, S2 = clone(V), clone(W), clone(S)
    orc.plan_lif(None, dt, J, V, W, S, 2e-3, 0.02, 1.0, upsample=4)()
    any_spike = np.zeros(500, dtype=bool)
    sub = orc.plan_lif(None, dt / 4, J, V2, W2, S2, 2e-3, 0.02, 1.0)
    for _ in range(4):
        sub()
        any_spike |= S2[0][:, 0] > 0
    np.testing.assert_allclose(V[0], V2[0], atol=1e-6)
    np.testing.assert_allclose(W[0], W2[0], atol=1e-7)
    assert np.array_equal(S[0][:, 0] > 0, any_spike)
    assert set(np.unique(S[0])) <= {0.0, np.float32(1000.0)}  # amp/dt, not amp/(dt/4)


def test_lif_rate_closed_form():
    rng = np.random.RandomState(3)
    Jv = rng.normal(1, 10, size=5000).astype(np.float32)
    J, R = RA([Jv]), RA([np.zeros(Jv.size)])
    orc.plan_lif_rate(None, 1e-3, J, R, 2e-3, 0.03, 1.5)()
    j = np.maximum(Jv.astype(np.float64) - 1, 0)
    with np.errstate(divide="ignore"):
        expect = 1.5 / (2e-3 + 0.03 * np.log1p(1.0 / j))
    np.testing.assert_allclose(R[0][:, 0], expect, rtol=2e-6, atol=1e-6)
    assert np.all(R[0][Jv <= 1] == 0)
    assert np.array_equal(J[0][:, 0], Jv)


# --------------------------------------------------------------- filters
def test_lowpass_step_response():
    """y[n] = a y[n-1] + (1-a) x[n], a = exp(-dt/tau): unit step gives 1 - a^n."""
    dt, tau = 1e-3, 0.005
    a = np.exp(-dt / tau)
    X, Y = RA([np.ones(7)]), RA([np.zeros(7)])
    A, B = RA([[-a]]), RA([[1 - a]])
    (plan,) = orc.plan_linearfilter(None, X, Y, A, B, RA([np.zeros((1, 7))]), RA([np.zeros((1, 7))]))
    for n in range(1, 60):
        plan()
        np.testing.assert_allclose(Y[0][:, 0], 1 - a ** n, rtol=2e-6)


def test_general_filter_against_scipy():
    """Second-order (alpha) synapse, zero-order hold, in the reference's packing
    (simulator.py:1214-1227) against scipy.signal.lfilter; also a 2-D strided signal."""
    from scipy.signal import cont2discrete, lfilter

    dt, tau = 1e-3, 0.005
    numd, dend, _ = cont2discrete(([1.0], [tau * tau, 2 * tau, 1.0]), dt, method="zoh")
    num, den = numd.ravel()[1:], dend[1:]
    rng = np.random.RandomState(4)
    n_steps, shape = 50, (3, 4)
    xs = rng.normal(size=(n_steps,) + shape).astype(np.float32)
    base = RA([np.zeros((3, 6)), np.zeros(shape)])
    from nengo_ocl_amd.raggedarray import RaggedArray

    X = RaggedArray.from_buffer(base.buf, [base.starts[0] + 1], [3], [4], [6], [1])  # columns 1..4 of a 3x6
    Y = base[[1]]
    (plan,) = orc.plan_linearfilter(None, X, Y, RA([den]), RA([num]), RA([np.zeros((2, 12))]),
                                    RA([np.zeros((2, 12))]))
    ys = []
    for n in range(n_steps):
        base[0][:, 1:5] = xs[n]
        plan()
        ys.append(np.array(Y[0]))
    expect = lfilter(np.float32(num).astype(np.float64), np.concatenate([[1.0], np.float32(den)]),
                     xs.astype(np.float64), axis=0)
    np.testing.assert_allclose(np.array(ys), expect, rtol=1e-4, atol=1e-6)


def test_gain_only_filter():
    X, Y = RA([[1.0, -2.0, 3.0]]), RA([np.zeros(3)])
    (plan,) = orc.plan_linearfilter(None, X, Y, RA([[]]), RA([[2.0]]), RA([np.zeros((1, 3))]),
                                    RA([np.zeros((0, 3))]))
    plan()
    assert np.array_equal(Y[0][:, 0], [2.0, -4.0, 6.0])


# ------------------------------------------------- element-wise and copies
def test_elementwise_inc_against_numpy():
    rng = np.random.RandomState(6)
    Xs = [(3, 3), (32, 64), (45, 34), (1, 100)]
    As = [(3, 3), (1, 1), (45, 34), (100, 1)]
    A, X = RA([rng.normal(size=s) for s in As]), RA([rng.normal(size=s) for s in Xs])
    alpha = rng.normal(size=4).astype(np.float32)
    Y = RA([rng.normal(size=np.broadcast(A[i], X[i]).shape) for i in range(4)])
    for inc in (True, False):
        Yo = clone(Y)
        orc.plan_elementwise_inc(None, A, X, Yo, alpha=alpha, inc=inc)()
        for k in range(4):
            ax = (alpha[k] * A[k]) * X[k]
            assert np.array_equal(Yo[k], Y[k] + ax if inc else ax)


def test_outer_product_pes_form():
    rng = np.random.RandomState(7)
    err, pre = rng.normal(size=5).astype(np.float32), rng.normal(size=40).astype(np.float32)
    delta = RA([rng.normal(size=(5, 40))])
    alpha = np.array([-1e-4 * 1e-3 / 40], dtype=np.float32)
    orc.plan_elementwise_inc(None, RA([err]), RA([pre]), delta, alpha=alpha, outer=True, inc=False)()
    assert np.array_equal(delta[0], np.outer(alpha[0] * err, pre))


def test_copy_slicedcopy_reset_against_numpy():
    rng = np.random.RandomState(9)
    sizes = [(10, 1), (40, 64), (1, 100)]
    X, Y = RA([rng.normal(size=s) for s in sizes]), RA([rng.normal(size=s) for s in sizes])
    Y0 = clone(Y)
    orc.plan_copy(None, X, Y, np.array([1, 0, 1]))()
    for i, inc in enumerate([1, 0, 1]):
        assert np.array_equal(Y[i], Y0[i] + X[i] if inc else X[i])

    A, B = RA([rng.normal(size=30), rng.normal(size=50)]), RA([rng.normal(size=30), rng.normal(size=50)])
    ai = [rng.permutation(30)[:12].astype(np.int32), np.arange(10, dtype=np.int32)]
    bi = [rng.permutation(30)[:12].astype(np.int32), np.arange(40, 50, dtype=np.int32)]
    expect = clone(B)
    expect[0][bi[0], 0] += A[0][ai[0], 0]
    expect[1][bi[1], 0] = A[1][ai[1], 0]
    orc.plan_slicedcopy(None, A, B, RA(ai, dtype=np.int32), RA(bi, dtype=np.int32), np.array([1, 0]))()
    assert np.array_equal(B.buf, expect.buf)

    Z = RA([np.ones(1000), np.ones((10, 17)), np.ones((3, 3))])
    vals = np.array([0.5, -2.0, 7.0], dtype=np.float32)
    orc.plan_reset(None, Z, vals)()
    for i, v in enumerate(vals):
        assert np.all(Z[i] == v)


# ------------------------------------------------------- time, inputs, probes
def test_timeupdate_float32_counter():
    sig = RA([np.zeros(1), np.zeros(1)])
    plan = orc.plan_timeupdate(None, sig[[0]], sig[[1]], 0.001)
    for n in range(1, 3001):
        plan()
        assert sig[0][0, 0] == np.float32(n)
        assert sig[1][0, 0] == np.float32(0.001 * n)  # double product, rounded once


def test_presentinput_rows():
    rng = np.random.RandomState(10)
    tables = [rng.normal(size=(1000, 1)), rng.normal(size=(37, 5))]
    S, Y = RA(tables), RA([np.zeros(1), np.zeros(5)])
    for step in [0, 1, 36, 37, 999, 1000, 4321]:
        T = RA([[float(step)], [float(step)]])
        orc.plan_presentinput(None, Y, T, S, 0.001)()
        for i, t in enumerate(tables):
            assert np.array_equal(Y[i][:, 0], np.float32(t[step % t.shape[0]]))
    # with a presentation time: row = int((step - 0.5) * dt / pt) mod rows
    T = RA([[250.0], [250.0]])
    orc.plan_presentinput(None, Y, T, S, 0.001, pres_t=np.array([0.01, 0.05], dtype=np.float32))()
    assert np.array_equal(Y[0][:, 0], np.float32(tables[0][24]))
    assert np.array_equal(Y[1][:, 0], np.float32(tables[1][4]))


def test_probe_schedule_matches_trange_rule():
    """A probe with period p (in steps) fires at the steps n with n % p < 1
    (simulator.py:700-702), for integer and non-integer periods."""
    periods = [1.0, 2.0, 2.5, 10.0]
    X = RA([np.zeros(1)] * len(periods))
    Y = RA([np.zeros((64, 1))] * len(periods))
    plan = orc.plan_probes(None, periods, X, Y)
    fired = [[] for _ in periods]
    for n in range(1, 41):
        X.buf[:] = n
        before = plan.bufpositions.copy()
        plan()
        for i in range(len(periods)):
            if plan.bufpositions[i] > before[i]:
                fired[i].append(n)
    steps = np.arange(1, 41)
    for i, p in enumerate(periods):
        assert fired[i] == list(steps[steps % p < 1]), p
        assert np.array_equal(Y[i][: len(fired[i]), 0], fired[i])  # the sampled values, in order


UNARY = {"identity": lambda v: v, "sin": np.sin, "cos": np.cos, "tanh": np.tanh, "exp": np.exp,
         "square": np.square}


@pytest.mark.parametrize("name", sorted(UNARY))
def test_direct_unary(name):
    """Every opcode of the single-function node kernel against numpy in float64 (the
    functions differ pairwise at these points, so a swapped opcode fails)."""
    points = np.float32([0.731, 2.5, -1.25])
    x, y = RA([[v] for v in points]), RA([[0.0]] * 3)
    orc.plan_direct_unary(None, name, x, y)()
    want = UNARY[name](points.astype(np.float64))
    np.testing.assert_allclose(y.buf[[int(s) for s in y.starts]], want, rtol=3e-7)
    for other, fn in UNARY.items():
        if other != name:
            assert np.abs(fn(points.astype(np.float64)) - want).max() > 1e-2, other


# ------------------------------------------------------- further neuron types
def test_adaptive_lif_reduces_to_lif_and_adapts():
    """With inc_n = 0 and N = 0 adaptive LIF is LIF bit for bit; a constant N with a
    very slow tau_n shifts the sub-threshold voltage exactly like a smaller current;
    without spikes N decays as N0 (1 - dt/tau_n)^k; with spikes N approaches
    inc_n * rate and the rate drops below the unadapted one."""
    rng = np.random.RandomState(11)
    dt, n = 1e-3, 300
    J = RA([rng.uniform(-1, 4, size=n)])
    V0, W0 = RA([rng.uniform(0, 1, size=n)]), RA([rng.uniform(-dt, 2 * dt, size=n)])
    # (i) inc_n = 0, N = 0: identical to LIF
    Va, Wa, Sa, Na = clone(V0), clone(W0), RA([np.zeros(n)]), RA([np.zeros(n)])
    Vl, Wl, Sl = clone(V0), clone(W0), RA([np.zeros(n)])
    alif = orc.plan_lif(None, dt, J, Va, Wa, Sa, 0.002, 0.02, 1.0, N=Na, tau_n=0.5, inc_n=0.0)
    lif = orc.plan_lif(None, dt, J, Vl, Wl, Sl, 0.002, 0.02, 1.0)
    for _ in range(50):
        alif()
        lif()
    assert np.array_equal(Va.buf, Vl.buf) and np.array_equal(Wa.buf, Wl.buf)
    assert np.array_equal(Sa.buf, Sl.buf) and Sa.buf.sum() > 0 and not Na.buf.any()
    # (ii) sub-threshold: J - N - V with N held (tau_n huge) is LIF driven by J - N
    Jq = RA([rng.uniform(-1, 0.9, size=n)])
    Nq = RA([rng.uniform(0, 0.5, size=n)])
    Jshift = RA([(Jq.buf - Nq.buf).astype(np.float32)])
    Va, Wa, Sa = RA([np.zeros(n)]), RA([np.zeros(n)]), RA([np.zeros(n)])
    Vl, Wl, Sl = RA([np.zeros(n)]), RA([np.zeros(n)]), RA([np.zeros(n)])
    N_before = Nq.buf.copy()
    orc.plan_lif(None, dt, Jq, Va, Wa, Sa, 0.002, 0.02, 1.0, N=Nq, tau_n=1e30, inc_n=0.0)()
    orc.plan_lif(None, dt, Jshift, Vl, Wl, Sl, 0.002, 0.02, 1.0)()
    assert np.array_equal(Va.buf, Vl.buf) and np.array_equal(Nq.buf, N_before)
    # (iii) decay of N without spikes
    Nd = RA([np.full(n, 0.3)])
    step = orc.plan_lif(None, dt, RA([np.zeros(n)]), RA([np.zeros(n)]), RA([np.zeros(n)]),
                        RA([np.zeros(n)]), 0.002, 0.02, 1.0, N=Nd, tau_n=0.05, inc_n=0.1)
    for _ in range(100):
        step()
    np.testing.assert_allclose(Nd.buf, 0.3 * (1 - dt / 0.05) ** 100, rtol=1e-4)
    # (iv) adaptation lowers the rate and N settles near inc_n * rate
    Jc = RA([np.full(n, 3.0)])
    Va, Wa, Sa, Na = (RA([np.zeros(n)]) for _ in range(4))
    step = orc.plan_lif(None, dt, Jc, Va, Wa, Sa, 0.002, 0.02, 1.0, N=Na, tau_n=0.1, inc_n=0.01)
    counts = np.zeros(n)
    for k in range(3000):
        step()
        if k >= 2000:
            counts += Sa.buf * dt
    rate = counts.mean() / 1.0
    unadapted = 1.0 / (0.002 + 0.02 * np.log1p(1.0 / (3.0 - 1.0)))
    assert rate < 0.9 * unadapted
    assert abs(Na.buf.mean() - 0.01 * rate) < 0.05 * 0.01 * rate + 0.02


def test_adaptive_lif_rate_fixed_point():
    """inc_n = 0: the LIF rate curve bit for bit; otherwise N converges to the solution of
    N = inc_n * r(J - N)."""
    rng = np.random.RandomState(12)
    n, dt = 200, 1e-3
    J = RA([rng.uniform(0, 6, size=n)])
    Ra, Rl, N = RA([np.zeros(n)]), RA([np.zeros(n)]), RA([np.zeros(n)])
    orc.plan_lif_rate(None, dt, J, Ra, 0.002, 0.02, 1.0, N=N, tau_n=0.1, inc_n=0.0)()
    orc.plan_lif_rate(None, dt, J, Rl, 0.002, 0.02, 1.0)()
    assert np.array_equal(Ra.buf, Rl.buf) and not N.buf.any()
    step = orc.plan_lif_rate(None, dt, J, Ra, 0.002, 0.02, 1.0, N=N, tau_n=0.02, inc_n=0.01)
    for _ in range(2000):
        step()
    rate = lambda j: np.where(j > 1, 1.0 / (0.002 + 0.02 * np.log1p(1.0 / np.maximum(j - 1, 1e-30))), 0)
    j64 = J.buf.astype(np.float64)
    ok = np.abs(j64 - N.buf - 1) > 0.05  # the curve is infinitely steep at threshold
    assert ok.sum() > 150
    np.testing.assert_allclose(N.buf[ok], 0.01 * rate(j64 - N.buf)[ok], rtol=2e-3, atol=1e-4)
    np.testing.assert_allclose(Ra.buf[ok], rate(j64 - N.buf)[ok], rtol=2e-2, atol=1e-2)


def test_relu_spiking_relu_sigmoid():
    """Rectified linear against numpy (exact); spiking rectified linear: the spike count
    over time is floor of the integrated current and the state stays in [0, 1);
    sigmoid against float64 and at its cut-offs."""
    rng = np.random.RandomState(13)
    n, dt = 500, 1e-3
    J = RA([rng.normal(scale=3, size=n), rng.normal(scale=30, size=n)])
    amp = np.array([1.0, 0.5], dtype=np.float32)
    R = RA([np.zeros(n), np.zeros(n)])
    orc.plan_rectified_linear(None, J, R, amp)()
    for i in range(2):
        assert np.array_equal(R[i], amp[i] * np.maximum(J[i], 0))

    V, S = RA([np.zeros(n), np.zeros(n)]), RA([np.zeros(n), np.zeros(n)])
    Jc = RA([rng.uniform(-50, 900, size=n), rng.uniform(0, 2500, size=n)])
    step = orc.plan_spiking_rectified_linear(None, dt, Jc, V, S, amp)
    spikes = np.zeros(2 * n)
    for _ in range(1000):
        step()
        spikes += S.buf * dt / np.repeat(amp, n)
        assert np.all((V.buf >= 0) & (V.buf < 1))
    expect = np.maximum(Jc.buf.astype(np.float64), 0) * dt * 1000
    assert np.all(np.abs(spikes - expect) <= 1.0 + 1e-3 * expect)
    assert np.all(np.abs(spikes + V.buf - expect) < 1e-2 + 1e-4 * expect)  # nothing is lost
    assert spikes.max() > 2000  # several spikes per step occur

    Js = RA([np.concatenate([rng.uniform(-30, 14, size=n - 4), [-100.0, -88.5, 15.5, 40.0]])])
    Rs = RA([np.zeros(n)])
    orc.plan_sigmoid(None, Js, Rs, 0.0025)()
    j64 = Js.buf[:-4].astype(np.float64)
    np.testing.assert_allclose(Rs.buf[:-4], 1.0 / (0.0025 * (1 + np.exp(-j64))), rtol=1e-6)
    assert np.array_equal(Rs.buf[-4:], np.float32([0, 0, 1 / np.float32(0.0025), 1 / np.float32(0.0025)]))


# ------------------------------------------------------------------ sparse
def test_spmv_against_scipy():
    """The CSR product against scipy: exact for small integers (any order gives the same
    sums), float64 closeness otherwise; duplicate entries add up, empty rows give 0 (or
    keep y when incrementing), several matrices per call, increment and set."""
    import scipy.sparse as sp

    rng = np.random.RandomState(21)
    shapes = [(70, 50), (1, 9), (200, 200), (5, 3)]
    mats = [sp.random(m, n, density=0.2, random_state=rng, format="csr") for m, n in shapes]
    mats[2].data[:] = rng.randint(-4, 5, size=mats[2].nnz)            # integers: exact
    dup = sp.csr_matrix((np.float32([1, 2, 3]), np.int32([2, 2, 0]), np.int32([0, 2, 2, 3, 3, 3])),
                        shape=(5, 3))                                  # duplicate column, empty rows
    mats[3] = dup
    X = RA([rng.randint(-3, 4, size=n) if i == 2 else rng.normal(size=n) for i, (m, n) in enumerate(shapes)])
    Y0 = RA([rng.normal(size=m) for m, n in shapes])
    for inc in (False, True, [1, 0, 1, 0]):
        Y = clone(Y0)
        orc.plan_sparse_dot_inc(None, mats, X, Y, inc=inc).plans[0]()
        incs = np.broadcast_to(np.asarray(inc, dtype=bool), (4,))
        for i, mat in enumerate(mats):
            want = mat.astype(np.float64) @ X[i][:, 0].astype(np.float64) + (Y0[i][:, 0] if incs[i] else 0)
            if i == 2 and not incs[i]:
                assert np.array_equal(Y[i][:, 0], want.astype(np.float32))
            else:
                np.testing.assert_allclose(Y[i][:, 0], want, rtol=1e-5, atol=1e-5)
    Y = clone(Y0)
    orc.plan_sparse_dot_inc(None, [dup], RA([[1.0, 10.0, 100.0]]), Y[[3]], inc=False).plans[0]()
    assert np.array_equal(Y[3][:, 0], np.float32([300, 0, 3, 0, 0]))


# ------------------------------------------------------------------ learning rules
def _rule_operands(rng, shapes):
    pre = RA([rng.uniform(0, 200, size=n) for m, n in shapes])
    post = RA([rng.uniform(0, 200, size=m) for m, n in shapes])
    theta = RA([rng.uniform(0, 200, size=m) for m, n in shapes])
    mat = RA([rng.normal(scale=0.01, size=(m, n)) for m, n in shapes])
    delta = RA([rng.normal(size=(m, n)) for m, n in shapes])  # stale values must be overwritten
    return pre, post, theta, mat, delta


def test_learning_rules_against_float64_outer_forms():
    """BCM, Oja and Voja deltas against their matrix forms in float64: a swapped index,
    a wrong sign or a dropped factor changes the matrices far beyond rounding."""
    rng = np.random.RandomState(5)
    shapes = [(7, 5), (1, 9), (33, 70), (64, 1)]
    pre, post, theta, mat, delta = _rule_operands(rng, shapes)
    k = len(shapes)
    alpha = rng.uniform(1e-6, 1e-4, size=k).astype(np.float32)
    beta = rng.uniform(0.5, 2, size=k).astype(np.float32)
    f64 = lambda ra, i: ra[i].astype(np.float64)

    orc.plan_bcm(None, pre, post, theta, delta, alpha)()
    for i in range(k):
        po, th, pr = f64(post, i)[:, 0], f64(theta, i)[:, 0], f64(pre, i)[:, 0]
        np.testing.assert_allclose(delta[i], alpha[i] * np.outer(po * (po - th), pr), rtol=1e-5,
                                   atol=1e-12)

    orc.plan_oja(None, pre, post, mat, delta, alpha, beta)()
    for i in range(k):
        po, pr, w = f64(post, i)[:, 0], f64(pre, i)[:, 0], f64(mat, i)
        want = alpha[i] * (np.outer(po, pr) - beta[i] * w * (po ** 2)[:, None])
        np.testing.assert_allclose(delta[i], want, rtol=1e-4, atol=1e-9)

    learn = RA([[rng.uniform(0, 1)] for _ in shapes])
    scale = RA([rng.uniform(1, 30, size=m) for m, n in shapes])
    orc.plan_voja(None, pre, post, mat, delta, learn, scale, alpha)()
    for i in range(k):
        po, pr, enc = f64(post, i)[:, 0], f64(pre, i)[:, 0], f64(mat, i)
        want = alpha[i] * learn[i][0, 0] * po[:, None] * (np.outer(f64(scale, i)[:, 0], pr) - enc)
        np.testing.assert_allclose(delta[i], want, rtol=1e-4, atol=1e-9)


def test_learning_rule_fixed_points():
    """What the rules are for: BCM's delta vanishes where post == theta and changes sign
    there; Oja's vanishes for a unit-norm weight row aligned with the input (post = w.pre);
    Voja's vanishes where the encoder already equals the scaled input, and with a zero
    learning signal."""
    pre = RA([[1.0, 2.0, 3.0]])
    post = RA([[4.0, 6.0, 8.0]])
    theta = RA([[4.0, 7.0, 5.0]])
    delta = RA([np.ones((3, 3))])
    orc.plan_bcm(None, pre, post, theta, delta, np.float32([0.5]))()
    assert np.all(delta[0][0] == 0) and np.all(delta[0][1] < 0) and np.all(delta[0][2] > 0)

    x = np.float32([0.6, 0.8])  # unit norm
    w = RA([np.float32([x, 2 * x])])
    pre, post = RA([x]), RA([np.float32([x @ x, 2 * x @ x])])
    delta = RA([np.ones((2, 2))])
    orc.plan_oja(None, pre, post, w, delta, np.float32([1.0]), np.float32([1.0]))()
    np.testing.assert_allclose(delta[0][0], 0, atol=1e-7)       # |w| = 1: fixed point
    assert np.all(delta[0][1] * x < 0)                           # |w| = 2: pulled back

    enc = RA([np.float32([[2.0, 4.0], [1.0, 1.0]])])
    pre, post = RA([[1.0, 2.0]]), RA([[3.0, 3.0]])
    scale = RA([[2.0, 2.0]])
    for learn, moves in ((1.0, True), (0.0, False)):
        delta = RA([np.ones((2, 2))])
        orc.plan_voja(None, pre, post, enc, delta, RA([[learn]]), scale, np.float32([0.1]))()
        assert np.all(delta[0][0] == 0)
        assert np.all(delta[0][1] > 0) if moves else np.all(delta[0] == 0)


# ------------------------------------------------------------------ convolution, pooling
@pytest.mark.parametrize("channels_last", [True, False])
@pytest.mark.parametrize("padding,strides", [("valid", (1, 1)), ("same", (1, 1)), ("same", (2, 3)),
                                             ("valid", (2, 2)), ((2, 1), (1, 1))])
def test_conv2d_against_scipy(channels_last, padding, strides):
    """Convolution against scipy.signal.correlate2d per (channel, filter) pair: a zero-padded
    full correlation subsampled by the strides."""
    from scipy.signal import correlate2d

    rng = np.random.RandomState(8)
    nxi, nxj, nc, nf, si, sj = 9, 11, 3, 4, 3, 5
    sti, stj = strides
    if padding == "valid":
        pi, pj = 0, 0
    elif padding == "same":
        pi, pj = (si - 1) // 2, (sj - 1) // 2
    else:
        pi, pj = padding
    nyi, nyj = (nxi + 2 * pi - si) // sti + 1, (nxj + 2 * pj - sj) // stj + 1
    img = rng.normal(size=(nxi, nxj, nc))
    filt = rng.normal(size=(si, sj, nc, nf))
    X = RA([(img if channels_last else img.transpose(2, 0, 1)).ravel()])
    F = RA([filt.ravel()])
    Y = RA([np.full(nyi * nyj * nf, 7.0)])
    shape_in = (nxi, nxj, nc) if channels_last else (nc, nxi, nxj)
    shape_out = (nyi, nyj, nf) if channels_last else (nf, nyi, nyj)
    orc.plan_conv2d(None, X, Y, F, shape_in, shape_out, (si, sj), padding=padding,
                    strides=strides, channels_last=channels_last)()
    got = Y[0].reshape(shape_out)
    if not channels_last:
        got = got.transpose(1, 2, 0)
    padded = np.pad(img, ((pi, pi), (pj, pj), (0, 0)))
    for k in range(nf):
        want = sum(correlate2d(padded[:, :, c], filt[:, :, c, k], mode="valid") for c in range(nc))
        want = want[::sti, ::stj][:nyi, :nyj]
        np.testing.assert_allclose(got[:, :, k], want, rtol=1e-5, atol=1e-5)


def test_local_filtering_brute_force():
    rng = np.random.RandomState(9)
    nxi, nxj, nc, nf, si, sj = 5, 6, 2, 3, 2, 3
    nyi, nyj = nxi - si + 1, nxj - sj + 1
    img = rng.normal(size=(nc, nxi, nxj))
    filt = rng.normal(size=(nf, nc, si, sj, nyi, nyj))
    X, F, Y = RA([img.ravel()]), RA([filt.ravel()]), RA([np.zeros(nf * nyi * nyj)])
    orc.plan_conv2d(None, X, Y, F, (nc, nxi, nxj), (nf, nyi, nyj), (si, sj), conv=False,
                    channels_last=False)()
    want = np.zeros((nf, nyi, nyj))
    for k in range(nf):
        for i in range(nyi):
            for j in range(nyj):
                want[k, i, j] = np.sum(filt[k, :, :, :, i, j] * img[:, i:i + si, j:j + sj])
    np.testing.assert_allclose(Y[0].reshape(nf, nyi, nyj), want, rtol=1e-5, atol=1e-5)


def test_pool2d_block_means_and_edges():
    rng = np.random.RandomState(10)
    nc, nxi, nxj = 3, 8, 12
    img = rng.normal(size=(nc, nxi, nxj)).astype(np.float32)
    X, Y = RA([img.ravel()]), RA([np.zeros(nc * 4 * 4)])
    orc.plan_pool2d(None, X, Y, (nc, 4, 4, nxi, nxj), (2, 3), (2, 3))()
    want = img.reshape(nc, 4, 2, 4, 3).mean(axis=(2, 4))
    np.testing.assert_allclose(Y[0].reshape(nc, 4, 4), want, rtol=1e-6, atol=1e-6)
    # windows hanging over the bottom / right edge average what is inside; NaNs are skipped
    img2 = np.arange(25, dtype=np.float32).reshape(1, 5, 5)
    img2[0, 0, 1] = np.nan
    X, Y = RA([img2.ravel()]), RA([np.zeros(9)])
    orc.plan_pool2d(None, X, Y, (1, 3, 3, 5, 5), (2, 2), (2, 2))()
    got = Y[0].reshape(3, 3)
    assert got[0, 0] == np.float32((0 + 5 + 6) / 3)
    assert got[2, 2] == 24 and got[0, 2] == np.float32((4 + 9) / 2)
    assert got[2, 0] == np.float32((20 + 21) / 2)


# ------------------------------------------------------------------ noise
def test_philox_known_answers():
    rows = np.array([c + k for c, k, _ in PHILOX_KNOWN_ANSWERS], dtype=np.uint32)
    want = np.array([o for _, _, o in PHILOX_KNOWN_ANSWERS], dtype=np.uint32)
    assert np.array_equal(orc.philox4x32(rows), want)


def test_whitenoise_distributions_and_streams():
    """Uniform and Gaussian samples against their distributions (Kolmogorov-Smirnov),
    the 1/sqrt(dt) scaling, increment mode, independence between calls, elements and
    seeds, and the restart of the streams."""
    from scipy import stats

    n, dt = 20000, 1e-3
    Y = RA([np.zeros(n), np.zeros(n), np.zeros(n), np.ones(5)])
    enums = [0, 1, 1, 0]
    params = [(-2.0, 3.0), (1.5, 0.5), (0.0, 1.0), (0.0, 1.0)]
    plan = orc.plan_whitenoise(None, Y, enums, params, [0, 0, 1, 0], [0, 0, 0, 1], dt,
                               [1, 2, 3, 4])
    plan()
    first = np.array(Y.buf)
    assert stats.kstest(Y[0][:, 0], stats.uniform(-2, 5).cdf).pvalue > 1e-3
    assert Y[0].min() >= -2 and Y[0].max() < 3
    assert stats.kstest(Y[1][:, 0], stats.norm(1.5, 0.5).cdf).pvalue > 1e-3
    assert stats.kstest(Y[2][:, 0], stats.norm(0, np.sqrt(1 / dt)).cdf).pvalue > 1e-3
    assert np.all((Y[3] >= 1) & (Y[3] < 2))  # incremented, not set
    # neighbouring elements (which share a generator block) and consecutive calls are
    # uncorrelated
    z = (Y[1][:, 0] - 1.5) / 0.5
    for lag in (1, 2, 3, 4):
        assert abs(np.mean(z[:-lag] * z[lag:])) < 4 / np.sqrt(n)
    plan()
    z2 = (Y[1][:, 0] - 1.5) / 0.5
    assert abs(np.mean(z * z2)) < 4 / np.sqrt(n)
    assert not np.array_equal(first[:n], Y.buf[:n])
    # restart: same samples again; another seed: other samples
    plan.reset_streams()
    Y.buf[-5:] = 1
    plan()
    assert np.array_equal(Y.buf, first)
    Y2 = RA([np.zeros(n)])
    orc.plan_whitenoise(None, Y2, [0], [(-2.0, 3.0)], [0], [0], dt, [99])()
    assert abs(np.corrcoef(Y2[0][:, 0], first[:n])[0, 1]) < 4 / np.sqrt(n)
