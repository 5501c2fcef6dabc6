"""GPU parity of the non-GEMV timestep kernels against the CPU oracle.

Cases follow nengo_ocl/tests/test_clra_nonlinearities.py: test_lif_step :35-91,
test_lif_rate :141-173, test_copy :176-191, test_elementwise_inc :194-227,
test_elementwise_inc_outer :230-251, test_reset :254-279, test_slicedcopy
:282-326, test_linearfilter :329-406.  Index / copy / fill / single-rounding
arithmetic is compared bit for bit, and so is the LIF / LIFRate state: expm1 and
log1p are evaluated in double and rounded once on both sides, so the result does
not depend on the math library.
"""

import numpy as np
import pytest

from helpers import RA, clone, run_plans, to_dev

pytestmark = pytest.mark.gpu


def nl():
    from nengo_ocl_amd import hipra_nonlinearities

    return hipra_nonlinearities


def orc():
    from oracle import oracle

    return oracle


@pytest.mark.parametrize("param_kind", ["float", "ragged_const", "ragged_varying"])
@pytest.mark.parametrize("upsample", [1, 4])
def test_lif_step(queue, rng, upsample, param_kind):
    dt = 1e-3
    n_neurons = [12345, 23456, 34567]
    J = RA([rng.normal(scale=1.2, size=n) for n in n_neurons])
    V = RA([rng.uniform(low=0, high=1, size=n) for n in n_neurons])
    W = RA([rng.uniform(low=-5 * dt, high=5 * dt, size=n) for n in n_neurons])
    OS = RA([np.zeros(n) for n in n_neurons])
    ref, amp = 2e-3, 1.0
    taus = rng.uniform(low=15e-3, high=80e-3, size=len(n_neurons))

    if param_kind == "ragged_varying":
        # per-neuron taus: the oracle takes one value per item, so check each neuron
        # against an oracle run on single-tau items instead
        tau_arrays = [rng.choice([0.02, 0.05], size=n) for n in n_neurons]
    else:
        tau_arrays = [t * np.ones(n) for t, n in zip(taus, n_neurons)]

    dJ, dV, dW, dOS = (to_dev(queue, x) for x in (J, V, W, OS))
    if param_kind == "float":
        taus = np.full(len(n_neurons), 0.02)
        tau_arrays = [0.02 * np.ones(n) for n in n_neurons]
        plan = nl().plan_lif(queue, dt, dJ, dV, dW, dOS, ref, 0.02, amp, upsample=upsample)
    else:
        dTau = to_dev(queue, RA(tau_arrays))
        plan = nl().plan_lif(queue, dt, dJ, dV, dW, dOS, ref, dTau, amp, upsample=upsample)
    plan()

    # oracle: split every item by tau value so that each oracle item has one tau
    Vo, Wo, So = clone(V), clone(W), clone(OS)
    for i, n in enumerate(n_neurons):
        for tau in np.unique(np.float32(tau_arrays[i])):
            sel = np.nonzero(np.float32(tau_arrays[i]) == tau)[0]
            j, v, w, s = (RA([x[i].ravel()[sel]]) for x in (J, V, W, OS))
            orc().plan_lif(None, dt, j, v, w, s, ref, float(tau), amp, upsample=upsample)()
            Vo[i][sel, 0], Wo[i][sel, 0], So[i][sel, 0] = v[0].ravel(), w[0].ravel(), s[0].ravel()

    gV, gW, gS = dV.to_host(), dW.to_host(), dOS.to_host()
    assert np.array_equal(dJ.buf, J.buf)
    assert So.buf.sum() > 0, "spiking mechanism not exercised"
    # every operation is a single correctly rounded float32 operation on both sides
    # (expm1 / log1p via double), so the state agrees bit for bit
    assert np.array_equal(gS.buf, So.buf)
    assert np.array_equal(gV.buf, Vo.buf)
    assert np.array_equal(gW.buf, Wo.buf)
    assert set(np.unique(gS.buf)) <= {0.0, np.float32(amp / dt)}


def test_lif_rate(queue, rng):
    n_neurons = [123459, 23456, 34567]
    J = RA([rng.normal(loc=1, scale=10, size=n) for n in n_neurons])
    R = RA([np.zeros(n) for n in n_neurons])
    ref, amp = 2e-3, 1.0
    taus = list(rng.uniform(low=15e-3, high=80e-3, size=len(n_neurons)))
    tau_ra = RA([t * np.ones(n) for t, n in zip(taus, n_neurons)])

    dJ, dR = to_dev(queue, J), to_dev(queue, R)
    nl().plan_lif_rate(queue, 1e-3, dJ, dR, ref, to_dev(queue, tau_ra), amp)()
    Ro = clone(R)
    orc().plan_lif_rate(None, 1e-3, J, Ro, ref, tau_ra, amp)()
    got = dR.to_host()
    assert np.array_equal(dJ.buf, J.buf)
    assert Ro.buf.sum() > 1.0
    assert np.array_equal(got.buf, Ro.buf)  # log1p correctly rounded on both sides: bit-exact


@pytest.mark.parametrize("align", [False, True])
def test_copy(queue, rng, align):
    """`align`: items start on 64-byte boundaries, so those made of whole quads take the
    16-byte path (with blocks of 1024 elements: whole, short and ragged last blocks)."""
    sizes = [(10, 1), (40, 64), (457, 342), (1, 100), (3000, 1), (2000, 32), (8, 1), (1, 1028)]
    X = RA([rng.normal(size=s) for s in sizes], align=align)
    Y0 = RA([rng.normal(size=s) for s in sizes], align=align)
    incs = np.array([0, 1, 1, 0, 1, 1, 1, 0], dtype=np.int32)
    dX, dY = to_dev(queue, X), to_dev(queue, Y0)
    nl().plan_copy(queue, dX, dY, incs)()
    Yo = clone(Y0)
    orc().plan_copy(None, X, Yo, incs)()
    got = dY.to_host()
    assert np.array_equal(got.buf, Yo.buf)
    for i, inc in enumerate(incs):
        assert np.array_equal(got[i], Y0[i] + X[i] if inc else X[i])


def test_copy_strided_rows(queue, rng):
    """Source and target are column slices of wider matrices (row stride > columns)."""
    from nengo_ocl_amd.raggedarray import RaggedArray

    base = RA([rng.normal(size=(30, 50)), rng.normal(size=(30, 70))])
    s = base.starts
    X = RaggedArray.from_buffer(base.buf, [s[0] + 5], [30], [20], [50], [1])
    Y = RaggedArray.from_buffer(base.buf, [s[1] + 40], [30], [20], [70], [1])
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray

    d = to_dev(queue, base)
    dX = HIPRaggedArray.from_buffer(queue, d.dev_buf, X.starts, X.shape0s, X.shape1s, X.stride0s, X.stride1s)
    dY = HIPRaggedArray.from_buffer(queue, d.dev_buf, Y.starts, Y.shape0s, Y.shape1s, Y.stride0s, Y.stride1s)
    nl().plan_copy(queue, dX, dY, np.array([1], dtype=np.int32))()
    expect = np.array(base.buf)
    e = RaggedArray.from_buffer(expect, base.starts, base.shape0s, base.shape1s, base.stride0s, base.stride1s)
    e[1][:, 40:60] += e[0][:, 5:25]
    assert np.array_equal(d.buf, expect)


@pytest.mark.parametrize("use_alpha", [False, True])
@pytest.mark.parametrize("inc", [True, False])
def test_elementwise_inc(queue, rng, inc, use_alpha):
    Xsizes = [(3, 3), (32, 64), (457, 342), (1, 100)]
    Asizes = [(3, 3), (1, 1), (457, 342), (100, 1)]
    A = RA([rng.normal(size=s) for s in Asizes])
    X = RA([rng.normal(size=s) for s in Xsizes])
    alpha = rng.normal(size=len(Xsizes)).astype(np.float32) if use_alpha else None
    Yshapes = [np.broadcast(A[i], X[i]).shape for i in range(len(Xsizes))]
    Y = RA([rng.normal(size=s) for s in Yshapes])

    dY = to_dev(queue, Y)
    nl().plan_elementwise_inc(queue, to_dev(queue, A), to_dev(queue, X), dY, alpha=alpha, inc=inc)()
    Yo = clone(Y)
    orc().plan_elementwise_inc(None, A, X, Yo, alpha=alpha, inc=inc)()
    got = dY.to_host()
    assert np.array_equal(got.buf, Yo.buf)
    for k in range(len(Y)):  # library expression, float32: (alpha*a)*x then one add
        al = np.float32(1.0) if alpha is None else alpha[k]
        ax = (al * A[k]) * X[k]
        assert np.array_equal(got[k], Y[k] + ax if inc else ax), k


@pytest.mark.parametrize("align", [False, True])
def test_elementwise_inc_outer(queue, rng, align):
    """`align`: items start on 64-byte boundaries, so products whose rows are whole quads
    take the 16-byte path (rows shorter and longer than a block of 1024 elements)."""
    Xsizes = [3, 9, 15, 432, 2000, 16, 4]
    Asizes = [9, 42, 10, 124, 32, 8, 700]
    alpha = rng.normal(size=len(Xsizes)).astype(np.float32)
    A = RA([rng.normal(size=s) for s in Asizes], align=align)
    X = RA([rng.normal(size=s) for s in Xsizes], align=align)
    Y = RA([rng.normal(size=(a, x)) for a, x in zip(Asizes, Xsizes)], align=align)
    for inc in (True, False):
        dY = to_dev(queue, Y)
        nl().plan_elementwise_inc(queue, to_dev(queue, A), to_dev(queue, X), dY, alpha=alpha,
                                  outer=True, inc=inc)()
        got = dY.to_host()
        for k in range(len(Y)):
            ax = np.outer(alpha[k] * A[k].ravel(), X[k].ravel())
            assert np.array_equal(got[k], Y[k] + ax if inc else ax)


def _outer_filter_case(queue, rng, shapes, broadcast_row=None, extra_filters=(), unfiltered=()):
    """Device arrays and plans for "W += (alpha a) (x) f; f <- filter(s)": item k of `vec` is
    the filter output f_k and the column operand of outer product k (products listed in
    `unfiltered` have a column operand that no filter writes); `extra_filters` are lengths of
    further filters that feed no product."""
    n = len(shapes)
    cols = [c for _, c in shapes]
    vec = RA([rng.normal(size=c) for c in cols] + [rng.normal(size=m) for m in extra_filters],
             align=True)
    spikes = RA([rng.normal(size=c) for c in cols] + [rng.normal(size=m) for m in extra_filters],
                align=True)
    rows = [1 if k == broadcast_row else r for k, (r, _) in enumerate(shapes)]
    A = RA([rng.normal(size=r) for r in rows], align=True)
    W = RA([rng.normal(size=s) for s in shapes], align=True)
    alpha = rng.normal(size=n).astype(np.float32)
    filtered = [k for k in range(n) if k not in unfiltered] + list(range(n, n + len(extra_filters)))
    kinds = ["lowpass" if k % 3 else "gain" for k in range(len(filtered))]
    coefs = [_filter_coefficients(kind) for kind in kinds]
    FA, FB = RA([den for _, den in coefs]), RA([num for num, _ in coefs])
    sizes = [vec.sizes[k] for k in filtered]
    Xbuf = RA([np.zeros((1, m)) for m in sizes])
    Ybuf = RA([np.zeros((len(den), m)) for (_, den), m in zip(coefs, sizes)])
    return dict(vec=vec, spikes=spikes, A=A, W=W, alpha=alpha, FA=FA, FB=FB, Xbuf=Xbuf, Ybuf=Ybuf,
                filtered=filtered, n=n)


def _outer_filter_plans(queue, case, where):
    """(weights, vectors, spikes, [outer-product plan, filter plan]) on the device
    (`where` = the device module) or on the host (the oracle module)."""
    c, n, filtered = case, case["n"], case["filtered"]
    if where is nl():
        put = lambda ra: to_dev(queue, ra)
        q = queue
    else:
        put, q = clone, None
    vec, spikes, W = put(c["vec"]), put(c["spikes"]), put(c["W"])
    A, FA, FB = put(c["A"]), put(c["FA"]), put(c["FB"])
    ew = where.plan_elementwise_inc(q, A, vec[list(range(n))], W, alpha=c["alpha"], outer=True,
                                    inc=True)
    lf = where.plan_linearfilter(q, spikes[filtered], vec[filtered], FA, FB, put(c["Xbuf"]),
                                 put(c["Ybuf"]))
    return W, vec, spikes, [ew] + list(lf)


def test_outer_product_with_the_filter_of_its_column_operand(queue, rng):
    """`nhip_outer_filter`: the weight update of a learning rule and the filter step of the
    activities it has just read, in one launch, against the two launches it replaces and
    against the oracle's two kernels -- bit for bit over several calls with fresh filter
    inputs.  Shapes: the benchmark's 32 x 2000, tiles that are not full, a single row, a row
    operand that is one value for all rows, a product whose column operand nothing filters,
    filters that feed no product."""
    shapes = [(32, 2000), (8, 128), (256, 4), (1, 260), (17, 64), (5, 388)]
    case = _outer_filter_case(queue, rng, shapes, broadcast_row=4, extra_filters=(300, 5),
                              unfiltered=(1,))
    W1, vec1, spikes1, two = _outer_filter_plans(queue, case, nl())
    W2, vec2, spikes2, pair = _outer_filter_plans(queue, case, nl())
    Wo, veco, spikeso, oplans = _outer_filter_plans(queue, case, orc())
    fused = nl().fuse_outer_filter(pair[0], pair[1])
    assert fused is not None and fused.name == "hip_outer_filter"
    assert fused.fused_filters == [0, 1, 2, 3, 4]  # the filters of products 0, 2, 3, 4, 5
    for call in range(4):
        for k in range(len(case["spikes"])):
            fresh = rng.normal(size=case["spikes"].sizes[k]).astype(np.float32)
            spikes1[k] = fresh
            spikes2[k] = fresh
            spikeso[k] = fresh[:, None]
        run_plans(two)
        fused()
        run_plans(oplans)
        assert np.array_equal(W2.buf, W1.buf) and np.array_equal(vec2.buf, vec1.buf), call
        assert np.array_equal(W2.buf, Wo.buf) and np.array_equal(vec2.buf, veco.buf), call
    assert not np.array_equal(W2.buf, case["W"].buf)


def test_outer_product_and_filter_stay_apart_where_the_launch_cannot_take_them(queue, rng):
    # a filter output read by two outer products: neither work-group may overwrite it
    case = _outer_filter_case(queue, rng, [(8, 64), (8, 64)])
    W, vec, spikes, (ew, lf) = _outer_filter_plans(queue, case, nl())
    A = to_dev(queue, case["A"])
    shared = nl().plan_elementwise_inc(queue, A, vec[[0, 0]], W, alpha=case["alpha"], outer=True)
    assert nl().fuse_outer_filter(shared, lf) is None
    assert nl().fuse_outer_filter(ew, lf) is not None
    # more rows than a work-group's tile takes; rows that are not whole quads
    for shapes in ([(300, 64)], [(8, 66)]):
        case = _outer_filter_case(queue, rng, shapes)
        _, _, _, (ew, lf) = _outer_filter_plans(queue, case, nl())
        assert nl().fuse_outer_filter(ew, lf) is None
    # a second-order filter
    case = _outer_filter_case(queue, rng, [(8, 64)])
    num, den = _filter_coefficients("alpha")
    case["FA"], case["FB"] = RA([den]), RA([num])
    case["Xbuf"], case["Ybuf"] = RA([np.zeros((len(num), 64))]), RA([np.zeros((len(den), 64))])
    _, _, _, (ew, lf) = _outer_filter_plans(queue, case, nl())
    assert nl().fuse_outer_filter(ew, lf) is None
    # an element-wise product that is no outer product
    d = to_dev(queue, RA([rng.normal(size=(4, 8))] * 3))
    plain = nl().plan_elementwise_inc(queue, d[[0]], d[[1]], d[[2]])
    assert nl().fuse_outer_filter(plain, lf) is None


def test_reset(queue, rng):
    Yshapes = [(1000000,), (1000, 1700), (3, 3), (1,), (4097,)]
    values = rng.uniform(size=len(Yshapes)).astype(np.float32)
    dY = to_dev(queue, RA([np.ones(s) for s in Yshapes]))
    nl().plan_reset(queue, dY, values)()
    got = dY.to_host()
    for i, v in enumerate(values):
        assert np.all(got[i] == v)


def test_slicedcopy(queue, rng):
    sizes = rng.randint(20, 200, size=10)
    A = RA([rng.normal(size=s) for s in sizes])
    B = RA([rng.normal(size=s) for s in sizes])
    incs = rng.randint(0, 2, size=len(sizes)).astype(np.int32)
    Ainds, Binds = [], []
    for k, size in enumerate(sizes):
        r = np.arange(size, dtype=np.int32)
        u = k % 3
        if u == 0:
            Ainds.append(r)
            Binds.append(r)
        elif u == 1:
            Ainds.append(r[:10])
            Binds.append(r[-10:])
        else:
            n = rng.randint(2, size - 2)
            Ainds.append(rng.permutation(size)[:n])
            Binds.append(rng.permutation(size)[:n])
    Ainds, Binds = RA(Ainds, dtype=np.int32), RA(Binds, dtype=np.int32)

    dB = to_dev(queue, B)
    nl().plan_slicedcopy(queue, to_dev(queue, A), dB, to_dev(queue, Ainds), to_dev(queue, Binds), incs)()
    Bo = clone(B)
    orc().plan_slicedcopy(None, A, Bo, Ainds, Binds, incs)()
    expect = clone(B)
    for i in range(len(sizes)):
        ai, bi = Ainds[i].ravel(), Binds[i].ravel()
        if incs[i]:
            expect[i][bi, 0] += A[i][ai, 0]
        else:
            expect[i][bi, 0] = A[i][ai, 0]
    got = dB.to_host()
    assert np.array_equal(got.buf, expect.buf)
    assert np.array_equal(Bo.buf, expect.buf)


def _filter_coefficients(kind, dt=1e-3):
    """(num, den) of the discrete filter in the reference's packing
    (simulator.py:1214-1227): zero-order-hold discretisation, leading zero of the
    numerator and leading one of the denominator dropped."""
    from scipy.signal import cont2discrete

    if kind == "gain":
        return np.array([2.0]), np.array([])
    tau = 0.005
    num, den = ([1.0], [tau, 1.0]) if kind == "lowpass" else ([1.0], [tau * tau, 2 * tau, 1.0])
    numd, dend, _ = cont2discrete((num, den), dt, method="zoh")
    numd = numd.ravel() / dend[0]
    dend = dend / dend[0]
    numd = numd[1:] if numd[0] == 0 else numd
    return numd, dend[1:]


@pytest.mark.parametrize("n_per_kind", [(100000, 0, 0), (0, 100000, 0), (0, 0, 100000),
                                        (10000, 10000, 10000)])
def test_linearfilter(queue, rng, n_per_kind):
    from scipy.signal import lfilter

    kinds = [(k, n) for k, n in zip(("gain", "lowpass", "alpha"), n_per_kind) if n > 0]
    coefs = [_filter_coefficients(k) for k, _ in kinds]
    A = RA([den for _, den in coefs])
    B = RA([num for num, _ in coefs])
    n_calls = 5
    xs = [[rng.normal(size=n) for _, n in kinds] for _ in range(n_calls)]
    X = RA(xs[0])
    Y = RA([np.zeros(n) for _, n in kinds])
    Xbuf = RA([np.zeros(s) for s in zip(B.sizes, X.sizes)])
    Ybuf = RA([np.zeros(s) for s in zip(A.sizes, Y.sizes)])

    dX, dY = to_dev(queue, X), to_dev(queue, Y)
    plans = nl().plan_linearfilter(queue, dX, dY, to_dev(queue, A), to_dev(queue, B),
                                   to_dev(queue, Xbuf), to_dev(queue, Ybuf))
    Xo, Yo = clone(X), clone(Y)
    oplans = orc().plan_linearfilter(None, Xo, Yo, A, B, clone(Xbuf), clone(Ybuf))
    for c in range(n_calls):
        for i in range(len(kinds)):
            dX[i] = xs[c][i]
            Xo[i] = xs[c][i][:, None]
        for p in plans:
            p()
        for p in oplans:
            p()
        assert np.array_equal(dY.buf, Yo.buf), "call %d" % c

    # independent check of the recurrence: scipy's direct-form filter in float64 on the
    # float32-rounded coefficients.  The step maps x[n] to y[n] with no extra delay:
    # y[n] = sum_p b[p] x[n-p] - sum_p a[p] y[n-1-p]  ==  lfilter(b, [1, a...], x)
    got = dY.to_host()
    for i, (kind, n) in enumerate(kinds):
        num, den = (np.float32(c).astype(np.float64) for c in coefs[i])
        m = min(n, 100)
        x_hist = np.array([np.float32(xs[c][i][:m]) for c in range(n_calls)], dtype=np.float64)
        y = lfilter(num, np.concatenate([[1.0], den]), x_hist, axis=0)
        np.testing.assert_allclose(got[i][:m, 0], y[-1], rtol=1e-5, atol=1e-6)


def test_timeupdate(queue):
    sig = RA([np.zeros(1), np.zeros(1)])
    d = to_dev(queue, sig)
    plan = nl().plan_timeupdate(queue, d[[0]], d[[1]], 0.001)
    for _ in range(1234):
        plan.enqueue()
    plan.wait()
    assert d[0][0, 0] == np.float32(1234)
    assert d[1][0, 0] == np.float32(0.001 * 1234)


@pytest.mark.parametrize("with_pres_t", [False, True])
def test_presentinput(queue, rng, with_pres_t):
    dt = 0.001
    tables = [rng.normal(size=(1000, 1)), rng.normal(size=(37, 32)), rng.normal(size=(5, 300))]
    S = RA(tables)
    Y = RA([np.zeros(t.shape[1]) for t in tables])
    pres = np.array([0.01, 0.05, 0.003], dtype=np.float32) if with_pres_t else None
    for step in [0, 1, 36, 37, 999, 1000, 123456]:
        T = RA([np.array([step], dtype=np.float32)] * len(tables))
        dY = to_dev(queue, Y)
        nl().plan_presentinput(queue, dY, to_dev(queue, T), to_dev(queue, S), dt, pres_t=pres)()
        Yo = clone(Y)
        orc().plan_presentinput(None, Yo, T, S, dt, pres_t=pres)()
        assert np.array_equal(dY.buf, Yo.buf)
        if not with_pres_t:
            for i, t in enumerate(tables):
                assert np.array_equal(dY[i].ravel(), np.float32(t[step % t.shape[0]]))


def test_direct_sin(queue):
    t = RA([np.array([0.731], dtype=np.float32)])
    y = RA([np.zeros(1)])
    dy = to_dev(queue, y)
    plan = nl().plan_direct(queue, "OUTPUT__[0] = sin(t[0]);", "", ["t"], [to_dev(queue, t)], dy)
    plan()
    np.testing.assert_allclose(dy[0][0, 0], np.sin(np.float32(0.731)), rtol=1e-6)
    with pytest.raises(NotImplementedError):
        nl().plan_direct(queue, "OUTPUT__[0] = t[0] * x[0];", "", ["t"], [to_dev(queue, t)], dy)


def test_probes(queue, rng):
    """Periods 1, 2.5 (non-integer) and 10 over 40 steps with 32 buffer rows; strided source."""
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray
    from nengo_ocl_amd.raggedarray import RaggedArray

    base = RA([np.zeros(7), np.zeros((6, 10)), np.zeros(300)])
    s = base.starts
    src_meta = ([s[0], s[1] + 2, s[2]], [7, 6, 300], [1, 4, 1], [1, 10, 1], [1, 1, 1])
    periods = [1.0, 2.5, 10.0]
    n_buf = 32
    Xh = RaggedArray.from_buffer(base.buf, *src_meta)
    Yh = RA([np.zeros((n_buf, 7)), np.zeros((n_buf, 24)), np.zeros((n_buf, 300))])
    d = to_dev(queue, base)
    dX = HIPRaggedArray.from_buffer(queue, d.dev_buf, *src_meta)
    dYp = to_dev(queue, Yh)
    plan = nl().plan_probes(queue, periods, dX, dYp)
    oplan = orc().plan_probes(None, periods, Xh, Yh)
    for step in range(30):
        vals = rng.normal(size=base.buf.size).astype(np.float32)
        base.buf[:] = vals
        d.dev_buf.set(vals)
        plan()
        oplan()
    pos = plan.dev_bufpositions.get()
    assert np.array_equal(pos, oplan.bufpositions)
    assert list(pos) == [30, 12, 3]
    assert np.array_equal(plan.dev_countdowns.get(), oplan.countdowns)
    assert np.array_equal(dYp.buf, Yh.buf)


@pytest.mark.parametrize("upsample", [1, 3])
def test_adaptive_lif_and_rate(queue, rng, upsample):
    """Adaptive LIF (state V, W, N) and adaptive LIF rate against the oracle, several
    steps, one parameter set per population: bit for bit."""
    dt = 1e-3
    sizes = [1000, 2345, 17]
    J = RA([rng.normal(loc=1.5, scale=1.5, size=n) for n in sizes])
    V = RA([rng.uniform(0, 1, size=n) for n in sizes])
    W = RA([rng.uniform(-3 * dt, 3 * dt, size=n) for n in sizes])
    N = RA([rng.uniform(0, 0.3, size=n) for n in sizes])
    S = RA([np.zeros(n) for n in sizes])
    tau = np.float32([0.02, 0.03, 0.05])
    ref = np.float32([0.002, 0.001, 0.003])
    amp = np.float32([1.0, 0.5, 2.0])
    tau_n = np.float32([0.1, 0.5, 1.0])
    inc_n = np.float32([0.01, 0.1, 0.05])
    dV, dW, dN, dS, dJ = (to_dev(queue, x) for x in (V, W, N, S, J))
    plan = nl().plan_lif(queue, dt, dJ, dV, dW, dS, ref, tau, amp, N=dN, tau_n=tau_n, inc_n=inc_n,
                         upsample=upsample)
    Vo, Wo, No, So = clone(V), clone(W), clone(N), clone(S)
    oplan = orc().plan_lif(None, dt, J, Vo, Wo, So, ref, tau, amp, N=No, tau_n=tau_n, inc_n=inc_n,
                           upsample=upsample)
    total = 0.0
    for _ in range(20):
        plan()
        oplan()
        total += So.buf.sum()
        for got, want in ((dV, Vo), (dW, Wo), (dN, No), (dS, So)):
            assert np.array_equal(got.buf, want.buf)
    assert total > 0

    R, Nr = RA([np.zeros(n) for n in sizes]), clone(N)
    dR, dNr = to_dev(queue, R), to_dev(queue, Nr)
    plan = nl().plan_lif_rate(queue, dt, dJ, dR, ref, tau, amp, N=dNr, tau_n=tau_n, inc_n=inc_n)
    oplan = orc().plan_lif_rate(None, dt, J, R, ref, tau, amp, N=Nr, tau_n=tau_n, inc_n=inc_n)
    for _ in range(20):
        plan()
        oplan()
        assert np.array_equal(dR.buf, R.buf) and np.array_equal(dNr.buf, Nr.buf)
    assert R.buf.sum() > 0


def test_relu_spiking_relu_sigmoid(queue, rng):
    """The one-line neuron types against the oracle (bit for bit), with one parameter
    per population and, for the rectified linear type, per neuron."""
    dt = 1e-3
    sizes = [3000, 777, 5]
    J = RA([rng.normal(scale=s, size=n) for n, s in zip(sizes, (2, 40, 400))])
    amp = np.float32([1.0, 0.25, 3.0])
    dJ = to_dev(queue, J)

    R = RA([np.zeros(n) for n in sizes])
    dR = to_dev(queue, R)
    nl().plan_rectified_linear(queue, dJ, dR, amp)()
    orc().plan_rectified_linear(None, J, R, amp)()
    assert np.array_equal(dR.buf, R.buf) and R.buf.max() > 0

    amps = RA([rng.uniform(0.5, 2, size=n) for n in sizes])
    dR2 = to_dev(queue, RA([np.zeros(n) for n in sizes]))
    nl().plan_rectified_linear(queue, dJ, dR2, to_dev(queue, amps))()
    got = dR2.to_host()
    for i in range(len(sizes)):
        assert np.array_equal(got[i], amps[i] * np.maximum(J[i], 0))

    V, S = RA([rng.uniform(0, 1, size=n) for n in sizes]), RA([np.zeros(n) for n in sizes])
    dV, dS = to_dev(queue, V), to_dev(queue, S)
    plan = nl().plan_spiking_rectified_linear(queue, dt, dJ, dV, dS, amp)
    oplan = orc().plan_spiking_rectified_linear(None, dt, J, V, S, amp)
    for _ in range(30):
        plan()
        oplan()
        assert np.array_equal(dV.buf, V.buf) and np.array_equal(dS.buf, S.buf)
    assert S.buf.max() > 0

    Rs = RA([np.zeros(n) for n in sizes])
    dRs = to_dev(queue, Rs)
    ref = np.float32([0.0025, 0.002, 0.01])
    nl().plan_sigmoid(queue, dJ, dRs, ref)()
    orc().plan_sigmoid(None, J, Rs, ref)()
    assert np.array_equal(dRs.buf, Rs.buf)
    assert (Rs.buf == 0).any() and (Rs[2] == 1 / ref[2]).any()  # both cut-offs are reached


# ------------------------------------------------------------------ learning rules
@pytest.mark.parametrize("rule", ["bcm", "oja", "voja"])
def test_learning_rules(queue, rng, rule):
    """Delta matrices of many connections of different shapes in one launch, bit for bit
    (every product and difference is rounded separately on both sides)."""
    shapes = [(7, 5), (1, 9), (300, 70), (64, 1), (1000, 513), (33, 1100)]
    k = len(shapes)
    pre = RA([rng.uniform(0, 200, size=n) for m, n in shapes])
    post = RA([rng.uniform(0, 200, size=m) for m, n in shapes])
    theta = RA([rng.uniform(0, 200, size=m) for m, n in shapes])
    mat = RA([rng.normal(scale=0.01, size=(m, n)) for m, n in shapes])
    delta = RA([rng.normal(size=(m, n)) for m, n in shapes])
    learn = RA([[rng.uniform(0, 1)] for _ in shapes])
    scale = RA([rng.uniform(1, 30, size=m) for m, n in shapes])
    alpha = rng.uniform(1e-6, 1e-4, size=k).astype(np.float32)
    beta = rng.uniform(0.5, 2, size=k).astype(np.float32)

    d = {name: to_dev(queue, x) for name, x in dict(pre=pre, post=post, theta=theta, mat=mat,
                                                    delta=delta, learn=learn, scale=scale).items()}
    want = clone(delta)
    if rule == "bcm":
        plan = nl().plan_bcm(queue, d["pre"], d["post"], d["theta"], d["delta"], alpha)
        orc().plan_bcm(None, pre, post, theta, want, alpha)()
    elif rule == "oja":
        plan = nl().plan_oja(queue, d["pre"], d["post"], d["mat"], d["delta"], alpha, beta)
        orc().plan_oja(None, pre, post, mat, want, alpha, beta)()
    else:
        plan = nl().plan_voja(queue, d["pre"], d["post"], d["mat"], d["delta"], d["learn"],
                              d["scale"], alpha)
        orc().plan_voja(None, pre, post, mat, want, learn, scale, alpha)()
    plan()
    got = d["delta"].to_host()
    assert np.abs(want.buf).max() > 0
    assert np.array_equal(got.buf, want.buf)
    for name, host in (("pre", pre), ("post", post), ("mat", mat)):
        assert np.array_equal(d[name].buf, host.buf), "%s was modified" % name


def test_learning_rule_on_views(queue, rng):
    """Operands that are strided views of one buffer (what the simulator passes): rows of
    a wider matrix as delta / weights, every other element as pre."""
    m, n = 40, 24
    big = RA([rng.normal(size=(m, 2 * n)), rng.normal(size=(m, 2 * n)), rng.uniform(0, 9, size=2 * n),
              rng.uniform(0, 9, size=m)])
    from nengo_ocl_amd.raggedarray import RaggedArray

    s = big.starts
    host = lambda start, s0, s1, st0: RaggedArray.from_buffer(big.buf, [start], [s0], [s1], [st0], [1])
    dbig = to_dev(queue, big)
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray

    dev = lambda start, s0, s1, st0: HIPRaggedArray.from_buffer(
        queue, dbig.dev_buf, np.int32([start]), np.int32([s0]), np.int32([s1]), np.int32([st0]),
        np.int32([1]))
    specs = dict(delta=(s[0] + n, m, n, 2 * n), weights=(s[1], m, n, 2 * n), pre=(s[2], n, 1, 2),
                 post=(s[3], m, 1, 1))
    h = {k: host(*v) for k, v in specs.items()}
    g = {k: dev(*v) for k, v in specs.items()}
    alpha, beta = np.float32([1e-3]), np.float32([1.5])
    orc().plan_oja(None, h["pre"], h["post"], h["weights"], h["delta"], alpha, beta)()
    nl().plan_oja(queue, g["pre"], g["post"], g["weights"], g["delta"], alpha, beta)()
    assert np.array_equal(dbig.buf, big.buf)


# ------------------------------------------------------------------ convolution, pooling
CONV_CASES = [
    # shape_in (i, j, c), n_filters, kernel, strides, padding
    ((28, 28, 1), 32, (3, 3), (1, 1), "valid"),
    ((14, 14, 32), 64, (3, 3), (2, 2), "same"),
    ((9, 11, 3), 4, (3, 5), (2, 3), "same"),
    ((1, 100, 6), 5, (1, 7), (1, 2), "valid"),       # a 1-D convolution as the simulator poses it
    ((33, 17, 70), 3, (5, 5), (1, 1), (2, 1)),       # more channels than one LDS chunk holds
    ((6, 6, 2), 300, (6, 6), (1, 1), "valid"),       # one output pixel, many filters
]


@pytest.mark.parametrize("channels_last", [True, False])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d(queue, rng, case, channels_last):
    """Bit-identical to the oracle: per output the same fused multiply-adds in the same
    order (channel, kernel row, kernel column), whatever the tiling."""
    (nxi, nxj, nc), nf, (si, sj), (sti, stj), padding = case
    if padding == "valid":
        pi, pj = 0, 0
    elif padding == "same":
        pi, pj = (si - 1) // 2, (sj - 1) // 2
    else:
        pi, pj = padding
    nyi, nyj = (nxi + 2 * pi - si) // sti + 1, (nxj + 2 * pj - sj) // stj + 1
    shape_in = (nxi, nxj, nc) if channels_last else (nc, nxi, nxj)
    shape_out = (nyi, nyj, nf) if channels_last else (nf, nyi, nyj)
    # the image and kernel sit between other signals of one buffer, as in the simulator
    data = RA([rng.normal(size=5), rng.normal(size=nxi * nxj * nc),
               rng.normal(size=si * sj * nc * nf), rng.normal(size=nyi * nyj * nf),
               rng.normal(size=3)])
    dev = to_dev(queue, data)
    nl().plan_conv2d(queue, dev[[1]], dev[[3]], dev[[2]], shape_in, shape_out, (si, sj),
                     padding=padding, strides=(sti, stj), channels_last=channels_last)()
    orc().plan_conv2d(None, data[[1]], data[[3]], data[[2]], shape_in, shape_out, (si, sj),
                      padding=padding, strides=(sti, stj), channels_last=channels_last)()
    assert np.array_equal(dev.buf, data.buf)


def test_local_filtering(queue, rng):
    nxi, nxj, nc, nf, si, sj = 12, 10, 3, 5, 3, 2
    nyi, nyj = nxi - si + 1, nxj - sj + 1
    for channels_last in (True, False):
        data = RA([rng.normal(size=nxi * nxj * nc), rng.normal(size=nf * nc * si * sj * nyi * nyj),
                   np.zeros(nf * nyi * nyj)])
        dev = to_dev(queue, data)
        shape_in = (nxi, nxj, nc) if channels_last else (nc, nxi, nxj)
        shape_out = (nyi, nyj, nf) if channels_last else (nf, nyi, nyj)
        nl().plan_conv2d(queue, dev[[0]], dev[[2]], dev[[1]], shape_in, shape_out, (si, sj),
                         conv=False, channels_last=channels_last)()
        orc().plan_conv2d(None, data[[0]], data[[2]], data[[1]], shape_in, shape_out, (si, sj),
                          conv=False, channels_last=channels_last)()
        assert np.abs(data[2]).max() > 0
        assert np.array_equal(dev.buf, data.buf)


def test_conv2d_rejects_bad_arguments(queue, rng):
    data = RA([np.zeros(50), np.zeros(9), np.zeros(18)])
    dev = to_dev(queue, data)
    with pytest.raises(AssertionError):  # X is not the size shape_in says
        nl().plan_conv2d(queue, dev[[0]], dev[[2]], dev[[1]], (5, 5, 1), (3, 3, 2), (3, 3))
    with pytest.raises(ValueError):
        nl().plan_conv2d(queue, dev[[0]], dev[[2]], dev[[1]], (5, 10, 1), (3, 6, 1), (3, 3),
                         padding="full")
    with pytest.raises(AssertionError):  # biases are not supported, as in the reference
        nl().plan_conv2d(queue, dev[[0]], dev[[2]], dev[[1]], (5, 10, 1), (3, 6, 1), (3, 3),
                         biases=dev[[1]])


@pytest.mark.parametrize("shape,pool,strides", [((3, 4, 4, 8, 12), (2, 3), (2, 3)),
                                                ((1, 3, 3, 5, 5), (2, 2), (2, 2)),
                                                ((16, 14, 14, 28, 28), (2, 2), (2, 2)),
                                                ((5, 9, 7, 20, 15), (3, 3), (2, 2))])
def test_pool2d(queue, rng, shape, pool, strides):
    nc, nyi, nyj, nxi, nxj = shape
    img = rng.normal(size=nc * nxi * nxj)
    img[rng.randint(0, img.size, size=5)] = np.nan  # skipped by the mean
    data = RA([np.zeros(3), img, np.zeros(nc * nyi * nyj)])
    dev = to_dev(queue, data)
    nl().plan_pool2d(queue, dev[[1]], dev[[2]], shape, pool, strides)()
    orc().plan_pool2d(None, data[[1]], data[[2]], shape, pool, strides)()
    assert np.array_equal(dev.buf, data.buf, equal_nan=True)


# ------------------------------------------------------------------ noise
def test_philox_known_answers(queue):
    """The generator's published test vectors, on the device."""
    import ctypes

    from nengo_ocl_amd import _lib
    from nengo_ocl_amd.hipraggedarray import to_device
    from helpers import PHILOX_KNOWN_ANSWERS

    rows = np.array([c + k for c, k, _ in PHILOX_KNOWN_ANSWERS], dtype=np.uint32)
    want = np.array([o for _, _, o in PHILOX_KNOWN_ANSWERS], dtype=np.uint32)
    extra = np.random.RandomState(0).randint(0, 2 ** 32, size=(500, 6), dtype=np.uint64).astype(np.uint32)
    rows = np.concatenate([rows, extra])
    d_in = to_device(queue, rows.view(np.int32))
    d_out = to_device(queue, np.zeros((len(rows), 4), dtype=np.int32))
    _lib.check(queue.lib.nhip_philox4x32(queue.handle, d_in.ptr, d_out.ptr, len(rows)))
    queue.finish()
    got = d_out.get().view(np.uint32)
    assert np.array_equal(got[:3], want)
    assert np.array_equal(got, orc().philox4x32(rows))


def test_whitenoise(queue):
    """Same streams as the oracle: uniform samples bit for bit; Gaussian samples go through
    double-precision log / sqrt / sin / cos of two math libraries and one final rounding,
    so they agree to the last float32 bit except where the double result lies within an
    ulp of a rounding boundary (tolerance: 1 float32 ulp, mismatches reported)."""
    dt = 1e-3
    sizes = [20000, 7, 1, 3000, 257]
    enums = [1, 0, 1, 0, 1]
    params = [(0.0, 1.0), (-2.0, 3.0), (1.5, 0.5), (0.0, 1.0), (0.0, 2.0)]
    scale, inc, seeds = [1, 0, 0, 1, 0], [0, 0, 1, 1, 0], [11, 12, 13, 14, 2 ** 31 + 5]
    Y = RA([np.full(n, 0.25) for n in sizes])
    dev = to_dev(queue, Y)
    gplan = nl().plan_whitenoise(queue, dev, np.int32(enums), np.float32(params), scale, inc, dt,
                                 seeds)
    oplan = orc().plan_whitenoise(None, Y, enums, params, scale, inc, dt, seeds)
    for call in range(3):
        gplan()
        oplan()
        got = dev.to_host()
        for i, e in enumerate(enums):
            if e == 0:
                assert np.array_equal(got[i], Y[i])
            else:
                ulp = np.spacing(np.abs(Y[i]))
                assert np.all(np.abs(got[i] - Y[i]) <= ulp)
                mismatch = np.mean(got[i] != Y[i])
                assert mismatch < 1e-3, "Gaussian samples differing in the last bit: %g" % mismatch
        dev.dev_buf.set(Y.buf)  # same starting point for the incrementing items
    assert np.array_equal(gplan.counters.get()[:len(sizes)], np.full(len(sizes), 3))
    gplan.reset_streams()
    oplan.reset_streams()
    Y.buf[:] = 0.25
    dev.dev_buf.set(Y.buf)
    gplan()
    oplan()
    assert np.allclose(dev.buf, Y.buf, rtol=1e-6, atol=0)


# ------------------------------------------------------------------ compiled function nodes
def test_plan_direct_compiled_functions(queue, rng):
    """Traced functions compiled at run time and launched over many node instances: the
    device's float32 result against the Python function in double precision (rtol 1e-5 /
    atol 2e-6: float32 evaluation of up to a dozen operations and library functions; the
    reference's own check of translated functions allows rtol 1e-5 / atol 2e-7 on single
    functions, tests/test_ast_conversion.py:198-200)."""
    from nengo_ocl_amd import fn_trace as ft
    from test_fn_trace import CASES

    n = 300  # instances: several waves
    skip_discontinuous = {20, 31}  # floor / mod / round: a float32 input next to a step
    for case, (fn, t_in, x_dim, out_dim) in enumerate(CASES):
        traced = ft.trace(fn, t_in, x_dim, out_dim)
        T = RA([[rng.uniform(0, 2)] for _ in range(n)])
        X = RA([rng.uniform(-3, 4, size=x_dim or 1) for _ in range(n)])
        Y = RA([np.zeros(out_dim) for _ in range(n)])
        dT, dX, dY = (to_dev(queue, a) for a in (T, X, Y))
        inputs = ([dT] if t_in else []) + ([dX] if x_dim else [])
        plan = nl().plan_direct(queue, traced.code, traced.init, traced.input_names, inputs, dY)
        assert plan.name == "hip_direct_compiled"
        plan()
        got = dY.to_host()
        if case in skip_discontinuous:
            continue
        for k in range(n):
            args = ([float(T[k][0, 0])] if t_in else []) + ([X[k][:, 0].astype(np.float64)] if x_dim else [])
            want = np.asarray(fn(*args), dtype=np.float64).ravel()
            np.testing.assert_allclose(got[k][:, 0], want, rtol=1e-5, atol=2e-6,
                                       err_msg="case %d instance %d" % (case, k))
        assert np.array_equal(dX.buf, X.buf) and np.array_equal(dT.buf, T.buf)


def test_plan_direct_unary_table_still_precompiled(queue):
    T = RA([[0.3], [1.2]])
    Y = RA([[0.0], [0.0]])
    dT, dY = to_dev(queue, T), to_dev(queue, Y)
    plan = nl().plan_direct(queue, "OUTPUT__[0] = sin(t[0]);", "", ["t"], [dT], dY)
    assert plan.name == "hip_direct"
    plan()
    np.testing.assert_allclose(dY.buf, np.sin(np.float32([0.3, 1.2])), rtol=1e-6)
    with pytest.raises(NotImplementedError, match="does not compile"):
        nl().plan_direct(queue, "OUTPUT__[0] = undefined_function(t[0]);", "", ["t"], [dT], dY)


# ------------------------------------------------------------------ many short signals
@pytest.mark.parametrize("size,lanes", [(1, 1), (2, 2), (3, 4), (6, 8), (11, 16), (25, 32),
                                        (50, 64), (200, 256), (2000, 256)])
def test_many_short_items_every_lane_width(queue, rng, size, lanes):
    """Models with very many very short signals: rows are handled by 1, 2, ... 64 lanes
    each instead of a 256-thread group (the width follows the median item size; longer
    items are cut into several rows).  Every element-wise operation, the
    filters (all three forms, several steps, so that ring positions advance), input
    playback, probes and unary functions against the oracle, bit for bit."""
    n_items = 700 if size <= 200 else 5
    sizes = np.maximum(1, rng.randint(size - size // 4, size + size // 4 + 1, size=n_items))
    sizes[1] = size          # (the median stays `size`)
    sizes[0] = 9 * size + 1  # one long item among them: cut into several rows
    vec = lambda: RA([rng.normal(size=n) for n in sizes])
    plans = []  # (device plan, oracle plan)

    # reset / copy / sliced copy / elementwise
    Y1 = vec(); dY1 = to_dev(queue, Y1)
    values = rng.normal(size=n_items).astype(np.float32)
    plans.append((nl().plan_reset(queue, dY1, values), orc().plan_reset(None, Y1, values)))
    X2, Y2 = vec(), vec(); dX2, dY2 = to_dev(queue, X2), to_dev(queue, Y2)
    incs = rng.randint(0, 2, size=n_items).astype(np.int32)
    plans.append((nl().plan_copy(queue, dX2, dY2, incs), orc().plan_copy(None, X2, Y2, incs)))
    XI = RA([rng.permutation(n)[: max(1, n // 2)] for n in sizes], dtype=np.int32)
    YI = RA([rng.permutation(n)[: max(1, n // 2)] for n in sizes], dtype=np.int32)
    X3, Y3 = vec(), vec(); dX3, dY3 = to_dev(queue, X3), to_dev(queue, Y3)
    plans.append((nl().plan_slicedcopy(queue, dX3, dY3, to_dev(queue, XI), to_dev(queue, YI), incs),
                  orc().plan_slicedcopy(None, X3, Y3, XI, YI, incs)))
    A4 = RA([[rng.normal()] for _ in sizes]); X4, Y4 = vec(), vec()
    dY4 = to_dev(queue, Y4)
    plans.append((nl().plan_elementwise_inc(queue, to_dev(queue, A4), to_dev(queue, X4), dY4),
                  orc().plan_elementwise_inc(None, A4, X4, Y4)))

    # filters: gain, lowpass and second-order items mixed
    kinds = [("gain", "lowpass", "alpha")[k % 3] for k in range(n_items)]
    coefs = [_filter_coefficients(k) for k in kinds]
    A5, B5 = RA([den for _, den in coefs]), RA([num for num, _ in coefs])
    X5, Y5 = vec(), RA([np.zeros(n) for n in sizes])
    Xbuf, Ybuf = RA([np.zeros(s) for s in zip(B5.sizes, X5.sizes)]), RA(
        [np.zeros(s) for s in zip(A5.sizes, Y5.sizes)])
    dX5, dY5 = to_dev(queue, X5), to_dev(queue, Y5)
    gf = nl().plan_linearfilter(queue, dX5, dY5, to_dev(queue, A5), to_dev(queue, B5),
                                to_dev(queue, Xbuf), to_dev(queue, Ybuf))
    of = orc().plan_linearfilter(None, X5, Y5, A5, B5, Xbuf, Ybuf)
    plans += list(zip(gf, of[:len(gf)]))
    extra_oracle = of[len(gf):]  # the oracle's separate position update, if any

    # input playback and probes: rows cannot be cut, the width follows the largest item
    small = np.minimum(sizes, 300)
    tables = [rng.normal(size=(7, n)) for n in small]
    S6, Y6 = RA(tables), RA([np.zeros(n) for n in small])
    T6 = RA([[3.0]] * n_items)
    dY6 = to_dev(queue, Y6)
    plans.append((nl().plan_presentinput(queue, dY6, to_dev(queue, T6), to_dev(queue, S6), 1e-3),
                  orc().plan_presentinput(None, Y6, T6, S6, 1e-3)))
    n_buf = 6
    P7 = RA([np.zeros((n_buf, n)) for n in sizes]); dP7 = to_dev(queue, P7)
    periods = rng.choice([1.0, 2.0, 2.5], size=n_items)
    gp, op = nl().plan_probes(queue, periods, dX5, dP7), orc().plan_probes(None, periods, X5, P7)
    plans.append((gp, op))

    widths = {p.name: p.args[{"hip_linearfilter": 3}.get(p.name, 2)] for p, _ in plans}
    assert widths["hip_reset"] == widths["hip_copy"] == widths["hip_linearfilter"] == lanes, widths
    for step in range(4):
        x_new = rng.normal(size=X5.buf.size).astype(np.float32)
        X5.buf[:] = x_new
        dX5.dev_buf.set(x_new)
        for g, o in plans:
            g()
            o()
        for o in extra_oracle:
            o()
        for dev, host in ((dY1, Y1), (dY2, Y2), (dY3, Y3), (dY4, Y4), (dY5, Y5), (dY6, Y6), (dP7, P7)):
            assert np.array_equal(dev.buf, host.buf), "step %d" % step
    assert np.array_equal(gp.dev_bufpositions.get(), op.bufpositions)
