"""GPU parity of the ragged gather-GEMV against the CPU oracle.

Shapes, seeds and parameters follow the reference's own GEMV tests
(nengo_ocl/tests/test_clra_gemv.py: test_basic :60-93, _test_random :96-145,
check_from_shapes :165-217 and the shape cases :220-289).  Every case runs
through all planner classes.  Tolerance: rtol 1e-4 / atol 1e-5 against the
oracle (block summation order of the reference) and against a float64
accumulate; the summation order of the HIP kernels differs from the oracle's,
so this comparison is tolerance based, not bit based.
"""

import numpy as np
import pytest

from helpers import RA, clone, to_dev

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def planners():
    from nengo_ocl_amd import hipra_gemv as g

    return [g.plan_block_gemv, g.plan_ragged_gather_gemv, g.plan_reduce_gemv,
            g.plan_many_dots_gemv, g.plan_ref_gemv]


PLANNER_NAMES = ["block", "ragged_gather", "reduce", "many_dots", "ref"]


def run_case(queue, planner, alpha, beta, gamma, A, X, Y, A_js, X_js, Y_in=None):
    from oracle import oracle as orc

    # float64 expectation
    expect = []
    Yin_host = Y if Y_in is None else Y_in
    for i in range(len(Y)):
        acc = np.zeros(Y[i].shape, dtype=np.float64)
        for aj, xj in zip(np.asarray(A_js[i]).ravel(), np.asarray(X_js[i]).ravel()):
            acc += A[int(aj)].astype(np.float64) @ X[int(xj)].astype(np.float64)
        a = np.asarray(alpha, dtype=np.float64).reshape(-1)
        b = np.asarray(beta, dtype=np.float64).reshape(-1)
        g = np.asarray(gamma, dtype=np.float64).reshape(-1)
        expect.append(g[i % g.size] + b[i % b.size] * Yin_host[i].astype(np.float64)
                      + a[i % a.size] * acc)

    # oracle (reference block order, float32)
    Yo = clone(Y)
    Yo_in = Yo if Y_in is None else clone(Y_in)
    orc.plan_block_gemv(None, alpha, A, A_js, X, X_js, beta, Yo, Y_in=Yo_in, gamma=gamma).plans[0]()

    dA, dX, dY = to_dev(queue, A), to_dev(queue, X), to_dev(queue, Y)
    dYin = None if Y_in is None else to_dev(queue, Y_in)
    prog = planner(queue, alpha, dA, A_js, dX, X_js, beta, dY, Y_in=dYin, gamma=gamma)
    assert len(prog.plans) >= 1
    for plan in prog.plans:
        plan()
    got = dY.to_host()
    for i in range(len(Y)):
        scale = max(1.0, float(np.abs(expect[i]).max()) if expect[i].size else 1.0)
        np.testing.assert_allclose(got[i], Yo[i], rtol=RTOL, atol=ATOL * scale)
        np.testing.assert_allclose(got[i], expect[i], rtol=RTOL, atol=ATOL * scale)
    # inputs untouched
    assert np.array_equal(dA.buf, A.buf) and np.array_equal(dX.buf, X.buf)
    return prog


@pytest.mark.parametrize("pi", range(5), ids=PLANNER_NAMES)
def test_basic_literal(queue, pi):
    """Literal vectors of test_clra_gemv.py:60-93: Y0 = 4.5, Y1 = [3.3, 5.9]."""
    A = RA([[[0.1, 0.2], [0.3, 0.4]], [[0.5, 0.6]]])
    X = RA([[3, 5]])
    Y = RA([[0.0], [2, 3]])
    A_js = RA([[1], [0]], dtype=np.int32)
    X_js = RA([[0], [0]], dtype=np.int32)
    dA, dX, dY = to_dev(queue, A), to_dev(queue, X), to_dev(queue, Y)
    prog = planners()[pi](queue, 1.0, dA, A_js, dX, X_js, 1.0, dY)
    for plan in prog.plans:
        plan()
    np.testing.assert_allclose(dY[0].ravel(), [4.5], rtol=1e-6)
    np.testing.assert_allclose(dY[1].ravel(), [3.3, 5.9], rtol=1e-6)


def _random_case(queue, planner, k, p, m, n, align):
    rng = np.random.RandomState(3294)
    aa = [rng.normal(size=(m, n)) for _ in range(k)]
    xx = [rng.normal(size=n) for _ in range(k)]
    yy = [rng.normal(size=m) for _ in range(k)]
    ajs = [rng.randint(k, size=p) for _ in range(k)]
    xjs = [rng.randint(k, size=p) for _ in range(k)]
    run_case(queue, planner, 0.5, 0.1, 0.0, RA(aa, align=align), RA(xx), RA(yy),
             RA(ajs, dtype=np.int32), RA(xjs, dtype=np.int32))


@pytest.mark.parametrize("align", [False, True], ids=["packed", "aligned"])
@pytest.mark.parametrize("pi", range(5), ids=PLANNER_NAMES)
@pytest.mark.parametrize("k,p,m,n", [(4, 1, 10, 10), (10, 1, 550, 550), (4, 4, 10, 10),
                                     (4, 4, 2000, 1000)],
                         ids=["small", "large", "many_dots_small", "many_dots_large"])
def test_random(queue, pi, k, p, m, n, align):
    _random_case(queue, planners()[pi], k, p, m, n, align)


def _from_shapes(queue, planner, alpha, beta, gamma, A_shapes, X_shapes, A_js, X_js, align=False):
    rng = np.random.RandomState(1234)
    A = RA([0.1 + rng.rand(*shp) for shp in A_shapes], align=align)
    X = RA([0.1 + rng.rand(*shp) for shp in X_shapes])
    Y = RA([0.1 + rng.rand(A_shapes[A_js[i][0]][0], X_shapes[X_js[i][0]][1])
            for i in range(len(A_js))])
    run_case(queue, planner, alpha, beta, gamma, A, X, Y,
             RA([list(a) for a in A_js], dtype=np.int32), RA([list(x) for x in X_js], dtype=np.int32))


@pytest.mark.parametrize("pi", range(5), ids=PLANNER_NAMES)
@pytest.mark.parametrize("rows", [1, 10, 2001])
def test_one_segment(queue, pi, rows):
    _from_shapes(queue, planners()[pi], 0.5, 0.6, 0.7, [(rows, 1)], [(1, 1)], [[0]], [[0]])


@pytest.mark.parametrize("pi", range(5), ids=PLANNER_NAMES)
@pytest.mark.parametrize("ND", [2, 20, 100])
def test_one_short_segment_many_dots(queue, pi, ND):
    _from_shapes(queue, planners()[pi], 0.5, 0.6, 0.7,
                 [(10, 1 + i % 2) for i in range(ND)], [(1 + i % 2, 1) for i in range(ND)],
                 [range(ND)], [range(ND)])


@pytest.mark.parametrize("pi", range(5), ids=PLANNER_NAMES)
@pytest.mark.parametrize("ND", [2, 20, 100])
def test_one_short_segment_many_longer_dots(queue, pi, ND):
    _from_shapes(queue, planners()[pi], 0.5, 0.6, 0.7,
                 [(2000, i + 1) for i in range(ND)], [(i + 1, 1) for i in range(ND)],
                 [range(ND)], [range(ND)], align=True)


@pytest.mark.parametrize("pi", [0, 2, 3], ids=["block", "reduce", "many_dots"])
def test_ensemble_shapes(queue, pi):
    """The shapes the benchmark configurations produce: encoders (n x d, tall and
    thin), decoders (d x n, short and wide), per-neuron scalars, single dots."""
    rng = np.random.RandomState(7)
    shapes = [(4096, 64), (64, 4096), (100, 1), (1, 100), (100, 2), (2, 100), (2000, 32),
              (32, 2000), (132, 64), (64, 132), (5, 5000), (3, 7), (1, 1), (300, 9000), (600, 16),
              (600, 20), (3000, 4), (700, 50), (700, 130)]
    A = RA([rng.normal(size=s) for s in shapes], align=True)
    X = RA([rng.normal(size=s[1]) for s in shapes], align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes], align=True)
    js = RA([[i] for i in range(len(shapes))], dtype=np.int32)
    prog = run_case(queue, planners()[pi], 1.0, 1.0, 0.0, A, X, Y, js, js)
    if pi == 0:
        classes = {p.kernel_class for p in prog.plans}
        # compile-time shapes (6: stages of 8 / 16 as well as of 512 columns), 4 columns
        # (a power of two), rows that are not 16-byte aligned (back to back with at most 64
        # columns: read in quads all the same; otherwise 4-byte loads), small
        assert classes == {(3, 6, 4), (3, 1, 4), (3, 7, 4), (3, 0, 1), (2, 4, 1)}


def test_strided_views_and_yin(queue):
    """A is a column slice of a wider matrix (row stride > columns, one aligned and
    one unaligned), X and Y are strided views of vectors, Y_in differs from Y, and
    alpha / beta / gamma differ per item."""
    from nengo_ocl_amd import hipra_gemv as g
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray
    from nengo_ocl_amd.raggedarray import RaggedArray
    from oracle import oracle as orc

    rng = np.random.RandomState(11)
    base = RA([rng.normal(size=(40, 96)), rng.normal(size=(200,)), rng.normal(size=(80,)),
               rng.normal(size=(70,)), rng.normal(size=(70, 33))], align=True)
    s = base.starts
    # items 5..8: A0 = base0[:, 32:80]; X0 = base1[0::4][:48]; A1 = base4[:, 1:33]; X1 = base1[3::5][:32]
    base.add_views([s[0] + 32, s[1], s[4] + 1, s[1] + 3], [40, 48, 70, 32], [48, 1, 32, 1],
                   [96, 4, 33, 5], [1, 1, 1, 1])
    A_js = RA([[5], [7]], dtype=np.int32)
    X_js = RA([[6], [8]], dtype=np.int32)
    y_meta = ([s[2], s[3]], [40, 70], [1, 1], [2, 1], [1, 1])  # Y0 = base2[::2], Y1 = base3
    Yin = RA([rng.normal(size=40), rng.normal(size=70)])
    alpha, beta, gamma = [0.5, -1.5], [1.0, 0.25], [0.0, 2.0]

    host = clone(base)
    Yo = RaggedArray.from_buffer(host.buf, *y_meta)
    orc.plan_block_gemv(None, alpha, host, A_js, host, X_js, beta, Yo, Y_in=clone(Yin),
                        gamma=gamma).plans[0]()

    dbase = to_dev(queue, base)
    dY = HIPRaggedArray.from_buffer(queue, dbase.dev_buf, *y_meta)
    prog = g.plan_block_gemv(queue, alpha, dbase, A_js, dbase, X_js, beta, dY,
                             Y_in=to_dev(queue, Yin), gamma=gamma)
    for plan in prog.plans:
        plan()
    got = dbase.buf
    np.testing.assert_allclose(got, host.buf, rtol=RTOL, atol=1e-4)
    changed = got != base.buf
    expect_changed = np.zeros_like(changed)
    expect_changed[s[2]:s[2] + 80:2] = True
    expect_changed[s[3]:s[3] + 70] = True
    assert np.array_equal(changed, expect_changed)  # nothing outside Y was written


def test_empty_dot_list_and_zero_rows(queue):
    """An output with no dot products is just beta*Y_in + gamma; zero-length outputs are skipped."""
    from nengo_ocl_amd import hipra_gemv as g

    A = RA([np.ones((3, 2))])
    X = RA([np.ones(2)])
    Y = RA([np.arange(3.0), np.arange(5.0)])
    A_js = [np.array([0], dtype=np.int32), np.array([], dtype=np.int32)]
    X_js = [np.array([0], dtype=np.int32), np.array([], dtype=np.int32)]
    dY = to_dev(queue, Y)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), A_js, to_dev(queue, X), X_js, 2.0, dY,
                             gamma=1.0)
    for plan in prog.plans:
        plan()
    np.testing.assert_allclose(dY[0].ravel(), 2 * np.arange(3.0) + 1 + 2)
    np.testing.assert_allclose(dY[1].ravel(), 2 * np.arange(5.0) + 1)


def test_bad_arguments_raise(queue):
    from nengo_ocl_amd import hipra_gemv as g

    A = to_dev(queue, RA([np.ones((3, 2))]))
    X = to_dev(queue, RA([np.ones(3)]))
    Y = to_dev(queue, RA([np.zeros(3)]))
    js = RA([[0]], dtype=np.int32)
    with pytest.raises(ValueError):
        g.plan_block_gemv(queue, 1.0, A, js, X, js, 1.0, Y)  # 2 columns vs 3-vector


def test_linearity_at_full_size(queue):
    """Size-independent property at the large configuration's shapes: the GEMV is
    linear in X, so A@(2x) - 2*(A@x) == 0 up to rounding, and A@e_k picks column k
    bit-exactly (gather check)."""
    from nengo_ocl_amd import hipra_gemv as g

    rng = np.random.RandomState(5)
    n_ens, n, d = 8, 4096, 64
    enc = [rng.normal(size=(n, d)).astype(np.float32) for _ in range(n_ens)]
    dec = [rng.normal(size=(d, n)).astype(np.float32) for _ in range(n_ens)]
    k_enc, k_dec = 37, 2049
    ex, dx = np.zeros(d, np.float32), np.zeros(n, np.float32)
    ex[k_enc], dx[k_dec] = 1.0, 1.0
    A = RA(enc + dec, align=True)
    X = RA([ex] * n_ens + [dx] * n_ens, align=True)
    Y = RA([np.zeros(n)] * n_ens + [np.zeros(d)] * n_ens, align=True)
    js = RA([[i] for i in range(2 * n_ens)], dtype=np.int32)
    dY = to_dev(queue, Y)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), js, to_dev(queue, X), js, 0.0, dY)
    for plan in prog.plans:
        plan()
    for i in range(n_ens):
        assert np.array_equal(dY[i].ravel(), enc[i][:, k_enc])
        assert np.array_equal(dY[n_ens + i].ravel(), dec[i][:, k_dec])


def test_small_items_bit_exact(queue):
    """Small items run in the reference's summation order: with alpha = beta = 1 and
    gamma = 0 (what the simulator produces) the result equals the oracle bit for bit,
    including outputs that sum several dot products and rows longer than one tile."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(99)
    shapes = [(100, 1), (1, 100), (100, 2), (2, 100), (1, 1), (7, 300), (16, 129), (3, 512),
              (40, 17), (64, 128)]
    A = RA([rng.normal(size=s) for s in shapes] + [rng.normal(size=(10, 5)) for _ in range(6)])
    X = RA([rng.normal(size=s[1]) for s in shapes] + [rng.normal(size=5) for _ in range(6)])
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=10)])
    n = len(shapes)
    A_js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + 6, dtype=np.int32)]
    X_js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + 6, dtype=np.int32)]
    for beta in (1.0, 0.0):
        Yo = clone(Y)
        orc.plan_block_gemv(None, 1.0, A, A_js, X, X_js, beta, Yo).plans[0]()
        dY = to_dev(queue, Y)
        prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), A_js, to_dev(queue, X), X_js, beta, dY)
        assert {p.kernel_class for p in prog.plans} == {(2, 4, 1)}
        for plan in prog.plans:
            plan()
        assert np.array_equal(dY.buf, Yo.buf)


@pytest.mark.parametrize("beta", [1.0, 0.0])
def test_large_items_bit_exact(queue, beta):
    """Large items are staged through LDS and summed in the reference's order too:
    bit-identical to the oracle for every shape class the configurations produce,
    for unaligned and odd shapes, rows longer than one stage, several dot products
    of different widths per output, and a Y_in different from Y."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(4242)
    shapes = [(4096, 64), (64, 4096), (2000, 32), (32, 2000), (300, 9000), (5, 5000), (550, 550),
              (1000, 130), (70, 33), (257, 129), (9000, 3), (3, 9000), (129, 1025), (2049, 5)]
    A = RA([rng.normal(size=s) for s in shapes] + [rng.normal(size=(500, n)) for n in (64, 700, 3, 128, 2500)],
           align=True)
    X = RA([rng.normal(size=s[1]) for s in shapes] + [rng.normal(size=n) for n in (64, 700, 3, 128, 2500)],
           align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=500)], align=True)
    Yin = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=500)], align=True)
    n = len(shapes)
    js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + 5, dtype=np.int32)]
    for use_yin in (False, True):
        Yo = clone(Y)
        orc.plan_block_gemv(None, 1.0, A, js, X, js, beta, Yo, Y_in=clone(Yin) if use_yin else None).plans[0]()
        dY = to_dev(queue, Y)
        prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), js, to_dev(queue, X), js, beta, dY,
                                 Y_in=to_dev(queue, Yin) if use_yin else None)
        assert {p.kernel_class[0] for p in prog.plans} == {2, 3}
        for plan in prog.plans:
            plan()
        got = dY.to_host()
        for i in range(len(Y)):
            assert np.array_equal(got[i], Yo[i]), (i, use_yin)


@pytest.mark.parametrize("beta", [1.0, 0.5])
def test_pow2_items_bit_exact(queue, beta):
    """Power-of-two column counts: every width from 4 to 16384, row counts that leave
    partial row blocks and partial tasks, outputs that sum dot products of different
    power-of-two widths, and matrix views with a row stride larger than the width --
    bit-identical to the oracle.  Items with a 4-column dot product take the staged
    kernel for powers of two, the others the one with compile-time shapes."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(777)
    shapes = [(5001, 4), (3003, 8), (1111, 16), (999, 32), (4096, 64), (777, 64), (301, 128),
              (130, 256), (67, 512), (33, 1024), (64, 4096), (9, 8192), (1, 16384), (257, 2048)]
    multi = (64, 128, 1024, 4, 512)
    mats = [rng.normal(size=s) for s in shapes] + [rng.normal(size=(300, n)) for n in multi]
    A = RA(mats, align=True)
    X = RA([rng.normal(size=m.shape[1]) for m in mats], align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=300)], align=True)
    n = len(shapes)
    js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + len(multi), dtype=np.int32)]
    Yo = clone(Y)
    orc.plan_block_gemv(None, 1.0, A, js, X, js, beta, Yo).plans[0]()
    dY = to_dev(queue, Y)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), js, to_dev(queue, X), js, beta, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 1, 4), (3, 6, 4)}
    for plan in prog.plans:
        plan()
    got = dY.to_host()
    for i in range(len(Y)):
        assert np.array_equal(got[i], Yo[i]), i

    # column blocks of a wider matrix: row stride 640, widths 128 and 512
    wide = rng.normal(size=(700, 640)).astype(np.float32)
    Aw = RA([wide], align=True)
    Av = Aw[[0]]  # shares the buffer
    Av.add_views([Aw.starts[0], Aw.starts[0] + 128], [700, 700], [128, 512], [640, 640], [1, 1])
    Xw = RA([rng.normal(size=128), rng.normal(size=512)], align=True)
    Yw = RA([rng.normal(size=700)], align=True)
    jA, jX = [np.array([1, 2], dtype=np.int32)], [np.array([0, 1], dtype=np.int32)]
    Yo = clone(Yw)
    orc.plan_block_gemv(None, 1.0, Av, jA, Xw, jX, beta, Yo).plans[0]()
    dY = to_dev(queue, Yw)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, Av), jA, to_dev(queue, Xw), jX, beta, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 4, 4)}
    for plan in prog.plans:
        plan()
    assert np.array_equal(dY.to_host()[0], Yo[0])
    expect = beta * Yw[0][:, 0] + wide[:, :128] @ Xw[0][:, 0] + wide[:, 128:] @ Xw[1][:, 0]
    assert np.allclose(Yo[0][:, 0], expect, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("beta", [1.0, 0.5])
@pytest.mark.parametrize("widths", ["to-64", "to-64-and-from-512", "from-32", "from-8-to-64", "all"])
def test_compile_time_shape_items_bit_exact(queue, beta, widths):
    """Column counts that are multiples of 4 from 8 up take the kernel whose stage
    shapes are compile-time constants (stages of 8, 16, 32, 64, 128 or 512 columns; one
    instance per set of stage widths a launch needs): row counts that leave partial
    row blocks, widths that leave a narrower last or only column stage, tasks of one to
    many stages, outputs that sum dot products of several such widths, a Y_in different
    from Y -- bit-identical to the oracle."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(31337)
    narrow = [(999, 32), (513, 32), (8200, 32), (4096, 64), (777, 64), (2049, 64), (257, 64),
              (1000, 36), (700, 48), (4100, 60), (300, 52), (2000, 44)]
    wide = [(67, 512), (131, 512), (33, 1024), (64, 4096), (6, 4096), (9, 8192), (1, 16384),
            (257, 2048), (3, 32768),
            # not a power of two: last column stages of 4 ... 508 columns
            (32, 2000), (300, 9000), (5, 5000), (64, 516), (9, 1028), (40, 700), (7, 520),
            (21, 1660), (130, 1020)]
    middle = [(301, 128), (130, 256), (700, 100), (300, 132), (260, 300), (1000, 500), (90, 508),
              (513, 68), (400, 260)]
    tiny = [(4096, 16), (4096, 8), (3000, 24), (5000, 12), (1037, 8), (999, 16), (2000, 28),
            (515, 20), (8300, 8), (2057, 12), (1029, 16), (7000, 16)]
    shapes, multi, expected = {
        "to-64": (narrow, (64, 32, 48, 64, 36), (3, 3, 4)),
        "to-64-and-from-512": (narrow + wide, (64, 1024, 32, 512, 64, 2000, 644, 40), (3, 2, 4)),
        "from-32": (narrow + wide + middle, (64, 1024, 300, 32, 512, 128, 2000, 68), (3, 4, 4)),
        "from-8-to-64": (tiny + narrow, (16, 64, 8, 32, 12, 48, 16, 8, 24), (3, 5, 4)),
        "all": (tiny + narrow[:6] + wide[::3] + middle[::2],
                (8, 1024, 300, 16, 512, 12, 128, 2000, 68, 8, 32), (3, 6, 4)),
    }[widths]
    mats = [rng.normal(size=s) for s in shapes] + [rng.normal(size=(300, n)) for n in multi]
    A = RA(mats, align=True)
    X = RA([rng.normal(size=m.shape[1]) for m in mats], align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=300)], align=True)
    Yin = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=300)], align=True)
    n = len(shapes)
    js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + len(multi), dtype=np.int32)]
    for use_yin in (False, True):
        Yo = clone(Y)
        orc.plan_block_gemv(None, 0.75, A, js, X, js, beta, Yo, Y_in=clone(Yin) if use_yin else None,
                            gamma=0.125).plans[0]()
        dY = to_dev(queue, Y)
        prog = g.plan_block_gemv(queue, 0.75, to_dev(queue, A), js, to_dev(queue, X), js, beta, dY,
                                 Y_in=to_dev(queue, Yin) if use_yin else None, gamma=0.125)
        assert {p.kernel_class for p in prog.plans} == {expected}
        for plan in prog.plans:
            plan()
        got = dY.to_host()
        for i in range(len(Y)):
            assert np.array_equal(got[i], Yo[i]), (i, use_yin)


@pytest.mark.parametrize("beta", [1.0, 0.5])
def test_compile_time_shape_views_bit_exact(queue, beta):
    """Matrix views with a row stride larger than the width and strided X vectors."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(4711)
    # column blocks of a wider matrix (row stride 1200: widths 64, 600 and 32) times
    # every second / third element of longer vectors
    wide = rng.normal(size=(700, 1200)).astype(np.float32)
    Aw = RA([wide], align=True)
    Av = Aw[[0]]  # shares the buffer
    s0 = int(Aw.starts[0])
    Av.add_views([s0, s0 + 64, s0 + 664], [700, 700, 700], [64, 600, 32], [1200] * 3, [1] * 3)
    xs = [rng.normal(size=64 * 2), rng.normal(size=600 * 3), rng.normal(size=32)]
    Xw = RA(xs, align=True)
    Xv = Xw[[0]]
    Xv.add_views([int(Xw.starts[0]), int(Xw.starts[1]), int(Xw.starts[2])], [64, 600, 32], [1] * 3,
                 [2, 3, 1], [1] * 3)
    Yw = RA([rng.normal(size=700)], align=True)
    jA, jX = [np.array([1, 2, 3], dtype=np.int32)], [np.array([1, 2, 3], dtype=np.int32)]
    Yo = clone(Yw)
    orc.plan_block_gemv(None, 1.0, Av, jA, Xv, jX, beta, Yo).plans[0]()
    dY = to_dev(queue, Yw)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, Av), jA, to_dev(queue, Xv), jX, beta, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 2, 4)}
    for plan in prog.plans:
        plan()
    assert np.array_equal(dY.to_host()[0], Yo[0])
    expect = (beta * Yw[0][:, 0] + wide[:, :64] @ xs[0][::2] + wide[:, 64:664] @ xs[1][::3]
              + wide[:, 664:696] @ xs[2])
    assert np.allclose(Yo[0][:, 0], expect, rtol=1e-4, atol=1e-3)


def test_compile_time_shape_odd_width_views_bit_exact(queue):
    """Column blocks of a wider matrix whose widths are no multiple of 4 (50, 333 and 601
    columns at a row stride of 1200, rows 16-byte aligned) take the same kernel: the
    16-byte loads run into the columns next to the block, which are not summed."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(99)
    wide = rng.normal(size=(700, 1200)).astype(np.float32)
    Aw = RA([wide], align=True)
    Av = Aw[[0]]
    s0 = int(Aw.starts[0])
    Av.add_views([s0, s0 + 52, s0 + 388], [700, 700, 700], [50, 333, 601], [1200] * 3, [1] * 3)
    xs = [rng.normal(size=50), rng.normal(size=333), rng.normal(size=601)]
    Xw = RA(xs, align=True)
    Yw = RA([rng.normal(size=700), rng.normal(size=700)], align=True)
    jA = [np.array([1, 2, 3], dtype=np.int32), np.array([1], dtype=np.int32)]
    jX = [np.array([0, 1, 2], dtype=np.int32), np.array([0], dtype=np.int32)]
    Yo = clone(Yw)
    orc.plan_block_gemv(None, 1.0, Av, jA, Xw, jX, 0.5, Yo).plans[0]()
    dY = to_dev(queue, Yw)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, Av), jA, to_dev(queue, Xw), jX, 0.5, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 4, 4)}
    for plan in prog.plans:
        plan()
    got = dY.to_host()
    assert np.array_equal(got[0], Yo[0]) and np.array_equal(got[1], Yo[1])
    expect = (0.5 * Yw[0][:, 0] + wide[:, :50] @ xs[0] + wide[:, 52:385] @ xs[1]
              + wide[:, 388:989] @ xs[2])
    assert np.allclose(Yo[0][:, 0], expect, rtol=1e-4, atol=1e-3)
    # widths from 5 up: 5, 9, 14 and 17 columns of a matrix with 48
    slim = rng.normal(size=(3000, 48)).astype(np.float32)
    As = RA([slim], align=True)
    Av = As[[0]]
    s0 = int(As.starts[0])
    cols, widths = [0, 8, 20, 28], [5, 9, 14, 17]
    Av.add_views([s0 + c for c in cols], [3000] * 4, widths, [48] * 4, [1] * 4)
    xs = [rng.normal(size=w) for w in widths]
    Xs = RA(xs, align=True)
    Ys = RA([rng.normal(size=3000), rng.normal(size=3000)], align=True)
    jA = [np.array([1, 2, 3, 4], dtype=np.int32), np.array([2], dtype=np.int32)]
    jX = [np.array([0, 1, 2, 3], dtype=np.int32), np.array([1], dtype=np.int32)]
    Yo = clone(Ys)
    orc.plan_block_gemv(None, 1.0, Av, jA, Xs, jX, 0.5, Yo).plans[0]()
    dY = to_dev(queue, Ys)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, Av), jA, to_dev(queue, Xs), jX, 0.5, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 5, 4)}
    for plan in prog.plans:
        plan()
    got = dY.to_host()
    assert np.array_equal(got[0], Yo[0]) and np.array_equal(got[1], Yo[1])
    expect = 0.5 * Ys[0][:, 0] + sum(slim[:, c:c + w] @ x for c, w, x in zip(cols, widths, xs))
    assert np.allclose(Yo[0][:, 0], expect, rtol=1e-4, atol=1e-3)
    # a contiguous matrix of such a width at the very end of its buffer has nothing readable
    # behind its last row: general kernel
    A = RA([rng.normal(size=(700, 50))], align=True)
    X = RA([rng.normal(size=50)], align=True)
    Y = RA([rng.normal(size=700)], align=True)
    js = [np.array([0], dtype=np.int32)]
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), js, to_dev(queue, X), js, 0.0, to_dev(queue, Y))
    assert {p.kernel_class for p in prog.plans} == {(3, 0, 1)}


@pytest.mark.parametrize("beta", [1.0, 0.5])
def test_back_to_back_rows_bit_exact(queue, beta):
    """Matrices of at most 64 columns whose rows are not 16-byte aligned but lie back to
    back (10, 50, 30, 5, 6, 13, 63 columns) are read in 16-byte quads block by block: row
    counts that leave partial blocks, partial last quads and short last tasks, outputs
    that sum several such dot products (one of them with aligned rows), a Y_in different
    from Y -- bit-identical to the oracle.  Wider ones, and a column block of a wider
    matrix with such a width, stay on 4-byte loads."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(2718)
    shapes = [(4096, 10), (4097, 50), (1001, 30), (2500, 5), (333, 63), (5003, 6), (999, 37),
              (1026, 13), (300, 62), (8190, 9)]
    multi = (10, 50, 64, 7, 62)
    mats = [rng.normal(size=s) for s in shapes] + [rng.normal(size=(1030, n)) for n in multi]
    mats.append(np.zeros((1, 8)))  # something readable behind the last matrix
    A = RA(mats, align=True)
    X = RA([rng.normal(size=m.shape[1]) for m in mats], align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=1030)], align=True)
    Yin = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=1030)], align=True)
    n = len(shapes)
    js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + len(multi), dtype=np.int32)]
    for use_yin in (False, True):
        Yo = clone(Y)
        orc.plan_block_gemv(None, 0.75, A, js, X, js, beta, Yo, Y_in=clone(Yin) if use_yin else None,
                            gamma=0.125).plans[0]()
        dY = to_dev(queue, Y)
        prog = g.plan_block_gemv(queue, 0.75, to_dev(queue, A), js, to_dev(queue, X), js, beta, dY,
                                 Y_in=to_dev(queue, Yin) if use_yin else None, gamma=0.125)
        assert {p.kernel_class for p in prog.plans} == {(3, 7, 4)}
        for plan in prog.plans:
            plan()
        got = dY.to_host()
        for i in range(len(Y)):
            assert np.array_equal(got[i], Yo[i]), (i, use_yin)
    expect = 0.75 * (mats[0].astype(np.float32) @ X[0][:, 0]) + beta * Yin[0][:, 0] + 0.125
    assert np.allclose(Yo[0][:, 0], expect, rtol=1e-4, atol=1e-3)

    # 50 columns of a matrix with 70 whose block starts at column 2: neither aligned rows
    # nor rows back to back
    wide = rng.normal(size=(700, 70)).astype(np.float32)
    Aw = RA([wide], align=True)
    Av = Aw[[0]]
    Av.add_views([int(Aw.starts[0]) + 2], [700], [50], [70], [1])
    Xw = RA([rng.normal(size=50)], align=True)
    Yw = RA([rng.normal(size=700)], align=True)
    jA, jX = [np.array([1], dtype=np.int32)], [np.array([0], dtype=np.int32)]
    Yo = clone(Yw)
    orc.plan_block_gemv(None, 1.0, Av, jA, Xw, jX, beta, Yo).plans[0]()
    dY = to_dev(queue, Yw)
    prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, Av), jA, to_dev(queue, Xw), jX, beta, dY)
    assert {p.kernel_class for p in prog.plans} == {(3, 0, 1)}
    for plan in prog.plans:
        plan()
    assert np.array_equal(dY.to_host()[0], Yo[0])


@pytest.mark.parametrize("tau_kind", ["per-population", "per-neuron"])
def test_gemv_with_lif_epilogue(queue, tau_kind):
    """GEMV + LIF in one launch: the currents, voltages, refractory times and spikes
    equal those of the oracle's GEMV followed by its LIF bit for bit, for
    power-of-two and odd widths, several steps in a row, items without neurons in
    the same launch, a population without any input item (rides along), a population
    fed by a small item (keeps its own launch), and per-neuron time constants; a
    launch whose inputs include the spikes it would write is left unfused."""
    from nengo_ocl_amd import hipra_gemv as g
    from nengo_ocl_amd import hipra_nonlinearities as nl
    from oracle import oracle as orc

    rng = np.random.RandomState(31)
    dt = 1e-3
    # GEMV items: four large ones with neurons, a small one with neurons, a large one without
    shapes = [(4096, 64), (3000, 4), (3000, 12), (520, 130), (60, 8), (300, 64)]
    pop_sizes = [4096, 3000, 3000, 520, 60, 700]  # the last population has no input item
    n, n_pop = len(shapes), len(pop_sizes)
    mats = [rng.normal(scale=0.4, size=s) for s in shapes]
    xs = [rng.normal(size=s[1]) for s in shapes]
    bias = [rng.normal(loc=1.0, scale=1.0, size=s[0]) for s in shapes]
    Jz = [np.zeros(s[0]) for s in shapes] + [rng.normal(loc=1.5, size=700)]
    Vz = [rng.uniform(0, 1, size=m) for m in pop_sizes]
    Wz = [rng.uniform(-2 * dt, 2 * dt, size=m) for m in pop_sizes]
    Sz = [np.zeros(m) for m in pop_sizes]
    taus = [0.02, 0.03, 0.015, 0.05, 0.02, 0.025]
    tau_vecs = [rng.choice([0.02, 0.04], size=m) if tau_kind == "per-neuron" else t * np.ones(m)
                for t, m in zip(taus, pop_sizes)]
    R = RA(mats + xs + bias + Jz + Vz + Wz + Sz + tau_vecs, align=True)
    iA, iX, iB = (list(range(k * n, (k + 1) * n)) for k in range(3))
    iJ = list(range(3 * n, 4 * n + 1))
    base = 4 * n + 1
    iV, iW, iS, iT = (list(range(base + k * n_pop, base + (k + 1) * n_pop)) for k in range(4))
    iJpop = iJ[:5] + [iJ[6]]  # currents of the six populations
    A_js = [np.array([i], dtype=np.int32) for i in iA]
    X_js = [np.array([i], dtype=np.int32) for i in iX]

    def build(ra, mod_gemv, mod_nl, q):
        prog = mod_gemv.plan_block_gemv(q, 1.0, ra, A_js, ra, X_js, 1.0, ra[iJ[:n]], Y_in=ra[iB])
        tau = ra[iT] if tau_kind == "per-neuron" else np.array(taus, dtype=np.float32)
        lif = mod_nl.plan_lif(q, dt, ra[iJpop], ra[iV], ra[iW], ra[iS], 0.002, tau, 1.0)
        return prog, lif

    host = clone(R)
    dev = to_dev(queue, R)
    prog, lif = build(dev, g, nl, queue)
    fused = g.fuse_lif(prog, lif)
    assert fused is not None
    names = sorted(p.name for p in fused)
    # three large-item classes (the input-less population joins the one with compile-time
    # shapes) and the small item's launch, each updating the neurons it feeds: no neuron
    # launch
    assert names == ["hipra_gemv.tile_lif"] * 3 + ["hipra_gemv.wave_ref_lif"]
    assert {p.kernel_class for p in fused if p.name == "hipra_gemv.tile_lif"} == {
        (3, 5, 4), (3, 1, 4), (3, 0, 1)}
    for step in range(3):
        for p in fused:
            p()
    got = dev.to_host()
    s0 = slice(int(got.starts[iS[0]]), int(got.starts[iS[0]]) + 4096)
    s5 = slice(int(got.starts[iS[5]]), int(got.starts[iS[5]]) + 700)
    if tau_kind == "per-population":
        # the oracle, with the neuron update after every GEMV
        for step in range(3):
            oprog = orc.plan_block_gemv(None, 1.0, host, A_js, host, X_js, 1.0, host[iJ[:n]],
                                        Y_in=host[iB])
            for p in oprog.plans:
                p()
            orc.plan_lif(None, dt, host[iJpop], host[iV], host[iW], host[iS], 0.002,
                         np.array(taus, dtype=np.float32), 1.0)()
        assert np.array_equal(got.buf, host.buf)
    else:
        # the oracle takes one tau per population: compare with separate device launches,
        # which the neuron-kernel test pins against the oracle for per-neuron taus
        dev2 = to_dev(queue, R)
        prog2, lif2 = build(dev2, g, nl, queue)
        for step in range(3):
            for p in prog2.plans:
                p()
            lif2()
        assert np.array_equal(got.buf, dev2.to_host().buf)
    assert got.buf[s0].sum() > 0 and got.buf[s5].sum() > 0, "no spikes"

    # a launch that reads the spikes the update would write must stay unfused
    prog3 = g.plan_block_gemv(queue, 1.0, dev, [A_js[1]], dev, [X_js[1]], 1.0, dev[[iJ[1]]],
                              Y_in=dev[[iS[1]]])
    lif3 = nl.plan_lif(queue, dt, dev[[iJ[1]]], dev[[iV[1]]], dev[[iW[1]]], dev[[iS[1]]], 0.002, 0.02, 1.0)
    assert g.fuse_lif(prog3, lif3) is None
    prog4 = g.plan_block_gemv(queue, 1.0, dev, [A_js[1]], dev, [X_js[1]], 1.0, dev[[iJ[1]]])
    assert g.fuse_lif(prog4, lif3) is not None


def test_gemv_with_filter_epilogue(queue):
    """GEMV + first-order filters in one launch: every decoded vector and every filter
    output equals the oracle's GEMV followed by its filter step bit for bit over
    several steps -- several filters per GEMV item, a pure gain, a filter fed by a
    small item (epilogue of the small-item launch) and a second-order filter (keeps a
    launch of its own)."""
    from nengo_ocl_amd import hipra_gemv as g
    from nengo_ocl_amd import hipra_nonlinearities as nl
    from oracle import oracle as orc

    rng = np.random.RandomState(5)
    shapes = [(64, 4096), (64, 2048), (3000, 12), (16, 8), (2500, 4), (300, 30)]
    n = len(shapes)
    mats = [rng.normal(scale=0.1, size=s) for s in shapes]
    xs = [rng.normal(size=s[1]) for s in shapes]
    outs = [np.zeros(s[0]) for s in shapes]
    # (GEMV item, denominator, numerator)
    lowpass = lambda tau: (np.array([-np.exp(-0.001 / tau)]), np.array([1 - np.exp(-0.001 / tau)]))
    filters = [(0,) + lowpass(0.005), (0,) + lowpass(0.1), (0,) + lowpass(0.02),
               (1, np.zeros(0), np.array([0.5])), (2,) + lowpass(0.01), (3,) + lowpass(0.01),
               (0, np.array([-1.2, 0.4]), np.array([0.1, 0.1])), (4,) + lowpass(0.03),
               (4,) + lowpass(0.002), (5,) + lowpass(0.02)]
    f_out = [rng.normal(size=shapes[b][0]) for b, _, _ in filters]
    R = RA(mats + xs + outs + f_out, align=True)
    iA, iX, iY = (list(range(k * n, (k + 1) * n)) for k in range(3))
    iF = list(range(3 * n, 3 * n + len(filters)))
    A_js = [np.array([i], dtype=np.int32) for i in iA]
    X_js = [np.array([i], dtype=np.int32) for i in iX]
    from nengo_ocl_amd.raggedarray import RaggedArray

    # an empty denominator (a pure gain) is a ragged item of shape (0, 1)
    den = RaggedArray([np.asarray(f[1], dtype=np.float32).reshape(-1, 1) if f[1].size
                       else np.zeros((0, 1), dtype=np.float32) for f in filters], dtype=np.float32)
    num = RaggedArray([np.asarray(f[2], dtype=np.float32).reshape(-1, 1) for f in filters],
                      dtype=np.float32)
    fx = [iY[b] for b, _, _ in filters]
    xbuf = RaggedArray([np.zeros((f[2].size, shapes[f[0]][0]), dtype=np.float32) for f in filters],
                       dtype=np.float32)
    ybuf = RaggedArray([np.zeros((f[1].size, shapes[f[0]][0]), dtype=np.float32) for f in filters],
                       dtype=np.float32)

    def build(ra, mod_gemv, mod_nl, q, up):
        prog = mod_gemv.plan_block_gemv(q, 1.0, ra, A_js, ra, X_js, 0.0, ra[iY])
        lf = mod_nl.plan_linearfilter(q, ra[fx], ra[iF], up(den), up(num), up(clone(xbuf)),
                                      up(clone(ybuf)))
        return prog, lf

    host = clone(R)
    dev = to_dev(queue, R)
    prog, lf = build(dev, g, nl, queue, lambda a: to_dev(queue, a))
    result = g.fuse_linearfilter(prog.plans, lf[0])
    assert result is not None
    fused, residual = result
    # compile-time shapes (4096, 2048, 12), 4 columns, rows not 16-byte aligned but back to
    # back (30), small
    assert sorted(p.name for p in fused) == ["hipra_gemv.tile_filter"] * 3 + [
        "hipra_gemv.wave_ref_filter"]
    assert {p.kernel_class for p in fused if p.name == "hipra_gemv.tile_filter"} == {
        (3, 6, 4), (3, 1, 4), (3, 7, 4)}
    assert [p.name for p in residual] == ["hip_linearfilter"]
    oprog, olf = build(host, orc, orc, None, lambda a: a)
    for step in range(4):
        for i in iX:  # new inputs every step
            v = rng.normal(size=R.shape0s[i])
            dev[i] = v
            host[i] = v[:, None]
        for p in fused + residual:
            p()
        for p in oprog.plans + olf:
            p()
        assert np.array_equal(dev.to_host().buf, host.buf), step


def test_sparse_products(queue):
    """Many sparse matrices in one launch (64-row slices, rows summed in column order):
    bit-identical to the oracle's CSR product for row counts that are no multiple of
    64, empty rows and empty matrices, duplicate entries, rows much longer than their
    neighbours, incrementing and setting items side by side; the layout is checked
    against the matrices it came from."""
    import scipy.sparse as sp

    from nengo_ocl_amd import hipra_spmv
    from oracle import oracle as orc

    rng = np.random.RandomState(8)
    shapes = [(1000, 700), (64, 64), (65, 10), (1, 300), (300, 1), (130, 4000), (40, 40)]
    mats = [sp.random(m, n, density=d, random_state=rng, format="csr", dtype=np.float32)
            for (m, n), d in zip(shapes, (0.05, 0.5, 0.3, 0.9, 0.5, 0.02, 0.0))]
    long_row = sp.lil_matrix(mats[5].shape, dtype=np.float32)
    long_row[7, :] = rng.normal(size=4000)          # one full row among sparse ones
    mats[5] = sp.csr_matrix(mats[5] + long_row.tocsr())
    mats[1].indices[:] = rng.randint(64, size=mats[1].nnz)  # unsorted, with duplicates
    X = RA([rng.normal(size=n) for m, n in shapes], align=True)
    Y = RA([rng.normal(size=m) for m, n in shapes], align=True)
    inc = [1, 0, 1, 0, 1, 0, 1]

    slice_rows, row_len, cols, vals = hipra_spmv.sell_layout([hipra_spmv.HostSparseMatrix(m) for m in mats])
    k = [r for r in slice_rows if r[0] == 0][3]     # fourth slice of the first matrix
    _, start, width, len_start, n_rows, row0 = k
    csr = hipra_spmv.HostSparseMatrix(mats[0]).csr
    for r in (0, 17, 63):
        n = row_len[len_start + r]
        lo = csr.indptr[row0 + r]
        assert n == csr.indptr[row0 + r + 1] - lo
        assert np.array_equal(cols[hipra_spmv.sell_index(start, r, np.arange(n))], csr.indices[lo:lo + n])
        assert np.array_equal(vals[hipra_spmv.sell_index(start, r, np.arange(n))], csr.data[lo:lo + n])

    Yo = clone(Y)
    oplan = orc.plan_sparse_dot_inc(None, mats, X, Yo, inc=inc).plans[0]
    dX, dY = to_dev(queue, X), to_dev(queue, Y)
    plan = hipra_spmv.plan_sparse_dot_inc(queue, mats, dX, dY, inc=inc).plans[0]
    for _ in range(3):  # the incrementing items accumulate
        plan()
        oplan()
        assert np.array_equal(dY.to_host().buf, Yo.buf)
    with pytest.raises(ValueError):
        hipra_spmv.plan_sparse_dot_inc(queue, mats[:2], dX[[0, 2]], dY[[0, 1]])


@pytest.mark.parametrize("wave_tasks", [True, False], ids=["wave-tasks", "row-tasks"])
def test_thin_items_lane_per_row(queue, monkeypatch, wave_tasks):
    """Many rows of dot products with one to four columns take the lane-per-row class (a
    wave per task of up to 64 rows, or a task record per row): bit-identical to the oracle
    for sums of several such terms, strided operands and a scalar X shared by all rows."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    monkeypatch.setattr(g, "WAVE_TASKS", wave_tasks)

    rng = np.random.RandomState(17)
    shapes = [(40000, 1), (30000, 4), (5000, 3), (33, 2)]
    A = RA([rng.normal(size=s) for s in shapes] + [rng.normal(size=(40000, 1)) for _ in range(5)],
           align=True)
    X = RA([rng.normal(size=s[1]) for s in shapes] + [rng.normal(size=1) for _ in range(5)],
           align=True)
    Y = RA([rng.normal(size=s[0]) for s in shapes] + [rng.normal(size=40000)], align=True)
    n = len(shapes)
    js = [np.array([i], dtype=np.int32) for i in range(n)] + [np.arange(n, n + 5, dtype=np.int32)]
    for beta, gamma in ((1.0, 0.0), (0.0, 0.25)):
        Yo = clone(Y)
        orc.plan_block_gemv(None, 1.0, A, js, X, js, beta, Yo, gamma=gamma).plans[0]()
        dY = to_dev(queue, Y)
        prog = g.plan_block_gemv(queue, 1.0, to_dev(queue, A), js, to_dev(queue, X), js, beta, dY,
                                 gamma=gamma)
        assert {p.kernel_class for p in prog.plans} == {(2, 1, 1)}
        assert {p.args[1] for p in prog.plans} == {64 if wave_tasks else 1}
        for plan in prog.plans:
            plan()
        assert np.array_equal(dY.buf, Yo.buf)


@pytest.mark.parametrize("inc, long_row, sparsity, shape", [
    (True, False, 0.02, 511), (False, False, 0.1, 511), (False, False, 0.02, 5000),
    (False, True, 0.02, 5000), (True, False, 0.1, 5000), (False, False, 0.02, (2047, 5007)),
    (True, True, 0.07, (2048, 5003)), (True, False, 0.02, (2057, 5981)),
    (False, False, 0.02, (1, 4999)), (False, False, 0.02, (5001, 1))])
def test_sparse_reference_cases(queue, rng, inc, long_row, sparsity, shape):
    """The cases of the reference's test_sparse (tests/test_clra_gemv.py:383-462): random
    masks, optionally ten rows with a run of 1025 entries, set and increment; checked
    like there against scipy's product, and bit for bit against the oracle."""
    import scipy.sparse as sp

    from nengo_ocl_amd import hipra_spmv
    from oracle import oracle as orc

    shape = (shape, shape) if isinstance(shape, int) else shape
    mask = rng.uniform(size=shape) < sparsity
    if long_row:
        rows = np.unique(rng.randint(0, shape[0], size=10))
        mask[rows, :min(1025, shape[1])] = True
    ii, jj = mask.nonzero()
    assert len(ii) > 0
    A = sp.coo_matrix((rng.uniform(0, 1, size=len(ii)), (ii, jj)), shape=shape)
    X = RA([rng.uniform(0, 1, size=shape[1])])
    Y = RA([rng.uniform(0, 1, size=shape[0])])
    dX, dY = to_dev(queue, X), to_dev(queue, Y)
    prog = hipra_spmv.plan_sparse_dot_inc(queue, hipra_spmv.HostSparseMatrix(A.tocsr()), dX, dY, inc=inc)
    for plan in prog.plans:
        plan()
    ref = (Y[0][:, 0].astype(np.float64) if inc else 0) + A.astype(np.float64).dot(X[0][:, 0].astype(np.float64))
    got = dY.to_host()[0][:, 0]
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)
    Yo = clone(Y)
    orc.plan_sparse_dot_inc(None, A.tocsr(), X, Yo, inc=inc).plans[0]()
    assert np.array_equal(got, Yo[0][:, 0])


@pytest.mark.parametrize("inc", [True, False])
@pytest.mark.parametrize("density", [0.0, 0.06, 0.5, 1.0])
def test_sparse_products_pass_over_zero_operands(queue, rng, inc, density):
    """The launch for vectors that are mostly zero (spikes): several matrices reading one
    X, rows longer than a slice is wide, an X with zeros, negative zeros and denormals in
    it; bit-identical (signs of zero included) to the oracle's sequential product at every
    density, also after X changes between two launches and with a stored value that is not
    finite.  Matrices with different X take the ordinary launch."""
    import scipy.sparse as sp

    from nengo_ocl_amd import hipra_spmv
    from oracle import oracle as orc

    n_cols = 70001  # not a multiple of 128: the last mask words are partly used
    shapes = [(3000, n_cols), (130, n_cols), (1, n_cols)]
    mats = []
    for m, n in shapes:
        A = sp.random(m, n, density=0.002, random_state=rng, format="lil", dtype=np.float32)
        A[min(5, m - 1), :3000] = rng.normal(size=3000)  # a long row among short ones
        A = A.tocsr()
        A.data[:] = rng.normal(size=A.nnz) * 10.0 ** rng.randint(-30, 5, size=A.nnz)
        mats.append(A)

    def draw_x():
        x = np.where(rng.uniform(size=n_cols) < density, rng.normal(size=n_cols), 0.0).astype(np.float32)
        x[rng.randint(0, n_cols, size=50)] = -0.0
        x[rng.randint(0, n_cols, size=50)] = 1e-42  # denormal: not zero
        return x

    x = draw_x()
    Xh = RA([x])
    Y = RA([rng.normal(size=m) * (rng.uniform(size=m) < 0.5) for m, _ in shapes])
    Yo = clone(Y)
    dX, dY = to_dev(queue, Xh), to_dev(queue, Y)
    idx = [0, 0, 0]
    prog = hipra_spmv.plan_sparse_dot_inc(queue, mats, dX[idx], dY, inc=inc, x_mostly_zero=True)
    assert prog.plans[0].skips_zero_x
    oplan = orc.plan_sparse_dot_inc(None, mats, Xh[idx], Yo, inc=inc).plans[0]
    for _ in range(3):
        prog.plans[0]()
        oplan()
        got, want = dY.buf, Yo.buf
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        x = draw_x()
        Xh[0] = x.reshape(-1, 1)
        dX[0] = x.reshape(-1, 1)
    # cases that keep the ordinary launch
    two_x = to_dev(queue, RA([x, x]))
    plain = hipra_spmv.plan_sparse_dot_inc(queue, mats[:2], two_x, dY[[0, 1]], x_mostly_zero=True)
    assert not plain.plans[0].skips_zero_x
    bad = mats[0].copy()
    bad.data[3] = np.inf  # inf * 0 is not a number in both launches
    outs = []
    for flag in (True, False):
        d = to_dev(queue, Y)
        prog = hipra_spmv.plan_sparse_dot_inc(queue, [bad], dX, d[[0]], x_mostly_zero=flag)
        assert prog.plans[0].skips_zero_x == flag
        prog.plans[0]()
        outs.append(d.to_host()[0])
    assert np.array_equal(outs[0], outs[1], equal_nan=True)
    plain = hipra_spmv.plan_sparse_dot_inc(queue, mats, dX[idx], dY, x_mostly_zero=[True, False, True])
    assert not plain.plans[0].skips_zero_x


@pytest.mark.parametrize("mostly_zero", [False, True])
def test_sparse_products_with_filter_epilogue(queue, mostly_zero):
    """Sparse product + the first-order filters on its output in one launch, for both
    sparse kernels: two matrices reading one X, two filters and a pure gain on the first
    output, none on the second, a second-order filter that keeps a launch of its own; every
    product and filter output equals the oracle's separate kernels bit for bit over steps."""
    import scipy.sparse as sp

    from nengo_ocl_amd import hipra_nonlinearities as nl
    from nengo_ocl_amd import hipra_spmv
    from nengo_ocl_amd.raggedarray import RaggedArray
    from oracle import oracle as orc

    rng = np.random.RandomState(11)
    n_cols, rows = 5000, [3001, 257]
    mats = [sp.random(m, n_cols, density=0.01, random_state=rng, format="csr", dtype=np.float32)
            for m in rows]
    lowpass = lambda tau: (np.array([-np.exp(-0.001 / tau)]), np.array([1 - np.exp(-0.001 / tau)]))
    filters = [(0,) + lowpass(0.1), (0,) + lowpass(0.005), (0, np.zeros(0), np.array([0.25])),
               (0, np.array([-1.2, 0.4]), np.array([0.1, 0.1]))]
    f_out = [rng.normal(size=rows[b]) for b, _, _ in filters]
    R = RA([np.zeros(n_cols)] + [np.zeros(m) for m in rows] + f_out, align=True)
    iY, iF = [1, 2], list(range(3, 3 + len(filters)))
    den = RaggedArray([np.asarray(f[1], dtype=np.float32).reshape(-1, 1) if f[1].size
                       else np.zeros((0, 1), dtype=np.float32) for f in filters], dtype=np.float32)
    num = RaggedArray([np.asarray(f[2], dtype=np.float32).reshape(-1, 1) for f in filters],
                      dtype=np.float32)
    xbuf = RaggedArray([np.zeros((f[2].size, rows[f[0]]), dtype=np.float32) for f in filters],
                       dtype=np.float32)
    ybuf = RaggedArray([np.zeros((f[1].size, rows[f[0]]), dtype=np.float32) for f in filters],
                       dtype=np.float32)
    fx = [iY[b] for b, _, _ in filters]

    def build(ra, spmv, mod_nl, q, up, **kw):
        prog = spmv(q, mats, ra[[0, 0]], ra[iY], inc=False, **kw)
        lf = mod_nl.plan_linearfilter(q, ra[fx], ra[iF], up(den), up(num), up(clone(xbuf)),
                                      up(clone(ybuf)))
        return prog, lf

    host, dev = clone(R), to_dev(queue, R)
    prog, lf = build(dev, hipra_spmv.plan_sparse_dot_inc, nl, queue, lambda a: to_dev(queue, a),
                     x_mostly_zero=mostly_zero)
    assert prog.plans[0].skips_zero_x == mostly_zero
    fused, residual = hipra_spmv.fuse_linearfilter(prog.plans[0], lf[0])
    assert [p.name for p in fused] == ["hip_spmv_filter"]
    assert [p.name for p in residual] == ["hip_linearfilter"] and residual[0].unfused_items == [3]
    oprog, olf = build(host, orc.plan_sparse_dot_inc, orc, None, lambda a: a)
    for step in range(4):
        v = np.where(rng.uniform(size=n_cols) < 0.1, rng.normal(size=n_cols), 0.0)
        dev[0] = v
        host[0] = v[:, None]
        for p in fused + residual:
            p()
        for p in oprog.plans + olf:
            p()
        assert np.array_equal(dev.to_host().buf.view(np.uint32), host.buf.view(np.uint32)), step


@pytest.mark.parametrize("activity", [0.0, 0.08, 1.0])
def test_products_with_spike_vectors_visit_active_columns_only(queue, activity, monkeypatch):
    """Items flagged as "X mostly zero, A constant" take the launch that reads only the
    columns of A whose x is not zero (matrices transposed on the device): 64 x 4096,
    32 x 2000 (columns no multiple of the tile), 64 x 512, 19 x 1000, 16 x 10000 (three runs of
    columns), with coefficients;
    bit-identical to the oracle's dense product at every activity, with negative zeros and
    denormals in X, over steps in which X changes; 100 x 4096 as two groups of rows.  Flagged
    items that do not fit (two dot products, few columns) keep the dense kernels, in the same
    program."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(23)
    shapes = [(64, 4096), (32, 2000), (64, 512), (19, 1000), (100, 4096), (64, 4096), (16, 300),
              (16, 10000)]
    n = len(shapes)
    mats = [rng.normal(scale=0.01, size=s) for s in shapes] + [rng.normal(size=(64, 4096))]
    xs = [np.zeros(s[1]) for s in shapes] + [np.zeros(4096)]
    outs = [rng.normal(size=s[0]) for s in shapes]
    R = RA(mats + xs + outs, align=True)
    iA = list(range(n + 1))
    iX = list(range(n + 1, 2 * n + 2))
    iY = list(range(2 * n + 2, 3 * n + 2))
    A_js = [np.array([i], dtype=np.int32) for i in iA[:n]]
    X_js = [np.array([i], dtype=np.int32) for i in iX[:n]]
    A_js[5] = np.array([iA[5], iA[n]], dtype=np.int32)  # two dot products: stays dense
    X_js[5] = np.array([iX[5], iX[n]], dtype=np.int32)
    alpha = [1.0, 0.5, 1.0, -2.0, 1.0, 1.0, 1.0, 0.75]
    beta = [0.0, 1.0, 0.25, 0.0, 1.0, 0.0, 1.0, 1.0]
    gamma = [0.0, 0.0, 0.125, 0.0, 0.0, 0.0, 0.0, 0.0]
    flagged = [0, 1, 2, 3, 4, 5, 6, 7]

    host, dev = clone(R), to_dev(queue, R)
    # a few MB of matrices next to a dense launch that stays: not worth a launch of its own
    prog = g.plan_block_gemv(queue, alpha, dev, A_js, dev, X_js, beta, dev[iY], gamma=gamma,
                             event_items=flagged)
    assert not any(p.name == "hipra_gemv.events" for p in prog.plans)
    monkeypatch.setattr(g, "EVENT_MIN_SPLIT_BYTES", 0)
    prog = g.plan_block_gemv(queue, alpha, dev, A_js, dev, X_js, beta, dev[iY], gamma=gamma,
                             event_items=flagged)
    events = [p for p in prog.plans if p.name == "hipra_gemv.events"]
    assert len(events) == 1 and events[0].members == [0, 1, 2, 3, 4, 7]
    assert events[0].n_tasks == 7  # 100 rows are two records
    assert sorted(b for p in prog.plans if p.name != "hipra_gemv.events" for b in p.members) == [5, 6]
    oprog = orc.plan_block_gemv(None, alpha, host, A_js, host, X_js, beta, host[iY], gamma=gamma)
    for step in range(3):
        for i in iX:
            m = R.shape0s[i]
            v = np.where(rng.uniform(size=m) < activity, 1000.0 * rng.choice([1.0, 0.5], size=m), 0.0)
            v[rng.randint(0, m, size=5)] = -0.0
            if activity > 0:
                v[rng.randint(0, m, size=3)] = 1e-42
            dev[i] = v
            host[i] = v[:, None]
        for p in prog.plans:
            p()
        for p in oprog.plans:
            p()
        assert np.array_equal(dev.to_host().buf.view(np.uint32), host.buf.view(np.uint32)), step


@pytest.mark.parametrize("activity", [0.0, 0.08, 1.0])
def test_active_columns_from_one_bit_per_column(queue, activity, monkeypatch):
    """The same launch with X handed over as one bit per column (`x_bits` in the record: the
    value of a set bit; 64-bit words at the start of the vector's memory): 64 x 4096,
    32 x 2000 and 19 x 1000 (a partial last word), 100 x 4096 (two records), 16 x 10000 (three
    runs of columns), with coefficients -- Y equals, bit for bit, the oracle's dense product
    with the floats the bits stand for, over steps in which the bits change."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(29)
    shapes = [(64, 4096), (32, 2000), (19, 1000), (100, 4096), (16, 10000)]
    values = [1000.0, 500.0, 1000.0, 0.25, 1000.0]
    n = len(shapes)
    mats = [rng.normal(scale=0.01, size=s) for s in shapes]
    xs = [np.zeros(s[1]) for s in shapes]
    outs = [rng.normal(size=s[0]) for s in shapes]
    R = RA(mats + xs + outs, align=True)
    iA, iX, iY = list(range(n)), list(range(n, 2 * n)), list(range(2 * n, 3 * n))
    A_js = [np.array([i], dtype=np.int32) for i in iA]
    X_js = [np.array([i], dtype=np.int32) for i in iX]
    alpha, beta = [1.0, 0.5, -2.0, 1.0, 0.75], [0.0, 1.0, 0.25, 1.0, 1.0]
    gamma = [0.0, 0.0, 0.125, 0.0, 0.0]
    host, dev = clone(R), to_dev(queue, R)
    monkeypatch.setattr(g, "EVENT_MIN_SPLIT_BYTES", 0)
    prog = g.plan_block_gemv(queue, alpha, dev, A_js, dev, X_js, beta, dev[iY], gamma=gamma,
                             event_items=list(range(n)))
    assert [p.name for p in prog.plans] == ["hipra_gemv.events"]
    plan = prog.plans[0]
    for k, b in enumerate(plan.event_record_item):
        assert plan.event_table[k, 4] % 2 == 0  # 64-bit words
        plan.event_table[k, 15] = int(np.array([values[b]], dtype=np.float32).view(np.int32)[0])
    plan.dev_event_table.set(plan.event_table.astype(np.int32).ravel())
    oprog = orc.plan_block_gemv(None, alpha, host, A_js, host, X_js, beta, host[iY], gamma=gamma)
    for step in range(3):
        for b, i in enumerate(iX):
            m = R.shape0s[i]
            active = rng.uniform(size=m) < activity
            host[i] = np.where(active, values[b], 0.0)[:, None]
            words = np.packbits(active, bitorder="little")
            words = np.concatenate([words, np.zeros(-len(words) % 8, dtype=np.uint8)])
            # the memory behind the words is never read: anything may be there
            image = rng.normal(size=m).astype(np.float32)
            image[:len(words) // 4] = words.view(np.float32)
            dev[i] = image
        plan()
        for p in oprog.plans:
            p()
        got, want = dev.to_host(), host
        for i in iY:
            assert np.array_equal(np.asarray(got[i]).view(np.uint32),
                                  np.asarray(want[i]).view(np.uint32)), (step, i)


def test_gemv_lif_forms_its_input_sums(queue):
    """Sums of vectors -> encoders -> LIF in one launch: inputs that are sums of one to
    eleven vectors times scalars (64, 40 and 8 elements), an ensemble whose input is a
    plain vector in the same launch, and two sums that nothing in the launch reads; the
    sums, currents and neuron states equal the oracle's three separate kernels bit for bit
    over several steps in which the summed vectors change."""
    from nengo_ocl_amd import hipra_gemv as g
    from nengo_ocl_amd import hipra_nonlinearities as nl
    from oracle import oracle as orc

    rng = np.random.RandomState(77)
    dt = 1e-3
    dims = [64, 64, 40, 8, 64]        # input dimension of the five ensembles
    n_neurons = [4096, 1000, 2048, 2048, 300]
    fan_in = [4, 11, 1, 3, 0]         # the last ensemble reads its input vector as it is
    spare = [64, 5]                   # sums that no encoder reads (probe inputs)
    srcs = [rng.normal(size=64) for _ in range(12)]
    scal = [np.array([v]) for v in (1.0, 1.0, 0.5, -2.0)]
    ins = [rng.normal(size=d) for d in dims] + [rng.normal(size=d) for d in spare]
    enc = [rng.normal(scale=0.5, size=(m, d)) for m, d in zip(n_neurons, dims)]
    bias = [rng.normal(loc=1.0, size=m) for m in n_neurons]
    J = [np.zeros(m) for m in n_neurons]
    V = [rng.uniform(0, 1, size=m) for m in n_neurons]
    W = [rng.uniform(-2 * dt, 2 * dt, size=m) for m in n_neurons]
    S = [np.zeros(m) for m in n_neurons]
    R = RA(srcs + scal + ins + enc + bias + J + V + W + S, align=True)
    n_e = len(dims)
    i_src = list(range(12))
    i_scal = list(range(12, 16))
    i_in = list(range(16, 16 + n_e + 2))
    at = 16 + n_e + 2
    i_enc, i_bias, i_J, i_V, i_W, i_S = (list(range(at + k * n_e, at + (k + 1) * n_e))
                                         for k in range(6))
    # which vectors each sum adds up (a source longer than the sum is used through a view)
    picks = [rng.choice(12, size=f, replace=False) for f in fan_in[:4]] + [
        rng.choice(12, size=2, replace=False), rng.choice(12, size=3, replace=False)]
    sum_items = [0, 1, 2, 3, 5, 6]    # positions in `ins` that are sums
    sum_lens = [dims[0], dims[1], dims[2], dims[3]] + spare

    def build(ra, mg, mn, q, second_reader=False):
        # A of the sums: the first n elements of each source as an n x 1 matrix
        views, A_js, X_js = [], [], []
        for length, pk in zip(sum_lens, picks):
            a_idx = []
            for src in pk:
                views.append((int(ra.starts[i_src[src]]), length))
                a_idx.append(len(views) - 1)
            A_js.append(np.array(a_idx, dtype=np.int32))
            X_js.append(np.array([i_scal[k % 4] for k in range(len(pk))], dtype=np.int32))
        from_buffer = type(ra).from_buffer
        buf = ra.dev_buf if hasattr(ra, "dev_buf") else ra.buf
        mk = (lambda *m: from_buffer(q, buf, *m)) if hasattr(ra, "dev_buf") else (
            lambda *m: from_buffer(buf, *m))
        starts = np.array([v[0] for v in views])
        lens = np.array([v[1] for v in views])
        ones = np.ones(len(views), dtype=int)
        A_sum = mk(starts, lens, ones, ones, ones)
        Y_sum = ra[[i_in[k] for k in sum_items]]
        sums = mg.plan_block_gemv(q, 1.0, A_sum, A_js, ra, X_js, 0.0, Y_sum)
        e_A = [np.array([i], dtype=np.int32) for i in i_enc]
        e_X = [np.array([i_in[k]], dtype=np.int32) for k in range(n_e)]
        if second_reader:  # the last ensemble also reads the first one's input sum
            e_A[4] = np.array([i_enc[4], i_enc[4]], dtype=np.int32)
            e_X[4] = np.array([i_in[4], i_in[0]], dtype=np.int32)
        encs = mg.plan_block_gemv(q, 1.0, ra, e_A, ra, e_X, 1.0, ra[i_J], Y_in=ra[i_bias])
        lif = mn.plan_lif(q, dt, ra[i_J], ra[i_V], ra[i_W], ra[i_S], 0.002,
                          np.float32([0.02, 0.03, 0.02, 0.05, 0.02]), 1.0)
        return sums, encs, lif

    host = clone(R)
    dev = to_dev(queue, R)
    sums, encs, lif = build(dev, g, nl, queue)
    assert [p.name for p in sums.plans] == ["hipra_gemv.wave_ref"]
    with_lif = g.fuse_lif(encs, lif)
    assert [p.name for p in with_lif] == ["hipra_gemv.tile_lif"]
    fused = g.fuse_input_sums(sums.plans[0], with_lif[0])
    assert fused is not None and fused.input_sums == 6
    assert fused.n_tasks == with_lif[0].n_tasks + 2   # the two sums nothing reads
    osums, oencs, olif = build(host, orc, orc, None)
    for step in range(4):
        fused()
        for p in osums.plans + oencs.plans:
            p()
        olif()
        got = dev.to_host()
        assert np.array_equal(got.buf, host.buf), step
        # new source vectors for the next step, the same on both sides
        for i in i_src:
            v = rng.normal(size=64)
            host[i] = v[:, None]
            dev[i] = v
    assert host.buf[int(host.starts[i_S[0]]):][:4096].any()

    # refused: a sum that a second dot product of the launch reads as well
    dev2 = to_dev(queue, R)
    sums2, encs2, lif2 = build(dev2, g, nl, queue, second_reader=True)
    with_lif2 = g.fuse_lif(encs2, lif2)
    assert with_lif2 is not None
    assert all(g.fuse_input_sums(sums2.plans[0], p) is None for p in with_lif2)


@pytest.mark.parametrize("planner", ["plan_csr", "plan_ellpack", "plan_ellpack_tree",
                                     "plan_ellpack_twostep", "spmv_prog"])
def test_sparse_planner_names_of_the_reference(queue, rng, planner, monkeypatch):
    """The reference's sparse planner classes (its test_sparse is run over plan_ellpack and
    plan_csr, tests/test_clra_gemv.py:40-49, 383-462) exist with its constructor and give
    the oracle's product bit for bit -- also for rows longer than a work-group, which the
    reference's tree planner refuses; `algorithm` strings are checked like there."""
    import scipy.sparse as sp

    from nengo_ocl_amd import hipra_spmv
    from oracle import oracle as orc

    shape = (2057, 5981)
    mask = rng.uniform(size=shape) < 0.02
    mask[rng.randint(0, shape[0], size=5), :1025] = True
    ii, jj = mask.nonzero()
    A = sp.coo_matrix((rng.uniform(0, 1, size=len(ii)), (ii, jj)), shape=shape).tocsr()
    X, Y = RA([rng.uniform(0, 1, size=shape[1])]), RA([rng.uniform(0, 1, size=shape[0])])
    hA = hipra_spmv.HostSparseMatrix(A)
    for inc in (False, True):
        dX, dY = to_dev(queue, X), to_dev(queue, Y)
        prog = getattr(hipra_spmv, planner)(queue, hA, dX, dY, inc=inc)
        for plan in prog.plans:
            plan()
        Yo = clone(Y)
        orc.plan_sparse_dot_inc(None, A, X, Yo, inc=inc).plans[0]()
        assert np.array_equal(dY.to_host()[0][:, 0], Yo[0][:, 0])
    dX, dY = to_dev(queue, X), to_dev(queue, Y)
    assert hipra_spmv.spmv_algorithm_heuristic(queue, hA) == "ELLPACK"
    hipra_spmv.plan_sparse_dot_inc(queue, hA, dX, dY, algorithm="CSR")
    with pytest.raises(KeyError):
        hipra_spmv.plan_sparse_dot_inc(queue, hA, dX, dY, algorithm="COO")
    monkeypatch.setenv("NENGO_OCL_SPMV_ALGORITHM", "nonsense")
    with pytest.raises(KeyError):
        hipra_spmv.plan_sparse_dot_inc(queue, hA, dX, dY)


@pytest.mark.parametrize("n_ens, wave_tasks", [(24, True), (700, True), (700, False)],
                         ids=["inline-task-records", "wave-tasks", "plain-task-records"])
def test_small_item_lif_forms_its_input_sums(queue, monkeypatch, n_ens, wave_tasks):
    """The same fusion for ensembles of 100 neurons with 1-D and 2-D inputs (the small-item
    kernel; a row per task with the item inline in its record for few rows; for many rows a
    lane per row, with tasks of up to 64 rows that a wave takes whole or, that switched off,
    a plain record per row): sums of one to twelve terms, a sum nothing reads, several steps
    with changing sources -- all bit-identical to the oracle's three kernels."""
    from nengo_ocl_amd import hipra_gemv as g

    monkeypatch.setattr(g, "WAVE_TASKS", wave_tasks)
    from nengo_ocl_amd import hipra_nonlinearities as nl
    from oracle import oracle as orc

    rng = np.random.RandomState(5)
    dt, n_neurons, n_src = 1e-3, 100, 40
    dims = [1 + (k % 2) for k in range(n_ens)]
    srcs = [rng.normal(size=2) for _ in range(n_src)]
    scal = [np.array([v]) for v in (1.0, 0.25)]
    ins = [rng.normal(size=d) for d in dims] + [rng.normal(size=2)]   # the last: read by nothing
    enc = [rng.normal(scale=1.5, size=(n_neurons, d)) for d in dims]
    bias = [rng.normal(loc=1.0, size=n_neurons) for _ in dims]
    zeros = lambda: [np.zeros(n_neurons) for _ in dims]
    V = [rng.uniform(0, 1, size=n_neurons) for _ in dims]
    W = [rng.uniform(-2 * dt, 2 * dt, size=n_neurons) for _ in dims]
    R = RA(srcs + scal + ins + enc + bias + zeros() + V + W + zeros(), align=True)
    i_src = list(range(n_src))
    i_scal = [n_src, n_src + 1]
    i_in = list(range(n_src + 2, n_src + 2 + n_ens + 1))
    at = i_in[-1] + 1
    i_enc, i_bias, i_J, i_V, i_W, i_S = (list(range(at + k * n_ens, at + (k + 1) * n_ens))
                                         for k in range(6))
    sum_lens = dims + [2]
    picks = [rng.choice(n_src, size=1 + (k * 5) % 12, replace=False) for k in range(n_ens + 1)]

    def build(ra, mg, mn, q):
        views, A_js, X_js = [], [], []
        for length, pk in zip(sum_lens, picks):
            a_idx = []
            for src in pk:
                views.append((int(ra.starts[i_src[src]]), length))
                a_idx.append(len(views) - 1)
            A_js.append(np.array(a_idx, dtype=np.int32))
            X_js.append(np.array([i_scal[k % 2] for k in range(len(pk))], dtype=np.int32))
        on_device = hasattr(ra, "dev_buf")
        starts, lens = np.array([v[0] for v in views]), np.array([v[1] for v in views])
        ones = np.ones(len(views), dtype=int)
        A_sum = (type(ra).from_buffer(q, ra.dev_buf, starts, lens, ones, ones, ones) if on_device
                 else type(ra).from_buffer(ra.buf, starts, lens, ones, ones, ones))
        sums = mg.plan_block_gemv(q, 1.0, A_sum, A_js, ra, X_js, 0.0, ra[i_in])
        e_A = [np.array([i], dtype=np.int32) for i in i_enc]
        e_X = [np.array([i_in[k]], dtype=np.int32) for k in range(n_ens)]
        encs = mg.plan_block_gemv(q, 1.0, ra, e_A, ra, e_X, 1.0, ra[i_J], Y_in=ra[i_bias])
        lif = mn.plan_lif(q, dt, ra[i_J], ra[i_V], ra[i_W], ra[i_S], 0.002, 0.02, 1.0)
        return sums, encs, lif

    host = clone(R)
    dev = to_dev(queue, R)
    sums, encs, lif = build(dev, g, nl, queue)
    assert [p.name for p in sums.plans] == ["hipra_gemv.wave_ref"]
    with_lif = g.fuse_lif(encs, lif)
    assert [p.name for p in with_lif] == ["hipra_gemv.wave_ref_lif"]
    lanes, task_words = with_lif[0].args[:2]
    if n_ens == 24:
        assert (lanes, task_words) == (4, 16)
    else:  # a lane per row: 64 rows per task with the item inline, or a plain record per row
        assert with_lif[0].kernel_class == (2, 1, 1)
        assert (lanes, task_words) == ((64, 16) if wave_tasks else (1, 4))
        assert with_lif[0].n_tasks == (2 * n_ens if wave_tasks else 100 * n_ens)
    fused = g.fuse_input_sums(sums.plans[0], with_lif[0])
    assert fused is not None and fused.input_sums == n_ens + 1
    # the sum nothing reads: two rows of their own, or one task of two rows
    assert fused.n_tasks == with_lif[0].n_tasks + (1 if lanes == 64 else 2)
    osums, oencs, olif = build(host, orc, orc, None)
    for step in range(3):
        fused()
        for p in osums.plans + oencs.plans:
            p()
        olif()
        assert np.array_equal(dev.to_host().buf, host.buf), step
        for i in i_src:
            v = rng.normal(size=2)
            host[i] = v[:, None]
            dev[i] = v
    assert any(host.buf[int(host.starts[i]):][:n_neurons].any() for i in i_S)


@pytest.mark.parametrize("coefs", [(0.1, 0.3, 0.7), (0.1, [0.3, 0.25, 0.1, 1.0], 0.0),
                                   ([0.5, 0.1, 0.2, 1.0], 0.6, [0.7, 0.0, 0.0, 0.1])],
                         ids=["literals", "beta-per-item", "alpha-gamma-per-item"])
def test_literal_coefficients_bit_exact(queue, coefs):
    """Coefficients that float32 does not hold exactly and that are the same for every item
    are double literals in the reference's kernel text (clra_gemv.py:17-32): the product of
    alpha with a tile sum, of beta with y_in and the sum with gamma are double operations
    rounded once.  Such launches take the kernel that does the same -- small and large items,
    several dot products, strided y_in -- and equal the oracle bit for bit; coefficients
    float32 holds keep the fast kernels."""
    from nengo_ocl_amd import hipra_gemv as g
    from oracle import oracle as orc

    rng = np.random.RandomState(77)
    shapes = [(7, 3), (300, 130), (64, 1024), (1000, 64)]
    A = RA([rng.normal(size=s) for s in shapes] + [rng.normal(size=(300, 5))], align=True)
    X = RA([rng.normal(size=s[1]) for s in shapes] + [rng.normal(size=5)])
    Y = RA([rng.normal(size=s[0]) for s in shapes])
    Yin = RA([rng.normal(size=s[0]) for s in shapes])
    A_js = [np.array([0]), np.array([1, 4]), np.array([2]), np.array([3])]
    X_js = [np.array([0]), np.array([1, 4]), np.array([2]), np.array([3])]
    alpha, beta, gamma = coefs
    Yo = clone(Y)
    orc.plan_block_gemv(None, alpha, A, A_js, X, X_js, beta, Yo, Y_in=clone(Yin), gamma=gamma).plans[0]()
    dY = to_dev(queue, Y)
    prog = g.plan_block_gemv(queue, alpha, to_dev(queue, A), A_js, to_dev(queue, X), X_js, beta, dY,
                             Y_in=to_dev(queue, Yin), gamma=gamma)
    assert [p.name for p in prog.plans] == ["hipra_gemv.wave_ref_literal"]
    for plan in prog.plans:
        plan()
    assert np.array_equal(dY.buf, Yo.buf)
    # the same problem with coefficients float32 holds: the usual kernels, the same bits
    Yo = clone(Y)
    orc.plan_block_gemv(None, 0.5, A, A_js, X, X_js, 0.25, Yo, Y_in=clone(Yin), gamma=2.0).plans[0]()
    dY = to_dev(queue, Y)
    prog = g.plan_block_gemv(queue, 0.5, to_dev(queue, A), A_js, to_dev(queue, X), X_js, 0.25, dY,
                             Y_in=to_dev(queue, Yin), gamma=2.0)
    assert "hipra_gemv.wave_ref_literal" not in [p.name for p in prog.plans]
    for plan in prog.plans:
        plan()
    assert np.array_equal(dY.buf, Yo.buf)
