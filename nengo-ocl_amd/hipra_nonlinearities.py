"""Plan builders for every non-GEMV step of the timestep, on HIP.

Counterpart of the reference's ``nengo_ocl/clra_nonlinearities.py`` for the
functions the timestep path uses; each keeps the reference's call signature
(``queue`` is a `hipraggedarray.Queue`) and returns a `Plan`:

=====================  =============================================  ==========
this module            reference (clra_nonlinearities.py)             C entry
=====================  =============================================  ==========
plan_timeupdate        plan_timeupdate :113-144                       nhip_timeupdate
plan_reset             plan_reset :147-214                            nhip_reset
plan_copy              plan_copy :217-304                             nhip_copy
plan_slicedcopy        plan_slicedcopy :307-411                       nhip_slicedcopy
plan_elementwise_inc   plan_elementwise_inc :414-574                  nhip_elementwise_inc
plan_linearfilter      plan_linearfilter :577-803                     nhip_linearfilter
plan_probes            plan_probes :806-951                           nhip_probes
plan_direct            plan_direct :954-1025                          nhip_direct_unary, nhip_rtc_*
plan_lif               plan_lif :1028-1146                            nhip_lif, nhip_alif
plan_lif_rate          plan_lif_rate :1149-1197                       nhip_lif_rate, nhip_alif_rate
plan_rectified_linear  :1238-1258 (and spiking :1200-1235, sigmoid)   nhip_relu, ...
plan_whitenoise        plan_whitenoise :1578-1675 (own generator)     nhip_whitenoise
plan_presentinput      plan_presentinput :1678-1759                   nhip_presentinput
plan_conv2d / pool2d   plan_conv2d :1762-1969, plan_pool2d :1972-2079  nhip_conv2d, nhip_pool2d
plan_bcm / oja / voja  :2082-2169, :2172-2277, :2280-2405             nhip_learning_rule
=====================  =============================================  ==========

Where the reference's kernels index ``*_starts[n]`` device arrays, these build
one int32 work list per plan (a row per block of <= ``BLOCK`` elements of one
item) at plan time; argument checks raise the same exception types the
reference's asserts / raises produce (AssertionError, NotImplementedError).
"""

import logging
import re

import numpy as np

from . import _lib
from .hipraggedarray import DeviceArray, HIPRaggedArray, _torch, to_device
from .plan import Plan
from .utils import f32_bits, is_number

logger = logging.getLogger(__name__)

WG = 256
BLOCK = 1024  # elements of one item handled by one work-group


def blockify(sizes, max_size=BLOCK):
    """Cut items of the given sizes into blocks of <= max_size elements.

    Returns int32 arrays ``(item index, offset inside the item, count)``, one
    entry per block, items in order; empty items get no block.  (The
    reference's ``blockify_ij`` / ``blockify_vectors`` :22-110 do this with
    Python loops; this is the vectorised equivalent.)
    """
    sizes = np.asarray(sizes, dtype=np.int64).reshape(-1)
    n_blocks = -(-sizes // max_size)
    inds = np.repeat(np.arange(sizes.size), n_blocks)
    first = np.cumsum(n_blocks) - n_blocks
    k = np.arange(int(n_blocks.sum())) - np.repeat(first, n_blocks)
    offsets = k * max_size
    counts = np.minimum(sizes[inds] - offsets, max_size)
    return inds.astype(np.int32), offsets.astype(np.int32), counts.astype(np.int32)


def lanes_for(size):
    """Threads that share one work-list row of `size` elements: the next power of two up
    to a wave (64), beyond that a whole group (256)."""
    lanes = 1
    while lanes < size and lanes < 64:
        lanes *= 2
    return lanes if size <= lanes else WG


def rows_for(sizes, max_size=BLOCK):
    """`blockify` with the row length fitted to the items: the lanes per row follow the
    median item size (one element per lane; longer items are cut into several rows), so
    that models with very many very short signals get a few lanes -- not a 256-thread
    group -- per signal, and a group works on 256 / lanes rows side by side.  Items
    longer than a group keep rows of `max_size` elements.
    Returns ``(item index, offset, count, lanes)``."""
    sizes = np.asarray(sizes, dtype=np.int64).reshape(-1)
    used = sizes[sizes > 0]
    lanes = lanes_for(int(np.median(used))) if used.size else WG
    return blockify(sizes, max_size if lanes == WG else lanes) + (lanes,)


def _row_iterations(counts, lanes):
    """Elements the busiest lane handles one after the other."""
    return int(-(-int(np.max(counts)) // lanes)) if len(counts) else 1


def _gsize(n_rows, lanes):
    return (WG * max(-(-n_rows // (WG // lanes)), 1),)


def _check(*named):
    """Bounds-check ragged operands on the host before any kernel is bound to them."""
    for name, ra in named:
        if isinstance(ra, HIPRaggedArray):
            ra.check_bounds(name)


def _description(ra):
    sizes = ra.sizes
    if len(sizes) == 0:
        return "groups: 0"
    return "groups: %d; items: %d; items/group: %0.1f [%d, %d]" % (
        len(ra), sizes.sum(), sizes.mean(), sizes.min(), sizes.max())


def _host(values):
    return values.get() if isinstance(values, DeviceArray) else np.asarray(values)


def _bits(values):
    """float32 bit patterns of an array, as int32."""
    return np.asarray(values, dtype=np.float32).view(np.int32)


def _dev_table(queue, columns, width):
    """Stack per-block int32 columns into a (n_blocks, width) device table."""
    n = len(columns[0]) if columns else 0
    table = np.zeros((max(n, 1), width), dtype=np.int32)
    for c, col in enumerate(columns):
        if n:
            table[:n, c] = col
    return to_device(queue, table), n


# ---------------------------------------------------------------- time update
def plan_timeupdate(queue, step, time, dt):
    assert len(step) == len(time) == 1
    assert step.ctype == time.ctype == "float"
    assert step.shape0s[0] == step.shape1s[0] == 1
    assert time.shape0s[0] == time.shape1s[0] == 1
    _check(("step", step), ("time", time))
    args = (step.ptr, int(step.starts[0]), time.ptr, int(time.starts[0]), float(dt))
    return Plan(queue, queue.lib.nhip_timeupdate, args, gsize=(64,), lsize=(64,),
                full_args=(step.dev_buf, time.dev_buf), name="hip_timeupdate")


# ---------------------------------------------------------------- reset
def plan_reset(queue, Y, values, tag=None):
    values = _host(values).astype(np.float32).reshape(-1)
    assert len(Y) == len(values)
    assert (Y.stride0s == Y.shape1s).all()
    assert (Y.stride1s == 1).all()
    assert Y.ctype == "float"
    _check(("Y", Y))

    inds, offsets, counts, lanes = rows_for(Y.sizes, 4 * BLOCK)
    table, n = _dev_table(queue, [Y.starts[inds] + offsets, counts, _bits(values[inds])], 4)
    plan = Plan(queue, queue.lib.nhip_reset, (table.ptr, n, lanes, Y.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,), full_args=(table, Y.dev_buf),
                name="hip_reset", tag=tag)
    plan.bw_per_call = Y.nbytes + values.nbytes + table.nbytes
    plan.description = _description(Y)
    plan.row_iterations = _row_iterations(counts, lanes)
    return plan


# ---------------------------------------------------------------- copy
def plan_copy(queue, X, Y, incs, tag=None):
    assert len(X) == len(Y)
    assert (X.shape0s == Y.shape0s).all()
    assert (X.shape1s == Y.shape1s).all()
    assert (X.stride1s == 1).all()
    assert (Y.stride1s == 1).all()
    assert X.ctype == Y.ctype
    incs = np.asarray(incs, dtype=np.int32).reshape(-1)
    assert incs.shape == (len(X),)
    _check(("X", X), ("Y", Y))

    inds, offsets, counts, lanes = rows_for(Y.sizes)
    table, n = _dev_table(queue, [X.starts[inds], Y.starts[inds], X.shape1s[inds],
                                  X.stride0s[inds], Y.stride0s[inds], offsets, counts,
                                  incs[inds]], 8)
    plan = Plan(queue, queue.lib.nhip_copy, (table.ptr, n, lanes, X.ptr, Y.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, X.dev_buf, Y.dev_buf), name="hip_copy", tag=tag)
    plan.bw_per_call = X.nbytes + Y.nbytes
    plan.description = _description(X)
    plan.row_iterations = _row_iterations(counts, lanes)
    return plan


# ---------------------------------------------------------------- sliced copy
def plan_slicedcopy(queue, X, Y, Xinds, Yinds, incs, tag=None):
    assert len(X) == len(Y) == len(Xinds) == len(Yinds)
    for arr in [X, Y, Xinds, Yinds]:
        assert (arr.shape1s == 1).all()
        assert (arr.stride1s == 1).all()
    for arr in [Xinds, Yinds]:
        assert (arr.stride0s == 1).all()
    assert (Xinds.shape0s == Yinds.shape0s).all()
    assert X.ctype == Y.ctype
    assert Xinds.ctype == Yinds.ctype == "int"
    incs = np.asarray(incs, dtype=np.int32).reshape(-1)
    assert incs.shape == (len(X),)
    _check(("X", X), ("Y", Y), ("Xinds", Xinds), ("Yinds", Yinds))
    xi_host, yi_host = Xinds.to_host(), Yinds.to_host()
    for k in range(len(X)):  # every index must address an element of its vector
        if Xinds.shape0s[k]:
            assert 0 <= xi_host[k].min() and xi_host[k].max() < X.shape0s[k], "Xinds[%d] out of range" % k
            assert 0 <= yi_host[k].min() and yi_host[k].max() < Y.shape0s[k], "Yinds[%d] out of range" % k

    inds, offsets, counts, lanes = rows_for(Xinds.shape0s)
    table, n = _dev_table(queue, [X.starts[inds], X.stride0s[inds], Y.starts[inds],
                                  Y.stride0s[inds], Xinds.starts[inds] + offsets,
                                  Yinds.starts[inds] + offsets, counts, incs[inds]], 8)
    plan = Plan(queue, queue.lib.nhip_slicedcopy,
                (table.ptr, n, lanes, X.ptr, Y.ptr, Xinds.ptr, Yinds.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, X.dev_buf, Y.dev_buf, Xinds.dev_buf, Yinds.dev_buf),
                name="hip_slicedcopy", tag=tag)
    plan.bw_per_call = 2 * (Xinds.nbytes + int(Xinds.sizes.sum()) * X.dtype.itemsize)
    plan.description = _description(Xinds)
    plan.row_iterations = _row_iterations(counts, lanes)
    return plan


# ---------------------------------------------------------------- elementwise inc
def plan_elementwise_inc(queue, A, X, Y, alpha=None, outer=False, inc=True, tag=None):
    """``Y (+)= alpha * A * X`` element-wise with broadcasting, or (``outer``) the
    outer product of vectors A and X."""
    assert len(Y) == len(X) == len(A)
    for arr in [A, X, Y]:
        assert (arr.stride1s == 1).all()
    if outer:
        assert (A.shape1s == 1).all()
        assert (X.shape1s == 1).all()
        assert ((A.shape0s == 1) | (A.shape0s == Y.shape0s)).all()
        assert ((X.shape0s == 1) | (X.shape0s == Y.shape1s)).all()
    else:
        assert ((X.shape0s == 1) | (X.shape0s == Y.shape0s)).all()
        assert ((X.shape1s == 1) | (X.shape1s == Y.shape1s)).all()
        assert ((A.shape0s == 1) | (A.shape0s == Y.shape0s)).all()
        assert ((A.shape1s == 1) | (A.shape1s == Y.shape1s)).all()
    assert X.ctype == Y.ctype
    assert A.ctype == Y.ctype
    if alpha is not None:
        assert isinstance(alpha, np.ndarray)
        assert alpha.shape == (len(Y),)
        alphas = alpha.astype(np.float32)
    else:
        alphas = np.ones(len(Y), dtype=np.float32)
    _check(("A", A), ("X", X), ("Y", Y))

    # large outer products (learning rules over whole weight matrices): rows of 4096
    # elements, four 16-byte accesses per lane issued together
    big = outer and int(Y.sizes.sum()) >= (1 << 20)
    inds, offsets, counts, lanes = rows_for(Y.sizes, max_size=4 * BLOCK if big else BLOCK)
    flags = np.full(len(inds), (1 if outer else 0) | (2 if inc else 0), dtype=np.int32)
    table, n = _dev_table(queue, [
        A.starts[inds], A.shape0s[inds], A.shape1s[inds], A.stride0s[inds],
        X.starts[inds], X.shape0s[inds], X.shape1s[inds], X.stride0s[inds],
        Y.starts[inds], Y.shape1s[inds], Y.stride0s[inds], offsets,
        counts, _bits(alphas[inds]), flags], 16)
    plan = Plan(queue, queue.lib.nhip_elementwise_inc, (table.ptr, n, lanes, A.ptr, X.ptr, Y.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, A.dev_buf, X.dev_buf, Y.dev_buf),
                name="hip_elementwise_inc", tag=tag)
    plan.flops_per_call = 2 * int(Y.sizes.sum())
    plan.bw_per_call = A.nbytes + X.nbytes + Y.nbytes + (0 if alpha is None else alphas.nbytes)
    plan.description = _description(Y)
    plan.row_iterations = _row_iterations(counts, lanes)
    # what `fuse_outer_filter` needs to run the filters of the column operands in this launch
    plan.ew_spec = dict(A=A, X=X, Y=Y, alphas=alphas, outer=outer, inc=inc)
    return plan


# ---------------------------------------------------------------- outer product + filter
OF_INC, OF_FILTER, OF_FILTER_HAS_A, OF_NO_OUTER = 1, 2, 4, 8  # flags of csrc/elementwise.hip
OF_MAX_COLS, OF_MAX_ROWS = 128, 256


def _interval(ra, i):
    """[first, last + 1) element of item i of a ragged array (empty items: None)."""
    n0, n1 = int(ra.shape0s[i]), int(ra.shape1s[i])
    if n0 == 0 or n1 == 0:
        return None
    first = int(ra.starts[i])
    return first, first + (n0 - 1) * int(ra.stride0s[i]) + (n1 - 1) * int(ra.stride1s[i]) + 1


def _apart(reason):
    logger.debug("outer product and filter stay launches of their own: %s", reason)
    return None


def _touch(iv, others):
    return iv is not None and any(o is not None and iv[0] < o[1] and o[0] < iv[1] for o in others)


def fuse_outer_filter(ew_plan, lf_plan):
    """One launch for "W (+)= (alpha a) (x) f; f <- filter(s)" (clra_nonlinearities.py
    `plan_elementwise_inc` with outer=True followed by `plan_linearfilter`): the end of a
    PES step, where the filter of the pre-synaptic activities may only run once the weight
    update has read their old values.  A work-group of `nhip_outer_filter` owns all rows of
    up to 128 columns of a matrix and steps the filter elements of those columns after
    writing them.

    Fused when every outer product has at most 256 rows and 16-byte aligned rows, every
    filter has one numerator and at most one denominator coefficient over contiguous
    vectors, and each filter output is either the column operand of exactly one outer
    product (same start and length) or touched by none of them; nothing the filters write
    may be a row operand or another operand of the launch.  Returns the plan that replaces
    both, or None.
    """
    ew, lf = getattr(ew_plan, "ew_spec", None), getattr(lf_plan, "lf_spec", None)
    if ew is None or lf is None or not ew["outer"]:
        return _apart("no outer product or no simple filter plan")
    A, X, Y, alphas, inc = ew["A"], ew["X"], ew["Y"], ew["alphas"], ew["inc"]
    S, F, FA, FB = lf["X"], lf["Y"], lf["A"], lf["B"]
    queue = ew_plan.queue
    n_outer, n_filters = len(Y), len(F)
    if n_outer == 0 or n_filters == 0:
        return _apart("nothing to fuse")
    # shapes the kernel takes
    for i in range(n_outer):
        rows, cols = int(Y.shape0s[i]), int(Y.shape1s[i])
        if rows > OF_MAX_ROWS or rows == 0 or cols == 0:
            return _apart("an outer product with more than 256 rows or an empty one")
        if (int(Y.starts[i]) | int(Y.stride0s[i]) | cols) & 3:
            return _apart("rows of an outer product are not whole aligned quads")
    for k in range(n_filters):
        simple = int(FB.shape0s[k]) == 1 and int(FA.shape0s[k]) <= 1
        vector = all(int(r.shape1s[k]) == 1 and int(r.stride0s[k]) == 1 for r in (S, F))
        if not (simple and vector and int(S.shape0s[k]) == int(F.shape0s[k])):
            return _apart("a filter of higher order or over strided vectors")
    same = lambda p, q: p.ptr.value == q.ptr.value
    f_iv = [_interval(F, k) for k in range(n_filters)]
    x_iv = [_interval(X, i) for i in range(n_outer)]
    a_iv = [_interval(A, i) for i in range(n_outer)]
    y_iv = [_interval(Y, i) for i in range(n_outer)]
    s_iv = [_interval(S, k) for k in range(n_filters)]
    # filter outputs: the column operand of exactly one outer product, or of none
    owner = {}  # filter -> outer product
    for k in range(n_filters):
        users = [i for i in range(n_outer) if same(F, X) and _touch(f_iv[k], [x_iv[i]])]
        if same(F, A) and _touch(f_iv[k], a_iv):
            return _apart("a filter output is a row operand of the launch")
        if same(F, Y) and _touch(f_iv[k], y_iv):
            return _apart("a filter output overlaps a matrix of the launch")
        if same(F, S) and _touch(f_iv[k], [s_iv[q] for q in range(n_filters) if q != k]):
            return _apart("a filter output is another filter's input")
        if not users:
            continue
        i = users[0]
        exact = (len(users) == 1 and int(X.shape0s[i]) == int(Y.shape1s[i])
                 and int(X.stride0s[i]) == 1 and x_iv[i] == f_iv[k])
        if not exact:
            return _apart("a filter output is not exactly the column operand of one outer product")
        owner[k] = i
    if len(set(owner.values())) != len(owner):
        return _apart("two filters feed the column operand of one outer product")
    if same(S, Y) and any(_touch(iv, y_iv) for iv in s_iv):
        return _apart("a filter input overlaps a matrix of the launch")
    if not owner:
        return _apart("no filter output is a column operand of the launch")
    filter_of = {i: k for k, i in owner.items()}

    a_host, b_host = FA.to_host(), FB.to_host()

    def filter_words(k):
        na = int(FA.shape0s[k])
        a0 = np.float32(a_host[k][0, 0]) if na else np.float32(0)
        b0 = np.float32(b_host[k][0, 0])
        flags = OF_FILTER | (OF_FILTER_HAS_A if na else 0)
        return flags, int(S.starts[k]), int(F.starts[k]), int(a0.view(np.int32)), int(b0.view(np.int32))

    records = []
    for i in range(n_outer):
        rows, cols = int(Y.shape0s[i]), int(Y.shape1s[i])
        a_stride = 0 if int(A.shape0s[i]) == 1 else int(A.stride0s[i])
        x_stride = 0 if int(X.shape0s[i]) == 1 else int(X.stride0s[i])
        alpha_bits = int(np.float32(alphas[i]).view(np.int32))
        flags, s0, f0, fa, fb = (0, 0, 0, 0, 0)
        if i in filter_of:
            flags, s0, f0, fa, fb = filter_words(filter_of[i])
        for col0 in range(0, cols, OF_MAX_COLS):
            records.append((int(A.starts[i]), a_stride, int(X.starts[i]), x_stride,
                            int(Y.starts[i]), int(Y.stride0s[i]), rows, col0,
                            min(OF_MAX_COLS, cols - col0), alpha_bits,
                            flags | (OF_INC if inc else 0), s0, f0, fa, fb, 0))
    for k in range(n_filters):
        if k in owner:
            continue
        flags, s0, f0, fa, fb = filter_words(k)
        for col0 in range(0, int(F.shape0s[k]), OF_MAX_COLS):
            records.append((0, 0, 0, 0, 0, 0, 0, col0, min(OF_MAX_COLS, int(F.shape0s[k]) - col0),
                            0, flags | OF_NO_OUTER, s0, f0, fa, fb, 0))
    table = to_device(queue, np.array(records, dtype=np.int32).reshape(-1, 16))
    n = len(records)
    plan = Plan(queue, queue.lib.nhip_outer_filter,
                (table.ptr, n, A.ptr, X.ptr, Y.ptr, S.ptr, F.ptr),
                gsize=(n * WG,), lsize=(WG,),
                full_args=tuple(ew_plan.full_args) + tuple(lf_plan.full_args) + (table,),
                name="hip_outer_filter", tag=ew_plan.tag)
    plan.flops_per_call = (ew_plan.flops_per_call or 0) + (lf_plan.flops_per_call or 0)
    plan.bw_per_call = (ew_plan.bw_per_call or 0) + (lf_plan.bw_per_call or 0)
    plan.description = ew_plan.description
    plan.fused_filters = sorted(owner)
    return plan


# ---------------------------------------------------------------- linear filter
def plan_linearfilter(queue, X, Y, A, B, Xbuf, Ybuf, tag=None):
    """``y[n+1] + a[0] y[n] + ... = b[0] x[n] + ... + b[j] x[n-j]`` per element.

    Returns a one-element list: the ring-buffer positions advance inside the
    same launch (the reference returns a second ``linearfilter_inc`` plan when
    any filter has order > 1, :781-803).
    """
    assert len(X) == len(Y) == len(A) == len(B) == len(Xbuf) == len(Ybuf)
    assert (X.shape0s == Y.shape0s).all()
    assert (X.shape1s == Y.shape1s).all()
    for arr in [A, B, Xbuf, Ybuf]:
        assert (arr.shape1s == arr.stride0s).all()
        assert (arr.stride1s == 1).all()
    for arr in [A, B]:
        assert (arr.shape1s == 1).all()
    assert (B.shape0s >= 1).all()
    assert ((B.shape0s == 1) | (Xbuf.shape0s == B.shape0s)).all()
    assert ((A.shape0s == 1) | (Ybuf.shape0s == A.shape0s)).all()
    assert (Xbuf.shape1s == X.sizes).all()
    assert (Ybuf.shape1s == Y.sizes).all()
    assert X.ctype == Xbuf.ctype
    assert Y.ctype == Ybuf.ctype
    _check(("X", X), ("Y", Y), ("A", A), ("B", B), ("Xbuf", Xbuf), ("Ybuf", Ybuf))

    inds, offsets, counts, lanes = rows_for(X.sizes)
    table, n = _dev_table(queue, [
        X.starts[inds], X.stride0s[inds], X.stride1s[inds], Y.starts[inds],
        Y.stride0s[inds], Y.stride1s[inds], X.shape1s[inds], offsets,
        counts, A.shape0s[inds], B.shape0s[inds], A.starts[inds],
        B.starts[inds], Xbuf.starts[inds], Ybuf.starts[inds], X.sizes[inds]], 16)
    pos = to_device(queue, np.zeros((max(n, 1), 2), dtype=np.int32))
    plan = Plan(queue, queue.lib.nhip_linearfilter,
                (table.ptr, pos.ptr, n, lanes, X.ptr, Y.ptr, A.ptr, B.ptr, Xbuf.ptr, Ybuf.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, pos, X.dev_buf, Y.dev_buf, A.dev_buf, B.dev_buf,
                           Xbuf.dev_buf, Ybuf.dev_buf),
                name="hip_linearfilter", tag=tag)
    plan.bw_per_call = (X.nbytes + Y.nbytes + A.nbytes + B.nbytes + Xbuf.nbytes + Ybuf.nbytes)
    plan.description = _description(Y)
    plan.row_iterations = _row_iterations(counts, lanes)
    plan.bufpos = pos  # zeroed again by Simulator.reset()
    plan.higher_order = bool(((A.shape0s > 1) | (B.shape0s > 1)).any())  # ring buffers in use
    # what a GEMV that produces X needs to run simple filters as its epilogue
    plan.lf_spec = dict(X=X, Y=Y, A=A, B=B, Xbuf=Xbuf, Ybuf=Ybuf)
    return [plan]


# ---------------------------------------------------------------- probes
def plan_probes(queue, periods, X, Y, tag=None):
    """Every ``periods[i]`` steps copy signal ``X[i]`` into row ``bufpositions[i]``
    of ``Y[i]`` (shape ``(buf_len, X[i].size)``)."""
    assert len(X) == len(Y)
    assert len(X) == len(periods)
    assert X.ctype == Y.ctype
    N = len(X)
    assert (X.shape0s * X.shape1s == Y.shape1s).all()
    assert (Y.stride0s == Y.shape1s).all()
    assert (Y.stride1s == 1).all()
    _check(("X", X), ("Y", Y))

    periods = np.asarray(periods, dtype=np.float32)
    dev_periods = to_device(queue, periods)
    dev_countdowns = to_device(queue, periods - 1)
    dev_bufpositions = to_device(queue, np.zeros(N, dtype=np.int32))
    table, n = _dev_table(queue, [X.starts, X.shape0s, X.shape1s, X.stride0s, X.stride1s,
                                  Y.starts, Y.shape0s], 8)
    widest = int((X.shape0s * X.shape1s).max()) if N else 1
    lanes = lanes_for(widest)  # a probe is one row
    plan = Plan(queue, queue.lib.nhip_probes,
                (table.ptr, n, lanes, dev_countdowns.ptr, dev_bufpositions.ptr, dev_periods.ptr,
                 X.ptr, Y.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, dev_countdowns, dev_bufpositions, dev_periods, X.dev_buf,
                           Y.dev_buf), name="hip_probes", tag=tag)
    plan.dev_bufpositions = dev_bufpositions
    plan.cl_bufpositions = dev_bufpositions  # the reference's attribute name
    plan.dev_countdowns = dev_countdowns
    plan.periods = periods
    plan.Y = Y
    plan.row_iterations = -(-widest // lanes)
    plan.bw_per_call = (2 * X.nbytes + dev_periods.nbytes + dev_countdowns.nbytes
                        + dev_bufpositions.nbytes)
    plan.description = _description(X)
    return plan


class ProbeDrain:
    """End-of-batch transfer of the step counter, the clock and the buffered probe rows
    in one device-to-host copy (`nhip_probes_drain`); what `Simulator._probe` does in the
    reference with one transfer per probe (simulator.py:499-520).

    ``probe_plan`` is the plan returned by `plan_probes` (or None for a model without
    probes: the drain then fetches the clock only); ``signals`` the ragged array holding
    the step counter (item ``step_idx``) and the clock (``time_idx``)."""

    STAGING_BYTES = 16 * 1024 * 1024  # larger drains are read buffer by buffer

    def __init__(self, queue, probe_plan, signals, step_idx, time_idx):
        import ctypes

        torch = _torch()
        self.queue, self.plan, self.signals = queue, probe_plan, signals
        self.step_start = int(signals.starts[step_idx])
        self.time_start = int(signals.starts[time_idx])
        if probe_plan is not None:
            Y = probe_plan.Y
            widths = np.asarray(Y.shape1s, dtype=np.int64)
            self.capacities = np.asarray(Y.shape0s, dtype=np.int64)
            self.n = len(Y)
        else:
            widths = np.zeros(0, dtype=np.int64)
            self.capacities = np.zeros(0, dtype=np.int64)
            self.n = 0
        self.widths = widths
        self.wprefix = np.concatenate([[0], np.cumsum(widths)[:-1]]).astype(np.int64) if self.n else widths
        self.total_width = int(widths.sum())
        self.max_width = int(widths.max()) if self.n else 0
        self.header = (self.n + 2 + 63) // 64 * 64
        full = self.header + int(self.capacities.max() if self.n else 0) * self.total_width
        self.words = int(min(full, max(self.STAGING_BYTES // 4, self.header + self.total_width)))
        if self.n:
            self.table, _ = _dev_table(queue, [Y.starts, widths, self.wprefix, self.capacities], 4)
        else:
            self.table = None
        with queue.context():
            self.staging = torch.zeros(self.words, dtype=torch.float32, device=queue.device)
        self.host = torch.zeros(self.words, dtype=torch.float32, pin_memory=True)
        self.host_np = self.host.numpy()
        self._p = ctypes.c_void_p

    def max_rows(self):
        """Most rows per probe one transfer can carry."""
        if not self.n:
            return 0
        return (self.words - self.header) // max(self.total_width, 1)

    def __call__(self, rows_bound):
        """Returns ``(step, time, counts, rows)``: ``rows[i]`` is an array of shape
        ``(min(counts[i], rows_bound), width_i)`` (a copy).  Buffer positions are zero
        afterwards."""
        p = self._p
        rows_bound = int(min(rows_bound, self.capacities.max())) if self.n else 0
        plan = self.plan
        _lib.check(self.queue.lib.nhip_probes_drain(
            self.queue.handle, self.table.ptr if self.n else None, self.n, self.total_width,
            self.max_width, rows_bound, plan.dev_bufpositions.ptr if self.n else None,
            plan.Y.ptr if self.n else None, self.signals.ptr, self.step_start, self.time_start,
            p(self.staging.data_ptr()), self.words, p(self.host.data_ptr())), "probe drain")
        out = self.host_np
        counts = out[2:2 + self.n].view(np.int32).copy()
        rows = []
        for i in range(self.n):
            k = int(min(counts[i], rows_bound, self.capacities[i]))
            w = int(self.widths[i])
            a = self.header + rows_bound * int(self.wprefix[i])
            rows.append(out[a:a + k * w].reshape(k, w).copy())
        return float(out[0]), float(out[1]), counts, rows


# ---------------------------------------------------------------- function nodes
UNARY_OPCODES = {"identity": 0, "sin": 1, "cos": 2, "tanh": 3, "exp": 4, "square": 5}
_DIRECT_RE = re.compile(
    r"^\s*OUTPUT__\[0\]\s*=\s*(?P<fn>[a-z]+)\(\s*(?P<arg>\w+)\[0\]\s*\)\s*;\s*$")


def plan_direct(queue, code, init, input_names, inputs, output, tag=None):
    """A function node on the device: ``code`` (C statements assigning ``OUTPUT__[i]``
    from the inputs ``name[i]``, after the declarations in ``init``) runs once per
    output item, one thread each (reference ``plan_direct`` :954-1025).

    ``OUTPUT__[0] = f(name[0]);`` with f in the unary table goes to a precompiled kernel
    (which can share a launch with other short operations); any other code is compiled
    at run time.  Compilation errors raise NotImplementedError, on which the Simulator
    falls back to a host callback, as the reference does when its translator fails
    (simulator.py:955-964)."""
    assert len(input_names) == len(inputs)
    for x in inputs:
        assert len(x) == len(output)
    for x in list(inputs) + [output]:
        assert (x.shape1s == 1).all() and (x.stride1s == 1).all()
        assert (x.stride0s == 1).all()
        assert x.ctype == "float"
    _check(*([("input", x) for x in inputs] + [("output", output)]))
    m = _DIRECT_RE.match(code or "")
    if (not (init or "").strip() and m is not None and m.group("fn") in UNARY_OPCODES
            and m.group("arg") in input_names):
        x = inputs[list(input_names).index(m.group("arg"))]
        assert (x.shape0s == 1).all() and (output.shape0s == 1).all()
        table, n = _dev_table(queue, [x.starts, output.starts, np.ones(len(output), np.int32)], 4)
        plan = Plan(queue, queue.lib.nhip_direct_unary,
                    (UNARY_OPCODES[m.group("fn")], table.ptr, n, 1, x.ptr, output.ptr),
                    gsize=_gsize(n, 1), lsize=(WG,),
                    full_args=(table, x.dev_buf, output.dev_buf), name="hip_direct", tag=tag)
        plan.description = _description(output)
        return plan
    return _plan_direct_compiled(queue, code, init, input_names, inputs, output, tag)


DIRECT_KERNEL = """\
// (the run-time compiler's headers do not bring the C macros for these along)
#ifndef INFINITY
#define INFINITY __builtin_inff()
#endif
#ifndef NAN
#define NAN __builtin_nanf("")
#endif
extern "C" __global__ void direct(int n__, const int* in0_starts__, const float* in0_data__,
                                  const int* in1_starts__, const float* in1_data__,
                                  const int* out_starts__, float* out_data__) {
    const int k__ = blockIdx.x * blockDim.x + threadIdx.x;
    if (k__ >= n__) return;
%(inputs)s
    float* OUTPUT__ = out_data__ + out_starts__[k__];
%(init)s
%(code)s
}
"""


def direct_kernel_source(code, init, input_names):
    """HIP source of the kernel ``plan_direct`` compiles for this code."""
    if len(input_names) > 2:
        raise NotImplementedError("function nodes take at most two inputs (time, vector)")
    lines = ["    const float* %s = in%d_data__ + in%d_starts__[k__];" % (name, i, i)
             for i, name in enumerate(input_names)]
    indent = lambda text: "\n".join("    " + line for line in (text or "").splitlines())
    return DIRECT_KERNEL % dict(inputs="\n".join(lines), init=indent(init), code=indent(code))


_compiled_programs = {}  # source text -> compiled program (kept for the life of the process)


def compile_direct(lib, source):
    """Compile (or look up) a function-node kernel; raises NotImplementedError with the
    compiler's messages if the source does not compile.  Needs no device."""
    import ctypes

    program = _compiled_programs.get(source)
    if program is None:
        handle = ctypes.c_void_p()
        log = ctypes.create_string_buffer(8192)
        err = lib.nhip_rtc_compile(source.encode(), b"gfx950", ctypes.byref(handle), log, len(log))
        if err != 0:
            raise NotImplementedError("the function's kernel does not compile:\n%s"
                                      % log.value.decode(errors="replace"))
        program = _compiled_programs[source] = handle
    return program


def _plan_direct_compiled(queue, code, init, input_names, inputs, output, tag):
    import ctypes

    source = direct_kernel_source(code, init, list(input_names))
    program = compile_direct(queue.lib, source)
    function = ctypes.c_void_p()
    _lib.check(queue.lib.nhip_rtc_load(program, b"direct", ctypes.byref(function)),
               "loading a function-node kernel")
    n = len(output)
    starts = [to_device(queue, np.ascontiguousarray(x.starts, dtype=np.int32)) for x in inputs]
    out_starts = to_device(queue, np.ascontiguousarray(output.starts, dtype=np.int32))
    pairs = [(s.ptr, x.ptr) for s, x in zip(starts, inputs)] + [(None, None)] * (2 - len(inputs))
    args = (function, n, pairs[0][0], pairs[0][1], pairs[1][0], pairs[1][1], out_starts.ptr,
            output.ptr)
    plan = Plan(queue, queue.lib.nhip_rtc_launch_direct, args, gsize=(64 * max(-(-n // 64), 1),),
                lsize=(64,), full_args=tuple(starts) + (out_starts, output.dev_buf, function)
                + tuple(x.dev_buf for x in inputs), name="hip_direct_compiled", tag=tag)
    plan.source = source
    plan.bw_per_call = output.nbytes + sum(x.nbytes for x in inputs)
    plan.description = _description(output)
    return plan


# ---------------------------------------------------------------- neurons
def _neuron_params(queue, params, sizes, inds, offsets):
    """Pack tau/ref/amp for the block table.

    A number, an ndarray with one value per item, or a ragged array whose items
    are each constant, becomes float bits in the table (one scalar per block, no per-neuron traffic).  Ragged
    arrays with varying values stay on the device and the table holds offsets.
    Returns (columns, pflags, device pointers, keepalive).
    """
    columns, ptrs, keep = [], [], []
    pflags = 0
    for k, p in enumerate(params):
        if is_number(p):
            columns.append(np.full(len(inds), f32_bits(p), dtype=np.int32))
            ptrs.append(None)
            continue
        if isinstance(p, np.ndarray) and p.shape == (len(sizes),):  # one value per item
            columns.append(_bits(p.astype(np.float32)[inds]))
            ptrs.append(None)
            continue
        if not isinstance(p, HIPRaggedArray):
            raise ValueError("Parameter must be a ragged device array or a float (got %s)" % type(p))
        assert len(p) == len(sizes)
        assert (p.shape1s == 1).all() and (p.stride1s == 1).all() and (p.stride0s == 1).all()
        assert ((p.shape0s == sizes) | (p.shape0s == 1)).all()
        host = p.to_host()
        firsts = np.array([host[i][0, 0] if host.sizes[i] else 0.0 for i in range(len(host))],
                          dtype=np.float32)
        constant = all(np.all(host[i] == firsts[i]) for i in range(len(host)))
        if constant:
            columns.append(_bits(firsts[inds]))
            ptrs.append(None)
        else:
            assert (p.shape0s == sizes).all(), "varying parameters need one value per neuron"
            columns.append(p.starts[inds] + offsets)
            ptrs.append(p.ptr)
            keep.append(p.dev_buf)
            pflags |= 1 << k
    return columns, pflags, ptrs, keep


def _check_vectors(ras):
    first = ras[0]
    for v in ras:
        assert len(v) == len(first)
        assert (v.shape0s == first.shape0s).all()
        assert (v.stride0s == v.shape1s).all()
        assert (v.stride1s == 1).all()
        assert (v.shape1s == 1).all()


def plan_lif(queue, dt, J, V, W, outS, ref, tau, amp, N=None, tau_n=None, inc_n=None,
             upsample=1, fastlif=False, tag=None, **kwargs):
    if N is not None or tau_n is not None or inc_n is not None:
        if fastlif:
            raise NotImplementedError("fastlif approximation")
        return _plan_alif(queue, dt, J, V, W, outS, ref, tau, amp, N, tau_n, inc_n, upsample, tag)
    if fastlif:
        raise NotImplementedError("fastlif approximation")
    assert J.ctype == "float"
    for x in [V, W, outS]:
        assert x.ctype == J.ctype
    _check_vectors([J, V, W, outS])
    _check(("J", J), ("V", V), ("W", W), ("outS", outS), ("tau", tau), ("ref", ref), ("amp", amp))

    inds, offsets, counts = blockify(J.shape0s, 2 * WG)
    pcols, pflags, pptrs, keep = _neuron_params(queue, [tau, ref, amp], J.shape0s, inds, offsets)
    table, n = _dev_table(queue, [
        J.starts[inds] + offsets, V.starts[inds] + offsets, W.starts[inds] + offsets,
        outS.starts[inds] + offsets, counts, pcols[0], pcols[1], pcols[2],
        np.full(len(inds), pflags, dtype=np.int32)], 12)
    args = (table.ptr, n, float(dt), int(upsample), J.ptr, V.ptr, W.ptr, outS.ptr,
            pptrs[0], pptrs[1], pptrs[2])
    plan = Plan(queue, queue.lib.nhip_lif, args, gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, V.dev_buf, W.dev_buf, outS.dev_buf) + tuple(keep),
                name="hip_lif", tag=tag)
    n_vec = bin(pflags).count("1")
    plan.bw_per_call = (J.nbytes + 2 * V.nbytes + 2 * W.nbytes + outS.nbytes + n_vec * J.nbytes)
    plan.description = _description(J)
    # what a GEMV that produces J needs to run this update as its epilogue
    plan.lif_spec = dict(dt=float(dt), upsample=int(upsample), J=J, V=V, W=W, outS=outS,
                         ref=ref, tau=tau, amp=amp)
    return plan


def lif_population_table(queue, spec):
    """Per-population rows {v_start, w_start, s_start, tau, ref, amp, pflags} (int32
    columns) of a `plan_lif` call, plus the parameter pointers and keep-alives."""
    J = spec["J"]
    n = len(J)
    inds = np.arange(n)
    zeros = np.zeros(n, dtype=np.int64)
    pcols, pflags, pptrs, keep = _neuron_params(
        queue, [spec["tau"], spec["ref"], spec["amp"]], J.shape0s, inds, zeros)
    cols = dict(v_start=spec["V"].starts, w_start=spec["W"].starts, s_start=spec["outS"].starts,
                tau=pcols[0], ref=pcols[1], amp=pcols[2],
                pflags=np.full(n, pflags, dtype=np.int32))
    return cols, pptrs, keep


def plan_lif_rate(queue, dt, J, R, ref, tau, amp, N=None, tau_n=None, inc_n=None, tag=None,
                  **kwargs):
    if N is not None or tau_n is not None or inc_n is not None:
        return _plan_alif_rate(queue, dt, J, R, ref, tau, amp, N, tau_n, inc_n, tag)
    assert J.ctype == "float"
    assert R.ctype == J.ctype
    _check_vectors([J, R])
    _check(("J", J), ("R", R), ("tau", tau), ("ref", ref), ("amp", amp))

    inds, offsets, counts = blockify(J.shape0s, 2 * WG)
    pcols, pflags, pptrs, keep = _neuron_params(queue, [tau, ref, amp], J.shape0s, inds, offsets)
    table, n = _dev_table(queue, [J.starts[inds] + offsets, R.starts[inds] + offsets, counts,
                                  pcols[0], pcols[1], pcols[2],
                                  np.full(len(inds), pflags, dtype=np.int32)], 8)
    args = (table.ptr, n, J.ptr, R.ptr, pptrs[0], pptrs[1], pptrs[2])
    plan = Plan(queue, queue.lib.nhip_lif_rate, args, gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, R.dev_buf) + tuple(keep), name="hip_lif_rate",
                tag=tag)
    plan.bw_per_call = J.nbytes + R.nbytes + bin(pflags).count("1") * J.nbytes
    plan.description = _description(J)
    return plan


# ---------------------------------------------------------------- further neuron types
def _neuron_table(queue, J, out, params, V=None, W=None, N=None):
    """Work list {j, out, v, w, n offsets, count, pflags, 0, p0..p4, 0, 0, 0} of the neuron
    kernels that share `NeuronDesc` (one row per block of <= 512 neurons)."""
    inds, offsets, counts = blockify(J.shape0s, 2 * WG)
    pcols, pflags, pptrs, keep = _neuron_params(queue, params, J.shape0s, inds, offsets)
    zeros = np.zeros(len(inds), dtype=np.int32)
    start = lambda ra: zeros if ra is None else ra.starts[inds] + offsets
    columns = [start(J), start(out), start(V), start(W), start(N), counts,
               np.full(len(inds), pflags, dtype=np.int32), zeros]
    columns += pcols + [zeros] * (8 - len(pcols))
    table, n = _dev_table(queue, columns, 16)
    n_vec = bin(pflags).count("1")
    return table, n, pptrs, keep, n_vec


def _plan_alif(queue, dt, J, V, W, outS, ref, tau, amp, N, tau_n, inc_n, upsample, tag):
    """Adaptive LIF (clra_nonlinearities.py `plan_lif` with N, tau_n, inc_n, :1028-1146)."""
    assert all(x is not None for x in [N, tau_n, inc_n])
    assert J.ctype == "float"
    for x in [V, W, outS, N]:
        assert x.ctype == J.ctype
    _check_vectors([J, V, W, outS, N])
    _check(("J", J), ("V", V), ("W", W), ("outS", outS), ("N", N), ("tau", tau), ("ref", ref),
           ("amp", amp), ("tau_n", tau_n), ("inc_n", inc_n))
    table, n, pp, keep, n_vec = _neuron_table(queue, J, outS, [tau, ref, amp, tau_n, inc_n],
                                              V=V, W=W, N=N)
    args = (table.ptr, n, float(dt), int(upsample), J.ptr, V.ptr, W.ptr, outS.ptr, N.ptr,
            pp[0], pp[1], pp[2], pp[3], pp[4])
    plan = Plan(queue, queue.lib.nhip_alif, args, gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, V.dev_buf, W.dev_buf, outS.dev_buf, N.dev_buf)
                + tuple(keep), name="hip_alif", tag=tag)
    plan.bw_per_call = (J.nbytes + 2 * V.nbytes + 2 * W.nbytes + 2 * N.nbytes + outS.nbytes
                        + n_vec * J.nbytes)
    plan.description = _description(J)
    return plan


def _plan_alif_rate(queue, dt, J, R, ref, tau, amp, N, tau_n, inc_n, tag):
    """Adaptive LIF rate (`plan_lif_rate` with N, tau_n, inc_n, :1149-1197)."""
    assert all(x is not None for x in [N, tau_n, inc_n])
    assert J.ctype == "float" and R.ctype == J.ctype and N.ctype == J.ctype
    _check_vectors([J, R, N])
    _check(("J", J), ("R", R), ("N", N), ("tau", tau), ("ref", ref), ("amp", amp),
           ("tau_n", tau_n), ("inc_n", inc_n))
    table, n, pp, keep, n_vec = _neuron_table(queue, J, R, [tau, ref, amp, tau_n, inc_n], N=N)
    args = (table.ptr, n, float(dt), J.ptr, R.ptr, N.ptr, pp[0], pp[1], pp[2], pp[3], pp[4])
    plan = Plan(queue, queue.lib.nhip_alif_rate, args, gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, R.dev_buf, N.dev_buf) + tuple(keep),
                name="hip_alif_rate", tag=tag)
    plan.bw_per_call = J.nbytes + R.nbytes + 2 * N.nbytes + n_vec * J.nbytes
    plan.description = _description(J)
    return plan


def plan_rectified_linear(queue, J, R, amp, tag=None, **kwargs):
    """``R = amp * max(J, 0)`` (clra_nonlinearities.py:1238-1258)."""
    assert J.ctype == "float" and R.ctype == J.ctype
    _check_vectors([J, R])
    _check(("J", J), ("R", R), ("amp", amp))
    table, n, pp, keep, n_vec = _neuron_table(queue, J, R, [amp])
    plan = Plan(queue, queue.lib.nhip_relu, (table.ptr, n, J.ptr, R.ptr, pp[0]),
                gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, R.dev_buf) + tuple(keep), name="hip_relu", tag=tag)
    plan.bw_per_call = J.nbytes + R.nbytes + n_vec * J.nbytes
    plan.description = _description(J)
    return plan


def plan_spiking_rectified_linear(queue, dt, J, V, outS, amp, tag=None, **kwargs):
    """``V += dt * max(J, 0); n = floor(V); V -= n; S = amp * n / dt``
    (clra_nonlinearities.py:1200-1235)."""
    assert J.ctype == "float"
    for x in [V, outS]:
        assert x.ctype == J.ctype
    _check_vectors([J, V, outS])
    _check(("J", J), ("V", V), ("outS", outS), ("amp", amp))
    table, n, pp, keep, n_vec = _neuron_table(queue, J, outS, [amp], V=V)
    plan = Plan(queue, queue.lib.nhip_spiking_relu,
                (table.ptr, n, float(dt), J.ptr, V.ptr, outS.ptr, pp[0]),
                gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, V.dev_buf, outS.dev_buf) + tuple(keep),
                name="hip_spikingrelu", tag=tag)
    plan.bw_per_call = J.nbytes + 2 * V.nbytes + outS.nbytes + n_vec * J.nbytes
    plan.description = _description(J)
    return plan


def plan_sigmoid(queue, J, R, ref, tag=None, **kwargs):
    """``R = 1 / (ref * (1 + exp(-J)))`` with the cut-offs of clra_nonlinearities.py:1261-1283."""
    assert J.ctype == "float" and R.ctype == J.ctype
    _check_vectors([J, R])
    _check(("J", J), ("R", R), ("ref", ref))
    table, n, pp, keep, n_vec = _neuron_table(queue, J, R, [ref])
    plan = Plan(queue, queue.lib.nhip_sigmoid, (table.ptr, n, J.ptr, R.ptr, pp[0]),
                gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=(table, J.dev_buf, R.dev_buf) + tuple(keep), name="hip_sigmoid", tag=tag)
    plan.bw_per_call = J.nbytes + R.nbytes + n_vec * J.nbytes
    plan.description = _description(J)
    return plan


# ---------------------------------------------------------------- table playback
def plan_presentinput(queue, Y, t, signals, dt, pres_t=None, tag=None):
    """``Y[k] = signals[k][row]`` with the row picked by the float32 step counter
    ``t[k]``: ``step % rows``, or ``int((step - 0.5) * (dt / pres_t)) % rows``."""
    N = len(Y)
    assert len(Y) == len(t) == len(signals)
    pres = None if pres_t is None else _host(pres_t).astype(np.float32).reshape(-1)
    assert pres is None or pres.shape == (N,)
    for arr in [Y, t, signals]:
        assert (arr.stride1s == 1).all()
    assert (Y.shape1s == 1).all()
    assert (Y.stride0s == 1).all()
    assert (t.shape0s == 1).all()
    assert (t.shape1s == 1).all()
    assert (Y.shape0s == signals.shape1s).all()
    assert (signals.stride0s == signals.shape1s).all()
    _check(("Y", Y), ("t", t), ("signals", signals))

    table, n = _dev_table(queue, [
        Y.starts, Y.shape0s, t.starts, signals.starts, signals.shape0s,
        np.zeros(N, np.int32) if pres is None else _bits(pres),
        np.full(N, 0 if pres is None else 1, dtype=np.int32)], 8)
    widest = int(Y.shape0s.max()) if N else 1
    lanes = lanes_for(widest)  # an input signal is one row
    plan = Plan(queue, queue.lib.nhip_presentinput,
                (table.ptr, n, lanes, float(np.float32(dt)), Y.ptr, t.ptr, signals.ptr),
                gsize=_gsize(n, lanes), lsize=(WG,),
                full_args=(table, Y.dev_buf, t.dev_buf, signals.dev_buf),
                name="hip_presentinput", tag=tag)
    plan.row_iterations = -(-widest // lanes)
    plan.description = _description(Y)
    return plan


# ---------------------------------------------------------------- learning rules
RULE_BCM, RULE_OJA, RULE_VOJA = 1, 2, 3


def _plan_rule(queue, rule, name, pre, post, aux, delta, alpha, beta=None, learn=None,
               scale=None, inc=False, flops_per_element=4, tag=None):
    N = len(pre)
    alpha = _host(alpha).astype(np.float32).reshape(-1)
    beta = np.zeros(N, dtype=np.float32) if beta is None else _host(beta).astype(
        np.float32).reshape(-1)
    assert alpha.size == N and beta.size == N
    operands = [("pre", pre), ("post", post), ("aux", aux), ("delta", delta)]
    if rule == RULE_VOJA:
        operands += [("learn", learn), ("scale", scale)]
    _check(*operands)

    inds, offsets, counts = blockify(delta.sizes)
    zeros = np.zeros(len(inds), dtype=np.int32)
    table, n = _dev_table(queue, [
        pre.starts[inds], pre.stride0s[inds], post.starts[inds], post.stride0s[inds],
        aux.starts[inds], aux.stride0s[inds], delta.starts[inds], delta.stride0s[inds],
        delta.shape1s[inds], offsets, counts, _bits(alpha[inds]),
        _bits(beta[inds]),
        learn.starts[inds] if learn is not None else zeros,
        scale.starts[inds] if scale is not None else zeros,
        scale.stride0s[inds] if scale is not None else zeros], 16)
    args = (rule, int(bool(inc)), table.ptr, n, pre.ptr, post.ptr, aux.ptr, delta.ptr,
            learn.ptr if learn is not None else None, scale.ptr if scale is not None else None)
    keep = [table, pre.dev_buf, post.dev_buf, aux.dev_buf, delta.dev_buf]
    keep += [ra.dev_buf for ra in (learn, scale) if ra is not None]
    plan = Plan(queue, queue.lib.nhip_learning_rule, args, gsize=(WG * max(n, 1),), lsize=(WG,),
                full_args=tuple(keep), name=name, tag=tag)
    plan.flops_per_call = flops_per_element * int(delta.sizes.sum())
    plan.bw_per_call = (sum(ra.nbytes for _, ra in operands) + alpha.nbytes
                        + (beta.nbytes if rule == RULE_OJA else 0) + (delta.nbytes if inc else 0))
    plan.description = _description(delta)
    return plan


def plan_bcm(queue, pre, post, theta, delta, alpha, inc=False, tag=None):
    """``delta = alpha * post * (post - theta) (outer) pre`` per connection
    (reference ``plan_bcm`` :2082-2169).  ``inc`` (here and for the two rules below, not
    in the reference): add the change to ``delta`` -- which may then be the learned
    matrix itself -- instead of storing it."""
    assert len(pre) == len(post) == len(theta) == len(delta) == np.size(_host(alpha))
    for arr in (pre, post, theta):  # vectors
        assert (arr.shape1s == 1).all()
    assert (delta.stride1s == 1).all()
    assert (post.shape0s == delta.shape0s).all()
    assert (pre.shape0s == delta.shape1s).all()
    assert (post.shape0s == theta.shape0s).all()
    assert pre.ctype == post.ctype == theta.ctype == delta.ctype == "float"
    return _plan_rule(queue, RULE_BCM, "hip_bcm", pre, post, theta, delta, alpha, inc=inc,
                      flops_per_element=4, tag=tag)


def plan_oja(queue, pre, post, weights, delta, alpha, beta, inc=False, tag=None):
    """``delta = alpha * post * (pre - beta * weights * post)`` per connection
    (reference ``plan_oja`` :2172-2277)."""
    assert (len(pre) == len(post) == len(weights) == len(delta) == np.size(_host(alpha))
            == np.size(_host(beta)))
    for arr in (pre, post):  # vectors
        assert (arr.shape1s == 1).all()
    for arr in (delta, weights):  # matrices
        assert (arr.stride1s == 1).all()
    assert (post.shape0s == weights.shape0s).all()
    assert (pre.shape0s == weights.shape1s).all()
    assert (weights.shape0s == delta.shape0s).all()
    assert (weights.shape1s == delta.shape1s).all()
    assert pre.ctype == post.ctype == weights.ctype == delta.ctype == "float"
    return _plan_rule(queue, RULE_OJA, "hip_oja", pre, post, weights, delta, alpha, beta=beta,
                      inc=inc, flops_per_element=6, tag=tag)


def plan_voja(queue, pre, post, enc, delta, learn, scale, alpha, inc=False, tag=None):
    """``delta = alpha * learn * post * (scale * pre - enc)`` per connection
    (reference ``plan_voja`` :2280-2405)."""
    assert (len(pre) == len(post) == len(enc) == len(delta) == len(learn)
            == np.size(_host(alpha)) == len(scale))
    assert (learn.shape0s == 1).all() and (learn.shape1s == 1).all()
    for arr in (pre, post, scale):  # vectors
        assert (arr.shape1s == 1).all()
    for arr in (enc, delta):  # matrices
        assert (arr.stride1s == 1).all()
    assert (post.shape0s == enc.shape0s).all()
    assert (pre.shape0s == enc.shape1s).all()
    assert (enc.shape0s == delta.shape0s).all()
    assert (enc.shape1s == delta.shape1s).all()
    assert (scale.shape0s == enc.shape0s).all()
    assert (pre.ctype == post.ctype == enc.ctype == delta.ctype == learn.ctype
            == scale.ctype == "float")
    return _plan_rule(queue, RULE_VOJA, "hip_voja", pre, post, enc, delta, alpha, learn=learn,
                      scale=scale, inc=inc, flops_per_element=5, tag=tag)


# ---------------------------------------------------------------- convolution, pooling
def _single_contiguous(ra, what):
    """(start, size) of a one-item ragged view whose item is one contiguous run."""
    assert len(ra) == 1, "%s: one signal expected" % what
    m, n = int(ra.shape0s[0]), int(ra.shape1s[0])
    assert ra.stride1s[0] == 1 or n == 1, "%s: not contiguous" % what
    assert ra.stride0s[0] == n or m == 1, "%s: not contiguous" % what
    return int(ra.starts[0]), m * n


def conv2d_tiles(shape_out_ijf, kernel_shape, strides, nc, channels_last):
    """Output tile (rows, columns, filters) of one work-group and the number of input
    channels staged in LDS at a time."""
    nyi, nyj, nf = shape_out_ijf
    si, sj = kernel_shape
    sti, stj = strides
    tile_f = 1
    if channels_last:  # filters run fastest over the lanes: take up to a wave of them
        while tile_f < min(nf, 64):
            tile_f *= 2
    tile_j = 1
    while tile_j * 2 * tile_f <= WG and tile_j < nyj:
        tile_j *= 2
    tile_j = min(tile_j, 32)
    tile_i = max(1, min(WG // (tile_j * tile_f), nyi))
    # LDS words per staged channel: the input patch and the taps of the group's filters
    per_channel = ((tile_i - 1) * sti + si) * ((tile_j - 1) * stj + sj) + si * sj * tile_f
    c_chunk = max(1, min(nc, (32 * 1024 // 4) // per_channel))
    assert (per_channel + si * sj) * 4 <= 60 * 1024, "convolution window too large for LDS"
    return tile_i, tile_j, tile_f, c_chunk


def plan_conv2d(queue, X, Y, filters, shape_in, shape_out, kernel_shape, conv=True, biases=None,
                padding=(0, 0), strides=(1, 1), channels_last=True, tag=None, transposed=False):
    """``Y = conv2d(X, filters)`` (``conv``) or local filtering of one image signal;
    X, Y and filters are one-item views (reference ``plan_conv2d`` :1762-1969).

    filters: ``(size_i, size_j, channels, n_filters)``; for local filtering
    ``(n_filters, channels, size_i, size_j, out_i, out_j)``."""
    assert biases is None, "Not tested with biases (strides may be wrong)"
    si, sj = (int(v) for v in kernel_shape)
    sti, stj = (int(v) for v in strides)
    if channels_last:
        nxi, nxj, nc = (int(v) for v in shape_in)
        nyi, nyj, nf = (int(v) for v in shape_out)
    else:
        nc, nxi, nxj = (int(v) for v in shape_in)
        nf, nyi, nyj = (int(v) for v in shape_out)
    if padding == "valid":
        pi, pj = 0, 0
    elif padding == "same":
        pi, pj = (si - 1) // 2, (sj - 1) // 2
    elif isinstance(padding, (tuple, list)) and len(padding) == 2:
        pi, pj = (int(v) for v in padding)
    else:
        raise ValueError("Unsupported padding (must be 'same', 'valid', or 2-tuple)")
    for ra in (X, Y, filters):
        assert ra.ctype == "float"
    _check(("X", X), ("Y", Y), ("filters", filters))
    x_start, x_size = _single_contiguous(X, "X")
    y_start, y_size = _single_contiguous(Y, "Y")
    f_start, f_size = _single_contiguous(filters, "filters")
    assert x_size == nxi * nxj * nc, "X does not have shape_in's size"
    assert y_size == nyi * nyj * nf, "Y does not have shape_out's size"
    assert f_size == si * sj * nc * nf * (1 if conv else nyi * nyj), "filters have the wrong size"
    # every output pixel's window must start inside the padded image
    assert (nyi - 1) * sti - pi < nxi and (nyj - 1) * stj - pj < nxj

    tile_i, tile_j, tile_f, c_chunk = conv2d_tiles((nyi, nyj, nf), (si, sj), (sti, stj), nc,
                                                   channels_last)
    geom = np.array([nxi, nxj, nc, nyi, nyj, nf, si, sj, sti, stj, pi, pj, x_start, y_start,
                     f_start, int(bool(channels_last)), int(not conv), tile_i, tile_j, tile_f,
                     c_chunk], dtype=np.int32)
    n_groups = (-(-nyi // tile_i)) * (-(-nyj // tile_j)) * (-(-nf // tile_f))
    plan = Plan(queue, queue.lib.nhip_conv2d, (geom.ctypes.data, X.ptr, filters.ptr, Y.ptr),
                gsize=(WG * n_groups,), lsize=(WG,),
                full_args=(geom, X.dev_buf, filters.dev_buf, Y.dev_buf), name="hip_conv2d", tag=tag)
    plan.flops_per_call = 2 * nyi * nyj * nf * nc * si * sj
    plan.bw_per_call = 4 * (x_size + f_size + y_size)
    plan.description = "shape_in=%s, shape_out=%s, kernel=%s, conv=%s" % (
        tuple(shape_in), tuple(shape_out), tuple(kernel_shape), conv)
    return plan


def plan_pool2d(queue, X, Y, shape, pool_size, strides, tag=None):
    """Average pooling of a channels-first image; ``shape = (channels, out_i, out_j,
    in_i, in_j)`` (reference ``plan_pool2d`` :1972-2079)."""
    nc, nyi, nyj, nxi, nxj = (int(v) for v in shape)
    si, sj = (int(v) for v in pool_size)
    sti, stj = (int(v) for v in strides)
    assert X.ctype == Y.ctype == "float"
    _check(("X", X), ("Y", Y))
    x_start, x_size = _single_contiguous(X, "X")
    y_start, y_size = _single_contiguous(Y, "Y")
    assert x_size == nc * nxi * nxj and y_size == nc * nyi * nyj
    geom = np.array([nc, nyi, nyj, nxi, nxj, si, sj, sti, stj, x_start, y_start], dtype=np.int32)
    n_groups = -(-(nc * nyi * nyj) // WG)
    plan = Plan(queue, queue.lib.nhip_pool2d, (geom.ctypes.data, X.ptr, Y.ptr),
                gsize=(WG * n_groups,), lsize=(WG,), full_args=(geom, X.dev_buf, Y.dev_buf),
                name="hip_pool2d", tag=tag)
    plan.flops_per_call = x_size
    plan.bw_per_call = 4 * (x_size + y_size)
    return plan


# ---------------------------------------------------------------- white noise
DIST_UNIFORM, DIST_GAUSSIAN = 0, 1


def plan_whitenoise(queue, Y, dist_enums, dist_params, scale, inc, dt, seeds, tag=None):
    """``Y[k] (=|+=) samples of distribution k``, scaled by ``1/sqrt(dt)`` where
    ``scale[k]`` (reference ``plan_whitenoise`` :1578-1675).

    ``dist_enums[k]`` is 0 (uniform; params low, high) or 1 (Gaussian; params mean,
    std) and ``seeds[k]`` the seed of process k (the reference takes a ragged array
    of generator states made by ``create_rngs`` / ``init_rngs`` in this place).  The
    plan owns one call counter per process; ``plan.reset_streams()`` zeroes them,
    which restarts every stream from its first sample."""
    N = len(Y)
    enums = np.asarray(_host(dist_enums), dtype=np.int32).reshape(-1)
    params = np.asarray(_host(dist_params), dtype=np.float32).reshape(N, 2)
    scale = np.asarray(_host(scale)).astype(bool).reshape(-1)
    inc = np.asarray(_host(inc)).astype(bool).reshape(-1)
    seeds = np.asarray(seeds, dtype=np.int64).reshape(-1)
    assert N == enums.size == scale.size == inc.size == seeds.size
    assert np.isin(enums, (DIST_UNIFORM, DIST_GAUSSIAN)).all()
    assert (Y.shape1s == 1).all() and (Y.stride0s == 1).all() and (Y.stride1s == 1).all()
    assert Y.ctype == "float"
    _check(("Y", Y))
    inds, offsets, counts = blockify(Y.shape0s, 4 * BLOCK)  # blocks start at multiples of 4
    flags = scale.astype(np.int32) | (inc.astype(np.int32) << 1)
    table, n = _dev_table(queue, [
        Y.starts[inds], counts, enums[inds], _bits(params[inds, 0]), _bits(params[inds, 1]),
        flags[inds], (seeds & 0xFFFFFFFF).astype(np.uint32).view(np.int32)[inds], offsets], 8)
    counters = to_device(queue, np.zeros(max(n, 1), dtype=np.int32))  # one per block
    plan = Plan(queue, queue.lib.nhip_whitenoise,
                (table.ptr, n, counters.ptr, 1.0 / np.sqrt(dt), Y.ptr),
                gsize=(WG * max(n, 1),), lsize=(WG,), full_args=(table, counters, Y.dev_buf),
                name="hip_whitenoise", tag=tag)
    plan.counters = counters
    plan.reset_streams = lambda: counters.fill(0)
    plan.bw_per_call = Y.nbytes
    plan.description = _description(Y)
    return plan
