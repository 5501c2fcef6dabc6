"""Python face of the CPU oracle (``oracle_kernels.c``).  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg
may import this module; it is the checker, never the thing shipped or measured.

It offers the reference's ``plan_*`` call signatures
(nengo_ocl/clra_gemv.py:1178-1195, nengo_ocl/clra_nonlinearities.py:113-1197,
1678-1759) over HOST ragged arrays: ``queue`` is ignored (pass ``None``), every
ragged argument is a ``RaggedArray`` whose ``buf`` is updated in place, and the
returned object is a host-callback plan (``plan()`` runs the step once).
Ragged metadata is handed to C exactly as the reference hands it to OpenCL
(starts / shapes / strides per item), independent of the HIP work lists.
"""

import ctypes
import os
import subprocess

import numpy as np

from nengo_ocl_amd.plan import PythonPlan
from nengo_ocl_amd.raggedarray import RaggedArray

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile oracle_kernels.c with gcc (OpenMP, no contraction, no fast-math)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + res.stdout + res.stderr)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _per_item(arg, n, dtype):
    v = np.asarray(arg, dtype=dtype)
    if v.ndim == 0:
        v = np.full(n, v, dtype=dtype)
    assert v.shape == (n,)
    return np.ascontiguousarray(v)


def _param_per_item(p, n):
    """tau/ref/amp: a number, or a ragged array constant within each item."""
    if isinstance(p, RaggedArray):
        vals = np.array([p[i].flat[0] for i in range(n)], dtype=np.float32)
        for i in range(n):
            assert np.all(p[i] == vals[i]), "the oracle takes one parameter value per item"
        return vals
    return _per_item(p, n, np.float32)


def _plan(fn, name, keep, tag=None):
    plan = PythonPlan(fn, name=name, tag=tag)
    plan.keep = keep  # arrays whose memory the bound C call reads
    return plan


# --------------------------------------------------------------------- GEMV
def _gemv_coefficient(arg, n):
    """alpha / beta / gamma per item as the doubles the reference's kernels compute with
    (clra_gemv.py:17-32 `float_cl_clra`): a Python float, or a list whose values are all
    equal, is written into the kernel text as a double literal; values that differ from
    item to item become a float32 device array."""
    v = np.asarray(arg, dtype=np.float64)
    if v.ndim == 0 or len(set(v.ravel().tolist())) == 1:
        return _per_item(v if v.ndim == 0 else v.ravel()[0], n, np.float64)
    return _per_item(np.asarray(arg, dtype=np.float32), n, np.float64)


class plan_block_gemv:
    """``Y = beta*Y_in + gamma + alpha * sum_j A[A_js[j]] @ X[X_js[j]]`` in the
    block order of clra_gemv.py:861-1175 (32x128 tiles, 4 strided partial sums)."""

    def __init__(self, queue, alpha, A, A_js, X, X_js, beta, Y, Y_in=None, gamma=0.0, tag=None):
        Y_in = Y if Y_in is None else Y_in
        n = len(Y)
        dot_ptr = [0]
        a_idx, x_idx = [], []
        for b in range(n):
            aj = np.asarray(A_js[b]).ravel().tolist()
            xj = np.asarray(X_js[b]).ravel().tolist()
            assert len(aj) == len(xj)
            for a, x in zip(aj, xj):
                assert A.shape0s[a] == Y.shape0s[b]
                assert A.shape1s[a] == X.shape0s[x] and X.shape1s[x] == 1
                assert A.stride1s[a] == 1 or A.shape1s[a] == 1
            a_idx += aj
            x_idx += xj
            dot_ptr.append(len(a_idx))
        a_idx = np.asarray(a_idx, dtype=np.int64)
        x_idx = np.asarray(x_idx, dtype=np.int64)
        args = [
            _i32(Y.starts), _i32(Y.stride0s), _i32(Y.shape0s), _i32(Y_in.starts),
            _i32(Y_in.stride0s), _i32(dot_ptr), _i32(A.starts[a_idx]), _i32(A.stride0s[a_idx]),
            _i32(A.shape1s[a_idx]), _i32(X.starts[x_idx]), _i32(X.stride0s[x_idx]),
            _gemv_coefficient(alpha, n), _gemv_coefficient(beta, n), _gemv_coefficient(gamma, n),
        ]
        fn = lib().orc_gemv_block

        def step():
            fn(ctypes.c_int(n), *[_p(a) for a in args], _p(A.buf), _p(X.buf), _p(Y_in.buf),
               _p(Y.buf))

        self.plans = [_plan(step, "oracle_gemv_block", args, tag)]


plan_ragged_gather_gemv = plan_block_gemv


# ------------------------------------------------------------------ neurons
def plan_lif(queue, dt, J, V, W, outS, ref, tau, amp, N=None, tau_n=None, inc_n=None,
             upsample=1, tag=None, **kwargs):
    assert not kwargs.get("fastlif")
    n = len(J)
    if N is not None:
        args = [_i32(J.shape0s), _i32(J.starts), _i32(V.starts), _i32(W.starts),
                _i32(outS.starts), _i32(N.starts), _param_per_item(tau, n),
                _param_per_item(ref, n), _param_per_item(amp, n), _param_per_item(tau_n, n),
                _param_per_item(inc_n, n)]
        fn = lib().orc_alif

        def step():
            fn(ctypes.c_int(n), *[_p(a) for a in args], ctypes.c_double(dt),
               ctypes.c_int(upsample), _p(J.buf), _p(V.buf), _p(W.buf), _p(outS.buf), _p(N.buf))

        return _plan(step, "oracle_alif", args, tag)
    args = [_i32(J.shape0s), _i32(J.starts), _i32(V.starts), _i32(W.starts), _i32(outS.starts),
            _param_per_item(tau, n), _param_per_item(ref, n), _param_per_item(amp, n)]
    fn = lib().orc_lif

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], ctypes.c_double(dt), ctypes.c_int(upsample),
           _p(J.buf), _p(V.buf), _p(W.buf), _p(outS.buf))

    return _plan(step, "oracle_lif", args, tag)


def plan_lif_rate(queue, dt, J, R, ref, tau, amp, N=None, tau_n=None, inc_n=None, tag=None,
                  **kwargs):
    n = len(J)
    if N is not None:
        args = [_i32(J.shape0s), _i32(J.starts), _i32(R.starts), _i32(N.starts),
                _param_per_item(tau, n), _param_per_item(ref, n), _param_per_item(amp, n),
                _param_per_item(tau_n, n), _param_per_item(inc_n, n)]
        fn = lib().orc_alif_rate

        def step():
            fn(ctypes.c_int(n), *[_p(a) for a in args], ctypes.c_double(dt), _p(J.buf), _p(R.buf),
               _p(N.buf))

        return _plan(step, "oracle_alif_rate", args, tag)
    args = [_i32(J.shape0s), _i32(J.starts), _i32(R.starts), _param_per_item(tau, n),
            _param_per_item(ref, n), _param_per_item(amp, n)]
    fn = lib().orc_lif_rate

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(J.buf), _p(R.buf))

    return _plan(step, "oracle_lif_rate", args, tag)


def _plan_simple_neurons(kind, name, dt, J, out, param, V=None, tag=None):
    n = len(J)
    args = [_i32(J.shape0s), _i32(J.starts), _i32(out.starts),
            _i32(V.starts if V is not None else np.zeros(n)), _param_per_item(param, n)]
    fn = lib().orc_simple_neurons
    vbuf = V.buf if V is not None else out.buf

    def step():
        fn(ctypes.c_int(kind), ctypes.c_int(n), *[_p(a) for a in args], ctypes.c_double(dt),
           _p(J.buf), _p(out.buf), _p(vbuf))

    return _plan(step, name, args, tag)


def plan_rectified_linear(queue, J, R, amp, tag=None, **kwargs):
    return _plan_simple_neurons(0, "oracle_relu", 1.0, J, R, amp, tag=tag)


def plan_spiking_rectified_linear(queue, dt, J, V, outS, amp, tag=None, **kwargs):
    return _plan_simple_neurons(1, "oracle_spikingrelu", dt, J, outS, amp, V=V, tag=tag)


def plan_sigmoid(queue, J, R, ref, tag=None, **kwargs):
    return _plan_simple_neurons(2, "oracle_sigmoid", 1.0, J, R, ref, tag=tag)


# ------------------------------------------------------------------ sparse
class plan_sparse_dot_inc:
    """``Y[b] (=|+=) A[b] @ X[b]`` from CSR, rows summed in column order
    (clra_gemv.py `spmv_csr_impl` :1570-1646)."""

    def __init__(self, queue, hA, X, Y, inc=False, tag=None, algorithm=None):
        import scipy.sparse

        mats = list(hA) if isinstance(hA, (list, tuple)) else [hA]
        csrs = []
        for m in mats:
            c = scipy.sparse.csr_matrix(m.csr if hasattr(m, "csr") else m)
            c.sort_indices()
            csrs.append(c)
        n = len(csrs)
        assert n == len(X) == len(Y)
        starts = np.cumsum([0] + [c.nnz for c in csrs])
        # each item's row pointers index the concatenated data: shift them by its offset
        indptr = np.concatenate([np.asarray(c.indptr, dtype=np.int64) + s
                                 for c, s in zip(csrs, starts)]).astype(np.int32)
        ptr_starts = np.cumsum([0] + [c.shape[0] + 1 for c in csrs])[:-1]
        args = [_i32([c.shape[0] for c in csrs]), _i32(ptr_starts), _i32(X.starts), _i32(Y.starts),
                _i32(np.broadcast_to(np.asarray(inc, dtype=np.int32), (n,))), indptr,
                _i32(np.concatenate([c.indices for c in csrs]) if n else []),
                np.ascontiguousarray(np.concatenate([c.data for c in csrs]) if n else [],
                                     dtype=np.float32)]
        fn = lib().orc_spmv_csr

        def step():
            fn(ctypes.c_int(n), *[_p(a) for a in args], _p(X.buf), _p(Y.buf))

        self.plans = [_plan(step, "oracle_spmv", args, tag)]


# ----------------------------------------------------------------- synapses
def plan_linearfilter(queue, X, Y, A, B, Xbuf, Ybuf, tag=None):
    n = len(X)
    xpos = np.zeros(n, dtype=np.int32)
    ypos = np.zeros(n, dtype=np.int32)
    args = [_i32(X.shape0s), _i32(X.shape1s), _i32(X.starts), _i32(X.stride0s), _i32(X.stride1s),
            _i32(Y.starts), _i32(Y.stride0s), _i32(Y.stride1s), _i32(A.shape0s), _i32(A.starts),
            _i32(B.shape0s), _i32(B.starts), _i32(Xbuf.starts), _i32(Ybuf.starts), xpos, ypos]
    fn = lib().orc_linearfilter

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(X.buf), _p(Y.buf), _p(A.buf), _p(B.buf),
           _p(Xbuf.buf), _p(Ybuf.buf))

    plan = _plan(step, "oracle_linearfilter", args, tag)
    plan.bufpos = (xpos, ypos)
    return [plan]


# -------------------------------------------------------------- elementwise
def plan_elementwise_inc(queue, A, X, Y, alpha=None, outer=False, inc=True, tag=None):
    n = len(Y)
    alphas = _per_item(1.0 if alpha is None else alpha, n, np.float32)
    args = [alphas, _i32(A.starts), _i32(A.shape0s), _i32(A.shape1s), _i32(A.stride0s),
            _i32(X.starts), _i32(X.shape0s), _i32(X.shape1s), _i32(X.stride0s),
            _i32(Y.starts), _i32(Y.shape0s), _i32(Y.shape1s), _i32(Y.stride0s)]
    fn = lib().orc_elementwise_inc

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], ctypes.c_int(bool(outer)),
           ctypes.c_int(bool(inc)), _p(A.buf), _p(X.buf), _p(Y.buf))

    return _plan(step, "oracle_elementwise_inc", args, tag)


def plan_copy(queue, X, Y, incs, tag=None):
    n = len(X)
    args = [_i32(X.shape0s), _i32(X.shape1s), _i32(X.starts), _i32(X.stride0s), _i32(Y.starts),
            _i32(Y.stride0s), _i32(incs)]
    fn = lib().orc_copy

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(X.buf), _p(Y.buf))

    return _plan(step, "oracle_copy", args, tag)


def plan_slicedcopy(queue, X, Y, Xinds, Yinds, incs, tag=None):
    n = len(X)
    args = [_i32(X.starts), _i32(X.stride0s), _i32(Y.starts), _i32(Y.stride0s),
            _i32(Xinds.shape0s), _i32(Xinds.starts), _i32(Yinds.starts), _i32(incs)]
    fn = lib().orc_slicedcopy

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(X.buf), _p(Y.buf), _p(Xinds.buf),
           _p(Yinds.buf))

    return _plan(step, "oracle_slicedcopy", args, tag)


def plan_reset(queue, Y, values, tag=None):
    n = len(Y)
    args = [_i32(Y.starts), _i32(Y.sizes), _f32(values)]
    fn = lib().orc_reset

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(Y.buf))

    return _plan(step, "oracle_reset", args, tag)


def plan_timeupdate(queue, step, time, dt):
    fn = lib().orc_timeupdate
    isz = 4

    def run():
        fn(ctypes.c_void_p(step.buf.ctypes.data + isz * int(step.starts[0])),
           ctypes.c_void_p(time.buf.ctypes.data + isz * int(time.starts[0])),
           ctypes.c_double(dt))

    return _plan(run, "oracle_timeupdate", [])


# --------------------------------------------------------- inputs / outputs
def plan_presentinput(queue, Y, t, signals, dt, pres_t=None, tag=None):
    n = len(Y)
    pres = None if pres_t is None else _f32(pres_t)
    args = [_i32(Y.starts), _i32(Y.shape0s), _i32(t.starts), _i32(signals.starts),
            _i32(signals.shape0s)]
    fn = lib().orc_presentinput

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(pres), ctypes.c_float(dt), _p(Y.buf),
           _p(t.buf), _p(signals.buf))

    return _plan(step, "oracle_presentinput", args + [pres], tag)


UNARY_OPCODES = {"identity": 0, "sin": 1, "cos": 2, "tanh": 3, "exp": 4, "square": 5}


def plan_direct_unary(queue, fn_name, x, output, tag=None):
    """y[0] = f(x[0]) per item for a named function of the unary table."""
    n = len(output)
    args = [_i32(x.starts), _i32(output.starts)]
    fn = lib().orc_direct_unary
    opcode = UNARY_OPCODES[fn_name]

    def step():
        fn(ctypes.c_int(opcode), ctypes.c_int(n), *[_p(a) for a in args], _p(x.buf),
           _p(output.buf))

    return _plan(step, "oracle_direct", args, tag)


def plan_probes(queue, periods, X, Y, tag=None):
    n = len(X)
    periods = _f32(periods)
    countdowns = periods - np.float32(1)
    bufpositions = np.zeros(n, dtype=np.int32)
    args = [countdowns, bufpositions, periods, _i32(X.starts), _i32(X.shape0s), _i32(X.shape1s),
            _i32(X.stride0s), _i32(X.stride1s), _i32(Y.starts)]
    fn = lib().orc_probes

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(X.buf), _p(Y.buf))

    plan = _plan(step, "oracle_probes", args, tag)
    plan.bufpositions = bufpositions
    plan.countdowns = countdowns
    plan.periods = periods
    plan.Y = Y
    return plan


# ------------------------------------------------- learning rules, convolution, noise
def _plan_rule(rule, name, pre, post, aux, delta, alpha, beta=None, learn=None, scale=None,
               inc=False, tag=None):
    n = len(pre)
    alphas = _per_item(alpha, n, np.float32)
    betas = _per_item(0.0 if beta is None else beta, n, np.float32)
    zeros = np.zeros(n, dtype=np.int32)
    args = [_i32(delta.shape0s), _i32(delta.shape1s), _i32(pre.starts), _i32(pre.stride0s),
            _i32(post.starts), _i32(post.stride0s), _i32(aux.starts), _i32(aux.stride0s),
            _i32(delta.starts), _i32(delta.stride0s), alphas, betas,
            zeros if learn is None else _i32(learn.starts),
            zeros if scale is None else _i32(scale.starts),
            zeros if scale is None else _i32(scale.stride0s)]
    fn = lib().orc_learning_rule

    def step():
        fn(ctypes.c_int(rule), ctypes.c_int(bool(inc)), ctypes.c_int(n), *[_p(a) for a in args],
           _p(pre.buf), _p(post.buf),
           _p(aux.buf), _p(delta.buf), None if learn is None else _p(learn.buf),
           None if scale is None else _p(scale.buf))

    return _plan(step, name, args, tag)


def plan_bcm(queue, pre, post, theta, delta, alpha, inc=False, tag=None):
    return _plan_rule(1, "oracle_bcm", pre, post, theta, delta, alpha, inc=inc, tag=tag)


def plan_oja(queue, pre, post, weights, delta, alpha, beta, inc=False, tag=None):
    return _plan_rule(2, "oracle_oja", pre, post, weights, delta, alpha, beta=beta, inc=inc,
                      tag=tag)


def plan_voja(queue, pre, post, enc, delta, learn, scale, alpha, inc=False, tag=None):
    return _plan_rule(3, "oracle_voja", pre, post, enc, delta, alpha, learn=learn, scale=scale,
                      inc=inc, tag=tag)


def plan_conv2d(queue, X, Y, filters, shape_in, shape_out, kernel_shape, conv=True, biases=None,
                padding=(0, 0), strides=(1, 1), channels_last=True, tag=None, transposed=False):
    assert biases is None
    si, sj = kernel_shape
    if channels_last:
        nxi, nxj, nc = shape_in
        nyi, nyj, nf = shape_out
    else:
        nc, nxi, nxj = shape_in
        nf, nyi, nyj = shape_out
    if padding == "valid":
        pi, pj = 0, 0
    elif padding == "same":
        pi, pj = (si - 1) // 2, (sj - 1) // 2
    else:
        pi, pj = padding
    geom = _i32([nxi, nxj, nc, nyi, nyj, nf, si, sj, strides[0], strides[1], pi, pj,
                 X.starts[0], Y.starts[0], filters.starts[0], bool(channels_last), not conv])
    fn = lib().orc_conv2d

    def step():
        fn(_p(geom), _p(X.buf), _p(filters.buf), _p(Y.buf))

    return _plan(step, "oracle_conv2d", [geom], tag)


def plan_pool2d(queue, X, Y, shape, pool_size, strides, tag=None):
    geom = _i32(list(shape) + list(pool_size) + list(strides) + [X.starts[0], Y.starts[0]])
    fn = lib().orc_pool2d

    def step():
        fn(_p(geom), _p(X.buf), _p(Y.buf))

    return _plan(step, "oracle_pool2d", [geom], tag)


def philox4x32(counters_keys):
    """Philox4x32-10 of ``(n, 6)`` uint32 rows (counter words 0-3, key words 0-1)."""
    rows = np.ascontiguousarray(counters_keys, dtype=np.uint32).reshape(-1, 6)
    out = np.zeros((len(rows), 4), dtype=np.uint32)
    lib().orc_philox4x32(_p(rows), _p(out), ctypes.c_int(len(rows)))
    return out


def plan_whitenoise(queue, Y, dist_enums, dist_params, scale, inc, dt, seeds, tag=None):
    n = len(Y)
    params = np.asarray(dist_params, dtype=np.float32).reshape(n, 2)
    args = [_i32(Y.starts), _i32(Y.shape0s), _i32(np.asarray(dist_enums).reshape(-1)),
            _f32(params[:, 0]), _f32(params[:, 1]), _i32(np.asarray(scale).astype(bool)),
            _i32(np.asarray(inc).astype(bool)),
            np.ascontiguousarray(np.asarray(seeds, dtype=np.int64) & 0xFFFFFFFF, dtype=np.uint32)]
    counters = np.zeros(max(n, 1), dtype=np.int32)
    fn = lib().orc_whitenoise

    def step():
        fn(ctypes.c_int(n), *[_p(a) for a in args], _p(counters),
           ctypes.c_double(1.0 / np.sqrt(dt)), _p(Y.buf))

    plan = _plan(step, "oracle_whitenoise", args, tag)
    plan.counters = counters
    plan.reset_streams = lambda: counters.fill(0)
    return plan
