"""Sparse matrix-vector products: host side of ``nhip_spmv_sell``.

Counterpart of the reference's ``plan_sparse_dot_inc`` (clra_gemv.py:1919-1948) and
its ``spmv_prog`` family (:1249-1567), which keep every matrix in CSR or ELLPACK on
the device and launch one kernel per matrix.  Here any number of matrices share one
launch: their rows are cut into slices of 64 (the wave width) and stored slice by
slice, four consecutive elements of every row of a slice side by side, so that a lane
reads values and column indices 16 bytes at a time, a wave in contiguous 1-KiB runs,
while each lane sums its row in column order.
"""

import os

import numpy as np

from .hipraggedarray import to_device
from .plan import Plan

WG, WAVE = 256, 64
QUAD = 4  # elements of a row stored side by side (one 16-byte access)
WINDOW = 1024  # consecutive elements of X a wave can keep in LDS (SPMV_WINDOW in csrc/spmv.hip)
SKIP_MAX_COLS = 32 * 36864  # longest X whose "is not zero" bits fit the LDS (SPMV_MASK_WORDS)


def slice_window(columns, n_cols, x_start):
    """First element of the run of `WINDOW` consecutive elements of X that a wave keeps
    in LDS for a slice with the given column indices, or -1 for none: the run is centred
    on the median column, starts on a multiple of 4 (16-byte reads; X itself must start
    on one) and lies inside X; it is used when it holds at least a quarter of the indices."""
    if columns.size == 0 or n_cols < WINDOW or x_start % QUAD:
        return -1
    lo = int(np.median(columns)) - WINDOW // 2
    lo = max(0, min(lo, n_cols - WINDOW)) // QUAD * QUAD
    inside = np.count_nonzero((columns >= lo) & (columns < lo + WINDOW))
    return lo if 4 * inside >= columns.size else -1


def sell_index(data_start, r, j):
    """Position in ``cols`` / ``vals`` of element ``j`` of row ``r`` of the slice that
    starts at ``data_start`` (``j`` may be an array)."""
    j = np.asarray(j)
    return data_start + WAVE * QUAD * (j // QUAD) + QUAD * r + j % QUAD


class HostSparseMatrix:
    """A sparse matrix on the host in CSR form (reference clra_gemv.py:1242-1247)."""

    def __init__(self, matrix):
        import scipy.sparse

        csr = matrix.csr if hasattr(matrix, "csr") else matrix
        self.csr = scipy.sparse.csr_matrix(csr)
        self.csr.sort_indices()
        self.shape = self.csr.shape


def sell_layout(matrices):
    """Sliced-ELLPACK arrays of a list of CSR matrices.

    Returns ``(slice_rows, row_len, cols, vals)``: ``slice_rows[k] = (item, data_start,
    width, len_start, n_rows, row0)``; ``width`` is the longest row of the slice rounded
    up to a multiple of 4, ``row_len`` is padded to 64 per slice; ``cols`` / ``vals``
    hold element j of row r of slice k at ``data_start + 256 (j // 4) + 4 r + j % 4``
    (see `sell_index`).
    """
    slice_rows, lens, cols, vals = [], [], [], []
    data_start = 0
    for item, m in enumerate(matrices):
        csr = m.csr
        indptr = np.asarray(csr.indptr, dtype=np.int64)
        indices = np.asarray(csr.indices, dtype=np.int32)
        data = np.asarray(csr.data, dtype=np.float32)
        row_counts = np.diff(indptr).astype(np.int32)
        for row0 in range(0, csr.shape[0], WAVE):
            n_rows = min(WAVE, csr.shape[0] - row0)
            counts = row_counts[row0:row0 + n_rows]
            width = -(-(int(counts.max()) if n_rows else 0) // QUAD) * QUAD
            block_c = np.zeros((width // QUAD, WAVE, QUAD), dtype=np.int32)
            block_v = np.zeros((width // QUAD, WAVE, QUAD), dtype=np.float32)
            # scatter the slice's elements: position inside its row, row inside the slice
            lo, hi = int(indptr[row0]), int(indptr[row0 + n_rows])
            r = np.repeat(np.arange(n_rows), counts)
            j = np.arange(lo, hi) - np.repeat(indptr[row0:row0 + n_rows], counts)
            block_c[j // QUAD, r, j % QUAD] = indices[lo:hi]
            block_v[j // QUAD, r, j % QUAD] = data[lo:hi]
            padded = np.zeros(WAVE, dtype=np.int32)
            padded[:n_rows] = counts
            slice_rows.append((item, data_start, width, len(lens) * WAVE, n_rows, row0))
            lens.append(padded)
            cols.append(block_c.ravel())
            vals.append(block_v.ravel())
            data_start += width * WAVE
    cat = lambda parts, dtype: (np.concatenate(parts) if parts else np.zeros(0, dtype)).astype(dtype)
    return slice_rows, cat(lens, np.int32), cat(cols, np.int32), cat(vals, np.float32)


class plan_sparse_dot_inc:
    """``Y[b] (=|+=) A[b] @ X[b]``; ``.plans`` holds the one launch.

    ``hA`` is a `HostSparseMatrix` (with X, Y of length 1: the reference's signature,
    clra_gemv.py:1919) or a list of them with one X and one Y item each.  ``inc``
    defaults to False like the reference's (whose Simulator thereby *sets* Y); the
    Simulator here passes True, the meaning of the operator.

    ``x_mostly_zero`` (one flag, or one per matrix) says that X is zero in most places
    most of the time -- the spikes of a population.  When it holds for every matrix and all
    read the same X of at most `SKIP_MAX_COLS` elements, the launch is
    `nhip_spmv_sell_skip`: one bit per element of X ("is not +0.0") is made first and kept
    in LDS, and where it is clear the operand is the constant instead of a look-up of X.
    Same bits as the ordinary launch whatever X holds; only faster when X is mostly zero.
    """

    def __init__(self, queue, hA, X, Y, inc=False, tag=None, algorithm=None, x_mostly_zero=False):
        # `algorithm` / NENGO_OCL_SPMV_ALGORITHM name one of the reference's planners
        # (clra_gemv.py:1937-1948); an unknown name is an error as there, a known one
        # changes nothing: they all are this launch
        if algorithm is None:
            algorithm = os.environ.get("NENGO_OCL_SPMV_ALGORITHM", None)
        if algorithm is not None and algorithm not in algostr_to_planner:
            raise KeyError(algorithm)
        matrices = list(hA) if isinstance(hA, (list, tuple)) else [hA]
        matrices = [m if isinstance(m, HostSparseMatrix) else HostSparseMatrix(m) for m in matrices]
        if not (len(matrices) == len(X) == len(Y)):
            raise ValueError("need one X and one Y item per matrix")
        for arr, name in ((X, "X"), (Y, "Y")):
            arr.check_bounds(name)
            if not ((arr.shape1s == 1).all() and (arr.stride0s == 1).all()):
                raise NotImplementedError("sparse products are matrix-vector only")
        for b, m in enumerate(matrices):
            if m.shape != (int(Y.shape0s[b]), int(X.shape0s[b])):
                raise ValueError("matrix %d is %s, Y has %d and X %d elements"
                                 % (b, m.shape, Y.shape0s[b], X.shape0s[b]))
            if m.csr.nnz and (m.csr.indices.min() < 0 or m.csr.indices.max() >= m.shape[1]):
                raise ValueError("matrix %d has column indices outside X" % b)
        incs = np.broadcast_to(np.asarray(inc, dtype=np.int32), (len(matrices),))
        slice_rows, row_len, cols, vals = sell_layout(matrices)
        table = np.zeros((max(len(slice_rows), 1), 8), dtype=np.int32)
        for k, (item, data_start, width, len_start, n_rows, row0) in enumerate(slice_rows):
            csr = matrices[item].csr
            window = slice_window(csr.indices[csr.indptr[row0]:csr.indptr[row0 + n_rows]],
                                  csr.shape[1], int(X.starts[item]))
            table[k] = (data_start, width, len_start, n_rows, int(X.starts[item]),
                        int(Y.starts[item]) + row0, int(incs[item]), window)
        if vals.size >= 2 ** 31:
            raise ValueError("more than 2^31 stored elements")
        n = len(slice_rows)
        dev = [to_device(queue, a) for a in (table, row_len if row_len.size else np.zeros(1, np.int32),
                                             cols if cols.size else np.zeros(1, np.int32),
                                             vals if vals.size else np.zeros(1, np.float32))]
        args = (dev[0].ptr, n, dev[1].ptr, dev[2].ptr, dev[3].ptr, X.ptr, Y.ptr)
        n_groups = max(1, -(-n // (WG // WAVE)))
        flags = np.broadcast_to(np.asarray(x_mostly_zero, dtype=bool), (len(matrices),))
        same_x = len({(int(X.starts[b]), int(X.shape0s[b])) for b in range(len(matrices))}) == 1
        skip = n > 0 and bool(flags.all()) and same_x and int(X.shape0s[0]) <= SKIP_MAX_COLS
        if skip:
            n_cols = int(X.shape0s[0])
            mask = to_device(queue, np.zeros(-(-n_cols // 128) * 4, dtype=np.int32))
            dev.append(mask)
            entry = queue.lib.nhip_spmv_sell_skip
            args = args + (int(X.starts[0]), n_cols, mask.ptr)
            gsize, lsize = (1024 * min(queue.n_compute_units, -(-n // 16)),), (1024,)
        else:
            entry, gsize, lsize = queue.lib.nhip_spmv_sell, (WG * n_groups,), (WG,)
        plan = Plan(queue, entry, args, gsize=gsize, lsize=lsize,
                    full_args=tuple(dev) + (X.dev_buf, Y.dev_buf), name="hip_spmv", tag=tag)
        plan.skips_zero_x = skip
        # what `fuse_linearfilter` needs to rebuild the launch with filters behind its rows
        plan.spmv = dict(X=X, Y=Y, slice_rows=slice_rows, dev=tuple(dev), n=n,
                         mask=(mask if skip else None),
                         x_start=int(X.starts[0]) if skip else 0,
                         n_cols=int(X.shape0s[0]) if skip else 0)
        nnz = int(sum(m.csr.nnz for m in matrices))
        plan.flops_per_call = 2 * nnz
        # reference accounting (clra_gemv.py:1552-1560): values, indices, row pointers, X, Y
        plan.bw_per_call = 8 * nnz + 4 * sum(m.shape[0] + 1 for m in matrices) + X.nbytes + Y.nbytes
        plan.stored_bytes = 8 * int(vals.size)
        plan.description = "groups: %d; nonzeros: %d; stored: %d" % (len(matrices), nnz, vals.size)
        self.plans = [plan]
        self.matrices = matrices


# The reference's planner classes (clra_gemv.py:1249-1567) differ in the storage format of
# the matrix (CSR, ELLPACK) and in how a row's products are reduced (one lane per row, a tree
# in LDS, two steps through global memory); its `plan_sparse_dot_inc` picks one from the
# ELLPACK footprint (padding every row to the longest can cost many times the CSR arrays).
# The sliced layout here pads a row only to the longest of its 64-row slice, so there is no
# such trade-off to decide and every name takes the same launch -- same constructor, same
# results (each row summed in column order); the names are kept so that code and tests
# written against the reference's planners run unchanged.
class spmv_prog(plan_sparse_dot_inc):
    """Reference constructor ``(queue, hA, X, Y, inc=False, tag=None)`` (clra_gemv.py:1271-1279)."""

    def __init__(self, queue, hA, X, Y, inc=False, tag=None):
        super().__init__(queue, hA, X, Y, inc=inc, tag=tag)


class plan_csr(spmv_prog):
    """clra_gemv.py:1494-1567."""


class plan_ellpack(spmv_prog):
    """clra_gemv.py:1322-1408."""


class plan_ellpack_tree(plan_ellpack):
    """clra_gemv.py:1411-1443 (there: rows of at most one work-group's length; no such limit here)."""


class plan_ellpack_twostep(plan_ellpack):
    """clra_gemv.py:1446-1491."""


#: names of `algorithm` / the NENGO_OCL_SPMV_ALGORITHM environment variable (clra_gemv.py:1991-1997)
algostr_to_planner = {
    "ELLPACK": plan_ellpack,
    "ELLPACK-tree": plan_ellpack_tree,
    "ELLPACK-twostep": plan_ellpack_twostep,
    "CSR": plan_csr,
}


def spmv_algorithm_heuristic(queue, hA, footprint_hard_limit=0.8, footprint_soft_limit=0.05,
                             soft_limit_ratio=0.1):
    """The reference's choice between "CSR" and "ELLPACK" from the footprint of the ELLPACK
    arrays relative to the device's memory (clra_gemv.py:1951-1988, the same rule): above the
    hard limit CSR, below the soft limit ELLPACK, in between CSR when it is smaller than
    `soft_limit_ratio` of ELLPACK.  Reported for callers that ask; the launch is the same."""
    csr = hA.csr
    ellwidth = max(np.diff(csr.indptr))
    ell_bytes = 2 * 4 * int(ellwidth) * csr.shape[1]
    csr_bytes = 2 * 4 * csr.nnz
    ell_device_ratio = ell_bytes / queue.global_mem_size
    if ell_device_ratio > footprint_hard_limit:
        return "CSR"
    if ell_device_ratio < footprint_soft_limit:
        return "ELLPACK"
    return "CSR" if csr_bytes / ell_bytes < soft_limit_ratio else "ELLPACK"


def fuse_linearfilter(spmv_plan, lf_plan):
    """One launch less for "Y = A X (sparse); filter step on Y": the product steps the
    first-order filters whose input is exactly one of its output vectors as soon as a row
    is final (`nhip_spmv_sell_filter`), with the arithmetic of the filter kernel's simple
    case.  Returns ``([plan replacing spmv_plan], plans replacing [lf_plan])`` -- the second
    list holds a filter launch for the items that were not fused (their indices in
    `lf_plan`: its ``unfused_items``), or is empty -- or None when nothing can be fused."""
    from .hipra_gemv import _overlaps, _span
    from .hipra_nonlinearities import plan_linearfilter

    spec, sp = getattr(lf_plan, "lf_spec", None), getattr(spmv_plan, "spmv", None)
    if spec is None or sp is None or sp["n"] == 0:
        return None
    queue = spmv_plan.queue
    X, F, A, B = spec["X"], spec["Y"], spec["A"], spec["B"]
    Y, SX = sp["Y"], sp["X"]
    if X.ptr.value != Y.ptr.value:
        return None
    outputs = {(int(Y.starts[b]), int(Y.shape0s[b])): b for b in range(len(Y))}
    a_host, b_host = A.to_host(), B.to_host()
    targets_of, rest = {}, []
    for i in range(len(X)):
        simple = int(B.shape0s[i]) == 1 and int(A.shape0s[i]) <= 1
        vector = (int(X.shape1s[i]) == 1 and int(X.stride0s[i]) == 1
                  and int(F.shape1s[i]) == 1 and int(F.stride0s[i]) == 1)
        b = outputs.get((int(X.starts[i]), int(X.shape0s[i]))) if simple and vector else None
        if b is None:
            rest.append(i)
            continue
        na = int(A.shape0s[i])
        a0 = np.float32(a_host[i][0, 0]) if na else np.float32(0)
        b0 = np.float32(b_host[i][0, 0])
        targets_of.setdefault(b, []).append(
            (int(F.starts[i]), int(a0.view(np.int32)), int(b0.view(np.int32)), na))
    if not targets_of:
        return None
    # a fused filter's output must be nothing the product reads or writes
    fused = [i for i in range(len(X)) if i not in set(rest)]
    written = [iv for iv in (_span(F, i) for i in fused) if iv]
    touched = []
    if F.ptr.value == SX.ptr.value:
        touched += [iv for iv in (_span(SX, b) for b in range(len(SX))) if iv]
    if F.ptr.value == Y.ptr.value:
        touched += [iv for iv in (_span(Y, b) for b in range(len(Y))) if iv]
    if _overlaps(written, touched):
        return None

    first, target_rows = {}, []
    for b, rows in sorted(targets_of.items()):
        first[b] = (len(target_rows), len(rows))
        target_rows.extend(rows)
    slice_epi = np.zeros((sp["n"], 4), dtype=np.int32)
    for k, (item, _, _, _, _, row0) in enumerate(sp["slice_rows"]):
        if item in first:
            slice_epi[k] = (first[item][0], first[item][1], row0, 0)
    dev_epi = to_device(queue, slice_epi)
    dev_targets = to_device(queue, np.array(target_rows, dtype=np.int32))
    mask = sp["mask"]
    args = tuple(spmv_plan.args[:7]) + (dev_epi.ptr, dev_targets.ptr, F.ptr, sp["x_start"],
                                        sp["n_cols"], mask.ptr if mask is not None else None)
    plan = Plan(queue, queue.lib.nhip_spmv_sell_filter, args, gsize=spmv_plan.gsize,
                lsize=spmv_plan.lsize,
                full_args=tuple(spmv_plan.full_args) + (dev_epi, dev_targets, F.dev_buf),
                name="hip_spmv_filter", tag=spmv_plan.tag)
    f_bytes = sum(8 * int(Y.shape0s[b]) * len(rows) for b, rows in targets_of.items())
    plan.flops_per_call = spmv_plan.flops_per_call
    plan.bw_per_call = spmv_plan.bw_per_call + f_bytes  # filter state in and out
    plan.stored_bytes = spmv_plan.stored_bytes
    plan.description = spmv_plan.description
    plan.skips_zero_x = spmv_plan.skips_zero_x
    plan.spmv = spmv_plan.spmv
    residual = []
    if rest:
        residual = plan_linearfilter(queue, X[rest], F[rest], A[rest], B[rest],
                                     spec["Xbuf"][rest], spec["Ybuf"][rest], tag=lf_plan.tag)
        residual[0].unfused_items = list(rest)
    return [plan], residual
