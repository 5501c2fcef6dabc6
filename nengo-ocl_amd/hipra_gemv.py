"""Plan builders for the ragged gather-GEMV on HIP.

Counterpart of the dense half of the reference's ``nengo_ocl/clra_gemv.py``:
``gemv_prog`` (:100-261), the planner classes ``plan_ref_gemv`` /
``plan_many_dots_gemv`` / ``plan_reduce_gemv`` / ``plan_block_gemv`` /
``plan_ragged_gather_gemv`` (:1178-1239) and the byte / flop accounting
(``bw_from_geometry`` :49-70, ``flops_from_geometry`` :35-46).  Same call
signature, same ``.plans`` attribute; what differs is the work decomposition:

* every output item is cut into *tasks* of whole rows; a task walks all dot
  products of its item and all their columns and writes final Y values, so a
  GEMV group is ONE launch per kernel class instead of ``fn`` + ``reduce``;
* items are sorted into kernel classes ``(flavor, lanes-per-row, vector width)``
  by shape and alignment, one launch per class that occurs.

For each item b:  ``Y[b] = beta[b]*Y_in[b] + gamma[b] + alpha[b] * sum_j A[A_js[b][j]] @ X[X_js[b][j]]``.
"""

import logging
import os
from collections import defaultdict

import numpy as np

from . import _lib
from .hipraggedarray import HIPRaggedArray, to_device
from .plan import Plan
from .utils import next_pow2

logger = logging.getLogger(__name__)

# items with at most this many matrix elements go to the wave-per-task kernel
SMALL_ITEM_ELEMS = 8192
# ... and so do items of few rows up to four times that size: the large-item kernel
# would give them a handful of waves that walk whole rows one after the other
SHORT_ITEM_ROWS = int(os.environ.get("NENGO_HIP_SHORT_ITEM_ROWS", 256))
SHORT_ITEM_ELEMS = 4 * SMALL_ITEM_ELEMS
# ... and among those, rows up to this length use the reference-order wave kernel
REF_ORDER_MAX_COLS = 512
# float32 words of one wave's LDS block in the reference-order kernel for large items
TILE_STAGE_WORDS = int(os.environ.get("NENGO_HIP_TILE_WORDS", 2176))
# the reference-order kernel wants at least this many (wave) tasks per launch
MIN_TILE_TASKS = int(os.environ.get("NENGO_HIP_TILE_MIN_TASKS", 2048))
TILE_TASK_BLOCKS = tuple(float(v) for v in os.environ.get(
    "NENGO_HIP_TILE_TASK_BLOCKS", "4,3.5,3,2.5,2,1.5,1").split(","))  # row blocks per task, tried in order
# items of the launch that visits only the columns with x != 0 (csrc/gemv_events.hip)
EVENT_MIN_COLS, EVENT_MAX_COLS, EVENT_MIN_ELEMS = 512, 1 << 20, 16384
EVENT_MIN_SPLIT_BYTES = 64 << 20  # matrix bytes that pay for a launch next to a dense one
TASK_OVERHEAD_BYTES = 8192.0  # what starting and finishing a task costs, in streamed bytes
# The large-item kernel with compile-time shapes takes dot products of STREAM_MIN_COLS
# columns or more whose rows are 16-byte aligned; its LDS block has STREAM_STAGE_WORDS words.
STREAM_MIN_COLS, STREAM_STAGE_WORDS = 5, 2176
STREAM_NARROW_MAX_ROWS = int(os.environ.get("NENGO_HIP_NARROW_ROWS", 128))
# instance of that kernel (`pow2_cols`) for matrices of at most FLAT_MAX_COLS columns
# whose rows are not 16-byte aligned but lie back to back: blocks of rows are read as
# aligned runs of memory
STREAM_FLAT, FLAT_MAX_COLS = 7, 64


def stream_class(stages):
    """The instance of the kernel with compile-time shapes (the `pow2_cols` argument of
    nhip_gemv_tile) that holds the stage widths `stages` (log2): 3 = 32 and 64 columns
    only (more waves fit a compute unit then), 5 = also 8 and 16, 2 = also 512, 4 = also
    128 and 512, 6 = all."""
    tiny, mid, wide = bool(stages & {3, 4}), 7 in stages, 9 in stages
    if tiny:
        return 6 if mid or wide else 5
    return 4 if mid else 2 if wide else 3


STREAM_CLASS_STAGES = {3: {5, 6}, 5: {3, 4, 5, 6}, 2: {5, 6, 9}, 4: {5, 6, 7, 9},
                       6: {3, 4, 5, 6, 7, 9}}


def stream_stage(n_cols):
    """(log2 of the stage width, rows of a block) the kernel with compile-time shapes
    uses for a dot product of `n_cols` columns: the smallest stage that holds it, 128
    columns wide from 65 to 511 columns, 512 from there up."""
    if n_cols <= 8:
        return 3, 128
    if n_cols <= 16:
        return 4, 64
    if n_cols <= 32:
        return 5, 32
    if n_cols <= 64:
        return 6, 32
    if n_cols < 512:
        return 7, 16
    return 9, 4
# small-item launches of at most this many rows get task records with the item and its
# coefficients inline (they are chains of dependent reads; larger ones are about traffic)
WIDE_TASK_MAX_ROWS = 65536
# launches with a lane per row: a wave takes a task of up to 64 rows of one item (switch for
# measurements: "0" keeps a task record per row)
WAVE_TASKS = os.environ.get("NENGO_HIP_WAVE_TASKS", "1") != "0"
WG, WAVE = 256, 64
THIN_MIN_ROWS, THIN_ROWS_FOR_LANE_PER_ROW = 32, 65536
LIF_POP_ENABLED, LIF_POP_DECAY, LIF_POP_NO_J = 1 << 8, 1 << 9, 1 << 10  # flag bits of a population row
LIF_POP_BITS = 1 << 11  # spikes stored as a bit per neuron (see `store_spikes_as_bits`)
LIF_COMPACT = os.environ.get("NENGO_HIP_LIF_COMPACT", "1") != "0"


def flops_from_geometry(geometry, items):
    """2 flops per matrix element + 3 per output (clra_gemv.py:35-46)."""
    flops = 0
    for i in items:
        g = geometry[i]
        flops += 2 * g["y_len"] * sum(d["a_shape1"] for d in g["dots"]) + 3 * g["y_len"]
    return int(flops)


def bw_from_geometry(geometry, items):
    """Algorithmic bytes: A and X of every dot, Y_in read, Y written, two scalars
    (clra_gemv.py:49-70).  This is the figure achieved-GB/s numbers are quoted on."""
    n_bytes = 0
    for i in items:
        g = geometry[i]
        for d in g["dots"]:
            n_bytes += 4 * d["a_shape1"] * g["y_len"] + 4 * d["a_shape1"]
        n_bytes += 8 + 4 * g["y_len"] + 4 * g["y_len"]
    return int(n_bytes)


def _per_item_floats(arg, n, what):
    """alpha/beta/gamma as a float32 vector of length n (scalar, list or ndarray)."""
    if isinstance(arg, HIPRaggedArray):
        raise NotImplementedError("%s given as a device ragged array" % what)
    vec = np.asarray(arg, dtype=np.float32)
    if vec.ndim == 0:
        vec = np.full(n, vec, dtype=np.float32)
    if vec.shape != (n,):
        raise ValueError("%s must be a scalar or have one value per output" % what)
    return vec


def _literal_coefficient(arg, n):
    """The double the reference writes into its kernel text for a coefficient that is the
    same for every item (a Python float, or a list of equal values: clra_gemv.py:17-32), or
    None for one that differs from item to item (a float32 array there)."""
    v = np.asarray(arg, dtype=np.float64)
    if v.ndim == 0:
        return float(v)
    if n and len(set(v.ravel().tolist())) == 1:
        return float(v.ravel()[0])
    return None


SPREAD_OVER_DIES = os.environ.get("NENGO_HIP_SPREAD_TASKS", "1") != "0"  # switch for measurements
N_DIES = 8  # accelerator dies of the device: work-group g runs on die g % 8


def spread_over_dies(tasks):
    """The 24-word task records of a large-item launch in an order that gives every
    accelerator die the same number of heavy tasks.

    Work-groups go to the dies in turn, and the kernels map them so that a die works through
    one contiguous range of the task list (`nhip_xcd_remap`).  Tasks without a matrix to stream
    (sums nothing else reads, populations without input) sit at the end of the list as it is
    built, so the last die got all of them and the first ones only heavy tasks: a launch of two
    rounds of groups per die then ran a third round on some dies.  Here the light tasks are
    dealt out over the ranges (at the end of each), so that the heavy ones divide evenly.
    Tasks are independent of each other (each owns its rows), so any order gives the same
    result."""
    per_group = WG // WAVE
    n = len(tasks)
    groups = -(-n // per_group)
    if not SPREAD_OVER_DIES or groups < 2 * N_DIES or tasks.shape[1] != 24:
        return tasks
    weight = tasks[:, 2].astype(np.int64) * np.maximum(tasks[:, 18], 1) * (tasks[:, 9] > 0)
    heavy = weight >= 0.25 * max(int(weight.max()), 1)
    if heavy.all() or not heavy.any():
        return tasks
    H, L = tasks[heavy], tasks[~heavy]
    per, rem = divmod(groups, N_DIES)  # (the partition nhip_xcd_remap makes)
    sizes = [(per + (1 if x < rem else 0)) * per_group for x in range(N_DIES)]
    sizes[-1] -= groups * per_group - n
    out, ih, il = [], 0, 0
    for x, size in enumerate(sizes):
        want = len(H) * (x + 1) // N_DIES
        want -= want % per_group if x < N_DIES - 1 else 0  # whole groups of heavy tasks
        h = max(0, min(want - ih, size, len(H) - ih))
        l = min(size - h, len(L) - il)
        h = min(size - l, len(H) - ih)  # (too few light tasks left: heavy ones fill the range)
        out += [H[ih:ih + h], L[il:il + l]]
        ih, il = ih + h, il + l
    out += [H[ih:], L[il:]]
    out = np.concatenate(out)
    assert len(out) == n
    return out


def _balanced_rows(M, cap):
    """Rows per task so that the tasks of an item are equally full (M = 4096, cap = 128
    stays 128; M = 100, cap = 64 becomes 50 instead of 64 + 36)."""
    n_tasks = -(-M // cap)
    return -(-M // n_tasks)


class gemv_prog:
    """Geometry + work lists of one ragged GEMV; subclasses pick the kernel classes."""

    # None = reference summation order (kernels "wave_ref" and "tile"); 0 = work-group
    # kernel and 1 = wave kernel with their own, faster-to-reduce order
    force_flavor = None
    force_scalar = False  # one lane per output, 4-byte loads (the plain fallback)

    def __init__(self, queue, alpha, A, A_js, X, X_js, beta, Y, Y_in=None, gamma=0.0, tag=None,
                 tile_items=(), event_items=()):
        self.queue = queue
        self.tile_items = frozenset(tile_items)  # items that take the large-item kernel regardless
        # items whose X is mostly zero (spikes) and whose A nothing ever writes: candidates
        # for the launch that only visits the columns with x != 0 (`_event_item`)
        self.event_items = frozenset(event_items)
        self._events_off = False
        self._host_A_cache = None
        self._finite_cache = {}
        self._many_thin_rows = False
        self.A, self.A_js, self.X, self.X_js = A, A_js, X, X_js
        self.Y = Y
        self.Y_in = Y if Y_in is None else Y_in
        self.tag = str(tag)
        n = len(Y)
        self.alpha = _per_item_floats(alpha, n, "alpha")
        self.beta = _per_item_floats(beta, n, "beta")
        self.gamma = _per_item_floats(gamma, n, "gamma")
        self.float_alpha = float(self.alpha[0]) if n and np.all(self.alpha == self.alpha[0]) else None
        self.float_beta = float(self.beta[0]) if n and np.all(self.beta == self.beta[0]) else None
        self.float_gamma = float(self.gamma[0]) if n and np.all(self.gamma == self.gamma[0]) else None
        # coefficients the reference computes with as double literals; where float32 does not
        # hold one of them exactly the launch takes the kernel that multiplies in double
        # (the kernels in their own summation order agree to a tolerance only anyway)
        self.literals = [_literal_coefficient(c, n) for c in (alpha, beta, gamma)]
        self._literal_kernel = (
            self.force_flavor is None and not self.force_scalar
            and any(c is not None and float(np.float32(c)) != c for c in self.literals))

        self.geometry = self._geometry()
        self.plans = self.choose_plans()
        self._host_A_cache = None  # (host copies of matrices: only needed while planning)

    # ------------------------------------------------------------ geometry
    def _geometry(self):
        A, X, Y, Y_in = self.A, self.X, self.Y, self.Y_in
        if len(Y_in) != len(Y):
            raise ValueError("Y_in and Y differ in length")
        if self.A_js is None or self.X_js is None:
            raise NotImplementedError("A_js / X_js are required")
        if len(self.A_js) != len(Y) or len(self.X_js) != len(Y):
            raise ValueError("need one A_js / X_js list per output")

        # kernels trust these offsets: fail on the host if a view leaves its buffer
        for name, ra in (("A", A), ("X", X), ("Y", Y), ("Y_in", Y_in)):
            ra.check_bounds(name)

        geometry = []
        for b in range(len(Y)):
            M = int(Y.shape0s[b])
            if int(Y.shape1s[b]) != 1 or int(Y_in.shape1s[b]) != 1:
                raise NotImplementedError("outputs must be column vectors")
            if int(Y_in.shape0s[b]) != M:
                raise ValueError("Y_in[%d] and Y[%d] differ in length" % (b, b))
            a_js = np.asarray(self.A_js[b]).ravel()
            x_js = np.asarray(self.X_js[b]).ravel()
            if a_js.size != x_js.size:
                raise ValueError("A_js[%d] and X_js[%d] differ in length" % (b, b))
            dots = []
            for j, (aj, xj) in enumerate(zip(a_js.tolist(), x_js.tolist())):
                if int(A.shape0s[aj]) != M:
                    raise ValueError("A[%d] has %d rows, Y[%d] has %d" % (aj, A.shape0s[aj], b, M))
                if int(A.shape1s[aj]) != int(X.shape0s[xj]) or int(X.shape1s[xj]) != 1:
                    raise ValueError("A[%d] and X[%d] do not conform" % (aj, xj))
                if int(A.stride1s[aj]) != 1 and int(A.shape1s[aj]) > 1:
                    raise NotImplementedError("A rows must be contiguous (stride1 == 1)")
                dots.append(
                    {
                        "j": j,
                        "a_j": aj,
                        "x_j": xj,
                        "a_start": int(A.starts[aj]),
                        "a_stride0": int(A.stride0s[aj]),
                        "a_shape1": int(A.shape1s[aj]),
                        "x_start": int(X.starts[xj]),
                        "x_stride0": int(X.stride0s[xj]),
                    }
                )
            geometry.append(
                {
                    "index": b,
                    "y_len": M,
                    "dots": dots,
                    "y_start": int(Y.starts[b]),
                    "y_stride0": int(Y.stride0s[b]),
                    "y_in_start": int(Y_in.starts[b]),
                    "y_in_stride0": int(Y_in.stride0s[b]),
                }
            )
        return geometry

    def geometry_summary(self, items=None):
        gg = self.geometry if items is None else [self.geometry[i] for i in items]
        if not gg:
            return "outputs: 0"
        dots = np.array([len(g["dots"]) for g in gg])
        m = np.array([g["y_len"] for g in gg])
        n = np.array([d["a_shape1"] for g in gg for d in g["dots"]] or [0])
        return "outputs: %d; dots: %0.1f [%d, %d]; shape: %0.1f [%d, %d] x %0.1f [%d, %d]" % (
            len(gg), dots.mean(), dots.min(), dots.max(),
            m.mean(), m.min(), m.max(), n.mean(), n.min(), n.max(),
        )

    # ------------------------------------------------------- class selection
    def _item_class(self, g):
        """(flavor, lanes per row, vector width) for one item."""
        if g["index"] in self.tile_items and not g["dots"]:
            return (3, 1, 4)  # no dot products: only Y = beta Y_in + gamma and the epilogue
        dots = g["dots"]
        M = g["y_len"]
        n_max = max([d["a_shape1"] for d in dots] or [1])
        n_sum = sum(d["a_shape1"] for d in dots)
        if self.force_scalar:
            return (1, 1, 1)
        if self.force_flavor is None and self._event_item(g):
            return (4, 0, 4)
        vec = 4
        if n_max < 4 or any(d["a_start"] % 4 or (d["a_stride0"] % 4 and M > 1) for d in dots):
            vec = 1
        flavor = self.force_flavor
        if flavor is None:
            # default: the reference's summation order, bit for bit -- small items one
            # wave per task, large items staged through LDS by a work-group
            if dots and n_max <= 4 and M >= THIN_MIN_ROWS and self._many_thin_rows:
                return (2, 1, 1)  # a lane per row: vector sums, scalar-times-vector terms
            if n_max <= REF_ORDER_MAX_COLS and (M * n_sum <= SMALL_ITEM_ELEMS or (
                    M <= SHORT_ITEM_ROWS and M * n_sum <= SHORT_ITEM_ELEMS)):
                return (2, 4, 1)
            pow2 = vec == 4 and all(
                d["a_shape1"] >= 4 and d["a_shape1"] & (d["a_shape1"] - 1) == 0
                and d["a_stride0"] < 2 ** 22 for d in dots)
            # second entry: 1 = every column count a power of two; 2 ... 6 = the kernel with
            # compile-time shapes, by the stage widths needed (`stream_class`)
            # (vec == 4: rows start on 16-byte boundaries; a row whose length is no multiple
            # of 4 must be followed by readable memory up to the next one: a column block
            # of a wider matrix)
            a_size = int(self.A.dev_buf.size)

            def quads_readable(d):  # 16-byte loads may run up to three columns past a row
                n4 = -(-d["a_shape1"] // 4) * 4
                return (d["a_shape1"] == n4 or (
                    M > 1 and d["a_stride0"] >= n4
                    and d["a_start"] + (M - 1) * d["a_stride0"] + n4 <= a_size))

            stream = (vec == 4 and TILE_STAGE_WORDS == STREAM_STAGE_WORDS and dots and all(
                d["a_stride0"] < 2 ** 22 and d["a_shape1"] >= STREAM_MIN_COLS
                and quads_readable(d) for d in dots))
            if stream:
                return (3, stream_class({stream_stage(d["a_shape1"])[0] for d in dots}), vec)
            # rows that are not 16-byte aligned but lie back to back, at most 64 columns: row
            # blocks are aligned runs of memory when tasks start at multiples of 4 rows
            # (the last quad of a matrix may reach 12 bytes past it)
            if (vec == 1 and TILE_STAGE_WORDS == STREAM_STAGE_WORDS and dots and all(
                    d["a_start"] % 4 == 0 and d["a_stride0"] == d["a_shape1"]
                    and STREAM_MIN_COLS <= d["a_shape1"] <= FLAT_MAX_COLS
                    and d["a_start"] + M * d["a_shape1"] + 3 <= a_size for d in dots)):
                return (3, STREAM_FLAT, 4)
            return (3, int(pow2), vec)
        if flavor == 0:
            # Matrix loads are non-temporal, so one wave instruction should take whole
            # 128-byte lines of a row: at least 8 lanes x 16 bytes per row, each lane then
            # walking further column quads of its row.  Measured on MI355X, encoders and
            # decoders of 256 ensembles alternating: 4096 x 64 -> 8 lanes per row, 5.75 TB/s;
            # 64 x 4096 -> the whole group per row, 5.85 TB/s.
            if vec == 4:
                lpr = min(WAVE, max(8, next_pow2(n_max // 16))) if n_max >= 32 else next_pow2(
                    -(-n_max // 4))
            else:
                lpr = min(WAVE, next_pow2(-(-n_max // 4)))
            if n_max >= 2048 and M <= 256:
                lpr = WG  # few, long rows: the whole group works on one row
        else:
            lpr = min(WAVE, next_pow2(-(-n_max // vec)))
        return (flavor, lpr, vec)

    def _event_item(self, g, any_size=False):
        """Does item `g` take the launch that visits only the columns with x != 0?  One
        dot product of `EVENT_MIN_COLS` to `EVENT_MAX_COLS` columns, a contiguous X, enough elements to be a large item, and the caller's word that X is
        mostly zero and A constant."""
        if self._events_off or g["index"] not in self.event_items or len(g["dots"]) != 1:
            return False
        d = g["dots"][0]
        return (g["y_len"] >= 1 and EVENT_MIN_COLS <= d["a_shape1"] <= EVENT_MAX_COLS
                and (any_size or g["y_len"] * d["a_shape1"] >= EVENT_MIN_ELEMS)
                and (d["x_stride0"] == 1 or d["a_shape1"] == 1)
                and self._finite_matrix(d["a_j"]))

    def _host_matrix(self, a_j):
        """Matrix `a_j` of A on the host (one transfer of that matrix, kept: the launch
        that visits active columns needs it again for its transposed copy)."""
        if self._host_A_cache is None:
            self._host_A_cache = {}
        if a_j not in self._host_A_cache:
            self._host_A_cache[a_j] = np.array(self.A[int(a_j)], dtype=np.float32)
        return self._host_A_cache[a_j]

    def _finite_matrix(self, a_j):
        """Skipping the columns whose x is zero equals the dense product only while no
        skipped product would be 0 * inf or 0 * nan: matrices with a non-finite entry keep
        the dense launch."""
        if a_j not in self._finite_cache:
            self._finite_cache[a_j] = bool(np.isfinite(self._host_matrix(a_j)).all())
        return self._finite_cache[a_j]

    def _event_plan(self, members):
        """The launch of `nhip_gemv_events` for `members`: their matrices transposed into a
        device buffer of their own (column c of an item: `mp` consecutive floats)."""
        queue, geometry = self.queue, self.geometry
        rows, parts, cursor, record_item = [], [], 0, []
        for b in members:
            g = geometry[b]
            d = g["dots"][0]
            M, N = g["y_len"], d["a_shape1"]
            mp = -(-M // 16) * 16
            block = self._host_matrix(d["a_j"]).reshape(M, N)
            t = np.zeros((N, mp), dtype=np.float32)
            t[:, :M] = block.T
            coefs = np.array([self.alpha[b], self.beta[b], self.gamma[b]], dtype=np.float32)
            for row0 in range(0, M, WAVE):  # a work-group per 64 rows
                rows.append((cursor, mp, min(WAVE, M - row0), N, d["x_start"], g["y_start"],
                             g["y_stride0"], g["y_in_start"], g["y_in_stride0"])
                            + tuple(coefs.view(np.int32).tolist()) + (0, 0, row0, 0))
                record_item.append(b)
            parts.append(t.ravel())
            cursor += N * mp
        if cursor >= 2 ** 31:
            raise ValueError("more than 2^31 elements of transposed matrices")
        table = np.array(rows, dtype=np.int32)
        dev_items = to_device(queue, table)
        dev_at = to_device(queue, np.concatenate(parts))
        n = len(rows)
        args = (dev_items.ptr, n, dev_at.ptr, self.X.ptr, self.Y_in.ptr, self.Y.ptr, None, None,
                int(table[:, 3].max()))
        plan = Plan(queue, queue.lib.nhip_gemv_events, args, gsize=(1024 * n,), lsize=(1024,),
                    full_args=(dev_items, dev_at, self.X.dev_buf, self.Y_in.dev_buf, self.Y.dev_buf),
                    name="hipra_gemv.events", tag="%s-events" % self.tag,
                    bw_per_call=bw_from_geometry(geometry, members),
                    flops_per_call=flops_from_geometry(geometry, members))
        plan.description = self.geometry_summary(members)
        plan.kernel_class = (4, 0, 4)
        plan.n_tasks = n
        plan.members = list(members)
        plan.prog = self
        plan.host_tasks = None
        plan.event_table = table
        plan.dev_event_table = dev_items
        plan.event_record_item = np.array(record_item, dtype=np.int64)  # Y item of each record
        plan.event_driven = True  # reads only the columns of A whose x is not zero
        return plan

    def _tile_tasks(self, members, max_rows=256, stream=False, row_multiple=1):
        """Tasks (item, first row, rows, 0) of the reference-order kernel for large items.

        A task is the rows one wave carries through all columns, a few row blocks of
        what fits its LDS stage.  Larger tasks reuse the gathered X more often and pay
        the start of a task (its record, the first loads, the epilogue: about what
        TASK_OVERHEAD_BYTES of streaming cost) less often; but the groups of a launch
        spread over the compute units in whole groups, and a launch of few groups (all
        resident at once, each lasting about as long as the launch) is only busy to the
        end when they spread evenly.  Among the task sizes that give enough tasks, the
        one with the smallest (groups per compute unit, rounded up) x (bytes of a task +
        overhead) wins.
        """
        lib, geometry = self.queue.lib, self.geometry
        blk = {b: min([stream_stage(dd["a_shape1"])[1] if stream else
                       lib.nhip_gemv_tile_rows(dd["a_shape1"], TILE_STAGE_WORDS)
                       for dd in geometry[b]["dots"]] or [WAVE]) for b in members}

        def tasks_for(per_task, whole_blocks_up):
            out = []
            for b in members:
                M = geometry[b]["y_len"]
                item_rows = max(1, min(int(blk[b] * per_task), max_rows))
                if M > item_rows:
                    item_rows = _balanced_rows(M, item_rows)
                    if item_rows >= 2 * blk[b]:
                        # whole row blocks: fewer rows per task, or more (fewer tasks, the
                        # last one of an item shorter); the cost below decides
                        if whole_blocks_up:
                            item_rows = min(-(-item_rows // blk[b]) * blk[b], max_rows)
                        else:
                            item_rows -= item_rows % blk[b]
                    # (tasks that must start at a multiple of so many rows)
                    item_rows = min(-(-item_rows // row_multiple) * row_multiple, max_rows)
                for r0 in range(0, M, item_rows):
                    out.append((b, r0, min(item_rows, M - r0), 0))
            return out

        n_cu = self.queue.n_compute_units
        best = None
        row_bytes = {b: 4.0 * sum(dd["a_shape1"] for dd in geometry[b]["dots"]) for b in members}
        for per_task, up in [(p, u) for p in TILE_TASK_BLOCKS for u in (False, True)]:
            tasks = tasks_for(per_task, up)
            groups = -(-len(tasks) // (WG // WAVE))
            task_bytes = sum(row_bytes[b] * n for b, _, n, _ in tasks) / max(len(tasks), 1)
            cost = -(-groups // n_cu) * (task_bytes + TASK_OVERHEAD_BYTES)
            enough = len(tasks) >= MIN_TILE_TASKS
            key = (not enough, cost)
            if best is None or key < best[0]:
                best = (key, tasks)
        return best[1]

    def _build(self, items):
        """Work lists for `items`; returns the list of plans (one per kernel class)."""
        lib = self.queue.lib
        geometry = self.geometry
        n_items = len(geometry)

        item_tab = np.zeros((max(n_items, 1), 8), dtype=np.int32)
        coef_tab = np.zeros((max(n_items, 1), 4), dtype=np.float32)
        dot_rows = []
        for b, g in enumerate(geometry):
            item_tab[b] = (g["y_start"], g["y_stride0"], g["y_in_start"], g["y_in_stride0"],
                           len(dot_rows), len(g["dots"]), g["y_len"], 0)
            coef_tab[b] = (self.alpha[b], self.beta[b], self.gamma[b], 0.0)
            for d in g["dots"]:
                n = d["a_shape1"]
                log2_n = n.bit_length() - 1 if n > 0 and n & (n - 1) == 0 else -1
                dot_rows.append((d["a_start"], d["a_stride0"], n, d["x_start"], d["x_stride0"],
                                 lib.nhip_gemv_tile_rows(n, TILE_STAGE_WORDS), log2_n,
                                 stream_stage(n)[0]))
        dot_tab = np.array(dot_rows or [(0,) * 8], dtype=np.int32)

        # Items whose dot products have at most four columns (sums of vectors, scalar
        # times vector) can give every row a lane of its own: consecutive lanes then
        # read consecutive elements and share the item's records.  That pays when there
        # is enough of it to be a throughput problem (c2's 2048 x 100 encoders: 10.2 ->
        # 6.7 us); a few thousand rows are latency bound and better spread over more
        # waves, four lanes per row (c3's 254 x 64 input sums: 7.9 vs 8.8 us).
        thin_rows = sum(geometry[b]["y_len"] for b in items
                        if geometry[b]["dots"] and geometry[b]["y_len"] >= THIN_MIN_ROWS
                        and max(d["a_shape1"] for d in geometry[b]["dots"]) <= 4)
        self._many_thin_rows = thin_rows >= THIN_ROWS_FOR_LANE_PER_ROW

        if self._literal_kernel:
            return self._literal_plans(items, item_tab, dot_tab)

        by_class = defaultdict(list)
        for b in items:
            if geometry[b]["y_len"] > 0:
                by_class[self._item_class(geometry[b])].append(b)
        # visiting only the columns with x != 0 is a launch of its own: next to a launch of
        # large items that stays anyway it must save more than it costs
        events = by_class.get((4, 0, 4), [])
        if events:
            # where that launch exists, candidates too small to ask for it join it rather
            # than keep a launch of large items alive
            for cls in [c for c in by_class if c[0] == 3]:
                join = [b for b in by_class[cls] if self._event_item(geometry[b], any_size=True)]
                if join:
                    events.extend(join)
                    by_class[cls] = [b for b in by_class[cls] if b not in set(join)]
                    if not by_class[cls]:
                        del by_class[cls]
            events.sort()
        if events and any(c[0] == 3 for c in by_class) and 4 * sum(
                geometry[b]["y_len"] * geometry[b]["dots"][0]["a_shape1"]
                for b in events) < EVENT_MIN_SPLIT_BYTES:
            del by_class[(4, 0, 4)]
            self._events_off = True
            for b in events:
                by_class[self._item_class(geometry[b])].append(b)
            self._events_off = False
            for members in by_class.values():
                members.sort()

        # the one instance of the compile-time-shape kernel that holds the stage widths of
        # all of them takes the items of several instances
        present = [c for c in by_class if c[0] == 3 and c[1] in STREAM_CLASS_STAGES]
        stream = (3, 3, 4)
        if present:
            stream = (3, stream_class(set().union(
                *(STREAM_CLASS_STAGES[c[1]] for c in present))), 4)
            by_class[stream] = sorted(b for c in present for b in by_class.pop(c))
        # ... and items without dot products (class (3, 1, 4)) ride with that launch
        if stream in by_class and (3, 1, 4) in by_class:
            bare = [b for b in by_class[(3, 1, 4)] if not geometry[b]["dots"]]
            by_class[stream] = sorted(by_class[stream] + bare)
            by_class[(3, 1, 4)] = [b for b in by_class[(3, 1, 4)] if geometry[b]["dots"]]
            if not by_class[(3, 1, 4)]:
                del by_class[(3, 1, 4)]

        dev_items = to_device(self.queue, item_tab)
        dev_coefs = to_device(self.queue, coef_tab)
        dev_dots = to_device(self.queue, dot_tab)

        plans = []
        for cls, members in sorted(by_class.items()):
            flavor, lpr, vec = cls[:3]
            if flavor == 4:
                plans.append(self._event_plan(members))
                continue
            passes = cls[3] if len(cls) > 3 else 0  # 0 = the class default
            if flavor == 3:
                rows = None  # per item, below
            elif flavor == 0:
                rows = lib.nhip_gemv_rows_per_task(flavor, lpr, vec, passes)
            elif flavor == 2:
                rows = 1  # a task is one row; a wave packs 64 / lpr of them, of any items
            else:
                rows = (WAVE // lpr) * 4  # four passes of a wave
            if rows is not None and rows <= 0:
                raise _lib.HipError("unknown GEMV class %r" % (cls,))
            if flavor == 3:
                # launches without wide dot products keep tasks to 128 rows (the kernel
                # then needs fewer registers and a fourth wave fits each SIMD)
                task_rows = self._tile_tasks(
                    members, STREAM_NARROW_MAX_ROWS if lpr in (3, 5, STREAM_FLAT) else 256,
                    stream=lpr >= 2, row_multiple=4 if lpr == STREAM_FLAT else 1)
            else:
                task_rows = []
                for b in (members if flavor != 2 else ()):
                    M = geometry[b]["y_len"]
                    for r0 in range(0, M, rows):
                        task_rows.append((b, r0, min(rows, M - r0), 0))
            lpr_arg = lpr
            if flavor == 2 and lpr == 1 and WAVE_TASKS:
                # a lane per row: tasks of up to 64 consecutive rows of an item that a wave
                # takes whole, so that the records are the wave's and not each row's
                lpr_arg = WAVE
                lens = np.array([geometry[b]["y_len"] for b in members], dtype=np.int64)
                per_item = -(-lens // WAVE)  # (built with numpy: there can be millions of rows)
                first = np.cumsum(per_item) - per_item
                row0 = (np.arange(int(per_item.sum())) - np.repeat(first, per_item)) * WAVE
                task_rows = np.zeros((len(row0), 4), dtype=np.int32)
                task_rows[:, 0] = np.repeat(np.array(members, dtype=np.int32), per_item)
                task_rows[:, 1] = row0
                task_rows[:, 2] = np.minimum(WAVE, np.repeat(lens, per_item) - row0)
            elif flavor == 2:  # built with numpy: there can be millions of rows
                counts = np.array([geometry[b]["y_len"] for b in members], dtype=np.int64)
                task_tab = np.zeros((int(counts.sum()), 4), dtype=np.int32)
                task_tab[:, 0] = np.repeat(np.array(members, dtype=np.int32), counts)
                task_tab[:, 1] = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
                task_tab[:, 2] = 1
                task_rows = task_tab
            task_tab = np.array(task_rows, dtype=np.int32)
            if flavor == 2 and (0 < len(task_tab) <= WIDE_TASK_MAX_ROWS or lpr_arg == WAVE):
                which = task_tab[:, 0]
                wide = np.zeros((len(task_tab), 16), dtype=np.int32)
                wide[:, 0:4] = task_tab
                wide[:, 4:12] = item_tab[which]
                wide[:, 12:16] = coef_tab[which].view(np.int32)
                wide[:, 15] = 0
                task_tab = wide
                passes = 16  # nhip_gemv: words of a task record
            if flavor == 3:
                # one record per task with its item, coefficients and first dot product
                # inline: a wave starts streaming after one read instead of three
                which = task_tab[:, 0]
                fat = np.zeros((len(task_tab), 24), dtype=np.int32)
                fat[:, 0:4] = task_tab
                fat[:, 4:12] = item_tab[which]
                fat[:, 12:16] = coef_tab[which].view(np.int32)
                has_dots = item_tab[which, 5] > 0
                fat[has_dots, 16:24] = dot_tab[item_tab[which[has_dots], 4]]
                task_tab = spread_over_dies(fat)
            dev_tasks = to_device(self.queue, task_tab)
            n_tasks = len(task_rows)
            if flavor == 0:
                n_groups = n_tasks
            elif flavor == 2:
                n_groups = -(-n_tasks // ((WG // WAVE) * (WAVE // lpr_arg)))
            else:
                n_groups = -(-n_tasks // (WG // WAVE))
            tail = (dev_items.ptr, dev_coefs.ptr, dev_dots.ptr, dev_tasks.ptr, n_tasks, self.A.ptr,
                    self.X.ptr, self.Y_in.ptr, self.Y.ptr)
            if flavor == 3:
                kern, args = lib.nhip_gemv_tile, (vec, lpr, TILE_STAGE_WORDS) + tail
            else:
                kern, args = lib.nhip_gemv, (flavor, lpr_arg, vec, passes) + tail
            plan = Plan(
                self.queue, kern, args, gsize=(WG * n_groups,), lsize=(WG,),
                full_args=(dev_items, dev_coefs, dev_dots, dev_tasks, self.A.dev_buf,
                           self.X.dev_buf, self.Y_in.dev_buf, self.Y.dev_buf),
                name="hipra_gemv.%s" % ("wg", "wave", "wave_ref", "tile")[flavor],
                tag="%s-lpr%d-v%d" % (self.tag, lpr, vec),
                bw_per_call=bw_from_geometry(geometry, members),
                flops_per_call=flops_from_geometry(geometry, members),
            )
            plan.description = self.geometry_summary(members)
            plan.kernel_class = cls
            plan.n_tasks = n_tasks
            plan.members = list(members)
            plan.prog = self
            plan.host_tasks = task_tab if flavor == 3 or task_tab.shape[1] == 16 else None
            plan.host_tables = (item_tab, coef_tab, task_tab)  # (for plans that extend the launch)
            plans.append(plan)
        return plans

    def _literal_plans(self, items, item_tab, dot_tab):
        """One launch of `nhip_gemv_rows_literal` for all of `items`: a task per output row,
        the coefficients as doubles (the literal where the reference writes one, else the
        float32 value)."""
        queue, geometry = self.queue, self.geometry
        members = [b for b in items if geometry[b]["y_len"] > 0]
        if not members:
            return []
        dcoefs = np.zeros((len(geometry), 4), dtype=np.float64)
        for k, (lit, per_item) in enumerate(zip(self.literals, (self.alpha, self.beta, self.gamma))):
            dcoefs[:, k] = per_item.astype(np.float64) if lit is None else lit
        counts = np.array([geometry[b]["y_len"] for b in members], dtype=np.int64)
        task_tab = np.zeros((int(counts.sum()), 4), dtype=np.int32)
        task_tab[:, 0] = np.repeat(np.array(members, dtype=np.int32), counts)
        task_tab[:, 1] = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
        task_tab[:, 2] = 1
        # (device arrays are float32 or int32: the doubles travel as pairs of words)
        dev = [to_device(queue, t) for t in (item_tab, dcoefs.view(np.int32), dot_tab, task_tab)]
        n_tasks = len(task_tab)
        args = tuple(d.ptr for d in dev) + (n_tasks, self.A.ptr, self.X.ptr, self.Y_in.ptr, self.Y.ptr)
        plan = Plan(queue, queue.lib.nhip_gemv_rows_literal, args,
                    gsize=(WG * -(-n_tasks // ((WG // WAVE) * (WAVE // 4))),), lsize=(WG,),
                    full_args=tuple(dev) + (self.A.dev_buf, self.X.dev_buf, self.Y_in.dev_buf,
                                            self.Y.dev_buf),
                    name="hipra_gemv.wave_ref_literal", tag="%s-literal" % self.tag,
                    bw_per_call=bw_from_geometry(geometry, members),
                    flops_per_call=flops_from_geometry(geometry, members))
        plan.description = self.geometry_summary(members)
        plan.kernel_class = (5, 4, 1)
        plan.n_tasks = n_tasks
        plan.members = list(members)
        plan.prog = self
        plan.host_tasks = None
        return [plan]

    def choose_plans(self):
        return self._build(list(range(len(self.Y))))


class plan_block_gemv(gemv_prog):
    """The planner the Simulator uses (clra_gemv.py:1193-1195)."""


class plan_ragged_gather_gemv(gemv_prog):
    """Shape-driven choice between kernels (clra_gemv.py:1198-1239); here the
    per-item class selection already does that."""


class plan_reduce_gemv(gemv_prog):
    """Few long dots per output: always the LDS-staged work-group kernel."""

    force_flavor = 0


class plan_many_dots_gemv(gemv_prog):
    """Many shallow dots per output: always the wave-per-task kernel."""

    force_flavor = 1


class plan_ref_gemv(gemv_prog):
    """One lane per output element, scalar loads: the plain fallback kernel."""

    force_scalar = True


def _overlaps(a, b):
    """Does any half-open interval of `a` overlap one of `b`?  (lists of (lo, hi))"""
    if not a or not b:
        return False
    b = sorted(b)
    los = np.array([lo for lo, _ in b])
    his = np.maximum.accumulate(np.array([hi for _, hi in b]))
    for lo, hi in a:
        k = np.searchsorted(los, hi, side="left")  # intervals of b starting before hi
        if k > 0 and his[k - 1] > lo:
            return True
    return False


def _span(ra, i):
    """Half-open element interval item i of a ragged array may touch."""
    m, n = int(ra.shape0s[i]), int(ra.shape1s[i])
    if m == 0 or n == 0:
        return None
    lo = int(ra.starts[i])
    return lo, lo + (m - 1) * int(ra.stride0s[i]) + (n - 1) * int(ra.stride1s[i]) + 1


def _concat(ras):
    """Items of several views of one device buffer, as one ragged view."""
    first = ras[0]
    fields = [np.concatenate([getattr(ra, f) for ra in ras])
              for f in ("starts", "shape0s", "shape1s", "stride0s", "stride1s")]
    return HIPRaggedArray.from_buffer(first.queue, first.dev_buf, *fields)


def _subset_param(param, idx):
    """tau / ref / amp of `plan_lif` restricted to the populations `idx`."""
    if isinstance(param, HIPRaggedArray):
        return param[list(idx)]
    if isinstance(param, np.ndarray) and param.ndim == 1:
        return param[list(idx)]
    return param


def _takes_epilogue(plan):
    """Reference-order launches (large or small items) that do not have an epilogue yet."""
    return (plan.name in ("hipra_gemv.tile", "hipra_gemv.wave_ref")
            and getattr(plan, "kernel_class", (None,))[0] in (2, 3))


def _takes_filters(plan):
    """Launches that can step first-order filters on their fresh rows."""
    return _takes_epilogue(plan) or (plan.name == "hipra_gemv.events"
                                     and getattr(plan, "kernel_class", (None,))[0] == 4)


def _epilogue_call(lib, plan, kind, extras=None):
    """Entry point, leading arguments and device arrays to keep alive of `plan`'s launch
    with an epilogue.  `extras(item indices) -> int32[n, 3]`: what the epilogue wants to
    find in the spare words 3, 11, 15 of 16-word task records (small-item launches)."""
    if plan.kernel_class[0] == 3:
        return getattr(lib, "nhip_gemv_tile_" + kind), plan.args, ()
    # nhip_gemv's (flavor, lpr, vec, passes, items, coefs, dots, tasks, ...)
    #   -> (lpr, task_words, items, coefs, dots, tasks, ...)
    tables, keep = tuple(plan.args[4:]), ()
    task_words = 16 if plan.host_tasks is not None else 4
    if task_words == 16:
        tasks = plan.host_tasks.copy()
        tasks[:, [3, 11, 15]] = extras(tasks[:, 0])
        dev_tasks = to_device(plan.queue, tasks)
        tables = tables[:3] + (dev_tasks.ptr,) + tables[4:]
        keep = (dev_tasks,)
        plan.epilogue_tasks = tasks
    return getattr(lib, "nhip_gemv_rows_" + kind), (plan.args[1], task_words) + tables, keep


def fuse_lif(prog, lif_plan, unread_currents=()):
    """Fewer launches for "J = GEMV(...); LIF(J)" (clra_gemv.py `plan_block_gemv` followed
    by clra_nonlinearities.py `plan_lif`): the reference-order kernels update the neurons
    of a row (block) as soon as its currents are final, so the currents are not read
    back and the neuron kernel is not launched.

    A population is fused when its J is exactly the output of one item of a
    reference-order launch of `prog` (large or small items).  Populations whose J no
    item of `prog` writes (neurons without input connections) ride along as items
    without dot products.  Populations fed by launches of another kind keep a neuron
    launch of their own.  Nothing is fused when a state the
    update writes (voltage, refractory time, spikes) is read by a dot product of
    `prog`.  Returns the plans that replace ``prog.plans + [lif_plan]`` (same results
    bit for bit), or None.

    `unread_currents`: populations (indices into the neuron plan) whose input current the
    caller knows nothing else reads.  Where such a current is formed from operands other
    than itself (``J = bias + E x``, not ``J += ...``), the fused launch does not store it;
    every fused plan carries ``lazy_currents = (those populations, a plain GEMV over their
    items)``: running that GEMV puts the currents of the last step into their place, bit
    for bit what the launch would have stored.
    """
    from .hipra_nonlinearities import lif_population_table, plan_lif

    spec = getattr(lif_plan, "lif_spec", None)
    if spec is None or not prog.plans:
        return None
    queue, lib = prog.queue, prog.queue.lib
    J, V, W, S = spec["J"], spec["V"], spec["W"], spec["outS"]
    Y = prog.Y
    if any(ra.ptr.value != Y.ptr.value for ra in (J, V, W, S)):
        return None  # different device buffers: nothing to match offsets against
    large = {}
    for plan in prog.plans:
        if _takes_epilogue(plan):
            for b in plan.members:
                if int(Y.stride0s[b]) == 1:
                    large[(int(Y.starts[b]), int(Y.shape0s[b]))] = b
    y_spans = [iv for iv in (_span(Y, b) for b in range(len(Y))) if iv]
    matched, idle, rest = [], [], []
    for p in range(len(J)):
        b = large.get((int(J.starts[p]), int(J.shape0s[p])))
        if b is not None:
            matched.append((p, b))
        elif _span(J, p) and not _overlaps([_span(J, p)], y_spans):
            idle.append(p)
        else:
            rest.append(p)
    if not matched or len({b for _, b in matched}) != len(matched):
        return None

    # the update must not write what the launch still reads elsewhere
    fused_pops = [p for p, _ in matched] + idle
    written = [iv for ra in (V, W, S) for iv in (_span(ra, p) for p in fused_pops) if iv]
    read = []
    for g in prog.geometry:
        for d in g["dots"]:
            if prog.A.ptr.value == Y.ptr.value:
                read.append(_span(prog.A, d["a_j"]))
            if prog.X.ptr.value == Y.ptr.value:
                read.append(_span(prog.X, d["x_j"]))
    if prog.Y_in.ptr.value == Y.ptr.value:
        for b in range(len(Y)):
            if int(prog.Y_in.starts[b]) != int(Y.starts[b]):
                read.append(_span(prog.Y_in, b))
    written += y_spans  # and the currents themselves
    if _overlaps(written, [iv for iv in read if iv]):
        return None

    if idle:
        # the same GEMV with one more item per input-less population: Y = 1 * J + 0, no dots
        n_old = len(Y)
        extra = J[idle]
        none = np.zeros(0, dtype=np.int32)
        prog = type(prog)(
            queue, np.concatenate([prog.alpha, np.ones(len(idle), np.float32)]),
            prog.A, list(prog.A_js) + [none] * len(idle), prog.X, list(prog.X_js) + [none] * len(idle),
            np.concatenate([prog.beta, np.ones(len(idle), np.float32)]),
            _concat([Y, extra]), Y_in=_concat([prog.Y_in, extra]),
            gamma=np.concatenate([prog.gamma, np.zeros(len(idle), np.float32)]), tag=prog.tag,
            tile_items=range(n_old, n_old + len(idle)))
        matched = matched + [(p, n_old + k) for k, p in enumerate(idle)]
        Y = prog.Y

    # currents nobody reads are not stored, when the product that forms them can be run
    # again later with the same result: it must not read the current itself
    unread = set(unread_currents)
    lazy = [(p, b) for p, b in matched
            if p in unread and prog.geometry[b]["dots"] and (
                prog.beta[b] == 0 or _span(prog.Y_in, b) is None
                or not _overlaps([_span(prog.Y_in, b)], [_span(Y, b)]))
            and not any(_overlaps([_span(prog.X, d["x_j"])], [_span(Y, b)])
                        for d in prog.geometry[b]["dots"])]
    lazy_currents = None
    if lazy:
        sel = [b for _, b in lazy]
        lazy_prog = plan_block_gemv(
            queue, prog.alpha[sel], prog.A, [prog.A_js[b] for b in sel], prog.X,
            [prog.X_js[b] for b in sel], prog.beta[sel], Y[sel], Y_in=prog.Y_in[sel],
            gamma=prog.gamma[sel], tag="%s-currents-on-demand" % prog.tag)
        lazy_currents = ([p for p, _ in lazy], lazy_prog)
    no_store = {p for p, _ in lazy}

    cols, pptrs, keep = lif_population_table(queue, spec)
    table = np.zeros((len(Y), 8), dtype=np.int32)
    for p, b in matched:
        flags = int(cols["pflags"][p]) | LIF_POP_ENABLED | (LIF_POP_NO_J if p in no_store else 0)
        decay_bits = 0
        if not (flags & 1) and spec["upsample"] == 1 and LIF_COMPACT:
            # one time constant and no sub-steps: the decay factor of a whole step,
            # -expm1(-dt / tau) with the kernel's roundings (float quotient, expm1 in
            # double, rounded once), is the same for every neuron that is not refractory
            tau = np.int32(cols["tau"][p]).view(np.float32)
            dtu = np.float32(spec["dt"] / float(spec["upsample"]))
            quotient = np.float32(-dtu) / tau
            decay = np.float32(-np.float32(np.expm1(np.float64(quotient))))
            decay_bits = int(decay.view(np.int32))
            flags |= LIF_POP_DECAY
        table[b] = (cols["v_start"][p], cols["w_start"][p], cols["s_start"][p], decay_bits,
                    cols["tau"][p], cols["ref"][p], cols["amp"][p], flags)
    dev_pops = to_device(queue, table)
    lif_args = (dev_pops.ptr, spec["dt"], spec["upsample"], V.ptr, W.ptr, S.ptr,
                pptrs[0], pptrs[1], pptrs[2])
    pop_of = {b: p for p, b in matched}
    out = []
    for plan in prog.plans:
        if not _takes_epilogue(plan) or not any(b in pop_of for b in plan.members):
            out.append(plan)
            continue
        lif_bytes = sum(4 * int(J.shape0s[pop_of[b]]) for b in plan.members if b in pop_of)
        # (currents that are not stored are not traffic)
        unstored = sum(4 * int(J.shape0s[pop_of[b]]) for b in plan.members
                       if b in pop_of and pop_of[b] in no_store)
        entry, args, kept = _epilogue_call(lib, plan, "lif", lambda items: table[items][:, [0, 1, 7]])
        fused = Plan(queue, entry, args + lif_args, gsize=plan.gsize,
                     lsize=plan.lsize,
                     full_args=(plan.full_args + (dev_pops, V.dev_buf, W.dev_buf, S.dev_buf)
                                + tuple(keep) + kept),
                     name=plan.name + "_lif", tag=plan.tag,
                     # V and W in and out, spikes out
                     bw_per_call=plan.bw_per_call + 5 * lif_bytes - unstored,
                     flops_per_call=plan.flops_per_call)
        fused.description = plan.description
        fused.kernel_class, fused.n_tasks = plan.kernel_class, plan.n_tasks
        fused.members, fused.prog = plan.members, prog
        fused.gemv_bytes = plan.bw_per_call - unstored
        fused.host_pops = table
        fused.dev_pops = dev_pops
        fused.lif_written = [V, W, S]
        fused.lazy_currents = lazy_currents
        if plan.kernel_class[0] == 3:
            fused.host_tasks = plan.host_tasks
        else:  # small items: 16-word records as the launch takes them, or the 4-word table
            fused.host_tasks = getattr(plan, "epilogue_tasks", None)
            fused.host_tables = plan.host_tables
        out.append(fused)
    if rest:
        out.append(plan_lif(queue, spec["dt"], J[rest], V[rest], W[rest], S[rest],
                            _subset_param(spec["ref"], rest), _subset_param(spec["tau"], rest),
                            _subset_param(spec["amp"], rest), upsample=spec["upsample"],
                            tag=lif_plan.tag))
    return out


def fuse_input_sums(sum_plan, lif_plan):
    """One launch less for "x = sum of vectors; J = E x; LIF(J)": the launch with the LIF
    epilogue (`fuse_lif`) forms the vector operands it needs itself, when the small-item
    launch `sum_plan` right before it does nothing but form them.

    Fused when every item of `sum_plan` is ``Y = 0 * Y + 0 + sum_k v_k * s_k`` (one-column
    dot products: vectors times scalars, alpha = 1) of at most 64 elements with stride 1,
    is the vector operand of the FIRST dot product of an item of `lif_plan` and of nothing
    else in that GEMV, and no part ``v_k`` / ``s_k`` is something either launch writes; all
    in one device buffer.  `lif_plan` is a launch of the large-item kernel with compile-time
    shapes (a first dot product of at most 64 columns), or of the small-item kernel when no
    dot product of the launch has more than 4 columns (ensembles of one to four
    dimensions).  Sums that nothing in the launch reads become items without dot products.  The sums are formed with
    the roundings and in the order of the small-item kernel and stored where it stores them,
    so results are bit-identical as long as the sums' old values are finite (the 0 * Y
    term is not formed).  Returns the plan that replaces ``[sum_plan, lif_plan]``, or None.
    """
    S, E = getattr(sum_plan, "prog", None), getattr(lif_plan, "prog", None)
    if S is None or E is None or sum_plan.name != "hipra_gemv.wave_ref":
        return None
    large = (lif_plan.name == "hipra_gemv.tile_lif" and lif_plan.kernel_class[0] == 3
             and lif_plan.kernel_class[1] >= 2 and getattr(lif_plan, "host_tasks", None) is not None)
    small = (lif_plan.name == "hipra_gemv.wave_ref_lif" and lif_plan.kernel_class[0] == 2
             and getattr(lif_plan, "host_tables", None) is not None)
    if not (large or small):
        return None
    if small and any(d["a_shape1"] > 4 for b in lif_plan.members for d in E.geometry[b]["dots"]):
        return None  # the small-item kernel forms sums on its path for narrow dot products only
    queue, lib = E.queue, E.queue.lib
    buf = E.X.ptr.value
    if any(ra.ptr.value != buf for ra in (S.A, S.X, S.Y, S.Y_in, E.Y)):
        return None
    # the sums: start -> (length, parts)
    sums = {}
    for b in sum_plan.members:
        g = S.geometry[b]
        if (S.alpha[b] != 1 or S.beta[b] != 0 or S.gamma[b] != 0 or g["y_stride0"] != 1
                or g["y_in_start"] != g["y_start"] or not 1 <= g["y_len"] <= 64
                or not g["dots"] or g["y_start"] in sums):
            return None
        if any(d["a_shape1"] != 1 or (d["a_stride0"] != 1 and g["y_len"] > 1) for d in g["dots"]):
            return None
        sums[g["y_start"]] = (g["y_len"], [(d["a_start"], d["x_start"]) for d in g["dots"]])
    sum_spans = sorted((lo, lo + n) for lo, (n, _) in sums.items())
    # every dot product of the GEMV that touches a sum is the first one of an item of this
    # launch, reads the whole sum with stride 1, and has a single column stage
    used = set()
    members = set(lif_plan.members)
    for g in E.geometry:
        for k, d in enumerate(g["dots"]):
            span = (d["x_start"], d["x_start"] + (d["a_shape1"] - 1) * d["x_stride0"] + 1)
            if not _overlaps([span], sum_spans):
                continue
            want = sums.get(d["x_start"])
            if (k != 0 or g["index"] not in members or want is None or want[0] != d["a_shape1"]
                    or (d["x_stride0"] != 1 and d["a_shape1"] > 1)
                    or stream_stage(d["a_shape1"])[0] > 6):
                return None
            used.add(d["x_start"])
        # (matrices and old outputs that overlap a sum would be read while it is written)
        if _overlaps([(g["y_in_start"], g["y_in_start"] + (g["y_len"] - 1) * g["y_in_stride0"] + 1)],
                     sum_spans) and E.Y_in.ptr.value == buf:
            return None
    spare = sorted(set(sums) - used)  # sums nothing here reads: tasks of their own, below
    if not used:
        return None
    if E.A.ptr.value == buf and _overlaps(
            [iv for g in E.geometry for d in g["dots"] for iv in [_span(E.A, d["a_j"])] if iv],
            sum_spans):
        return None
    # no part is written by either launch
    written = list(sum_spans) + [iv for iv in (_span(E.Y, b) for b in lif_plan.members) if iv]
    for ra in getattr(lif_plan, "lif_written", ()):
        if ra.ptr.value == buf:
            written += [iv for iv in (_span(ra, p) for p in range(len(ra))) if iv]
    part_spans = [(a, a + n) for n, parts in sums.values() for a, _ in parts]
    part_spans += [(x, x + 1) for _, parts in sums.values() for _, x in parts]
    if _overlaps(part_spans, written):
        return None

    part_rows, where = [], {}
    for start, (_, parts) in sums.items():
        where[start] = (len(part_rows), len(parts))
        part_rows.extend(parts)
    dev_parts = to_device(queue, np.array(part_rows, dtype=np.int32))
    args = tuple(lif_plan.args)
    sum_bytes = sum_plan.bw_per_call or 0
    one = np.array([1.0, 0.0, 0.0, 0.0], dtype=np.float32).view(np.int32)
    new_pops = lif_plan.host_pops
    if large:
        tasks = lif_plan.host_tasks.copy()  # 24-word records: task, item, coefficients, first dot
        for row in tasks:
            if row[9] > 0 and int(row[19]) in where:  # has dot products; x_start of the first
                row[3], row[11] = where[int(row[19])]
        keep = ()
        if spare:
            # one task each, of an item without dot products and without neurons: Y = the sum
            pops = np.concatenate([lif_plan.host_pops, np.zeros((1, 8), dtype=np.int32)])
            extra = np.zeros((len(spare), 24), dtype=np.int32)
            for row, start in zip(extra, spare):
                first, count = where[start]
                row[0:4] = (len(pops) - 1, 0, sums[start][0], first)
                row[4:12] = (start, 1, start, 1, 0, 0, sums[start][0], count)
                row[12:16] = one
            tasks = np.concatenate([tasks, extra])
            dev_pops = to_device(queue, pops)
            new_pops = pops
            args = args[:12] + (dev_pops.ptr,) + args[13:]
            keep = (dev_pops,)
        tasks = spread_over_dies(tasks)
        dev_tasks = to_device(queue, tasks)
        n_groups = -(-len(tasks) // (WG // WAVE))
        args = args[:6] + (dev_tasks.ptr, len(tasks)) + args[8:] + (dev_parts.ptr,)
        entry = lib.nhip_gemv_tile_lif_sums
        keep = keep + (dev_tasks, dev_parts)
    else:
        # (lpr, task words, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y, pops, ...): the
        # ranges of parts go by item; sums nothing reads become items without dot products
        lpr, task_words = args[0], args[1]
        item_tab, coef_tab, plain_tasks = lif_plan.host_tables
        n_items = len(item_tab)
        tasks = (lif_plan.host_tasks if task_words == 16 else plain_tasks).copy()
        items = np.concatenate([item_tab, np.zeros((len(spare), 8), dtype=np.int32)])
        coefs = np.concatenate([coef_tab, np.zeros((len(spare), 4), dtype=np.float32)])
        pops = np.concatenate([lif_plan.host_pops[:n_items],
                               np.zeros((len(spare), 8), dtype=np.int32)])
        ranges = np.zeros((len(items), 2), dtype=np.int32)
        for b in lif_plan.members:
            dots = E.geometry[b]["dots"]
            if dots and dots[0]["x_start"] in where:
                ranges[b] = where[dots[0]["x_start"]]
        extra = []
        for k, start in enumerate(spare):
            b, n = n_items + k, sums[start][0]
            items[b] = (start, 1, start, 1, 0, 0, n, 0)
            coefs[b] = (1.0, 0.0, 0.0, 0.0)
            ranges[b] = where[start]
            if lpr == WAVE:  # a wave takes a task of up to 64 rows: the whole sum
                extra.append(np.concatenate([[b, 0, n, 0], items[b], one]).astype(np.int32))
                extra[-1][15] = 0
                continue
            for r in range(n):
                if task_words == 16:
                    extra.append(np.concatenate([[b, r, 1, 0], items[b], one]).astype(np.int32))
                    extra[-1][15] = 0
                else:
                    extra.append(np.array([b, r, 1, 0], dtype=np.int32))
        if extra:
            tasks = np.concatenate([tasks, np.array(extra, dtype=np.int32)])
        dev = [to_device(queue, t) for t in (items, coefs, tasks, pops, ranges)]
        rows_per_group = (WG // WAVE) * (WAVE // lpr)
        n_groups = -(-len(tasks) // rows_per_group)
        args = (lpr, task_words, dev[0].ptr, dev[1].ptr, args[4], dev[2].ptr, len(tasks)) + args[7:11] \
            + (dev[3].ptr,) + args[12:] + (dev[4].ptr, dev_parts.ptr)
        entry = lib.nhip_gemv_rows_lif_sums
        keep = tuple(dev) + (dev_parts,)
    fused = Plan(queue, entry, args, gsize=(WG * n_groups,), lsize=lif_plan.lsize,
                 full_args=tuple(lif_plan.full_args) + keep,
                 name=lif_plan.name, tag=lif_plan.tag,
                 bw_per_call=lif_plan.bw_per_call + sum_bytes,
                 flops_per_call=(lif_plan.flops_per_call or 0) + (sum_plan.flops_per_call or 0))
    fused.description = lif_plan.description + "; input sums: " + sum_plan.description
    fused.kernel_class, fused.n_tasks = lif_plan.kernel_class, len(tasks)
    fused.members, fused.prog = lif_plan.members, E
    fused.gemv_bytes = getattr(lif_plan, "gemv_bytes", lif_plan.bw_per_call)
    fused.host_tasks = tasks
    fused.input_sums = len(sums)
    fused.lazy_currents = getattr(lif_plan, "lazy_currents", None)
    fused.host_pops = new_pops if large else pops
    # (the device copy of the table, where it is the one the launch reads: large items)
    fused.dev_pops = (dev_pops if spare else getattr(lif_plan, "dev_pops", None)) if large else None
    return fused


def _learning_apart(which):
    logger.debug("fuse_learning: check %d did not hold", which)
    return None


def store_spikes_as_bits(enc_plan, items, event_records, dt):
    """Populations of a `tile_lif` launch whose spikes only launches that visit active columns
    read: the launch leaves one bit per neuron in the first words of the spike signal's memory
    instead of a float per neuron (`LIF_POP_BITS`), and the records of the reading launches say
    so (their `x_bits` word: the one value a spike has, amplitude / dt rounded as the neuron
    update rounds it).  `items`: rows of the launch's population table; `event_records`:
    ``{item: [(event plan, record index), ...]}``.  Returns ``{item: spike value}``.  The
    caller has checked that nothing else reads those spikes."""
    pops = enc_plan.host_pops
    dt_inv = np.float32(1.0 / dt)
    values = {}
    touched = []
    for b in items:
        amp = np.array([pops[b, 6]], dtype=np.int32).view(np.float32)[0]
        value = np.float32(amp * dt_inv)  # (__fmul_rn of two floats)
        if not np.isfinite(value) or value == 0:
            continue
        pops[b, 7] |= LIF_POP_BITS
        values[b] = value
        for plan, k in event_records[b]:
            plan.event_table[k, 15] = int(np.array([value], dtype=np.float32).view(np.int32)[0])
            if plan not in touched:
                touched.append(plan)
        n = int(sum(int(row[2]) for row in enc_plan.host_tasks if row[0] == b))
        if enc_plan.bw_per_call:
            enc_plan.bw_per_call -= 4 * n - n // 8
    if values:
        enc_plan.dev_pops.set(pops.astype(np.int32).ravel())
        for plan in touched:
            plan.dev_event_table.set(plan.event_table.astype(np.int32).ravel())
        enc_plan.tag = "%s + spikes as bits" % enc_plan.tag
    return values


def fuse_learning(enc_plan, dec_plan, ew_plan, lf_plan):
    """A step that ends with an outer-product learning rule -- ``W += (alpha e) (x) f`` and
    then ``f <- filter(spikes)`` (the reference: `_plan_SimPES`, simulator.py:1334-1345, with
    the copy that adds the result, and the `plan_linearfilter` of the rule's pre-synaptic
    synapse) -- without a launch for either:

    * the launch that decodes with the learned matrices (`dec_plan`, large items with the
      filter epilogue) writes every block of such a matrix back with the change added once
      the block has gone into its sums (``nhip_gemv_tile_filter_learn``): the matrix is read
      once per step;
    * the filters of the activities ``f`` are stepped by the NEXT step's launch that updates
      the neurons (`enc_plan`, large items with the LIF epilogue,
      ``nhip_gemv_tile_lif_deferred``), by the task that is about to replace the spikes they
      read.  Between steps ``f`` then holds the value from before the pending filter step.

    Fused when every outer product's matrix is the only matrix of an item of `dec_plan`
    (same start, shape and row stride; tasks of at most 64 rows; whole aligned quads), its
    row and column operands are contiguous vectors, every filter of `lf_plan` whose output is
    such a column operand reads exactly the spikes of a population of `enc_plan` and has one
    numerator and at most one denominator coefficient.  The caller checks what only it knows:
    that nothing else reads ``f``, that ``f`` and the spikes start at zero, and that no plan in
    between touches what moves.  Returns ``(new enc_plan, new dec_plan, plans for the filters
    that stay, {f start: (spike start, a0 bits or None, b0 bits, length)})`` or None.
    """
    from .hipra_nonlinearities import plan_linearfilter

    ew, lf = getattr(ew_plan, "ew_spec", None), getattr(lf_plan, "lf_spec", None)
    if ew is None or lf is None or not ew.get("outer") or not ew.get("inc"):
        return _learning_apart(1)
    if (enc_plan.name != "hipra_gemv.tile_lif" or tuple(enc_plan.kernel_class) != (3, 3, 4)
            or dec_plan.name != "hipra_gemv.tile_filter" or tuple(dec_plan.kernel_class) != (3, 2, 4)
            or getattr(dec_plan, "host_tasks", None) is None
            or getattr(enc_plan, "host_pops", None) is None):
        return _learning_apart(2)
    E, Fv, Wm, alphas = ew["A"], ew["X"], ew["Y"], ew["alphas"]
    S, F, FA, FB = lf["X"], lf["Y"], lf["A"], lf["B"]
    D = dec_plan.prog
    queue, lib = D.queue, D.queue.lib
    buf = D.A.ptr.value
    if any(ra.ptr.value != buf for ra in (E, Fv, Wm, S, F, D.X, D.Y, enc_plan.prog.Y)):
        return _learning_apart(3)
    # the matrices: each the only dot product of one item of the decoding launch
    by_matrix = {}
    for b in dec_plan.members:
        g = D.geometry[b]
        if len(g["dots"]) == 1:
            d = g["dots"][0]
            by_matrix[(d["a_start"], g["y_len"], d["a_shape1"], d["a_stride0"])] = b
    tasks = dec_plan.host_tasks
    learn_of_item = {}
    for i in range(len(Wm)):
        rows, cols = int(Wm.shape0s[i]), int(Wm.shape1s[i])
        key = (int(Wm.starts[i]), rows, cols, int(Wm.stride0s[i]) if rows > 1 else cols)
        b = by_matrix.get(key)
        if b is None or b in learn_of_item or int(Wm.stride1s[i]) != 1:
            return _learning_apart(4)
        if (key[0] | key[3] | cols) & 3 or cols < 512:  # aligned quads; the 512-column stages
            return _learning_apart(5)
        if not (int(E.shape0s[i]) == rows and (rows == 1 or int(E.stride0s[i]) == 1)
                and int(E.shape1s[i]) == 1 and int(Fv.shape0s[i]) == cols
                and int(Fv.stride0s[i]) == 1 and int(Fv.shape1s[i]) == 1
                and int(Fv.starts[i]) % 4 == 0):
            return _learning_apart(6)
        alpha = np.float32(alphas[i])
        learn_of_item[b] = (int(E.starts[i]), int(Fv.starts[i]), int(alpha.view(np.int32)), 1)
    if not learn_of_item or int(tasks[np.isin(tasks[:, 0], list(learn_of_item)), 2].max()) > WAVE:
        return _learning_apart(7)
    learn = np.zeros((len(tasks), 4), dtype=np.int32)
    for t, item in enumerate(tasks[:, 0]):
        if int(item) in learn_of_item:
            learn[t] = learn_of_item[int(item)]
    # the filters: those whose output is a column operand move to the neuron launch
    f_operands = {(int(Fv.starts[i]), int(Fv.shape0s[i])) for i in range(len(Wm))}
    pops = enc_plan.host_pops
    enc_geo = enc_plan.prog.geometry
    by_spikes = {(int(pops[b][2]), enc_geo[b]["y_len"]): b for b in enc_plan.members
                 if b < len(pops) and pops[b][7] & LIF_POP_ENABLED}
    a_host, b_host = FA.to_host(), FB.to_host()
    deferred = np.zeros((len(pops), 4), dtype=np.int32)
    moved, rest, pending = [], [], {}
    for k in range(len(F)):
        out = (int(F.starts[k]), int(F.shape0s[k]))
        if out not in f_operands:
            rest.append(k)
            continue
        simple = int(FB.shape0s[k]) == 1 and int(FA.shape0s[k]) <= 1
        vector = all(int(r.shape1s[k]) == 1 and int(r.stride0s[k]) == 1 for r in (S, F))
        b = by_spikes.get((int(S.starts[k]), int(S.shape0s[k]))) if simple and vector else None
        if b is None or deferred[b][3] or int(S.shape0s[k]) != out[1]:
            return _learning_apart(8)
        na = int(FA.shape0s[k])
        a0 = np.float32(a_host[k][0, 0]) if na else np.float32(0)
        b0 = np.float32(b_host[k][0, 0])
        deferred[b] = (out[0], int(a0.view(np.int32)), int(b0.view(np.int32)), 1 | (2 if na else 0))
        pending[out[0]] = (int(S.starts[k]), int(a0.view(np.int32)) if na else None,
                           int(b0.view(np.int32)), out[1])
        moved.append(k)
    if len(moved) != len(f_operands):
        return _learning_apart(9)  # a column operand that no filter of this plan produces: leave it all alone

    dev_learn, dev_deferred = to_device(queue, learn), to_device(queue, deferred)
    new_dec = Plan(queue, lib.nhip_gemv_tile_filter_learn, tuple(dec_plan.args) + (dev_learn.ptr,),
                   gsize=dec_plan.gsize, lsize=dec_plan.lsize,
                   full_args=tuple(dec_plan.full_args) + (dev_learn,) + tuple(ew_plan.full_args),
                   name=dec_plan.name, tag="%s + learning" % dec_plan.tag,
                   # the matrices are read by the decoding anyway: the update adds their write
                   # and its two vectors
                   bw_per_call=(dec_plan.bw_per_call or 0) + sum(
                       4 * int(Wm.shape0s[i]) * int(Wm.shape1s[i]) + 4 * int(Wm.shape0s[i])
                       + 4 * int(Wm.shape1s[i]) for i in range(len(Wm))),
                   flops_per_call=(dec_plan.flops_per_call or 0) + (ew_plan.flops_per_call or 0))
    enc_args = tuple(enc_plan.args)
    if getattr(enc_plan.kern, "__name__", "") == "nhip_gemv_tile_lif":
        enc_args += (None,)  # no input sums: no parts table
    elif getattr(enc_plan.kern, "__name__", "") != "nhip_gemv_tile_lif_sums":
        return _learning_apart(10)
    new_enc = Plan(queue, lib.nhip_gemv_tile_lif_deferred, enc_args + (dev_deferred.ptr, F.ptr),
                   gsize=enc_plan.gsize, lsize=enc_plan.lsize,
                   full_args=tuple(enc_plan.full_args) + (dev_deferred, F.dev_buf),
                   name=enc_plan.name, tag="%s + activity filters" % enc_plan.tag,
                   bw_per_call=(enc_plan.bw_per_call or 0) + sum(12 * int(F.shape0s[k]) for k in moved),
                   flops_per_call=enc_plan.flops_per_call)
    for new, old in ((new_dec, dec_plan), (new_enc, enc_plan)):
        for attr in ("description", "kernel_class", "n_tasks", "members", "prog", "gemv_bytes",
                     "host_tasks", "host_pops", "dev_pops", "lif_written", "lazy_currents",
                     "input_sums"):
            if hasattr(old, attr):
                setattr(new, attr, getattr(old, attr))
    new_dec.learned_matrices = len(learn_of_item)
    new_enc.deferred_filters = len(moved)
    residual = []
    if rest:
        residual = plan_linearfilter(queue, S[rest], F[rest], FA[rest], FB[rest],
                                     lf["Xbuf"][rest], lf["Ybuf"][rest], tag=lf_plan.tag)
        residual[0].unfused_items = list(rest)
    return new_enc, new_dec, residual, pending


def _read_spans(prog, ptr_value):
    """Element intervals a GEMV reads through A, X and a Y_in that is not its Y, in
    the device buffer at `ptr_value`."""
    read = []
    for g in prog.geometry:
        for d in g["dots"]:
            if prog.A.ptr.value == ptr_value:
                read.append(_span(prog.A, d["a_j"]))
            if prog.X.ptr.value == ptr_value:
                read.append(_span(prog.X, d["x_j"]))
    if prog.Y_in.ptr.value == ptr_value:
        for b in range(len(prog.Y)):
            if (int(prog.Y_in.starts[b]) != int(prog.Y.starts[b])
                    or prog.Y_in.ptr.value != prog.Y.ptr.value):
                read.append(_span(prog.Y_in, b))
    return [iv for iv in read if iv]


def fuse_linearfilter(gemv_plans, lf_plan):
    """Fewer launches for "Y = GEMV(...); filter step on Y" (clra_gemv.py
    `plan_block_gemv` followed by clra_nonlinearities.py `plan_linearfilter`): the
    reference-order kernels step the first-order filters whose input is one of their
    output items as soon as a row is final.

    `gemv_plans` are the plans of one GEMV (one `gemv_prog`).  A filter item is fused
    when it has one numerator and at most one denominator coefficient, its input is
    exactly the output of an item of a reference-order launch without another
    epilogue, and both vectors are contiguous.  Returns ``(plans replacing gemv_plans,
    plans replacing [lf_plan])`` -- the second list holds a filter launch for the items
    that were not fused (their indices in `lf_plan`: its ``unfused_items``), or is empty
    -- or None when nothing can be fused.
    """
    from .hipra_nonlinearities import plan_linearfilter

    spec = getattr(lf_plan, "lf_spec", None)
    if spec is None or not gemv_plans:
        return None
    prog = gemv_plans[0].prog
    queue, lib = prog.queue, prog.queue.lib
    X, F, A, B = spec["X"], spec["Y"], spec["A"], spec["B"]
    Y = prog.Y
    if X.ptr.value != Y.ptr.value:
        return None
    large = {}
    for plan in gemv_plans:
        if _takes_filters(plan):
            for b in plan.members:
                if int(Y.stride0s[b]) == 1:
                    large[(int(Y.starts[b]), int(Y.shape0s[b]))] = b
    if not large:
        return None
    a_host, b_host = A.to_host(), B.to_host()
    targets_of = defaultdict(list)
    rest = []
    for i in range(len(X)):
        simple = int(B.shape0s[i]) == 1 and int(A.shape0s[i]) <= 1
        vector = (int(X.shape1s[i]) == 1 and int(X.stride0s[i]) == 1
                  and int(F.shape1s[i]) == 1 and int(F.stride0s[i]) == 1)
        b = large.get((int(X.starts[i]), int(X.shape0s[i]))) if simple and vector else None
        if b is None:
            rest.append(i)
            continue
        na = int(A.shape0s[i])
        a0 = np.float32(a_host[i][0, 0]) if na else np.float32(0)
        b0 = np.float32(b_host[i][0, 0])
        targets_of[b].append((int(F.starts[i]), int(a0.view(np.int32)), int(b0.view(np.int32)), na))
    if not targets_of:
        return None
    fused_filters = [i for i in range(len(X)) if i not in set(rest)]
    written = [iv for iv in (_span(F, i) for i in fused_filters) if iv]
    if _overlaps(written, _read_spans(prog, F.ptr.value)):
        return None
    if F.ptr.value == Y.ptr.value and _overlaps(
            written, [iv for iv in (_span(Y, b) for b in range(len(Y))) if iv]):
        return None

    item_targets = np.zeros((len(Y), 2), dtype=np.int32)
    target_rows = []
    for b, rows in sorted(targets_of.items()):
        item_targets[b] = (len(target_rows), len(rows))
        target_rows.extend(rows)
    dev_items = to_device(queue, item_targets)
    dev_targets = to_device(queue, np.array(target_rows, dtype=np.int32))
    extra = (dev_items.ptr, dev_targets.ptr, F.ptr)
    out = []
    for plan in gemv_plans:
        if not _takes_filters(plan) or not any(b in targets_of for b in plan.members):
            out.append(plan)
            continue
        f_bytes = sum(8 * int(Y.shape0s[b]) * len(targets_of[b]) for b in plan.members
                      if b in targets_of)  # filter state in and out
        if plan.kernel_class[0] == 4:
            # the launch that visits only the columns with x != 0: an item's range of
            # targets goes into its record
            table = plan.event_table.copy()
            table[:, 12:14] = item_targets[plan.event_record_item]
            dev_table = to_device(queue, table)
            fused = Plan(queue, lib.nhip_gemv_events,
                         (dev_table.ptr,) + tuple(plan.args[1:6]) + (dev_targets.ptr, F.ptr,
                                                                      plan.args[8]),
                         gsize=plan.gsize, lsize=plan.lsize,
                         full_args=plan.full_args + (dev_table, dev_targets, F.dev_buf),
                         name=plan.name + "_filter", tag=plan.tag,
                         bw_per_call=plan.bw_per_call + f_bytes,
                         flops_per_call=plan.flops_per_call)
            fused.description = plan.description
            fused.kernel_class, fused.n_tasks = plan.kernel_class, plan.n_tasks
            fused.members, fused.prog = plan.members, prog
            fused.gemv_bytes = plan.bw_per_call
            fused.event_table, fused.event_driven = table, True
            fused.dev_event_table = dev_table
            fused.event_record_item = plan.event_record_item
            fused.host_tasks = None
            out.append(fused)
            continue
        entry, args, keep = _epilogue_call(
            lib, plan, "filter",
            lambda items: np.column_stack([item_targets[items], np.zeros(len(items), np.int32)]))
        if plan.kernel_class[0] == 3:
            # the large-item kernel finds an item's range of targets in the spare
            # fields of its task records (one read less before it can start)
            tasks = plan.host_tasks.copy()
            tasks[:, 3] = item_targets[tasks[:, 0], 0]
            tasks[:, 11] = item_targets[tasks[:, 0], 1]
            dev_tasks = to_device(queue, tasks)
            at = 6  # (vec, pow2, words, items, coefs, dots, tasks, ...)
            args = tuple(args[:at]) + (dev_tasks.ptr,) + tuple(args[at + 1:])
            keep = (dev_tasks,)
        fused = Plan(queue, entry, args + extra, gsize=plan.gsize,
                     lsize=plan.lsize,
                     full_args=plan.full_args + (dev_items, dev_targets, F.dev_buf) + keep,
                     name=plan.name + "_filter", tag=plan.tag,
                     bw_per_call=plan.bw_per_call + f_bytes, flops_per_call=plan.flops_per_call)
        fused.description = plan.description
        fused.kernel_class, fused.n_tasks = plan.kernel_class, plan.n_tasks
        fused.members, fused.prog = plan.members, prog
        fused.gemv_bytes = plan.bw_per_call
        if plan.kernel_class[0] == 3:
            fused.host_tasks = tasks
        out.append(fused)
    residual = []
    if rest:
        residual = plan_linearfilter(queue, X[rest], F[rest], A[rest], B[rest],
                                     spec["Xbuf"][rest], spec["Ybuf"][rest], tag=lf_plan.tag)
        residual[0].unfused_items = list(rest)
    return out, residual
