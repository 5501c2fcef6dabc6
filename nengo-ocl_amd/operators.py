"""Graph rewrites that feed the ragged GEMV: MultiDotInc and op simplification.

Counterpart of the reference's ``nengo_ocl/operators.py``: ``MultiDotInc``
(:19-194: ``convert_to`` :51, ``compress`` :112, ``get_views`` :159),
``signal_io_dicts`` (:197), ``remove_unmodified_resets`` (:226),
``remove_zero_incs`` (:265), ``simplify_operators`` / ``simplifications``
(:334-350).  Operator kinds are recognised by class name so that operators
built by nengo and by `ir` are treated alike.
"""

import numpy as np

from . import ir


def _is(op, name):
    return type(op).__name__ == name


class MultiDotInc(ir.Operator):
    r"""``Y <- gamma + beta * Y_in + \sum_i dot(A_i, X_i)``"""

    def __init__(self, Y, Y_in, beta, gamma, tag=None):
        super().__init__(tag=tag)
        if Y.ndim != 1:
            raise ValueError("Y must be a vector")
        if Y.shape != Y_in.shape:
            raise TypeError("Y and Y_in differ in shape")
        self.Y, self.Y_in = Y, Y_in

        if hasattr(beta, "shape") and hasattr(beta, "base"):  # a Signal
            if beta.shape != Y.shape:
                raise NotImplementedError("", (beta.shape, Y.shape))
            self._float_beta, self._signal_beta = None, beta
        else:
            self._float_beta = float(getattr(beta, "value", beta))
            self._signal_beta = None

        self.gamma = float(gamma)
        self.As, self.Xs = [], []
        self._incs_Y = self._signal_beta is None and self._float_beta == 1 and Y_in is Y

    @classmethod
    def convert_to(cls, op):
        """A plain DotInc becomes ``MultiDotInc(Y, Y, beta=1, gamma=0)`` with one pair."""
        if _is(op, "BsrDotInc"):
            raise NotImplementedError("BsrDotInc operations are not supported")
        if not _is(op, "DotInc"):
            return op
        new = cls(op.Y, op.Y, beta=1, gamma=0, tag=op.tag)
        new.add_AX(op.A, op.X)
        assert set(op.reads).issuperset(new.reads)
        assert list(new.incs) == list(op.incs) and list(new.sets) == list(op.sets)
        assert all(s.size for s in new.all_signals), op
        return new

    def add_AX(self, A, X):
        if X.ndim != 1:
            raise ValueError("X must be a vector")
        self.As.append(A)
        self.Xs.append(X)

    # sets / incs / reads are derived from the current state
    @property
    def reads(self):
        r = list(self.As) + list(self.Xs)
        if not self._incs_Y:
            if self._signal_beta is not None:
                r.append(self._signal_beta)
                if self.Y_in is not self.Y:
                    r.append(self.Y_in)
            elif self._float_beta != 0 and self.Y_in is not self.Y:
                r.append(self.Y_in)
        return r

    @reads.setter
    def reads(self, value):
        pass

    @property
    def incs(self):
        return [self.Y] if self._incs_Y else []

    @incs.setter
    def incs(self, value):
        pass

    @property
    def sets(self):
        return [] if self._incs_Y else [self.Y]

    @sets.setter
    def sets(self, value):
        pass

    @property
    def updates(self):
        return []

    @updates.setter
    def updates(self, value):
        pass

    def __repr__(self):
        beta = self._float_beta if self._signal_beta is None else self._signal_beta
        dots = ", ".join("dot(%s, %s)" % (A, X) for A, X in zip(self.As, self.Xs))
        return "<MultiDotInc(tag=%s, Y=%s, Y_in=%s, beta=%s, gamma=%s, dots=[%s]) at 0x%x>" % (
            self.tag, self.Y, self.Y_in, beta, self.gamma, dots, id(self))

    @classmethod
    def compress(cls, operators):
        """Merge MultiDotIncs that write the same Signal object into one op.

        Increments are folded into the op that sets the same signal, if any;
        the remaining increments on one signal are folded together.  Other
        operators keep their order and come first, as in the reference.
        """
        setters, incrementers, rest = {}, {}, []
        for op in operators:
            if not isinstance(op, cls):
                rest.append(op)
            elif op.sets:
                assert len(op.sets) == 1 and not op.incs
                setters.setdefault(op.sets[0], []).append(op)
            else:
                assert len(op.incs) == 1 and not op.sets
                incrementers.setdefault(op.incs[0], []).append(op)

        for view, set_ops in setters.items():
            (set_op,) = set_ops
            for inc_op in incrementers.pop(view, []):
                set_op.As.extend(inc_op.As)
                set_op.Xs.extend(inc_op.Xs)
            rest.append(set_op)

        for view, inc_ops in incrementers.items():
            first = inc_ops[0]
            for other in inc_ops[1:]:
                first.As.extend(other.As)
                first.Xs.extend(other.Xs)
            rest.append(first)
        return rest

    @staticmethod
    def _as2d(view):
        if view.ndim == 0:
            return view.reshape(1, 1)
        if view.ndim == 1:
            return view.reshape(view.shape[0], 1)
        if view.ndim == 2:
            return view
        raise ValueError("No support for tensors with %d dimensions" % view.ndim)

    def get_views(self):
        """2-D views ``(A_views, X_views, Y, Y_in, beta)`` in kernel orientation.

        A vector A with a vector X is a 1 x n row; a 1 x 1 (scalar) A is swapped
        with its X, so ``y += a * x`` runs as the GEMV ``x[n x 1] @ a[1]``.
        """
        Y_view, Y_in_view = self._as2d(self.Y), self._as2d(self.Y_in)
        beta_view = None if self._signal_beta is None else self._as2d(self._signal_beta)
        A_views, X_views = [], []
        for A, X in zip(self.As, self.Xs):
            X_view = self._as2d(X)
            A_view = A.reshape((1, A.shape[0])) if (A.ndim == 1 and X.ndim == 1) else self._as2d(A)
            if A_view.shape == (1, 1):
                A_view, X_view = X_view, A_view
            elif not (X_view.shape[0] == A_view.shape[1] and X_view.shape[1] == Y_view.shape[1]
                      and A_view.shape[0] == Y_view.shape[0]):
                raise ValueError("shape mismach (A: %s, X: %s, Y: %s)" % (A.shape, X.shape, self.Y.shape))
            A_views.append(A_view)
            X_views.append(X_view)
        return A_views, X_views, Y_view, Y_in_view, beta_view


def signal_io_dicts(operators):
    """Four dicts base-signal -> [ops that set / inc / read / update part of it]."""
    bases = {s.base for op in operators for s in op.all_signals}
    sets, incs, reads, updates = ({b: [] for b in bases} for _ in range(4))
    for op in operators:
        for table, sigs in ((sets, op.sets), (incs, op.incs), (reads, op.reads), (updates, op.updates)):
            for s in sigs:
                table[s.base].append(op)
    return sets, incs, reads, updates


def _overwrite_initial_value(sig, value):
    arr = sig.initial_value
    owner = sig.base.initial_value
    owner.setflags(write=True)
    arr.setflags(write=True)
    arr[...] = value
    arr.setflags(write=False)
    owner.setflags(write=False)


def remove_unmodified_resets(operators):
    """Drop every Reset whose target is never incremented or updated: the reset
    value becomes the signal's initial value instead."""
    _, incs, _, updates = signal_io_dicts(operators)
    kept = []
    for op in operators:
        if _is(op, "Reset") and not incs[op.dst.base] and not updates[op.dst.base]:
            _overwrite_initial_value(op.dst, op.value)
        else:
            kept.append(op)
    return kept


def remove_zero_incs(operators):
    """Drop DotInc / ElementwiseInc / Copy / ConvInc ops with an input known to be
    zero forever (only written by a ``Reset(0)``, or constant zero).  A dropped op
    that *set* its target is replaced by a Reset of that target.  Node outputs are
    never treated as constant."""

    def constant_zero(sig):
        data = sig.initial_value
        if getattr(sig, "sparse", False):
            data = data.tocoo().data if hasattr(data, "tocoo") else data.data
        return np.all(np.asarray(data) == 0)

    sets, incs, _, updates = signal_io_dicts(operators)
    kept = []
    for op in operators:
        if type(op).__name__ not in ("DotInc", "ElementwiseInc", "Copy", "ConvInc"):
            kept.append(op)
            continue
        for src in op.reads:
            if str(src.name).startswith("<Node"):
                continue
            writers = sets[src.base] + incs[src.base] + updates[src.base]
            if len(writers) == 1:
                w = writers[0]
                zero = _is(w, "Reset") and np.all(w.value == 0)
            else:
                zero = len(writers) == 0 and constant_zero(src)
            if zero:
                if len(op.sets) > 0:
                    kept.append(_make_reset(op, op.sets[0]))
                break
        else:
            kept.append(op)
    return kept


def _make_reset(like, dst):
    """A Reset of the same family (nengo's or `ir`'s) as operator ``like``."""
    if type(like).__module__.startswith("nengo."):
        from nengo.builder.operator import Reset

        return Reset(dst)
    return ir.Reset(dst)


def fuse_into_multidotinc(operators):
    """Express vector copies and resets that surround a GEMV as part of that GEMV.

    ``MultiDotInc`` computes ``Y = beta*Y_in + gamma + sum_i A_i @ X_i`` with
    ``Y_in`` allowed to differ from ``Y``; three common operator patterns are
    special cases of it and are rewritten so that `MultiDotInc.compress` can
    fold them into one operator per target (one kernel work item instead of
    several dependent launches):

    * ``Copy(src -> dst[slice], inc=True)`` on vectors is ``dst[slice] += src * 1``:
      a MultiDotInc with the pair ``(A = scalar one, X = src)`` (the scalar-A
      form of `get_views`).  All increments into one target then merge, where
      the planner would otherwise run colliding increments one group at a time.
    * ``Reset(dst, v)`` of a vector that receives MultiDotInc increments is the
      setter ``dst = 0*dst + v + sum(...)``.
    * ``Copy(src -> dst)`` (e.g. bias into the neuron input) of a vector that
      receives MultiDotInc increments is the setter ``dst = 1*src + 0 + sum(...)``.

    The order of floating-point additions per element is unchanged: first the
    set value, then the increments in operator order.
    """
    one = None
    views = {}

    def view_of(sig, sl):
        if sl is None:
            return sig
        key = (id(sig), sl.start, sl.stop, sl.step)
        if key not in views:
            views[key] = sig[sl]
        return views[key]

    basic = lambda sl: sl is None or isinstance(sl, slice)
    out = []
    for op in operators:
        if (_is(op, "Copy") and op.inc and basic(op.src_slice) and basic(op.dst_slice)
                and op.src.ndim == 1 and op.dst.ndim == 1):
            if one is None:
                one = type(op.src)(np.array(1.0), name="one", readonly=True)
            y = view_of(op.dst, op.dst_slice)
            new = MultiDotInc(y, y, beta=1, gamma=0, tag=op.tag)
            new.add_AX(one, view_of(op.src, op.src_slice))
            out.append(new)
        else:
            out.append(op)

    targets = {op.Y for op in out if isinstance(op, MultiDotInc) and op._incs_Y}
    setters = {}
    for op in out:
        if not isinstance(op, MultiDotInc):
            for sig in op.sets:
                setters.setdefault(sig, []).append(op)
    fused = []
    for op in out:
        if _is(op, "Reset") and op.dst in targets and op.dst.ndim == 1 and len(setters[op.dst]) == 1:
            fused.append(MultiDotInc(op.dst, op.dst, beta=0, gamma=op.value, tag=op.tag))
        elif (_is(op, "Copy") and not op.inc and op.src_slice is None and op.dst_slice is None
              and op.dst in targets and op.dst.ndim == 1 and op.src.shape == op.dst.shape
              and len(setters[op.dst]) == 1):
            fused.append(MultiDotInc(op.dst, op.src, beta=1, gamma=0, tag=op.tag))
        else:
            fused.append(op)
    return fused


class SparseDotSet(ir.Operator):
    """``Y = A @ X`` with a sparse matrix signal A: what ``Reset(Y, 0)`` followed by a
    ``SparseDotInc`` into Y is when nothing else writes Y."""

    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        self.A, self.X, self.Y = A, X, Y
        self.sets, self.reads = [Y], [A, X]


def sparse_products_set_their_target(operators):
    """``Reset(y, 0); SparseDotInc(y += A x)`` with no other writer of y becomes
    `SparseDotSet` (``y = A x``): one launch and one pass over y less per step.  The sum of a
    row starts from +0.0 either way, so the result has the same bits."""
    sets, incs, _, updates = signal_io_dicts(operators)
    drop, replace = set(), {}
    for op in operators:
        if not _is(op, "SparseDotInc") or op.Y.is_view:
            continue
        base = op.Y.base
        resets = [w for w in sets[base] if _is(w, "Reset")]
        if (len(sets[base]) != 1 or len(resets) != 1 or len(incs[base]) != 1
                or incs[base][0] is not op or updates[base]):
            continue
        reset = resets[0]
        if reset.dst.is_view or float(reset.value) != 0.0:
            continue
        drop.add(id(reset))
        replace[id(op)] = SparseDotSet(op.A, op.X, op.Y, tag=getattr(op, "tag", None))
    return [replace.get(id(op), op) for op in operators if id(op) not in drop]


def neurons_read_constant_input(operators, keep=()):
    """Neurons whose input current is only ever a copy of a constant (an ensemble
    without incoming connections: J = bias every step) read that constant directly,
    and the copy goes away.

    Applies to ``Copy(src -> J)`` (whole vectors, not an increment) when nothing else
    writes J, nothing writes src, and the neuron operator is the only reader of J;
    signals in `keep` (probed ones) are left alone.  The neuron update sees the same
    values, so results do not change; J itself is no longer refreshed.
    """
    import copy as _copy

    written = {}
    readers = {}
    for op in operators:
        for sig in list(op.sets) + list(op.incs) + list(op.updates):
            written.setdefault(sig.base, []).append(op)
        for sig in list(op.reads) + list(op.incs):
            readers.setdefault(sig.base, []).append(op)
    keep_bases = {sig.base for sig in keep}
    drop, replace = set(), {}
    for op in operators:
        if not _is(op, "SimNeurons") or not hasattr(op, "J"):
            continue
        J = op.J
        if J.base in keep_bases or getattr(J, "is_view", False):
            continue
        writers = written.get(J.base, [])
        if len(writers) != 1 or len(readers.get(J.base, [])) != 1:
            continue
        cp = writers[0]
        if not (_is(cp, "Copy") and not cp.inc and cp.src_slice is None and cp.dst_slice is None
                and cp.dst is J and cp.src.shape == J.shape and cp.src.base not in written
                and not getattr(cp.src, "is_view", False)):
            continue
        new = _copy.copy(op)
        new.J = cp.src
        new.reads = [cp.src if sig is J else sig for sig in op.reads]
        replace[op] = new
        drop.add(cp)
    if not replace:
        return operators
    return [replace.get(op, op) for op in operators if op not in drop]


def propagate_vector_copies(operators, keep=()):
    """Vectors that are only ever a copy of another vector are not copied: their readers
    read the source.

    After `fuse_into_multidotinc` and `MultiDotInc.compress`, ``Reset(y); Copy(x -> y,
    inc=True)`` -- what a passthrough node or an ensemble with a single unweighted input
    leaves in the graph -- is one operator ``y = 0*y + 0 + 1*x``.  When that operator is
    the only writer of ``y``, ``y`` is a whole signal that is not in `keep` (probed
    signals), and every reader of ``y`` is a MultiDotInc that uses it as a vector
    operand, those readers take ``x`` instead and the copy goes away: one launch less per
    link of such a chain (the reference runs each link as a GEMV of its own,
    simulator.py:746-816).  The planner orders the readers after the writers of ``x``
    and before its updates, which is when the copy read it.  Values are unchanged except
    that a copy turns -0.0 into +0.0, so a sum downstream may be -0.0 where it was +0.0.
    The copied signal is no longer part of the simulation (``sim.signals`` does not hold
    it), like the signals the reference's own simplifications remove.  The operators
    passed in are left as they are (readers are replaced by modified copies), so that the
    caller can keep the original list if the rewritten one does not plan better.
    """
    import copy as _copy

    keep_bases = {sig.base for sig in keep}
    ops = list(operators)
    # positions of the operators that write / read each base signal; kept current while
    # readers are redirected (a dropped operator leaves None at its position)
    writers, readers = {}, {}
    for pos, op in enumerate(ops):
        for sig in list(op.sets) + list(op.incs) + list(op.updates):
            writers.setdefault(sig.base, []).append(pos)
        for sig in op.reads:
            readers.setdefault(sig.base, []).append(pos)
    mine = set()  # positions holding copies made here (safe to modify)

    for pos in range(len(ops)):
        op = ops[pos]
        if not isinstance(op, MultiDotInc):
            continue
        if (op._incs_Y or op._signal_beta is not None or op._float_beta != 0 or op.gamma != 0
                or len(op.As) != 1):
            continue
        A, X, Y = op.As[0], op.Xs[0], op.Y
        base = Y.base
        if (getattr(Y, "is_view", False) or base in keep_bases or X.shape != Y.shape
                or X.base is base or A.size != 1 or not getattr(A, "readonly", False)
                or writers.get(A.base) or float(np.asarray(A.initial_value).ravel()[0]) != 1.0):
            continue
        if writers.get(base) != [pos]:
            continue
        users = sorted({q for q in readers.get(base, []) if q != pos and ops[q] is not None})
        if not users or not all(
                isinstance(ops[q], MultiDotInc) and any(x is Y for x in ops[q].Xs)
                and all(a is not Y for a in ops[q].As) and ops[q].Y_in is not Y
                and ops[q]._signal_beta is not Y for q in users):
            continue
        for q in users:
            if q not in mine:
                new = _copy.copy(ops[q])
                new.As, new.Xs = list(new.As), list(new.Xs)
                ops[q] = new
                mine.add(q)
            ops[q].Xs = [X if x is Y else x for x in ops[q].Xs]
            readers.setdefault(X.base, []).append(q)
        ops[pos] = None
        writers[base] = []
        readers[base] = []
    return [op for op in ops if op is not None]


def _exactly_disjoint(a, b):
    """Views of one signal that share no element (interleaved slices pass a test of their
    bounds and are still disjoint)."""
    if not a.may_share_memory(b):
        return True
    try:
        return not np.shares_memory(a.initial_value, b.initial_value, max_work=100000)
    except Exception:  # too hard to decide: assume the worst
        return False


def products_write_their_target(operators, keep=(), ahead=None):
    """``w = gamma + A x`` followed by ``v += 1 * w`` becomes ``v = gamma + A x``.

    A transform whose result is then added into a part ``v`` of a node's or ensemble's
    input leaves three operators behind: ``Reset(B)``, the product into its own vector
    ``w``, and the copy ``v += w`` (after `fuse_into_multidotinc`: a MultiDotInc with the
    constant one as its matrix).  When the views written that way are pairwise disjoint and
    together make up the whole of ``B``, nothing else writes ``B``, and each ``w`` is a whole
    signal outside `keep` that only its product writes and only its copy reads, the products
    write the views themselves and the copies and the Reset go: two operator groups less in
    a chain like "transform -> interleave -> ensembles" (the reference runs each link as a
    launch, simulator.py:746-816).  The same holds for a ``w`` that a process updates at the
    end of every step (the synapse of a connection into a part of a node's input: what an
    ensemble array's output node collects): the process writes ``v`` itself, unless ``B`` is
    in `keep` (a probe reads after the updates of a step).  Every operator then reads what it
    read before; only the host, looking at ``B`` between two steps, sees the value the next
    step will read where the reference shows the one the last step read -- such ``B`` are
    added to the set `ahead`.  Values are unchanged except that the copy turned -0.0 into
    +0.0.  The vectors ``w`` are no longer part of the simulation.  The operators
    passed in are left as they are.
    """
    import copy as _copy

    keep_bases = {sig.base for sig in keep}
    ops = list(operators)
    writers, readers = {}, {}
    for pos, op in enumerate(ops):
        for sig in list(op.sets) + list(op.incs) + list(op.updates):
            writers.setdefault(sig.base, []).append(pos)
        for sig in op.reads:
            readers.setdefault(sig.base, []).append(pos)

    def is_one(A):
        return (A.size == 1 and getattr(A, "readonly", False) and not writers.get(A.base)
                and float(np.asarray(A.initial_value).ravel()[0]) == 1.0)

    copies_into = {}
    for pos, op in enumerate(ops):
        if (isinstance(op, MultiDotInc) and op._incs_Y and op.gamma == 0 and len(op.As) == 1
                and is_one(op.As[0])):
            w = op.Xs[0]
            if (not getattr(w, "is_view", False) and w.base not in keep_bases
                    and w.shape == op.Y.shape and w.base is not op.Y.base):
                copies_into.setdefault(op.Y.base, []).append(pos)

    for base, copies in copies_into.items():
        resets = [q for q in writers.get(base, []) if _is(ops[q], "Reset")]
        if (len(resets) != 1 or float(ops[resets[0]].value) != 0.0
                or getattr(ops[resets[0]].dst, "is_view", False)
                or sorted(writers[base]) != sorted(resets + copies)):
            continue
        views = [ops[q].Y for q in copies]
        if sum(v.size for v in views) != base.size or not all(
                _exactly_disjoint(a, b) for i, a in enumerate(views) for b in views[i + 1:]):
            continue
        pairs = []
        for q in copies:
            w = ops[q].Xs[0]
            made_by = writers.get(w.base, [])
            producer = ops[made_by[0]] if len(made_by) == 1 else None
            if producer is None or readers.get(w.base, []) != [q]:
                break
            product = (isinstance(producer, MultiDotInc) and not producer._incs_Y
                       and producer.Y is w and producer._signal_beta is None
                       and producer._float_beta == 0
                       and not any(sig.base is base for sig in producer.reads))
            # a process that updates w at the end of a step (a synapse): what the copy adds
            # at the start of the next step is what the process can leave in v itself
            process = (_is(producer, "SimProcess") and getattr(producer, "mode", None) == "update"
                       and getattr(producer, "output", None) is w and base not in keep_bases
                       and not any(sig.base is base for sig in producer.all_signals))
            if not (product or process):
                break
            pairs.append((made_by[0], q, product))
        if len(pairs) != len(copies):
            continue
        for ppos, q, product in pairs:
            if product:
                new = _copy.copy(ops[ppos])
                new.As, new.Xs = list(new.As), list(new.Xs)
                new.Y = new.Y_in = ops[q].Y
                if getattr(ops[q], "tag", None) is not None:
                    new.tag = ops[q].tag
            else:
                w = ops[q].Xs[0]
                new = _replace_signals(ops[ppos], {w: ops[q].Y})
                _overwrite_initial_value(ops[q].Y, np.asarray(w.initial_value).reshape(ops[q].Y.shape))
                if ahead is not None:
                    ahead.add(base)
            ops[ppos] = new
            ops[q] = None
        ops[resets[0]] = None
    return [op for op in ops if op is not None]


LEARNING_RULES = ("SimPES", "SimBCM", "SimOja", "SimVoja")


def apply_learning_in_place(operators, keep=()):
    """Learning rules whose delta matrix only exists to be added to the learned matrix
    add their change to that matrix directly.

    The builder emits ``rule(... -> delta)`` (an update: its result is first seen in the
    next step) and ``Copy(delta -> target, inc=True)``.  The copy of step n+1 adds what
    the rule computed at the end of step n, and nothing can see the target in between,
    so adding the change at the end of step n gives every reader the same values -- in
    one pass over the matrix instead of a pass that writes the delta and another that
    reads delta and target and writes the target.  Rewritten when the copy is the only
    writer of the target and the only reader of the delta, both are whole signals (no
    views, no slices), and neither is in `keep` (probed signals; a probe samples at the
    very end of a step and would see the change one step early): the rule gets
    ``delta = target`` and ``apply_inc = True``, the copy goes away.  Sums are formed as
    before (change rounded, then added), so everything computed inside the simulation
    is bit-identical.  What differs: the delta signal is no longer written, and a host
    read of the target *between* steps already includes the change of the step just
    finished.
    """
    import copy as _copy

    writers, readers = {}, {}
    for op in operators:
        for sig in list(op.sets) + list(op.incs) + list(op.updates):
            writers.setdefault(sig.base, []).append(op)
        for sig in list(op.reads) + list(op.incs):
            readers.setdefault(sig.base, []).append(op)
    keep_bases = {sig.base for sig in keep}
    whole = lambda sig: not getattr(sig, "is_view", False)
    drop, replace = set(), {}
    for op in operators:
        if type(op).__name__ not in LEARNING_RULES or getattr(op, "apply_inc", False):
            continue
        delta = op.delta
        if not whole(delta) or delta.base in keep_bases or writers.get(delta.base) != [op]:
            continue
        users = readers.get(delta.base, [])
        if len(users) != 1:
            continue
        cp = users[0]
        if not (_is(cp, "Copy") and cp.inc and cp.src is delta and cp.src_slice is None
                and cp.dst_slice is None and whole(cp.dst) and cp.dst.shape == delta.shape
                and cp.dst.base not in keep_bases and writers.get(cp.dst.base) == [cp]):
            continue
        new = _copy.copy(op)
        new.delta, new.apply_inc = cp.dst, True
        new.updates = [cp.dst]
        new.reads = list(op.reads)
        replace[op] = new
        drop.add(cp)
    if not replace:
        return operators
    return [replace.get(op, op) for op in operators if op not in drop]


def _replace_signals(op, mapping):
    """A shallow copy of ``op`` in which every signal that is a key of ``mapping`` (by
    identity) is replaced by its value -- in attributes, and in lists, tuples and dicts held
    by attributes (nengo's operators keep their signals in the sets / incs / reads /
    updates lists, `ir`'s also in named attributes)."""
    import copy as _copy

    def swap(v):
        if isinstance(v, (list, tuple)):
            w = [swap(x) for x in v]
            return type(v)(w) if any(a is not b for a, b in zip(w, v)) else v
        if isinstance(v, dict):
            w = {k: swap(x) for k, x in v.items()}
            return w if any(w[k] is not v[k] for k in v) else v
        try:
            return mapping.get(v, v)
        except TypeError:  # unhashable attribute values (arrays) are not signals
            return v

    new = _copy.copy(op)
    for key, value in list(vars(new).items()):
        swapped = swap(value)
        if swapped is not value:
            setattr(new, key, swapped)
    return new


def _process_key(process):
    """What makes two synapse processes the same filter, or None for a process that is
    not a plain transfer function (noise, tables, anything with a seed)."""
    num, den = getattr(process, "num", None), getattr(process, "den", None)
    if num is None or den is None or getattr(process, "seed", None) is not None:
        return None
    return (type(process).__name__, tuple(np.atleast_1d(num).tolist()),
            tuple(np.atleast_1d(den).tolist()), bool(getattr(process, "analog", True)),
            str(getattr(process, "method", "")),
            repr(getattr(process, "initial_output", None)))


def merge_identical_chains(operators, keep=(), aliases=None):
    """Signals that are computed the same way from the same inputs are computed once.

    nengo's builder emits one weight signal, one ``Reset`` + ``DotInc`` and one synapse per
    Connection.  Connections that leave one ensemble with the same function, solver and
    transform carry bit-identical decoders and read the same activities, so their weighted
    sums -- and behind equal synapses their filtered values -- are the same numbers every
    step.  Here such duplicates are found and dropped, their readers redirected to the one
    that stays: the matrix is then stored and read once per step instead of once per
    connection (the reference keeps every copy: its `compress`, operators.py:112-146,
    merges by target signal only).

    A signal ``S`` is a candidate when every operator refers to it whole (no views), it is
    not in `keep` (probed signals), and each of its writers is one of ``Reset``,
    ``DotInc``, ``ElementwiseInc``, a whole ``Copy``, or a ``SimProcess`` (mode update)
    of a plain transfer function whose state signals nobody else touches.  Two candidates
    are duplicates when shape and initial value agree and their writer lists agree
    operator by operator: same kind, same parameters, and the same operand signals, where
    operands that are read-only constants nobody writes count as the same signal if their
    values are bit-identical.  Learned weights have a writer, so they never qualify.
    Repeated to a fixed point, so a chain (weighted sum, then synapse) folds link by link.

    Every reader then sees the values it saw before, bit for bit.  ``aliases`` (a dict,
    filled in place) maps each dropped signal to the one that replaces it, for whoever
    resolves signals afterwards (``sim.signals[dropped]``).
    """
    if aliases is None:
        aliases = {}
    keep_bases = {sig.base for sig in keep}
    ops = list(operators)
    const_canon = {}   # signal -> canonical equal-valued constant
    const_buckets = {}

    def canonical_constant(sig, writers):
        """`sig`, or the first constant seen with its shape and values."""
        if sig in const_canon:
            return const_canon[sig]
        out = sig
        if (not getattr(sig, "is_view", False) and getattr(sig, "readonly", False)
                and not getattr(sig, "sparse", False) and not writers.get(sig.base)
                and sig.base not in keep_bases):
            value = np.asarray(sig.initial_value)
            flat = value.reshape(-1)
            key = (value.shape, str(value.dtype), flat[:4].tobytes(), flat[-4:].tobytes())
            for other in const_buckets.setdefault(key, []):
                if np.array_equal(np.asarray(other.initial_value), value):
                    out = other
                    break
            else:
                const_buckets[key].append(sig)
        const_canon[sig] = out
        return out

    while True:
        writers, readers, partial = {}, {}, set()
        for pos, op in enumerate(ops):
            for sig in list(op.sets) + list(op.incs) + list(op.updates):
                writers.setdefault(sig.base, []).append(pos)
            for sig in op.reads:
                readers.setdefault(sig.base, []).append(pos)
            for sig in op.all_signals:
                if sig.base is not sig:
                    partial.add(sig.base)

        def exclusive_state(op, pos):
            """Initial values of the operator's state signals if only it touches them."""
            out = []
            for name in sorted(getattr(op, "state", None) or {}):
                st = op.state[name]
                if (st.base is not st or st.base in partial or st.base in keep_bases
                        or writers.get(st.base) != [pos]
                        or any(q != pos for q in readers.get(st.base, []))):
                    return None
                v = np.asarray(st.initial_value)
                out.append((name, v.shape, v.tobytes()))
            return tuple(out)

        def writer_key(pos, S):
            op = ops[pos]
            const = lambda sig: id(canonical_constant(sig, writers))
            if _is(op, "Reset") and op.dst is S:
                return ("Reset", float(op.value))
            if _is(op, "DotInc") and op.Y is S:
                return ("DotInc", const(op.A), const(op.X))
            if _is(op, "ElementwiseInc") and op.Y is S:
                return ("ElementwiseInc", const(op.A), const(op.X))
            if (_is(op, "Copy") and op.dst is S and op.src_slice is None
                    and op.dst_slice is None):
                return ("Copy", bool(op.inc), const(op.src))
            if (_is(op, "SimProcess") and op.output is S and op.mode == "update"
                    and op.input is not None):
                pkey = _process_key(op.process)
                state = exclusive_state(op, pos)
                if pkey is not None and state is not None:
                    return ("SimProcess", pkey, id(op.input), state)
            return None

        groups = {}
        for S, wpos in writers.items():
            if S in partial or S in keep_bases or getattr(S, "sparse", False):
                continue
            keys = []
            for pos in wpos:
                op = ops[pos]
                own_state = list((getattr(op, "state", None) or {}).values())
                outputs = list(op.sets) + list(op.incs) + list(op.updates)
                if any(sig is not S and all(sig is not st for st in own_state)
                       for sig in outputs):
                    keys = None  # the writer also writes something else
                    break
                k = writer_key(pos, S)
                if k is None:
                    keys = None
                    break
                keys.append(k)
            if not keys:
                continue
            v = np.asarray(S.initial_value)
            groups.setdefault((v.shape, v.tobytes(), tuple(keys)), []).append(S)

        mapping = {}
        for members in groups.values():
            for dup in members[1:]:
                mapping[dup] = members[0]
        if not mapping:
            break
        drop = {pos for dup in mapping for pos in writers[dup]}
        ops_before = ops
        touched = {pos for dup in mapping for pos in readers.get(dup, [])} - drop
        ops = [_replace_signals(op, mapping) if pos in touched else op
               for pos, op in enumerate(ops) if pos not in drop]
        for dup, rep in mapping.items():
            aliases[dup] = rep
            # what only the dropped writers used (their equal-valued constants, their
            # state) resolves to the surviving writers' operands
            for p_dup, p_rep in zip(writers[dup], writers[rep]):
                a_sigs = list(ops_before[p_dup].reads) + list(ops_before[p_dup].updates)
                b_sigs = list(ops_before[p_rep].reads) + list(ops_before[p_rep].updates)
                for a, b in zip(a_sigs, b_sigs):
                    if a is not b and a is not dup:
                        aliases.setdefault(a, b)
        for sig, rep in list(aliases.items()):  # chains of replacements end at a survivor
            while rep in aliases:
                rep = aliases[rep]
            aliases[sig] = rep
    return ops


merge_identical_chains.takes_context = True


def simplify_operators(operators, keep=(), aliases=None, skip=()):
    """Apply every function in ``simplifications`` in turn (those named in `skip`
    excepted).  `keep` (signals that must stay as they are: probed ones) and `aliases`
    (dict filled with dropped signal -> its replacement) go to the simplifications that
    take them."""
    for simplification in simplifications:
        if simplification.__name__ in skip:
            continue
        if getattr(simplification, "takes_context", False):
            operators = simplification(operators, keep=keep, aliases=aliases)
        else:
            operators = simplification(operators)
    return operators


# Modify this module-level list to change which simplifications run.
simplifications = [remove_unmodified_resets, remove_zero_incs, merge_identical_chains]
