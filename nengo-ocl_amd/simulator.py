"""The Simulator: builds the per-timestep plan list and runs it on one MI355X.

Counterpart of the reference's ``nengo_ocl/simulator.py`` (``ViewBuilder``
:72-143, ``Simulator`` :145-1449).  Kept: constructor arguments, operator
simplification / MultiDotInc conversion / planning (:248-265), packing of all
signals into one float32 ragged buffer with views (:269-335), the
``_plan_<OperatorType>`` dispatch (:733-734) with nested dispatch on neuron
class (:1035-1044) and process class (:1160-1177), ``run`` / ``run_steps`` /
``step`` / ``reset`` / ``trange`` / ``signals`` / ``data`` / ``close``, probe
buffering (:499-520, :705-731) and the profiling table (:1388-1449).

Changed on purpose: the plan list is replayed as a HIP graph instead of a
Python launch loop; signal bases are packed 64-byte aligned so matrix rows can
be read with 16-byte loads; LIF parameters travel as one scalar per population
instead of one array element per neuron; probe drains copy only the rows
that were written.

``network`` may be a nengo ``Network`` (needs nengo importable: its builder
produces the operator graph) or a `minibuilder.Network`; ``model`` may be a
nengo ``Model`` or an `ir.Model` that already holds operators.
"""

import inspect
import logging
import os
import time as _time
import warnings
from collections import defaultdict
from collections.abc import Mapping
from io import StringIO

import numpy as np

from . import operators as ops_mod
from .operators import MultiDotInc
from .plan import BasePlan, Plans, PythonPlan
from .planners import batching_planner, greedy_planner  # noqa: F401
from .raggedarray import RaggedArray
from .utils import get_closures, groupby, indent, split, stable_unique

logger = logging.getLogger(__name__)


class SimulatorClosed(RuntimeError):
    pass


class ReadonlyError(AttributeError):
    pass


class ValidationError(ValueError):
    pass


class HipBackend:
    """The device side of the ``plan_*`` boundary (everything below the Simulator)."""

    name = "hip"

    def __init__(self, device=0):
        from . import hipra_gemv, hipra_nonlinearities, hipraggedarray

        self.queue = hipraggedarray.Queue(device if device is not None else 0)
        self._ra = hipraggedarray
        for name in ("plan_timeupdate", "plan_reset", "plan_copy", "plan_slicedcopy",
                     "plan_elementwise_inc", "plan_linearfilter", "plan_probes", "plan_direct",
                     "plan_lif", "plan_lif_rate", "plan_presentinput", "plan_rectified_linear",
                     "plan_spiking_rectified_linear", "plan_sigmoid", "plan_bcm", "plan_oja",
                     "plan_voja", "plan_conv2d", "plan_pool2d", "plan_whitenoise"):
            setattr(self, name, getattr(hipra_nonlinearities, name))
        self.plan_block_gemv = hipra_gemv.plan_block_gemv
        self._fuse_lif = hipra_gemv.fuse_lif
        self._gemv = hipra_gemv
        # switch for measurements: "0" stores every input current
        self.skip_unread_currents = os.environ.get("NENGO_HIP_SKIP_CURRENTS", "1") != "0"
        # spikes that only launches visiting active columns read: a bit per neuron
        self.spikes_as_bits = os.environ.get("NENGO_HIP_SPIKE_BITS", "1") != "0"
        # switch for measurements: False keeps input sums a launch of their own
        self.input_sums_in_launch = os.environ.get("NENGO_HIP_INPUT_SUMS", "1") != "0"
        from . import hipra_sequence

        from . import hipra_spmv

        self.plan_sparse_dot_inc = hipra_spmv.plan_sparse_dot_inc
        # switch for measurements: "0" multiplies every stored element of a sparse matrix
        self.skips_zero_operands = os.environ.get("NENGO_HIP_SPMV_SKIP", "1") != "0"
        # switch for measurements: "0" multiplies every column of a matrix applied to spikes
        self.event_driven_products = os.environ.get("NENGO_HIP_EVENT_GEMV", "1") != "0"
        self.merge_small_plans = hipra_sequence.merge_small_plans
        if os.environ.get("NENGO_HIP_CARRY_SEQUENCES", "1") != "0":  # switch for measurements
            self.carry_sequences = hipra_sequence.carry_sequences
        self.plans_conflict = hipra_sequence._conflict
        self.fuse_gemv_filter = hipra_gemv.fuse_linearfilter
        self.fuse_spmv_filter = hipra_spmv.fuse_linearfilter
        if os.environ.get("NENGO_HIP_OUTER_FILTER", "1") != "0":  # switch for measurements
            self.fuse_outer_filter = hipra_nonlinearities.fuse_outer_filter
        if os.environ.get("NENGO_HIP_FOLD_LEARNING", "1") != "0":  # switch for measurements
            self.fuse_learning = hipra_gemv.fuse_learning

    def fuse_input_sums(self, sum_plan, lif_plan):
        """The plan replacing ``[sum_plan, lif_plan]`` when the first only forms vector
        operands of the second, or None."""
        if self.input_sums_in_launch and hasattr(sum_plan, "prog") and hasattr(lif_plan, "prog"):
            return self._gemv.fuse_input_sums(sum_plan, lif_plan)
        return None

    def store_spikes_as_bits(self, enc_plan, items, event_records, dt):
        return self._gemv.store_spikes_as_bits(enc_plan, items, event_records, dt)

    def fuse_gemv_neurons(self, gemv_plans, neuron_plans, unread_currents=()):
        """Plans replacing ``gemv_plans + neuron_plans`` by launches that update the
        neurons in the epilogue of the GEMV that produces their input, or None.
        `unread_currents`: populations of the neuron plan whose input current nothing else
        reads (the launch need not store it)."""
        progs = {id(getattr(p, "prog", None)) for p in gemv_plans}
        if len(neuron_plans) != 1 or len(progs) != 1 or not hasattr(gemv_plans[0], "prog"):
            return None
        if not self.skip_unread_currents:
            unread_currents = ()
        return self._fuse_lif(gemv_plans[0].prog, neuron_plans[0], unread_currents=unread_currents)

    def upload(self, host_ragged):
        return self._ra.HIPRaggedArray(self.queue, host_ragged)

    def probe_drain(self, probe_plan, signals, step_idx, time_idx):
        """Callable ``drain(rows_bound) -> (step, time, counts, rows)`` that fetches the
        clock and the buffered probe rows in one transfer and zeroes the positions."""
        from .hipra_nonlinearities import ProbeDrain

        return ProbeDrain(self.queue, probe_plan, signals, step_idx, time_idx)

    def array(self, values, dtype=np.float32):
        return self._ra.to_device(self.queue, np.asarray(values, dtype=dtype))

    def finish(self):
        self.queue.finish()

    def read_rows(self, ragged, i, n_rows):
        """First ``n_rows`` rows of contiguous item ``i`` of a device ragged array."""
        width = int(ragged.shape1s[i])
        flat = ragged.dev_buf.get_span(int(ragged.starts[i]), n_rows * width)
        return flat.reshape(n_rows, width)

    def write_all(self, ragged, host_buf):
        ragged.dev_buf.set(host_buf)

    def get_array(self, arr):
        return arr.get()

    def fill_array(self, arr, value):
        arr.fill(value)

    def set_array(self, arr, values):
        arr.set(values)


class ViewBuilder:
    """Collects every signal view an operator (or probe) touches as an extra ragged
    entry aliasing its base (reference simulator.py:72-143)."""

    def __init__(self, bases, rarray):
        self.sidx = {b: i for i, b in enumerate(bases)}
        assert len(bases) == len(self.sidx)
        self.rarray = rarray
        self.meta = ([], [], [], [], [])
        self.names = []
        self._A_views, self._X_views, self._YYB_views = {}, {}, {}

    def append_view(self, sig):
        if sig in self.sidx:
            return
        if not sig.is_view:
            raise ValueError("can only append views of known signals", sig)
        assert sig.size and sig.ndim <= 2
        idx = self.sidx[sig.base]
        shape0 = sig.shape[0] if sig.ndim > 0 else 1
        shape1 = sig.shape[1] if sig.ndim > 1 else 1
        for column, value in zip(self.meta, (
                int(self.rarray.starts[idx]) + sig.elemoffset, shape0, shape1,
                sig.elemstrides[0] if shape0 > 1 else 1,
                sig.elemstrides[1] if shape1 > 1 else 1)):
            column.append(int(value))
        self.names.append(getattr(sig, "name", ""))
        self.sidx[sig] = len(self.sidx)

    def setup_views(self, ops):
        views = [sig for op in ops for sig in op.all_signals]
        for op in ops:
            if isinstance(op, MultiDotInc):
                A_views, X_views, Y_view, Y_in_view, beta_view = op.get_views()
                views.extend(A_views + X_views + [Y_view, Y_in_view]
                             + ([beta_view] if beta_view is not None else []))
                self._A_views[op], self._X_views[op] = A_views, X_views
                self._YYB_views[op] = [Y_view, Y_in_view, beta_view]
        for view in views:
            if not getattr(view, "sparse", False):
                self.append_view(view)

    def add_views_to(self, rarray):
        if self.names:
            rarray.add_views(*self.meta, names=self.names)


class ProbeData(Mapping):
    """``sim.data``: probe -> array of samples (rows), plus build parameters."""

    def __init__(self, raw):
        self.raw = raw

    def __getitem__(self, key):
        value = self.raw[key]
        if isinstance(value, list):
            if len(value) == 0:
                return np.zeros((0,))
            return np.asarray(value)
        return value

    def __iter__(self):
        return iter(self.raw)

    def __len__(self):
        return len(self.raw)

    def reset(self):
        pass


# numpy functions of time alone that the device runs without a host callback;
# the translated code has the form the reference's translator emits for them
# neuron types whose output is zero except in the steps a neuron spikes
SPIKING_NEURON_TYPES = ("LIF", "AdaptiveLIF", "SpikingRectifiedLinear")

_DIRECT_FUNCTIONS = {np.sin: "sin", np.cos: "cos", np.tanh: "tanh", np.exp: "exp",
                     np.square: "square"}


class Simulator:
    """Simulator for running Nengo models on one MI355X (see module docstring).

    Parameters follow the reference (simulator.py:145-190): ``network, dt, seed,
    model, context, n_prealloc_probes, profiling, if_python_code, planner,
    progress_bar``.  ``context`` is the HIP device index here; ``n_prealloc_probes``
    defaults to what fits 64 MiB (32 to 4096 rows) instead of 32.  Not in the
    reference: ``backend`` replaces the device side of the ``plan_*`` boundary
    (the CPU oracle used by the tests plugs in there); ``use_graph=False`` runs
    the plan list as an eager launch loop; ``fuse=False`` keeps vector copies and
    resets as separate operators instead of folding them into the GEMVs
    (`operators.fuse_into_multidotinc`) and the neuron update as a separate launch
    instead of the epilogue of the GEMV that computes the input currents;
    ``branches=True`` (record the timestep as a graph in which kernels that touch
    different memory run side by side instead of one chain of kernels) is switched off
    and raises NotImplementedError: it was slower than the chain, and ending such a
    multi-stream recording crashed inside the runtime for one step shape;
    ``merge_small=False`` keeps every short
    operation (clock, inputs, small copies and filters, probes) as a launch of its
    own instead of binding runs of them into one launch; ``learn_in_place`` (on by
    default, with ``fuse``) lets learning rules whose delta matrix nothing but the
    builder's increment reads, and that is not probed, add their change to the learned
    matrix directly instead of writing a delta matrix that a copy adds in the next step:
    one pass over the matrix instead of two, identical values inside the simulation and
    in all probe data, but the delta signals are not written and ``sim.signals[weights]``
    read between steps already holds the change of the last step
    (`operators.apply_learning_in_place`); ``learn_in_place=False`` keeps the two passes;
    ``dedup=False`` keeps products and synapses that compute the same values from the same
    inputs as separate operators (`operators.merge_identical_chains`).

    What the host sees through ``sim.signals`` follows the reference whatever rewrites are
    on (`_host_state_rules`): a learned matrix that the rule updates in place and a node
    input that synapses write directly are read from a copy taken before the last step of
    every ``run_steps`` (the value the reference holds between two steps); signals that a
    rewrite no longer computes (the delta matrix of such a rule, a vector whose copy was
    cut out) raise ``ValueError`` when read instead of returning stale memory; writes to a
    learned matrix updated in place, to a signal that merged connections share or to a
    constant with a second device copy raise ``ValueError`` naming the constructor switch
    that makes them possible; spikes that only launches visiting active columns read are kept
    as one bit per neuron (`_store_spikes_as_bits`): reads give the reference's floats,
    writes raise ``ValueError``.  ``reference_host_state=True`` switches ``learn_in_place``,
    ``dedup``, the rewrites that move writes (``products_write_their_target``,
    ``propagate_vector_copies``), the second copies of constants and the spike bits off in
    one go: every signal is then readable and writable as in the reference.

    ``event_calibration_steps`` (default 32, 0 = off): products of a constant matrix with
    spikes visit only the columns of the neurons that spiked, which pays while few neurons
    spike per step and costs more than the dense product when most do.  When the plan list
    holds such launches and no host callback, the constructor runs that many steps, looks at
    the share of each population that spiked per step, resets, and -- if a population spiked
    above ``EVENT_MAX_SPIKING_SHARE`` (a quarter) of its neurons per step -- builds the plans
    again with the products of those populations dense.  ``sim.event_calibration`` holds what
    it saw.
    """

    def __init__(self, network, dt=0.001, seed=None, model=None, context=None,
                 n_prealloc_probes=None, profiling=None, if_python_code="none",
                 planner=batching_planner, progress_bar=True, backend=None, use_graph=True,
                 fuse=True, branches=False, merge_small=True, learn_in_place=True,
                 dedup=True, reference_host_state=False, event_calibration_steps=32,
                 _spike_sources_read_whole=()):
        self.closed = False
        self.model = None
        # what a second construction needs (see `_calibrate_event_launches`)
        self._init_args = dict(
            dt=dt, seed=seed, context=context, n_prealloc_probes=n_prealloc_probes,
            profiling=profiling, if_python_code=if_python_code, planner=planner,
            progress_bar=progress_bar, backend=backend, use_graph=use_graph, fuse=fuse,
            branches=branches, merge_small=merge_small, learn_in_place=learn_in_place,
            dedup=dedup, reference_host_state=reference_host_state)
        self._spike_sources_read_whole = frozenset(_spike_sources_read_whole)
        self.event_calibration = None
        if reference_host_state:
            learn_in_place = dedup = False
        self.reference_host_state = bool(reference_host_state)

        if profiling is None:
            profiling = int(os.getenv("NENGO_OCL_PROFILING", "0"))
        self.profiling = profiling
        if if_python_code not in ["none", "warn", "error"]:
            raise ValueError("%r not a valid value for `if_python_code`" % if_python_code)
        self.if_python_code = if_python_code
        self.n_prealloc_probes = n_prealloc_probes
        self.progress_bar = progress_bar
        self.use_graph = use_graph
        self.context = context

        # --- build
        t0 = _time.time()
        if model is None:
            if network is None:
                raise ValueError("need a network or a model")
            if hasattr(network, "build_model"):  # minibuilder.Network
                self.model = network.build_model(dt=float(dt))
            else:
                self.model = self._nengo_build(network, dt)
        else:
            self.model = model
            if network is not None:
                self.model.build(network)
        logger.info("Build in %0.3f s", _time.time() - t0)

        # --- operators
        t0 = _time.time()
        all_operators = list(self.model.operators)
        probed = [self.model.sig[p]["in"] for p in self.model.probes]
        self.signal_aliases = {}  # signal dropped as a duplicate -> the one computed
        self._copied_constants = set()  # constants that launches read from a copy of their own
        self.signals_a_step_ahead = set()
        operators = ops_mod.simplify_operators(
            all_operators, keep=probed, aliases=self.signal_aliases,
            skip=() if dedup else ("merge_identical_chains",))
        operators = list(map(MultiDotInc.convert_to, operators))
        if fuse:
            operators = ops_mod.fuse_into_multidotinc(operators)
            operators = ops_mod.sparse_products_set_their_target(operators)
            if not reference_host_state:
                operators = ops_mod.neurons_read_constant_input(operators, keep=probed)
            if learn_in_place:
                operators = ops_mod.apply_learning_in_place(operators, keep=probed)
        operators = MultiDotInc.compress(operators)
        op_groups = planner(operators)
        if fuse and not reference_host_state:
            # cutting vector copies out of the graph saves launches in chains of small
            # operators, but it can also split a group of like operators whose members no
            # longer depend on the same things: keep it only where the step gets shorter
            shorter = ops_mod.propagate_vector_copies(operators, keep=probed)
            ahead = set()
            shorter = ops_mod.products_write_their_target(shorter, keep=probed, ahead=ahead)
            if len(shorter) < len(operators):
                shorter_groups = planner(shorter)
                if len(shorter_groups) < len(op_groups):
                    operators, op_groups = shorter, shorter_groups
                    # signals that hold, between two steps, what the next step will read
                    self.signals_a_step_ahead = ahead
        assert len([t for t, _ in op_groups if t.__name__ == "Reset"]) < 2, \
            "All resets not planned together"
        self.operators = operators
        self.op_groups = op_groups
        logger.info("Planning in %0.3f s", _time.time() - t0)

        # --- signals: every base into one float32 ragged buffer, views appended
        t0 = _time.time()
        # the rewritten operator list may have introduced signals (the constant one)
        all_signals = stable_unique(sig for op in all_operators + operators
                                    for sig in op.all_signals)
        all_bases = stable_unique(sig.base for sig in all_signals)
        self._host_state_rules(all_operators, operators, probed)
        if self._not_computed:  # nothing reads or writes them any more: no device memory
            all_bases = [b for b in all_bases if b not in self._not_computed]
        if self.signal_aliases:
            # duplicates (and the constants only they read) take no device memory: they
            # resolve to the signal that replaces them
            live = {sig.base for op in operators for sig in op.all_signals}
            live |= {sig.base for sig in probed}
            gone = {sig.base for sig in self.signal_aliases}
            dropped = {id(op) for op in all_operators
                       if any(sig.base in gone for sig in
                              list(op.sets) + list(op.incs) + list(op.updates))}
            only_dropped = {}
            for op in all_operators:
                for sig in op.all_signals:
                    only_dropped[sig.base] = (only_dropped.get(sig.base, True)
                                              and id(op) in dropped)
            all_bases = [b for b in all_bases
                         if b in live or not (b in gone or only_dropped.get(b, False))]
        # sparse matrices are constants of the sparse products: they stay on the host
        # until `_plan_SparseDotInc` lays them out (reference simulator.py:281-329)
        sparse_bases = [b for b in all_bases if getattr(b, "sparse", False)]
        if any(getattr(s, "sparse", False) and s.base is not s for s in all_signals):
            raise NotImplementedError("views of sparse signals")
        all_bases = [b for b in all_bases if not getattr(b, "sparse", False)]
        all_values = self._initial_values(all_operators, all_bases + sparse_bases)
        self.sparse_data = {b: all_values[b] for b in sparse_bases}
        values = {b: all_values[b] for b in all_bases}

        self.base_reshapes = {}
        dense = []
        for base in all_bases:
            x = np.asarray(values[base])
            if x.ndim > 2:
                self.base_reshapes[base] = x.shape
                x = x.reshape(-1, 1)
            dense.append(x)
        dense_data = RaggedArray(dense, names=[getattr(b, "name", "") for b in all_bases],
                                 dtype=np.float32, align=True)
        view_builder = ViewBuilder(all_bases, dense_data)
        view_builder.setup_views(operators)
        for probe in self.model.probes:
            view_builder.append_view(self.model.sig[probe]["in"])
        view_builder.add_views_to(dense_data)

        self.all_bases = all_bases
        self.sidx = {k: np.int32(v) for k, v in view_builder.sidx.items()}
        for sig, rep in self.signal_aliases.items():
            if sig not in self.sidx and rep in self.sidx:
                self.sidx[sig] = self.sidx[rep]
        self._A_views = view_builder._A_views
        self._X_views = view_builder._X_views
        self._YYB_views = view_builder._YYB_views
        self._initial_buf = np.array(dense_data.buf)

        self.backend = HipBackend(context) if backend is None else backend
        self.queue = self.backend.queue
        self.all_data = self.backend.upload(dense_data)

        self._probe_outputs = dict(getattr(self.model, "params", {}))
        self.data = ProbeData(self._probe_outputs)
        logger.info("Signals in %0.3f s", _time.time() - t0)

        # --- seed
        if seed is None:
            net_seed = getattr(network, "seed", None) if network is not None else None
            seed = net_seed + 1 if net_seed is not None else np.random.randint(2 ** 31 - 1)
        self.seed = seed
        self.rng = np.random.RandomState(self.seed)

        # --- plans
        t0 = _time.time()
        self._raggedarrays_to_reset = []  # (device ragged, host initial)
        self._lazy_currents = {}  # signal base -> {"prog": GEMV that recomputes it, "at_step"}
        self._event_spike_sources = set()  # spike signals whose products may visit active columns
        # filter outputs whose last step is pending in device memory (`_fuse_learning`):
        # signal base -> (spike signal base, a0 or None, b0)
        self._pending_filters = {}
        self._n_steps = 0
        self._filter_positions = []
        self._noise_plans = []
        self._python_rngs = {}
        plans = []
        previous = None  # (type, plans) of the group planned last
        for op_type, op_list in op_groups:
            group_plans = self._plan_op_group(op_type, op_list)
            # memory blocks the group's kernels touch, for the executor's dependency graph
            reads = {sig.base for op in op_list for sig in list(op.reads) + list(op.incs)}
            writes = {sig.base for op in op_list
                      for sig in list(op.sets) + list(op.incs) + list(op.updates)}
            if (fuse and op_type.__name__ == "SimNeurons" and previous is not None
                    and previous[0].__name__ == "MultiDotInc" and previous[1]
                    and hasattr(self.backend, "fuse_gemv_neurons")):
                # neurons right behind the GEMV that computes their input current
                fused = self.backend.fuse_gemv_neurons(
                    previous[1], group_plans, unread_currents=self._unread_currents(op_list, probed))
                if fused is not None:
                    self._register_lazy_currents(fused, op_list)
                    reads = reads | previous[1][0].reads_mem
                    writes = writes | previous[1][0].writes_mem
                    del plans[len(plans) - len(previous[1]):]
                    group_plans = fused
            for plan in group_plans:
                own = getattr(plan, "planned_ops", None)
                if own is None:
                    plan.reads_mem, plan.writes_mem = reads, writes
                else:  # a plan that covers only part of the group
                    skip = set(getattr(plan, "unread_signals", ()))  # declared, not touched
                    plan.reads_mem = {sig.base for op in own
                                      for sig in list(op.reads) + list(op.incs) if sig not in skip}
                    plan.writes_mem = {sig.base for op in own
                                       for sig in list(op.sets) + list(op.incs) + list(op.updates)}
            plans.extend(group_plans)
            previous = (op_type, group_plans)
        probe_plans = self._plan_probes()
        for plan in probe_plans:  # sample buffers and counters are the plan's own
            plan.reads_mem = {self.model.sig[p]["in"].base for p in self.model.probes}
            plan.writes_mem = set()
        plans.extend(probe_plans)
        if fuse and hasattr(self.backend, "fuse_gemv_filter"):
            plans = self._fuse_filter_epilogues(plans)
        if fuse and hasattr(self.backend, "fuse_input_sums"):
            plans = self._fuse_input_sums(plans)
        if fuse and hasattr(self.backend, "fuse_learning"):
            plans = self._fuse_learning(plans)
        if fuse and hasattr(self.backend, "fuse_outer_filter"):
            plans = self._fuse_outer_filters(plans)
        if merge_small and hasattr(self.backend, "merge_small_plans"):
            plans = self.backend.merge_small_plans(plans)
            if fuse and hasattr(self.backend, "carry_sequences"):
                plans = self.backend.carry_sequences(plans)
        self._store_spikes_as_bits(plans)
        logger.info("Plans in %0.3f s", _time.time() - t0)

        self._plans = Plans(plans, self.profiling, use_graph=use_graph, branches=branches,
                            before_last=self._plan_host_view())
        self.rng = None
        self._drain = None
        if hasattr(self.backend, "probe_drain"):
            self._drain = self.backend.probe_drain(self._probe_plan, self.all_data,
                                                   self.sidx[self.model.step],
                                                   self.sidx[self.model.time])
        self._reset_probes()
        self._plans.prepare()  # record the step graphs now, not inside the first run
        if event_calibration_steps and not self._spike_sources_read_whole:
            self._calibrate_event_launches(int(event_calibration_steps))

    # share of a population's neurons that may spike per step before the launch that visits
    # only their columns loses to the dense product (measured on MI355X: 4.4 us with no spikes,
    # 8.7 us at 8 %, 20.3 us at 30 %, 50.3 us at 100 % against 45 us dense, for 256 matrices of
    # 64 x 4096)
    EVENT_MAX_SPIKING_SHARE = 0.25

    def _calibrate_event_launches(self, n_steps):
        """Runs `n_steps` steps, reads the spikes of the populations whose products visit
        active columns only after each quarter of them, resets; populations that spiked
        above `EVENT_MAX_SPIKING_SHARE` per step get dense products (the simulator is built
        again around the same model).  Skipped when a plan is a host callback: running the
        model before the user does would show in whatever the callback keeps."""
        plans = list(self._plans)
        event_plans = [p for p in plans if getattr(p, "event_driven", False)]
        if not event_plans or any(not hasattr(p, "enqueue") for p in plans):
            return
        sources = {}  # spike signal base -> its largest share seen
        for op in self.operators:
            if (type(op).__name__ == "SimNeurons"
                    and type(op.neurons).__name__ in SPIKING_NEURON_TYPES
                    and op.output.base in self._event_spike_sources):
                sources[op.output.base] = 0.0
        if not sources:
            return
        quarter = max(n_steps // 4, 1)
        for _ in range(0, n_steps, quarter):
            self.run_steps(quarter)
            for base in sources:
                spikes = np.asarray(self.signals[base])
                sources[base] = max(sources[base], float(np.count_nonzero(spikes)) / spikes.size)
        self.reset()
        for plan in plans:  # (the run leaves no trace in the profiling table either)
            if isinstance(plan, BasePlan):
                plan.atimes[:], plan.btimes[:], plan.ctimes[:] = [], [], []
                plan.n_calls = 0
        hot = [base for base, share in sources.items() if share > self.EVENT_MAX_SPIKING_SHARE]
        report = {"steps": n_steps, "populations": len(sources),
                  "largest_share_spiking_per_step": max(sources.values()),
                  "threshold": self.EVENT_MAX_SPIKING_SHARE,
                  "populations_switched_to_dense_products": len(hot)}
        if hot:
            logger.info("%d populations spike above %g of their neurons per step: their "
                        "products are read whole", len(hot), self.EVENT_MAX_SPIKING_SHARE)
            model, args = self.model, dict(self._init_args, seed=self.seed)
            self.close()
            self.__init__(None, model=model, event_calibration_steps=0,
                          _spike_sources_read_whole=hot, **args)
        self.event_calibration = report

    def _unread_currents(self, neuron_ops, probed):
        """Indices of the neuron operators whose input current only they read and that can
        be formed again after the step: a whole signal that is not probed, that no other
        operator reads, increments or updates, that one operator sets, and whose operands
        (matrices, vectors, the bias it starts from) nothing writes later in the step --
        a vector that a synapse updates at the end of the step no longer holds what the
        product read."""
        if self.reference_host_state or len({type(op.neurons) for op in neuron_ops}) != 1:
            return ()
        probed_bases = {sig.base for sig in probed}
        readers, writers = defaultdict(list), defaultdict(list)
        when = {}  # operator -> index of its group in the step
        for g, (_, ops) in enumerate(self.op_groups):
            for op in ops:
                when[id(op)] = g
        for op in self.operators:
            for sig in list(op.reads) + list(op.incs) + list(op.updates):
                readers[sig.base].append(op)
            for sig in list(op.sets) + list(op.incs) + list(op.updates):
                writers[sig.base].append(op)
        out = []
        for k, op in enumerate(neuron_ops):
            J = op.J
            if not (J.base is J and J.base not in probed_bases and readers[J.base] == [op]
                    and len(writers[J.base]) == 1 and J.base not in self._shared):
                continue
            product = writers[J.base][0]
            if all(when[id(w)] < when[id(product)]
                   for sig in product.reads for w in writers[sig.base]):
                out.append(k)
        return out

    def _register_lazy_currents(self, plans, neuron_ops):
        """Input currents the fused launches do not store: signal base -> the GEMV that
        puts them into their place when the host asks for them."""
        for plan in plans:
            lazy = getattr(plan, "lazy_currents", None)
            if lazy is None:
                continue
            populations, prog = lazy
            group = {"prog": prog, "at_step": None}
            for p in populations:
                self._lazy_currents[neuron_ops[p].J.base] = group

    def _refresh_lazy(self, base):
        """Make a current that its launch does not store hold the last step's value (the
        step counter tells whether that was done since the last step)."""
        group = self._lazy_currents.get(base)
        # (before the first step the signal holds its initial value, as in the reference)
        if group is None or self._n_steps == 0 or group["at_step"] == self._n_steps:
            return
        for plan in group["prog"].plans:
            plan()
        group["at_step"] = self._n_steps

    def _host_state_rules(self, all_operators, operators, probed):
        """Which signals the host cannot read or write as they lie in device memory, given
        the rewritten operator list (reference semantics of the accessor:
        nengo_ocl/simulator.py:427-471).

        ``_not_computed``: bases some operator of the model writes but no operator of the
        rewritten list touches (and that are neither probed nor aliases of a survivor):
        reading them raises.  ``_updated_in_place``: matrices a learning rule adds its
        change to directly; with ``signals_a_step_ahead`` they make up ``_host_view``, the
        bases read from a copy taken before the last step.  ``_shared``: bases that stand
        for several signals of the model (survivors of a merge and what resolves to them)."""
        written = lambda ops: {sig.base for op in ops
                               for sig in list(op.sets) + list(op.incs) + list(op.updates)}
        touched = {sig.base for op in operators for sig in op.all_signals}
        touched |= {sig.base for sig in probed}
        aliased = {sig.base for sig in self.signal_aliases}
        self._not_computed = {b for b in written(all_operators)
                              if b not in touched and b not in aliased}
        self._updated_in_place = {
            op.delta.base for op in operators
            if type(op).__name__ in ops_mod.LEARNING_RULES and getattr(op, "apply_inc", False)}
        self._shared = aliased | {sig.base for sig in self.signal_aliases.values()}
        self._host_view = stable_unique(
            [b for b in self._updated_in_place] + [b.base for b in self.signals_a_step_ahead])
        self._host_view_index = {b: k for k, b in enumerate(self._host_view)}
        self._host_view_copy = None

    def _plan_host_view(self):
        """The plan that copies every base of ``_host_view`` aside; the executor runs it
        before the last timestep of each ``run_steps``."""
        if not self._host_view:
            return []
        X = self.all_data[[self.sidx[b] for b in self._host_view]]
        self._host_view_copy = self.RaggedArray(
            [np.zeros((int(X.shape0s[k]), int(X.shape1s[k]))) for k in range(len(X))],
            dtype=np.float32)
        plan = self.backend.plan_copy(self.queue, X, self._host_view_copy,
                                      np.zeros(len(X), dtype=np.int32))
        self._host_view_plan = plan
        plan()  # nothing has run yet: the copy holds the initial values
        return [plan]

    def _store_spikes_as_bits(self, plans):
        """Spike signals that nothing but launches visiting active columns reads -- no other
        launch, no probe, no host copy; written by one large-item neuron launch in tasks that
        start at multiples of 32 rows; one amplitude per population; zero at the start -- are
        kept as one bit per neuron in the first words of their own memory
        (`hipra_gemv.store_spikes_as_bits`): `_spike_bits` maps such a base to
        (start, neurons, value of a spike).  The host reads them through `_spikes_from_bits`
        and may not write them."""
        self._spike_bits = {}
        if self.reference_host_state or not getattr(self.backend, "spikes_as_bits", False):
            return
        encs = [p for p in plans if getattr(p, "name", "") == "hipra_gemv.tile_lif"
                and getattr(p, "dev_pops", None) is not None
                and getattr(p, "host_tasks", None) is not None]
        events = [p for p in plans if getattr(p, "dev_event_table", None) is not None]
        if not encs or not events:
            return
        ra = self.all_data
        base_at = {}  # start in the buffer -> the (largest) base signal that starts there
        for b in self.all_bases:
            start = int(ra.starts[self.sidx[b]])
            if start not in base_at or int(b.size) > int(base_at[start].size):
                base_at[start] = b
        records = defaultdict(list)  # (x_start, columns) -> [(plan, record)]
        for q in events:
            for k, row in enumerate(q.event_table):
                records[(int(row[4]), int(row[3]))].append((q, k))
        for enc in encs:
            pops, tasks = enc.host_pops, enc.host_tasks
            items, hits = [], {}
            for b in sorted({int(t) for t in tasks[:, 0]}):
                if b >= len(pops):
                    continue
                flags, start = int(pops[b, 7]), int(pops[b, 2])
                # (bits of a population row: 4 = an amplitude per neuron, 0x100 = there is a
                # population, 0x200 = one decay factor, which selects the code that can do this)
                if (flags & 0x304) != 0x300 or start % 2:
                    continue
                mine = tasks[tasks[:, 0] == b]
                n = int(mine[:, 2].sum())
                base = base_at.get(start)
                checks = (base is not None and int(base.size) == n >= 64, (start, n) in records,
                          not np.any(mine[:, 1] % 32),
                          not np.any(self._initial_buf[start:start + n]),
                          base not in self._host_view_index, base not in enc.reads_mem)
                if not all(checks):
                    logger.debug("spikes of item %d stay floats: %s", b, checks)
                    continue
                ok = True
                for q in plans:
                    carried = getattr(q, "carried", None)
                    if carried is not None and base in getattr(carried, "reads_mem", {base}):
                        ok = False
                    if q is enc:
                        continue
                    if base in getattr(q, "writes_mem", {base}):
                        ok = False
                    if base in getattr(q, "reads_mem", {base}):
                        if q not in events:
                            ok = False
                        else:  # every record of that launch that reads the span reads all of it
                            for row in q.event_table:
                                a, m = int(row[4]), int(row[3])
                                if a < start + n and start < a + m and (a, m) != (start, n):
                                    ok = False
                if ok:
                    items.append(b)
                    hits[b] = records[(start, n)]
                else:
                    logger.debug("spikes of item %d stay floats: another launch reads or "
                                 "writes them", b)
            if not items:
                continue
            values = self.backend.store_spikes_as_bits(enc, items, hits, self.model.dt)
            for b, value in values.items():
                start = int(pops[b, 2])
                base = base_at[start]
                self._spike_bits[base] = (start, int(base.size), np.float32(value))

    def _spikes_from_bits(self, base):
        """The spike vector of a population whose spikes device memory holds as bits, as an
        (n, 1) array: the value of a spike where the bit is set."""
        start, n, value = self._spike_bits[base]
        raw = np.ascontiguousarray(np.asarray(self.all_data[self.sidx[base]], dtype=np.float32))
        words = raw.reshape(-1)[:2 * (-(-n // 64))]
        bits = np.unpackbits(words.view(np.uint8), bitorder="little")[:n]
        return (bits.astype(np.float32) * value).reshape(n, 1)

    def _fuse_input_sums(self, plans):
        """A launch that only adds up the decoded inputs of ensembles, right before the
        launch that encodes them and updates the neurons, becomes part of that launch
        (`hipra_gemv.fuse_input_sums`)."""
        out = []
        for plan in plans:
            fused = self.backend.fuse_input_sums(out[-1], plan) if out else None
            if fused is None:
                out.append(plan)
                continue
            fused.reads_mem = out[-1].reads_mem | plan.reads_mem
            fused.writes_mem = out[-1].writes_mem | plan.writes_mem
            out[-1] = fused
        return out

    def _fuse_learning(self, plans):
        """An outer-product learning rule that updates its matrix in place, and the filter of
        the activities it reads, without launches of their own (`hipra_gemv.fuse_learning`):
        the update rides in the launch that decodes with the learned matrices, the filter step
        in the next step's launch that updates the neurons.  Only where nothing else looks at
        what moves: no plan between the decoding launch and the rule touches the rule's
        operands or matrices, nothing but the rule reads the filtered activities (no probe, no
        other operator), no plan from the filter to the end of the step or from its start to
        the neuron launch touches them, and they and the spikes start at zero (the first
        deferred filter step then changes nothing, as the step it stands for never ran)."""
        plans = list(plans)
        conflict = self.backend.plans_conflict
        is_dec = lambda p: (getattr(p, "name", "") == "hipra_gemv.tile_filter"
                            and tuple(getattr(p, "kernel_class", ())) == (3, 2, 4))
        is_enc = lambda p: (getattr(p, "name", "") == "hipra_gemv.tile_lif"
                            and tuple(getattr(p, "kernel_class", ())) == (3, 3, 4))
        is_rule = lambda p: bool((getattr(p, "ew_spec", None) or {}).get("outer")
                                 and (getattr(p, "ew_spec", None) or {}).get("inc"))
        try:
            j = next(k for k, p in enumerate(plans) if is_dec(p))
            i = next(k for k in range(j - 1, -1, -1) if is_enc(plans[k]))
            r = next(k for k in range(j + 1, len(plans)) if is_rule(plans[k]))
            f = next(k for k in range(r + 1, len(plans)) if getattr(plans[k], "lf_spec", None))
        except StopIteration:
            return self._learning_apart(plans, 1)
        enc, dec, rule, lf = plans[i], plans[j], plans[r], plans[f]
        rule_ops = getattr(rule, "planned_ops", None)
        lf_ops = getattr(lf, "planned_ops", None)
        if not rule_ops or not lf_ops or len(lf_ops) != len(lf.lf_spec["X"]):
            return self._learning_apart(plans, 2)
        if any(conflict(rule, q) for q in plans[j + 1:r]):
            return self._learning_apart(plans, 3)
        activities = {op.pre_filtered.base for op in rule_ops if hasattr(op, "pre_filtered")}
        if len(activities) != len(rule_ops):
            return self._learning_apart(plans, 4)
        moving = [op for op in lf_ops if op.output.base in activities]
        probed = {self.model.sig[p]["in"].base for p in self.model.probes}
        for op in moving:
            out, spikes = op.output, op.input
            readers = [q for q in self.operators if q is not op and any(
                sig.base is out.base for sig in list(q.reads) + list(q.incs) + list(q.updates))]
            if (out.base is not out or spikes.base is not spikes or out.base in probed
                    or any(q not in rule_ops for q in readers) or out.base in self._shared
                    or np.any(np.asarray(out.initial_value)) or np.any(np.asarray(spikes.initial_value))):
                return self._learning_apart(plans, 5)
        moved = type("Moved", (), {"reads_mem": {op.input.base for op in moving},
                                   "writes_mem": {op.output.base for op in moving}})
        if any(conflict(moved, q) for q in plans[f + 1:] + plans[:i]):
            return self._learning_apart(plans, 6)
        # neither launch may touch on its own what the other part relies on
        if (dec.writes_mem & (rule.reads_mem | moved.writes_mem)) or (enc.reads_mem & moved.writes_mem):
            return self._learning_apart(plans, 7)
        result = self.backend.fuse_learning(enc, dec, rule, lf)
        if result is None:
            return self._learning_apart(plans, 8)
        new_enc, new_dec, residual, pending = result
        new_enc.reads_mem = enc.reads_mem | moved.reads_mem
        new_enc.writes_mem = enc.writes_mem | moved.writes_mem
        new_dec.reads_mem = dec.reads_mem | rule.reads_mem
        new_dec.writes_mem = dec.writes_mem | rule.writes_mem
        for p in residual:
            rest = [op for op in lf_ops if op not in moving]
            p.reads_mem = {op.input.base for op in rest}
            p.writes_mem = {op.output.base for op in rest}
            p.planned_ops = rest
        for op in moving:
            start = int(self.all_data.starts[self.sidx[op.output]])
            spike_start, a_bits, b_bits, n = pending[start]
            assert spike_start == int(self.all_data.starts[self.sidx[op.input]]) and n == op.output.size
            bits = lambda v: None if v is None else np.int32(v).view(np.float32)
            self._pending_filters[op.output.base] = (op.input.base, bits(a_bits), bits(b_bits))
        plans[f:f + 1] = residual
        del plans[r]
        plans[j] = new_dec
        plans[i] = new_enc
        return plans

    @staticmethod
    def _learning_apart(plans, which):
        logger.debug("learning rule and activity filters keep their launches (check %d of "
                     "`_fuse_learning` did not hold)", which)
        return plans

    def _with_pending_filter(self, base, stored):
        """The output of a filter whose last step is pending in device memory, as the
        reference holds it: that step applied (the two rounded operations of the kernel)."""
        spikes, a0, b0 = self._pending_filters[base]
        x = np.asarray(self.all_data[self.sidx[spikes]], dtype=np.float32).reshape(stored.shape)
        bx = np.float32(b0) * x
        return bx if a0 is None else bx - np.float32(a0) * np.asarray(stored, dtype=np.float32)

    def _fuse_outer_filters(self, plans):
        """An outer-product update (a learning rule's weight increment) and the launch behind
        it that filters its column operands become one launch
        (`hipra_nonlinearities.fuse_outer_filter`), when the plans between the two touch
        nothing that the one that moves reads or writes."""
        plans = list(plans)
        conflict = self.backend.plans_conflict
        j = 0
        while j < len(plans):
            lf = plans[j]
            j += 1
            if getattr(lf, "lf_spec", None) is None:
                continue
            i = j - 2
            while i >= 0 and not (getattr(plans[i], "ew_spec", None) or {}).get("outer"):
                i -= 1
            if i < 0:
                continue
            ew, between = plans[i], plans[i + 1:j - 1]
            # the filters move up to the outer product, or the outer product down to them
            if not any(conflict(lf, q) for q in between):
                at = i
            elif not any(conflict(ew, q) for q in between):
                at = j - 2
            else:
                continue
            fused = self.backend.fuse_outer_filter(ew, lf)
            if fused is None:
                continue
            fused.reads_mem = ew.reads_mem | lf.reads_mem
            fused.writes_mem = ew.writes_mem | lf.writes_mem
            del plans[j - 1]
            del plans[i]
            plans.insert(at, fused)
            j -= 1
        return plans

    def _fuse_filter_epilogues(self, plans):
        """Synapse filters whose input is the output of a large GEMV item become the
        epilogue of that GEMV (`hipra_gemv.fuse_linearfilter`), when no plan between
        the two touches what the filter reads or writes."""
        plans = list(plans)
        j = 0
        while j < len(plans):
            lf = plans[j]
            j += 1
            if getattr(lf, "lf_spec", None) is None:
                continue
            i = j - 2
            between = []  # plans the fused filters would move ahead of
            producer = lambda p: hasattr(p, "prog") or (
                hasattr(p, "spmv") and hasattr(self.backend, "fuse_spmv_filter"))
            while i >= 0 and not producer(plans[i]):
                if not hasattr(plans[i], "enqueue"):
                    i = -1
                    break
                between.append(plans[i])
                i -= 1
            if i < 0:
                continue
            lo = i
            if hasattr(plans[i], "spmv"):
                result = self.backend.fuse_spmv_filter(plans[i], lf)
            else:
                while lo > 0 and getattr(plans[lo - 1], "prog", None) is plans[i].prog:
                    lo -= 1
                result = self.backend.fuse_gemv_filter(plans[lo:i + 1], lf)
            if result is None:
                continue
            fused, residual = result
            # memory of the filters that moved into the GEMV / of those that stayed behind
            ops = getattr(lf, "planned_ops", None)
            rest = set(residual[0].unfused_items) if residual else set()
            if ops is not None and len(ops) == len(lf.lf_spec["X"]):
                mem = lambda sel: ({op.input.base for k, op in enumerate(ops) if sel(k)},
                                   {op.output.base for k, op in enumerate(ops) if sel(k)})
                (fr, fw), (rr, rw) = mem(lambda k: k not in rest), mem(lambda k: k in rest)
            else:
                (fr, fw), (rr, rw) = (lf.reads_mem, lf.writes_mem), (lf.reads_mem, lf.writes_mem)
            # only the filters that move must not touch what the plans in between touch
            # (the others stay where they are): a learning rule that reads a filtered
            # activity does not keep the synapses of decoded values out of the GEMV
            moved = type("Moved", (), {"reads_mem": fr, "writes_mem": fw})
            if any(self.backend.plans_conflict(moved, q) for q in between):
                continue
            for new, old in zip(fused, plans[lo:i + 1]):
                new.reads_mem = old.reads_mem | fr
                new.writes_mem = old.writes_mem | fw
            for p in residual:
                p.reads_mem, p.writes_mem = rr, rw
                if ops is not None and len(ops) == len(lf.lf_spec["X"]):
                    p.planned_ops = [op for k, op in enumerate(ops) if k in rest]
                if getattr(p, "bufpos", None) is not None:
                    self._filter_positions.append(p.bufpos)
            plans[j - 1:j] = residual
            plans[lo:i + 1] = fused
            j += len(residual) - 1
        return plans

    # ------------------------------------------------------------ build help
    @staticmethod
    def _nengo_build(network, dt):
        try:
            from nengo.builder import Model
            from nengo.cache import get_default_decoder_cache
        except ImportError as e:
            raise ImportError(
                "building a nengo Network needs the `nengo` package (>= 3.1); without it "
                "pass a minibuilder.Network or a ready ir.Model") from e
        from .builder import Builder
        from .version import check_nengo_version

        import nengo

        check_nengo_version(nengo)  # (the reference does this first, simulator.py:195-206)
        model = Model(dt=float(dt), label="%s, dt=%f" % (network, dt),
                      decoder_cache=get_default_decoder_cache(), builder=Builder())
        model.build(network)
        return model

    @staticmethod
    def _initial_values(all_operators, all_bases):
        if all_operators and type(all_operators[0]).__module__.startswith("nengo."):
            from nengo.builder.signal import SignalDict

            sigdict = SignalDict()
            for op in all_operators:
                op.init_signals(sigdict)
            # signals that only the rewritten operator list knows (the constant one of the
            # fused copies) are not among nengo's operators: their own initial value
            return {b: sigdict[b] if b in sigdict else np.array(b.initial_value)
                    for b in all_bases}
        return {b: b.initial_value for b in all_bases}

    def RaggedArray(self, listofarrays, **kwargs):
        kwargs.setdefault("align", True)
        return self.backend.upload(RaggedArray(listofarrays, **kwargs))

    def Array(self, val, dtype=np.float32):
        return self.backend.array(val, dtype=dtype)

    # ------------------------------------------------------------- lifecycle
    def __del__(self):
        if not getattr(self, "closed", True):
            warnings.warn("Simulator with model=%s was deallocated while open. Please close "
                          "simulators manually to ensure resources are properly freed."
                          % self.model, ResourceWarning)

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()

    def __getitem__(self, item):
        """Internally shaped (always 2-D) value of a signal."""
        return self.all_data[self.sidx[item]]

    def __getstate__(self):
        raise NotImplementedError("this simulator does not support pickling")

    def __setstate__(self, state):
        raise NotImplementedError("this simulator does not support pickling")

    @property
    def dt(self):
        return self.model.dt

    @dt.setter
    def dt(self, dummy):
        raise ReadonlyError("dt is read-only")

    @property
    def n_steps(self):
        return self._n_steps

    @property
    def time(self):
        return self._time

    @property
    def signals(self):
        """Get / set signal values in their own shape (0-, 1- or 2-D)."""
        sim = self

        class Accessor(Mapping):
            def __iter__(self):
                return iter(sim.all_bases)

            def __len__(self):
                return len(sim.all_bases)

            def __getitem__(self, item):
                base = item.base
                if base in sim._not_computed:
                    raise ValueError(
                        "%s is not computed by this simulator: a rewrite of the operator "
                        "graph folded it into another operator (a learning rule that updates "
                        "its matrix in place does not write its delta; a vector that was only "
                        "a copy is read at its source).  Simulator(reference_host_state=True) "
                        "keeps every signal of the model." % (item,))
                if base in sim._host_view_index:
                    # between two steps the reference holds what this signal was before
                    # the last step's update of it
                    full = np.array(sim._host_view_copy[sim._host_view_index[base]])
                    raw = full if base is item else sim._view_of(item, full)
                elif base in sim._pending_filters:
                    full = sim._with_pending_filter(base, np.array(sim.all_data[sim.sidx[base]]))
                    raw = full if base is item else sim._view_of(item, full)
                elif base in sim._spike_bits:
                    full = sim._spikes_from_bits(base)
                    raw = full if base is item else sim._view_of(item, full)
                else:
                    sim._refresh_lazy(base)
                    raw = sim.all_data[sim.sidx[item]]
                if item.ndim == 0:
                    return raw[0, 0]
                if item.ndim == 1:
                    return raw.ravel()
                if item.ndim == 2:
                    return raw
                raise NotImplementedError()

            def __setitem__(self, item, val):
                incoming = np.asarray(val)
                base = item.base
                sim._refresh_lazy(base)  # (a later read must not recompute over the write)
                if base in sim._shared:
                    raise ValueError(
                        "%s shares its memory with other signals of the model that compute "
                        "the same values (merged connections): a write would change all of "
                        "them.  Simulator(dedup=False) keeps them apart." % (item,))
                resolved = sim.signal_aliases.get(base, base)
                if base in sim._copied_constants or resolved in sim._copied_constants:
                    raise ValueError(
                        "%s is a constant whose device copy in another layout would go stale; "
                        "build the simulator with NENGO_HIP_EVENT_GEMV=0 (or "
                        "reference_host_state=True) to change it at run time" % (item,))
                if base in sim._not_computed:
                    raise ValueError(
                        "%s is not computed by this simulator (see reading it); "
                        "Simulator(reference_host_state=True) keeps every signal" % (item,))
                deferred = set(sim._pending_filters) | {v[0] for v in sim._pending_filters.values()}
                if base in deferred:
                    raise ValueError(
                        "%s belongs to a filter whose last step is still pending in device "
                        "memory (it runs with the next step's neuron update): a write would be "
                        "filtered once more or lost.  NENGO_HIP_FOLD_LEARNING=0 (or "
                        "Simulator(reference_host_state=True)) keeps the filter a launch of the "
                        "step it belongs to." % (item,))
                if base in sim._spike_bits:
                    raise ValueError(
                        "%s is kept as one bit per neuron in device memory (only launches that "
                        "visit the columns of the neurons that spiked read it).  "
                        "NENGO_HIP_SPIKE_BITS=0 (or Simulator(reference_host_state=True)) keeps "
                        "a float per neuron." % (item,))
                if base in sim._updated_in_place:
                    raise ValueError(
                        "%s is updated in place by its learning rule: the change of the last "
                        "step is already part of it and a write would lose it.  "
                        "Simulator(learn_in_place=False) keeps the reference's two passes."
                        % (item,))
                if base in sim._host_view_index:
                    # a node input that synapses write directly: the reference overwrites
                    # it at the start of the next step, so a host write only changes what
                    # the host reads back, not the simulation
                    k = sim._host_view_index[base]
                    full = np.array(sim._host_view_copy[k])
                    window = sim._view_of(item, full)
                    window[...] = incoming.reshape(window.shape)
                    sim._host_view_copy[k] = full
                    return
                if item.ndim == 0:
                    assert incoming.size == 1
                    sim.all_data[sim.sidx[item]] = incoming
                elif item.ndim == 1:
                    assert (item.size,) == incoming.shape
                    sim.all_data[sim.sidx[item]] = incoming[:, None]
                elif item.ndim == 2:
                    assert item.shape == incoming.shape
                    sim.all_data[sim.sidx[item]] = incoming
                else:
                    raise NotImplementedError()

            def __str__(self):
                sio = StringIO()
                for k in self:
                    print(k, self[k], file=sio)
                return sio.getvalue()

        return Accessor()

    def _view_of(self, sig, base_array):
        """The window of ``base_array`` (the 2-D image of ``sig.base``) that ``sig`` covers,
        in the 2-D shape the ragged index gives the view."""
        i, b = self.sidx[sig], self.sidx[sig.base]
        ra = self.all_data
        offset = int(ra.starts[i]) - int(ra.starts[b])
        flat = base_array.reshape(-1)
        return np.lib.stride_tricks.as_strided(
            flat[offset:], shape=(int(ra.shape0s[i]), int(ra.shape1s[i])),
            strides=(4 * int(ra.stride0s[i]), 4 * int(ra.stride1s[i])))

    def signal_buffer(self):
        """A host copy of the whole signal buffer as the reference holds it between two
        steps: currents that their launch does not store are brought up to date first, and
        signals that device memory holds a step ahead are taken from the copy made before
        the last step."""
        for base in list(self._lazy_currents):
            self._refresh_lazy(base)
        buf = np.array(self.all_data.buf)
        for base in self._pending_filters:
            i = self.sidx[base]
            start, n = int(self.all_data.starts[i]), int(base.size)
            buf[start:start + n] = self._with_pending_filter(base, buf[start:start + n]).reshape(-1)
        for base, k in self._host_view_index.items():
            i = self.sidx[base]
            start = int(self.all_data.starts[i])
            flat = np.asarray(self._host_view_copy[k], dtype=np.float32).reshape(-1)
            buf[start:start + flat.size] = flat
        for base, (start, n, value) in self._spike_bits.items():
            words = np.ascontiguousarray(buf[start:start + 2 * (-(-n // 64))])
            bits = np.unpackbits(words.view(np.uint8), bitorder="little")[:n]
            buf[start:start + n] = bits.astype(np.float32) * value
        return buf

    def clear_probes(self):
        for probe in self.model.probes:
            self._probe_outputs[probe] = []
        self.data.reset()

    def close(self):
        self.closed = True
        if getattr(self, "_plans", None) is not None:
            self._plans.close()
        self.context = None
        self.queue = None
        self.all_data = None
        self._plans = None
        self._raggedarrays_to_reset = None
        self._probe_plan = None
        self._drain = None
        self._host_view_copy = None
        self._host_view_plan = None

    # ---------------------------------------------------------------- probes
    def _probe(self, steps_since_drain=None):
        """Drain the device probe buffers into ``sim.data`` and refresh ``n_steps`` /
        ``time``.  ``steps_since_drain`` bounds the rows a probe can have buffered."""
        plan = self._probe_plan
        drain = self._drain
        if drain is not None:
            if plan is None:
                self._n_steps, self._time = (lambda r: (int(r[0]), r[1]))(drain(0))
                return
            if steps_since_drain is None:
                bound = int(plan.Y.shape0s.max())
            else:
                bound = int(steps_since_drain // max(int(self._min_period), 1)) + 1
            if bound <= drain.max_rows():
                step, time, counts, rows = drain(bound)
                self._n_steps, self._time = int(step), time
                complete = True
                for i, probe in enumerate(self.model.probes):
                    cap = int(plan.Y.shape0s[i])
                    if counts[i] > cap:
                        raise RuntimeError("probe buffer %d overran: %d samples for %d rows"
                                           % (i, counts[i], cap))
                    complete = complete and counts[i] == len(rows[i])
                if complete:
                    for i, probe in enumerate(self.model.probes):
                        shape = self.model.sig[probe]["in"].shape
                        if len(rows[i]):
                            self._probe_outputs[probe].extend(
                                rows[i].reshape((len(rows[i]),) + shape))
                    return
                # more rows than the bound (cannot happen with the bound above): the rows
                # are still in the buffers, only the positions were zeroed
                for i, probe in enumerate(self.model.probes):
                    shape = self.model.sig[probe]["in"].shape
                    n_buffered = int(counts[i])
                    if n_buffered:
                        got = self.backend.read_rows(plan.Y, i, n_buffered)
                        self._probe_outputs[probe].extend(got.reshape((n_buffered,) + shape))
                return
        self.backend.finish()
        self._probe_step_time()
        if plan is None:
            return
        bufpositions = self.backend.get_array(plan.dev_bufpositions)
        for i, probe in enumerate(self.model.probes):
            shape = self.model.sig[probe]["in"].shape
            n_buffered = int(bufpositions[i])
            if n_buffered:
                rows = self.backend.read_rows(plan.Y, i, n_buffered)
                self._probe_outputs[probe].extend(rows.reshape((n_buffered,) + shape))
        self.backend.fill_array(plan.dev_bufpositions, 0)
        self.backend.finish()

    def _probe_step_time(self):
        self._n_steps = int(self.signals[self.model.step].item())
        self._time = float(self.signals[self.model.time].item())

    def _reset_probes(self):
        if self._probe_plan is not None:
            self.backend.fill_array(self._probe_plan.dev_bufpositions, 0)
            # also restart the sampling phase (the reference leaves the countdowns as they are)
            self.backend.set_array(self._probe_plan.dev_countdowns,
                                   self._probe_plan.periods - np.float32(1))
        for probe in self.model.probes:
            self._probe_outputs[probe] = []
        self.data.reset()
        self._probes_drained = True
        self._probe_step_time()

    def reset(self, seed=None):
        """Back to the initial state (signals, filter memories, probe buffers)."""
        if self.closed:
            raise SimulatorClosed("Cannot reset closed Simulator.")
        if seed is not None:
            raise NotImplementedError("Seed changing not implemented")
        self.backend.write_all(self.all_data, self._initial_buf)
        for dev, host in self._raggedarrays_to_reset:
            self.backend.write_all(dev, host.buf)
        for pos in self._filter_positions:
            self.backend.fill_array(pos, 0)
        for plan in self._noise_plans:
            plan.reset_streams()
        for rng, state in self._python_rngs.items():
            rng.set_state(state)
        if self._host_view_copy is not None:
            self._host_view_plan()
        for group in self._lazy_currents.values():
            group["at_step"] = None
        self._reset_probes()

    # ------------------------------------------------------------------- run
    def run(self, time_in_seconds, progress_bar=None):
        """Advance by ``time_in_seconds`` (rounded to the nearest multiple of dt)."""
        if time_in_seconds < 0:
            raise ValidationError("Must be positive (got %g)" % (time_in_seconds,))
        steps = int(np.round(float(time_in_seconds) / self.dt))
        if steps == 0:
            warnings.warn("%g results in running for 0 timesteps. Simulator still at time %g."
                          % (time_in_seconds, self.time))
        else:
            self.run_steps(steps, progress_bar=progress_bar)

    def run_steps(self, steps, progress_bar=True):
        """Advance by ``steps`` timesteps, draining probe buffers every
        ``n_prealloc_probes * min(period)`` steps."""
        if self.closed:
            raise SimulatorClosed("Simulator cannot run because it is closed.")
        if self.n_steps + steps >= 2 ** 24:
            # the step counter is a float32 signal: beyond this n + 1 == n
            raise ValueError("Cannot handle more than 2**24 steps")
        if steps < 0:
            raise ValueError("Cannot run for negative steps (got %r)" % (steps,))
        # every path that runs steps drains afterwards, so the buffers are empty here
        assert self._probes_drained

        while steps > 0:
            B = min(steps, self._max_steps_between_probes)
            self._probes_drained = False
            if self._drain is not None and not self._plans.profiling:
                # the drain is queued right behind the steps and waits for both: one host
                # round trip per batch instead of two
                self._plans.enqueue_n_times(B)
            else:
                self._plans.call_n_times(B)
            self._probe(B)
            self._probes_drained = True
            steps -= B

        if self.profiling > 1:
            self.print_profiling()

    def step(self):
        return self.run_steps(1, progress_bar=False)

    def trange(self, sample_every=None, dt=None):
        """Times of the probed samples (starting at dt, not 0)."""
        if dt is not None:
            if sample_every is not None:
                raise ValidationError("Cannot specify both `dt` and `sample_every`.")
            warnings.warn("`dt` is deprecated. Use `sample_every` instead.", DeprecationWarning)
            sample_every = dt
        period = 1 if sample_every is None else sample_every / self.dt
        steps = np.arange(1, self.n_steps + 1)
        return self.dt * steps[steps % period < 1]

    # ------------------------------------------------------------- planning
    # probe rows buffered on the device when `n_prealloc_probes` is None: as many as fit
    # this many bytes, between the reference's 32 and 4096 (draining means a device
    # sync and several host copies, which cost tens of steps of a fast model)
    PROBE_BUFFER_BYTES = 64 * 1024 * 1024

    def _plan_probes(self):
        probes = self.model.probes
        if self.n_prealloc_probes is None:
            row_bytes = 4 * sum(self.model.sig[p]["in"].size for p in probes)
            rows = self.PROBE_BUFFER_BYTES // max(row_bytes, 1)
            self.n_prealloc_probes = int(min(4096, max(32, rows - rows % 32)))
        if len(probes) == 0:
            self._max_steps_between_probes = self.n_prealloc_probes
            self._probe_plan = None
            return []
        n_prealloc = self.n_prealloc_probes
        periods = [max(1 if p.sample_every is None else p.sample_every / self.dt, 1)
                   for p in probes]
        X = self.all_data[[self.sidx[self.model.sig[p]["in"]] for p in probes]]
        Y = self.RaggedArray([np.zeros((n_prealloc, self.model.sig[p]["in"].size))
                              for p in probes], dtype=np.float32)
        plan = self.backend.plan_probes(self.queue, periods, X, Y)
        self._max_steps_between_probes = n_prealloc * int(min(periods))
        self._min_period = int(min(periods))
        self._probe_plan = plan
        assert self._max_steps_between_probes >= 1
        return [plan]

    _cl_probe_plan = property(lambda self: self._probe_plan)

    def _plan_op_group(self, op_type, ops):
        return getattr(self, "_plan_" + op_type.__name__)(ops)

    def _plan_SimProbe(self, ops):
        return []

    def _plan_MultiDotInc(self, ops):
        constant_bs = [op for op in ops if op._float_beta is not None]
        if len(constant_bs) != len(ops):
            raise NotImplementedError("signal-valued beta")
        extra = {}
        if getattr(self.backend, "event_driven_products", False) and not self.reference_host_state:
            # products of a constant matrix with the spikes of a population: only the columns
            # of the neurons that spiked need to be visited
            spikes = {op2.output.base for op2 in self.operators
                      if type(op2).__name__ == "SimNeurons"
                      and type(op2.neurons).__name__ in SPIKING_NEURON_TYPES}
            # (populations a calibration run saw spiking too densely keep the dense product)
            spikes -= self._spike_sources_read_whole
            written = {s.base for op2 in self.operators
                       for s in list(op2.sets) + list(op2.incs) + list(op2.updates)}
            constant = lambda sig: getattr(sig.base, "readonly", False) and sig.base not in written
            extra["event_items"] = [
                k for k, op in enumerate(constant_bs)
                if len(self._A_views[op]) == 1 and self._X_views[op][0].base in spikes
                and constant(self._A_views[op][0])]
            self._event_spike_sources |= {self._X_views[constant_bs[k]][0].base
                                          for k in extra["event_items"]}
        return self._sig_gemv(
            constant_bs,
            lambda op: self._A_views[op], lambda op: self._X_views[op],
            lambda op: self._YYB_views[op][0], lambda op: self._YYB_views[op][1],
            beta=[op._float_beta for op in constant_bs],
            gamma=[op.gamma for op in constant_bs],
            tag="c-beta-%d" % len(constant_bs), **extra)

    def _sig_gemv(self, ops, A_js_fn, X_js_fn, Y_fn, Y_in_fn=None, alpha=1.0, beta=1.0,
                  gamma=0.0, tag=None, **extra):
        if len(ops) == 0:
            return []
        all_data, sidx = self.all_data, self.sidx
        A_js = [np.array([sidx[s] for s in A_js_fn(op)], dtype=np.int32) for op in ops]
        X_js = [np.array([sidx[s] for s in X_js_fn(op)], dtype=np.int32) for op in ops]
        Y_sigs = [Y_fn(op) for op in ops]
        Y_in_sigs = [Y_in_fn(op) for op in ops] if Y_in_fn else Y_sigs
        Y = all_data[[sidx[s] for s in Y_sigs]]
        Y_in = all_data[[sidx[s] for s in Y_in_sigs]]
        prog = self.backend.plan_block_gemv(self.queue, alpha, all_data, A_js, all_data, X_js,
                                            beta, Y, Y_in=Y_in, gamma=gamma, tag=tag, **extra)
        for plan in prog.plans:
            if getattr(plan, "event_driven", False):
                # these matrices have a second, transposed copy on the device
                self._copied_constants.update(
                    sig.base for b in plan.members for sig in A_js_fn(ops[b]))
        return prog.plans

    def _plan_SparseDotSet(self, ops):
        return self._plan_SparseDotInc(ops, inc=False)

    def _plan_SparseDotInc(self, ops, inc=True):
        """All sparse products of the group in one launch (the reference plans one
        launch per operator, simulator.py:877-892)."""
        matrices = []
        for op in ops:
            value = self.sparse_data[op.A]
            matrices.append(value.csr if hasattr(value, "csr") else value)
        X = self.all_data[[self.sidx[op.X] for op in ops]]
        Y = self.all_data[[self.sidx[op.Y] for op in ops]]
        extra = {}
        if getattr(self.backend, "skips_zero_operands", False):
            # vectors that are the spikes of a population are zero in most places
            spikes = {op2.output.base for op2 in self.operators
                      if type(op2).__name__ == "SimNeurons"
                      and type(op2.neurons).__name__ in SPIKING_NEURON_TYPES}
            extra["x_mostly_zero"] = [op.X.base in spikes for op in ops]
        return self.backend.plan_sparse_dot_inc(self.queue, matrices, X, Y, inc=inc, **extra).plans

    def _plan_TimeUpdate(self, ops):
        (op,) = ops
        step = self.all_data[[self.sidx[op.step]]]
        time = self.all_data[[self.sidx[op.time]]]
        return [self.backend.plan_timeupdate(self.queue, step, time, self.model.dt)]

    def _plan_Reset(self, ops):
        targets = self.all_data[[self.sidx[op.dst] for op in ops]]
        values = np.array([op.value for op in ops], dtype=np.float32)
        return [self.backend.plan_reset(self.queue, targets, values)]

    def _plan_Copy(self, ops):
        copies, sliced = split(ops, lambda op: op.src_slice is None and op.dst_slice is None)
        plans = []
        if copies:
            X = self.all_data[[self.sidx[op.src] for op in copies]]
            Y = self.all_data[[self.sidx[op.dst] for op in copies]]
            incs = np.array([op.inc for op in copies], dtype=np.int32)
            plans.append(self.backend.plan_copy(self.queue, X, Y, incs))
        if sliced:
            def inds(sig, sl):
                return np.arange(sig.size, dtype=np.int32)[Ellipsis if sl is None else sl]

            xinds = [inds(op.src, op.src_slice) for op in sliced]
            yinds = [inds(op.dst, op.dst_slice) for op in sliced]
            if any(len(i) != len(set(i.tolist())) for i in xinds + yinds):
                raise NotImplementedError("Duplicates in indices")
            X = self.all_data[[self.sidx[op.src] for op in sliced]]
            Y = self.all_data[[self.sidx[op.dst] for op in sliced]]
            Xinds = self.RaggedArray(xinds, dtype=np.int32, align=False)
            Yinds = self.RaggedArray(yinds, dtype=np.int32, align=False)
            incs = np.array([op.inc for op in sliced], dtype=np.int32)
            plans.append(self.backend.plan_slicedcopy(self.queue, X, Y, Xinds, Yinds, incs))
        return plans

    def _plan_ElementwiseInc(self, ops):
        A = self.all_data[[self.sidx[op.A] for op in ops]]
        X = self.all_data[[self.sidx[op.X] for op in ops]]
        Y = self.all_data[[self.sidx[op.Y] for op in ops]]
        return [self.backend.plan_elementwise_inc(self.queue, A, X, Y)]

    # --- function nodes
    def _plan_SimPyFunc(self, ops):
        plans = []
        for fn, group in groupby(ops, lambda op: op.fn):
            plans.extend(self._plan_python_fn(fn, ts=[op.t for op in group],
                                              xs=[op.x for op in group],
                                              ys=[op.output for op in group]))
        return plans

    def _found_python_code(self, message):
        if self.if_python_code == "error":
            raise RuntimeError(message)
        if self.if_python_code == "warn":
            warnings.warn(message, RuntimeWarning)

    def _plan_python_fn(self, fn, ts, xs, ys):
        assert len(ts) == len(xs) == len(ys)
        assert all(t is None for t in ts) or all(t is not None for t in ts)
        assert all(x is None for x in xs) or all(x is not None for x in xs)
        assert all(y is None for y in ys) or all(y is not None for y in ys)
        fn_name = fn.__name__ if inspect.isfunction(fn) else getattr(
            fn, "__name__", type(fn).__name__)
        size = lambda s: s.size if s is not None else None

        plans, unplanned = [], []
        for _, group in groupby(zip(ts, xs, ys), lambda s: size(s[1])):
            tt, xx, yy = zip(*group)
            if size(yy[0]) is None:
                self._found_python_code("Function %r has no outputs; it runs on the host."
                                        % fn_name)
                unplanned.extend(zip(tt, xx, yy))
                continue
            try:
                plans.append(self._plan_fn_on_device(fn, tt, xx, yy, fn_name))
            except NotImplementedError as e:
                self._found_python_code("Function %r could not be put on the device: %s"
                                        % (fn_name, e))
                unplanned.extend(zip(tt, xx, yy))
        if unplanned:
            tt, xx, yy = zip(*unplanned)
            plans.append(self._plan_fn_in_python(fn, tt, xx, yy, fn_name))
        return plans

    def _plan_fn_on_device(self, fn, tt, xx, yy, fn_name):
        """The function as a kernel: single unary functions of time from the precompiled
        table (``Node(np.sin)``), everything else traced and compiled at run time
        (reference ``_plan_fn_in_ocl``, simulator.py:968-1009)."""
        from . import fn_trace

        t_in, x_in = tt[0] is not None, xx[0] is not None
        x_dim = xx[0].size if x_in else None
        y_dim = yy[0].size
        assert all((x.size if x is not None else None) == x_dim for x in xx)
        assert all(y.size == y_dim for y in yy)
        vector = lambda s: s.ndim == 1 or (s.ndim == 2 and s.shape[1] == 1)
        if not all(vector(s) for s in list(yy) + (list(xx) if x_in else [])):
            raise NotImplementedError("function nodes on matrix signals")
        try:
            known = _DIRECT_FUNCTIONS.get(fn)
        except TypeError:
            known = None
        if known is not None and t_in and not x_in and y_dim == 1:
            code, init, names = "OUTPUT__[0] = %s(t[0]);" % known, "", ["t"]
        else:
            traced = fn_trace.trace(fn, t_in, x_dim, y_dim)
            code, init, names = traced.code, traced.init, traced.input_names
        inputs = []
        if t_in:
            inputs.append(self.all_data[[self.sidx[t] for t in tt]])
        if x_in:
            inputs.append(self.all_data[[self.sidx[x] for x in xx]])
        output = self.all_data[[self.sidx[y] for y in yy]]
        return self.backend.plan_direct(self.queue, code, init, names, inputs, output, tag=fn_name)

    def _plan_fn_in_python(self, fn, tt, xx, yy, fn_name):
        t_in = tt[0] is not None
        t_idx = self.sidx[self.model.time]
        ix_iy = [(self.sidx[x] if x is not None else None, self.sidx[y] if y is not None else None)
                 for x, y in zip(xx, yy)]

        def step():
            t = float(self.all_data[t_idx][0, 0]) if t_in else 0.0
            for ix, iy in ix_iy:
                args = [t] if t_in else []
                if ix is not None:
                    x = self.all_data[ix]
                    args.append(x[:, 0] if x.ndim == 2 and x.shape[1] == 1 else x)
                y = fn(*args)
                if iy is not None:
                    y = np.asarray(y, dtype=np.float32)
                    self.all_data[iy] = y[:, None] if y.ndim == 1 else y

        return PythonPlan(step, name="python_fn", tag=fn_name)

    # --- neurons
    def _plan_SimNeurons(self, all_ops):
        plans = []
        for neuron_class, ops in groupby(all_ops, lambda op: op.neurons.__class__):
            attr = "_plan_%s" % neuron_class.__name__
            if not hasattr(self, attr):
                raise ValueError("Unsupported neuron type '%s'" % neuron_class.__name__)
            plans.extend(getattr(self, attr)(ops))
        return plans

    def _plan_LIF(self, ops):
        if not all(op.neurons.min_voltage == 0 for op in ops):
            raise NotImplementedError("LIF min voltage")
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        V = self.all_data[[self.sidx[op.state["voltage"]] for op in ops]]
        W = self.all_data[[self.sidx[op.state["refractory_time"]] for op in ops]]
        S = self.all_data[[self.sidx[op.output] for op in ops]]
        # one value per population: the reference expands these to per-neuron arrays
        ref = np.array([op.neurons.tau_ref for op in ops], dtype=np.float32)
        tau = np.array([op.neurons.tau_rc for op in ops], dtype=np.float32)
        amp = np.array([op.neurons.amplitude for op in ops], dtype=np.float32)
        return [self.backend.plan_lif(self.queue, self.model.dt, J, V, W, S, ref, tau, amp)]

    def _plan_LIFRate(self, ops):
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        R = self.all_data[[self.sidx[op.output] for op in ops]]
        ref = np.array([op.neurons.tau_ref for op in ops], dtype=np.float32)
        tau = np.array([op.neurons.tau_rc for op in ops], dtype=np.float32)
        amp = np.array([op.neurons.amplitude for op in ops], dtype=np.float32)
        return [self.backend.plan_lif_rate(self.queue, self.model.dt, J, R, ref, tau, amp)]

    def _per_population(self, ops, attr):
        return np.array([getattr(op.neurons, attr) for op in ops], dtype=np.float32)

    def _plan_AdaptiveLIF(self, ops):
        if not all(getattr(op.neurons, "min_voltage", 0) == 0 for op in ops):
            raise NotImplementedError("LIF min voltage")
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        V = self.all_data[[self.sidx[op.state["voltage"]] for op in ops]]
        W = self.all_data[[self.sidx[op.state["refractory_time"]] for op in ops]]
        N = self.all_data[[self.sidx[op.state["adaptation"]] for op in ops]]
        S = self.all_data[[self.sidx[op.output] for op in ops]]
        par = lambda name: self._per_population(ops, name)
        return [self.backend.plan_lif(self.queue, self.model.dt, J, V, W, S, par("tau_ref"),
                                      par("tau_rc"), par("amplitude"), N=N, tau_n=par("tau_n"),
                                      inc_n=par("inc_n"))]

    def _plan_AdaptiveLIFRate(self, ops):
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        R = self.all_data[[self.sidx[op.output] for op in ops]]
        N = self.all_data[[self.sidx[op.state["adaptation"]] for op in ops]]
        par = lambda name: self._per_population(ops, name)
        return [self.backend.plan_lif_rate(self.queue, self.model.dt, J, R, par("tau_ref"),
                                           par("tau_rc"), par("amplitude"), N=N,
                                           tau_n=par("tau_n"), inc_n=par("inc_n"))]

    def _plan_RectifiedLinear(self, ops):
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        R = self.all_data[[self.sidx[op.output] for op in ops]]
        return [self.backend.plan_rectified_linear(self.queue, J, R,
                                                   self._per_population(ops, "amplitude"))]

    def _plan_SpikingRectifiedLinear(self, ops):
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        V = self.all_data[[self.sidx[op.state["voltage"]] for op in ops]]
        S = self.all_data[[self.sidx[op.output] for op in ops]]
        return [self.backend.plan_spiking_rectified_linear(
            self.queue, self.model.dt, J, V, S, self._per_population(ops, "amplitude"))]

    def _plan_Sigmoid(self, ops):
        J = self.all_data[[self.sidx[op.J] for op in ops]]
        R = self.all_data[[self.sidx[op.output] for op in ops]]
        return [self.backend.plan_sigmoid(self.queue, J, R, self._per_population(ops, "tau_ref"))]

    # --- processes
    def _plan_SimProcess(self, all_ops):
        plan_groups = defaultdict(list)
        python_ops = []
        for process_class, ops in groupby(all_ops, lambda op: type(op.process)):
            for cls in process_class.__mro__:
                attr = "_plan_" + cls.__name__
                if hasattr(self, attr):
                    plan_groups[attr].extend(ops)
                    break
            else:
                python_ops.extend(ops)
        plans = []
        for attr, ops in plan_groups.items():
            for p in getattr(self, attr)(ops):
                p.planned_ops = ops  # each process class touches its own signals only
                plans.append(p)
        plans += [p for op in python_ops for p in self._plan_python_process(op)]
        return plans

    def _plan_python_process(self, op):
        if not hasattr(op.process, "make_step"):
            raise NotImplementedError("process %r has no device plan" % type(op.process).__name__)
        shape = lambda s: s.shape if s is not None else (0,)
        rng = op.process.get_rng(self.rng)
        state = op.process.make_state(shape(op.input), shape(op.output), self.model.dt, dtype=None)
        fn = op.process.make_step(shape(op.input), shape(op.output), self.model.dt, rng=rng,
                                  state=state)
        plans = self._plan_python_fn(fn, [op.t], [op.input], [op.output])
        self._python_rngs[rng] = rng.get_state()
        return plans

    def _filter_tf(self, op):
        """(num, den) of one synapse in the packing the filter kernel takes."""
        if hasattr(op.process, "discrete_tf"):
            return op.process.discrete_tf(self.model.dt)
        # nengo synapse: state-space step -> transfer function (reference :1196-1227)
        from nengo.utils.filter_design import ss2tf

        state = op.process.make_state(op.input.shape, op.output.shape, self.model.dt, dtype=None)
        f = op.process.make_step(op.input.shape, op.output.shape, self.model.dt, rng=None,
                                 state=state)
        if f.A.size == 0:
            num, den = f.D, np.array([1.0])
        else:
            num, den = ss2tf(f.A, f.B, f.C, f.D)
        num = np.asarray(num).flatten()
        if den[0] != 1.0:
            raise ValidationError("First element of the denominator must be 1")
        return (num[1:] if num[0] == 0 else num), den[1:]

    def _plan_LinearFilter(self, ops):
        nums, dens = zip(*[self._filter_tf(op) for op in ops])
        A = self.RaggedArray(list(dens), dtype=np.float32, align=False)
        B = self.RaggedArray(list(nums), dtype=np.float32, align=False)
        X = self.all_data[[self.sidx[op.input] for op in ops]]
        Y = self.all_data[[self.sidx[op.output] for op in ops]]
        # one ring-buffer row per coefficient, as the reference allocates them (:1231-1236)
        Xbuf0 = RaggedArray([np.zeros(shape) for shape in zip(B.sizes, X.sizes)],
                            dtype=np.float32)
        Ybuf0 = RaggedArray([np.zeros(shape) for shape in zip(A.sizes, Y.sizes)],
                            dtype=np.float32)
        Xbuf, Ybuf = self.backend.upload(Xbuf0), self.backend.upload(Ybuf0)
        self._raggedarrays_to_reset.append((Xbuf, Xbuf0))
        self._raggedarrays_to_reset.append((Ybuf, Ybuf0))
        plans = self.backend.plan_linearfilter(self.queue, X, Y, A, B, Xbuf, Ybuf)
        for p in plans:
            pos = getattr(p, "bufpos", None)
            if pos is not None:
                self._filter_positions.extend(pos if isinstance(pos, tuple) else [pos])
            p.unread_signals = [op.t for op in ops]  # a filter step does not look at the clock
        return plans

    _plan_Lowpass = _plan_LinearFilter

    def _plan_WhiteSignal(self, ops):
        Y = self.all_data[[self.sidx[op.output] for op in ops]]
        t = self.all_data[[self.sidx[self.model.step] for _ in ops]]
        dt = self.model.dt
        signals = []
        for op in ops:
            assert op.input is None and op.output is not None
            if hasattr(op.process, "table"):
                seed = op.process.seed
                rng = np.random.RandomState(seed if seed is not None
                                            else self.rng.randint(2 ** 31 - 1))
                signals.append(op.process.table(dt, op.output.size, rng))
            else:  # nengo process: pull the table out of its step closure (reference :1263-1277)
                rng = op.process.get_rng(self.rng)
                state = op.process.make_state((0,), op.output.shape, dt, dtype=None)
                f = op.process.make_step((0,), op.output.shape, dt, rng, state)
                signals.append(get_closures(f)["signal"])
        signals = self.RaggedArray(signals, dtype=np.float32)
        return [self.backend.plan_presentinput(self.queue, Y, t, signals, dt)]

    def _plan_PresentInput(self, ops):
        ps = [op.process for op in ops]
        Y = self.all_data[[self.sidx[op.output] for op in ops]]
        t = self.all_data[[self.sidx[self.model.step] for _ in ops]]
        inputs = self.RaggedArray([p.inputs.reshape(p.inputs.shape[0], -1) for p in ps],
                                  dtype=np.float32)
        pres_t = np.array([p.presentation_time for p in ps], dtype=np.float32)
        return [self.backend.plan_presentinput(self.queue, Y, t, inputs, self.model.dt,
                                               pres_t=pres_t)]

    # --- learning
    def _plan_SimPES(self, ops):
        return self._plan_learning(ops, self._plan_pes_group)

    def _plan_pes_group(self, ops):
        pre = self.all_data[[self.sidx[op.pre_filtered] for op in ops]]
        error = self.all_data[[self.sidx[op.error] for op in ops]]
        delta = self.all_data[[self.sidx[op.delta] for op in ops]]
        alpha = np.array([-op.learning_rate * self.model.dt / op.pre_filtered.shape[0]
                          for op in ops])
        return [self.backend.plan_elementwise_inc(self.queue, error, pre, delta, alpha=alpha,
                                                  outer=True, inc=ops[0].apply_inc)]

    @staticmethod
    def _by_application(ops):
        """Learning operators split into those that store their change and those that
        add it to the learned matrix (`operators.apply_learning_in_place`)."""
        for op in ops:
            if not hasattr(op, "apply_inc"):
                op.apply_inc = False
        groups = [[op for op in ops if op.apply_inc == flag] for flag in (False, True)]
        return [g for g in groups if g]

    def _plan_learning(self, ops, plan_group):
        plans = []
        for group in self._by_application(ops):
            for plan in plan_group(group):
                plan.planned_ops = group
                plans.append(plan)
        return plans

    def _plan_SimBCM(self, ops):
        return self._plan_learning(ops, self._plan_bcm_group)

    def _plan_bcm_group(self, ops):
        pre = self.all_data[[self.sidx[op.pre_filtered] for op in ops]]
        post = self.all_data[[self.sidx[op.post_filtered] for op in ops]]
        theta = self.all_data[[self.sidx[op.theta] for op in ops]]
        delta = self.all_data[[self.sidx[op.delta] for op in ops]]
        alpha = np.array([op.learning_rate * self.model.dt for op in ops])
        return [self.backend.plan_bcm(self.queue, pre, post, theta, delta, alpha,
                                      inc=ops[0].apply_inc)]

    def _plan_SimOja(self, ops):
        return self._plan_learning(ops, self._plan_oja_group)

    def _plan_oja_group(self, ops):
        pre = self.all_data[[self.sidx[op.pre_filtered] for op in ops]]
        post = self.all_data[[self.sidx[op.post_filtered] for op in ops]]
        weights = self.all_data[[self.sidx[op.weights] for op in ops]]
        delta = self.all_data[[self.sidx[op.delta] for op in ops]]
        alpha = np.array([op.learning_rate * self.model.dt for op in ops])
        beta = np.array([op.beta for op in ops])
        return [self.backend.plan_oja(self.queue, pre, post, weights, delta, alpha, beta,
                                      inc=ops[0].apply_inc)]

    def _plan_SimRLS(self, ops):
        raise NotImplementedError("RLS learning rule not yet supported")

    def _plan_SimVoja(self, ops):
        return self._plan_learning(ops, self._plan_voja_group)

    def _plan_voja_group(self, ops):
        pre = self.all_data[[self.sidx[op.pre_decoded] for op in ops]]
        post = self.all_data[[self.sidx[op.post_filtered] for op in ops]]
        encoders = self.all_data[[self.sidx[op.scaled_encoders] for op in ops]]
        delta = self.all_data[[self.sidx[op.delta] for op in ops]]
        learning_signal = self.all_data[[self.sidx[op.learning_signal] for op in ops]]
        scale = self.RaggedArray([np.asarray(op.scale).reshape(-1) for op in ops],
                                 dtype=np.float32)
        alpha = np.array([op.learning_rate * self.model.dt for op in ops])
        return [self.backend.plan_voja(self.queue, pre, post, encoders, delta, learning_signal,
                                       scale, alpha, inc=ops[0].apply_inc)]

    # --- convolution
    def _plan_ConvInc(self, ops):
        plans = []
        for op in ops:
            conv = op.conv
            assert conv.dimensions in (1, 2)
            channels_last = conv.channels_last
            assert channels_last == conv.input_shape.channels_last
            assert channels_last == conv.output_shape.channels_last
            shape_in, shape_out = tuple(conv.input_shape.shape), tuple(conv.output_shape.shape)
            kernel_shape, strides = tuple(conv.kernel_size), tuple(conv.strides)
            if conv.dimensions == 1:  # a 1-D convolution is a 2-D one over a single row
                assert len(shape_in) == len(shape_out) == 2
                kernel_shape, strides = (1,) + kernel_shape, (1,) + strides
                if channels_last:
                    shape_in, shape_out = (1,) + shape_in, (1,) + shape_out
                else:
                    shape_in = (shape_in[0], 1, shape_in[1])
                    shape_out = (shape_out[0], 1, shape_out[1])
            plan = self.backend.plan_conv2d(
                self.queue, X=self.all_data[[self.sidx[op.X]]], Y=self.all_data[[self.sidx[op.Y]]],
                filters=self.all_data[[self.sidx[op.W]]], biases=None, shape_in=shape_in,
                shape_out=shape_out, kernel_shape=kernel_shape, padding=conv.padding.lower(),
                strides=strides, channels_last=channels_last, conv=True)
            plan.planned_ops = [op]
            plans.append(plan)
        return plans

    # --- noise
    def _plan_WhiteNoise(self, ops):
        assert all(op.input is None for op in ops)
        seeds = [self.rng.randint(2 ** 31 - 1) if op.process.seed is None else op.process.seed
                 for op in ops]
        Y = self.all_data[[self.sidx[op.output] for op in ops]]
        scale = [bool(op.process.scale) for op in ops]
        inc = [op.mode == "inc" for op in ops]
        enums, params = [], []
        for op in ops:
            dist = op.process.dist
            kind = type(dist).__name__
            if kind == "Uniform":
                enums.append(0)
                params.append((dist.low, dist.high))
            elif kind == "Gaussian":
                enums.append(1)
                params.append((dist.mean, dist.std))
            else:
                raise NotImplementedError("white noise with distribution %r" % kind)
        plan = self.backend.plan_whitenoise(self.queue, Y, np.array(enums, dtype=np.int32),
                                            np.array(params, dtype=np.float32), scale, inc,
                                            self.model.dt, seeds)
        self._noise_plans.append(plan)
        plan.unread_signals = [op.t for op in ops]
        return [plan]

    def _plan_FilteredNoise(self, ops):
        raise NotImplementedError()

    # ------------------------------------------------------------- reporting
    def print_plans(self):
        print(" Plans ".center(80, "-"))
        for plan in self._plans:
            print("%r" % plan)
            if hasattr(plan, "description"):
                print(indent(plan.description, 4))

    def profiling_table(self):
        """Rows ``(n_calls, seconds, GF/s, GB/s, plan)`` from the recorded event times."""
        table = []
        for p in self._plans:
            if isinstance(p, BasePlan):
                t = sum(p.ctimes)
                calls_per_sec = p.n_calls / t if t > 0 else np.nan
                gfps = 1e-9 * p.flops_per_call * calls_per_sec if p.flops_per_call else np.nan
                gbps = 1e-9 * p.bw_per_call * calls_per_sec if p.bw_per_call else np.nan
                table.append((p.n_calls, t, gfps, gbps, str(p)))
        return table

    def print_profiling(self, sort=None):
        """Per-plan call count, run time, GF/s and GB/s (needs ``profiling=True``)."""
        if not self.profiling:
            print("Profiling not enabled!")
            return
        table = self.profiling_table()
        if sort is not None:
            table.sort(key=lambda x: x[abs(sort)], reverse=sort >= 0)
        print(" Profiling ".center(80, "-"))
        print("%8s|%10s|%10s|%10s|" % ("n_calls", "runtime", "GF/s", "GB/s"))
        for r in table:
            print("%8d|%10.3f|%10.3f|%10.3f| %s" % r)
        print("-" * 80)
        times = np.array([r[1] for r in table], dtype=np.float64)

        def wmean(col):
            x = np.array([r[col] for r in table], dtype=np.float64)
            m = ~np.isnan(x)
            return (x[m] * times[m]).sum() / times[m].sum() if m.any() else np.nan

        print("totals:\t%2.3f\t%2.3f\t%2.3f" % (times.sum(), wmean(2), wmean(3)))
