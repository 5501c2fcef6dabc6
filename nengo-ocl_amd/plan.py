"""Plans (bound kernel launches) and the executor that replays a timestep.

Counterpart of the reference's ``nengo_ocl/plan.py`` (``BasePlan`` :12-38,
``PythonPlan`` :41-53, ``Plan`` :56-108, ``Plans`` :111-149).  A `Plan` binds one
C-ABI entry point of ``libnengo_hip.so`` to its arguments; the executor does
not issue one driver call per plan per step from Python: the plan sequence is
recorded once from the stream into a HIP graph and replayed ``n`` times by a
single C call.  Host-callback plans (`PythonPlan`) cannot be recorded, so they
split the sequence into graph segments with a stream sync on either side.
"""

import ctypes
import time

from . import _lib


class BasePlan:
    def __init__(self, name="", tag=None, flops_per_call=None, bw_per_call=None):
        self.name = name
        self.tag = tag
        self.atimes = []  # queued -> submitted (always 0 here: HIP events time execution only)
        self.btimes = []  # submitted -> started
        self.ctimes = []  # started -> ended, seconds
        self.n_calls = 0
        self.flops_per_call = flops_per_call
        self.bw_per_call = bw_per_call

    def _label(self):
        return "%s%s" % (self.name, ": %s" % self.tag if self.tag else "")

    def __str__(self):
        return "<%s>" % self._label()

    def __repr__(self):
        return "%s{%s}" % (type(self).__name__, self._label())

    def update_profiling(self):
        pass


class PythonPlan(BasePlan):
    """A host callback executed between device plans (forces a stream sync)."""

    def __init__(self, function, **kwargs):
        super().__init__(**kwargs)
        self.function = function

    def __call__(self, profiling=False):
        t0 = time.time() if profiling else 0.0
        self.function()
        if profiling:
            self.atimes.append(0)
            self.btimes.append(0)
            self.ctimes.append(time.time() - t0)
            self.n_calls += 1


class Plan(BasePlan):
    """One kernel launch with all arguments bound.

    ``kern`` is a ctypes function from ``libnengo_hip.so`` whose first parameter
    is the stream; ``args`` are the remaining arguments.  ``gsize``/``lsize`` are
    kept for display (grid in threads, group size), as in the reference.
    ``full_args`` pins every device array the launch reads so that Python does
    not free them.
    """

    LAUNCHES_WITHOUT_EVENTS = ("nhip_rtc_launch_direct",)

    def __init__(self, queue, kern, args, gsize, lsize=None, full_args=(), **kwargs):
        super().__init__(**kwargs)
        self.queue = queue
        self.kern = kern
        self.args = tuple(args)
        self.gsize = self._format_size(gsize)
        self.lsize = self._format_size(lsize) if lsize is not None else None
        self.full_args = tuple(full_args)
        self._events_to_profile = []
        # (function, arguments) of a call that prepares the launch and launches nothing
        # itself, made right before it (a sequence the launch carries)
        self.prelude = None

    @staticmethod
    def _format_size(size):
        size = tuple(int(s) for s in size)
        if len(size) == 0 or any(s <= 0 for s in size):
            raise ValueError("launch sizes must be positive, got %r" % (size,))
        return size

    def enqueue(self, wait_for=None, profiling=False):
        """Put the launch on the queue's stream; returns immediately."""
        lib = self.queue.lib
        handle = self.queue.handle
        if profiling:
            ev0, ev1 = ctypes.c_void_p(), ctypes.c_void_p()
            _lib.check(lib.nhip_event_create(ctypes.byref(ev0)))
            _lib.check(lib.nhip_event_create(ctypes.byref(ev1)))
            # the kernel carries its own start / stop events where the entry point
            # launches through the runtime API; otherwise events around the launch.  An
            # entry point that issues two launches puts the start event on its first and
            # the stop event on its last.
            own = getattr(self.kern, "__name__", "") not in self.LAUNCHES_WITHOUT_EVENTS
            if own:
                _lib.check(lib.nhip_time_next_launch(ev0, ev1))
            else:
                _lib.check(lib.nhip_event_record(ev0, handle))
        if self.prelude is not None:
            _lib.check(self.prelude[0](*self.prelude[1]), self.name)
        _lib.check(self.kern(handle, *self.args), self.name)
        if profiling:
            if own and lib.nhip_launch_events_pending():
                # the entry point returned without launching (an empty work list): the
                # events were never recorded and there is nothing to time
                _lib.check(lib.nhip_time_next_launch(None, None))
                lib.nhip_event_destroy(ev0)
                lib.nhip_event_destroy(ev1)
                return self
            if not own:
                _lib.check(lib.nhip_event_record(ev1, handle))
            self._events_to_profile.append((ev0, ev1))
        return self

    def wait(self):
        self.queue.finish()

    def __call__(self, profiling=False):
        self.enqueue(profiling=profiling)
        self.wait()

    def update_profiling(self):
        lib = self.queue.lib
        for ev0, ev1 in self._events_to_profile:
            ms = ctypes.c_float()
            _lib.check(lib.nhip_event_elapsed_ms(ev0, ev1, ctypes.byref(ms)))
            self.atimes.append(0.0)
            self.btimes.append(0.0)
            self.ctimes.append(1e-3 * ms.value)
            self.n_calls += 1
            lib.nhip_event_destroy(ev0)
            lib.nhip_event_destroy(ev1)
        self._events_to_profile[:] = []

    def __str__(self):
        return "<%s %s %s>" % (self._label(), self.gsize, self.lsize)

    def __repr__(self):
        return "%s{%s %s %s}" % (type(self).__name__, self._label(), self.gsize, self.lsize)


def plan_dependencies(plans):
    """For every plan, the earlier plans it has to wait for (indices into `plans`),
    transitively reduced.

    Two plans conflict when one writes memory the other reads or writes; `reads_mem`
    and `writes_mem` of a plan are sets of hashable memory-block keys (the Simulator
    uses the base signals of the operators behind the plan).  A plan without them is
    ordered against everything.  The list order of `plans` is a valid execution
    order, so a conflict always means "the later one waits for the earlier one".
    """
    deps, ancestors = [], []
    for i, p in enumerate(plans):
        ri, wi = getattr(p, "reads_mem", None), getattr(p, "writes_mem", None)
        direct = set()
        for j in range(i):
            rj, wj = getattr(plans[j], "reads_mem", None), getattr(plans[j], "writes_mem", None)
            if ri is None or wi is None or rj is None or wj is None:
                direct.add(j)
            elif (wj & ri) or (wj & wi) or (rj & wi):
                direct.add(j)
        reduced, anc = set(), set()
        for j in sorted(direct, reverse=True):
            if j not in anc:
                reduced.add(j)
                anc.add(j)
                anc |= ancestors[j]
        deps.append(reduced)
        ancestors.append(anc)
    return deps


class _GraphSegment:
    """A run of consecutive device plans recorded into executable graphs.

    Between two graph launches the device idles for several microseconds, so the run is
    recorded several times: as a long graph holding `unroll` consecutive timesteps, and
    as graphs of unroll/2, ..., 2, 1 timesteps for what is left over (n steps are then
    n // unroll launches of the long graph plus at most one launch of each shorter one).
    All of them are recorded, instantiated and uploaded to the device by `prepare`,
    before the first step runs, so that no call of `launch` ever records anything.
    """

    # timesteps recorded back to back into the long graph: as many as keep it within
    # MAX_GRAPH_NODES kernel nodes (a step of two launches: 128 steps; of ten: 16)
    MAX_UNROLL = 128
    MAX_GRAPH_NODES = 256

    def __init__(self, queue, plans, before_last=()):
        self.queue = queue
        self.plans = list(plans)
        # plans that run once per `launch`, between its last timestep and the one before
        self.before_last = list(before_last)
        self.execs = {}  # timesteps per graph -> executable graph
        self.tail_execs = {}  # the same with `before_last` recorded ahead of the last step
        unroll = 1
        while unroll * 2 <= self.MAX_UNROLL and unroll * 2 * len(self.plans) <= self.MAX_GRAPH_NODES:
            unroll *= 2
        self.unroll = unroll  # a power of two

    @property
    def sizes(self):
        """Timesteps per recorded graph, longest first."""
        out, n = [], self.unroll
        while n >= 1:
            out.append(n)
            n //= 2
        return out

    def capture(self, n_steps=1, tail=False):
        """Record `n_steps` consecutive timesteps into one executable graph (`tail`: with
        the `before_last` plans ahead of the last of them)."""
        lib = self.queue.lib
        _lib.check(lib.nhip_capture_begin(self.queue.handle), "graph capture begin")
        err = None
        try:
            for k in range(n_steps):
                if tail and k == n_steps - 1:
                    for plan in self.before_last:
                        plan.enqueue()
                for plan in self.plans:
                    plan.enqueue()
        except Exception as e:  # close the capture before re-raising
            err = e
        handle = ctypes.c_void_p()
        rc = lib.nhip_capture_end(self.queue.handle, ctypes.byref(handle))
        if err is not None:
            if rc == 0 and handle:
                lib.nhip_graph_destroy(handle)
            raise err
        _lib.check(rc, "graph capture end")
        (self.tail_execs if tail else self.execs)[n_steps] = handle

    def steps_of_every_graph(self):
        """A step count whose run launches each recorded graph once."""
        return sum(self.sizes)

    def prepare(self):
        """Record every graph `launch` can ask for and hand each to the device ahead of
        its first launch; nothing is executed."""
        for tail, execs in ((False, self.execs), (True, self.tail_execs)):
            if tail and not self.before_last:
                continue
            for n_steps in self.sizes:
                if n_steps not in execs:
                    self.capture(n_steps, tail=tail)
                    _lib.check(self.queue.lib.nhip_graph_upload(execs[n_steps], self.queue.handle),
                               "graph upload")

    @property
    def exec(self):
        return self.execs.get(1)

    def launch(self, n, tail=True):
        """Run `n` timesteps: n // unroll launches of the long graph plus the binary rest.
        With `before_last` plans (and `tail`), the graph that holds the last timestep is the
        variant with those plans recorded ahead of its last step."""
        lib = self.queue.lib
        self.prepare()
        times, rest = divmod(n, self.unroll)
        todo = [(self.unroll, times)] if times else []
        todo += [(n_steps, 1) for n_steps in self.sizes[1:] if rest & n_steps]
        if tail and self.before_last and todo:
            n_steps, count = todo[-1]
            todo[-1:] = ([(n_steps, count - 1)] if count > 1 else []) + [(n_steps, -1)]
        for n_steps, count in todo:
            execs = self.tail_execs if count < 0 else self.execs
            _lib.check(lib.nhip_graph_launch(execs[n_steps], self.queue.handle, abs(count)),
                       "graph launch")

    def destroy(self):
        for handle in list(self.execs.values()) + list(self.tail_execs.values()):
            self.queue.lib.nhip_graph_destroy(handle)
        self.execs, self.tail_execs = {}, {}


class Plans:
    """The ordered plan list of one timestep and its executor."""

    def __init__(self, planlist, profiling, use_graph=True, branches=False, before_last=()):
        if branches and use_graph:
            # Switched off: ending a multi-stream recording crashed inside the HIP runtime
            # (segmentation fault in the call that ends the capture) for a step whose
            # branches depend on each other back and forth (stream 1 -> 2 -> 1), and the
            # mode was slower than the single chain on this driver in every measurement.
            raise NotImplementedError(
                "recording independent kernels as parallel graph branches is switched off "
                "(the runtime did not survive ending such a recording); use branches=False")
        self.plans = list(planlist)
        # device plans that every `call_n_times(n)` runs once, after timestep n - 1 and
        # before timestep n (copies of what the host may ask for as it was before the last
        # step); not part of a timestep, not listed among `plans`
        self.before_last = list(before_last)
        self.profiling = profiling
        self.use_graph = use_graph
        self._segments = None  # list of _GraphSegment | PythonPlan

    def __call__(self):
        return self.call_n_times(1)

    def __len__(self):
        return len(self.plans)

    def __getitem__(self, i):
        return self.plans[i]

    def __iter__(self):
        return iter(self.plans)

    def _queue(self):
        for p in self.plans:
            if hasattr(p, "queue"):
                return p.queue
        return None

    def _build_segments(self):
        segments, run = [], []

        def close_run():
            if run:
                segments.append(_GraphSegment(run[0].queue, run, before_last=self.before_last))

        for plan in self.plans:
            if hasattr(plan, "enqueue"):
                run.append(plan)
            else:
                close_run()
                run = []
                segments.append(plan)
        close_run()
        self._segments = segments

    def steps_of_every_graph(self):
        """A step count whose run launches every recorded graph at least once (0 without
        graphs)."""
        if not self.use_graph:
            return 0
        if self._segments is None:
            self._build_segments()
        return max([seg.steps_of_every_graph() for seg in self._segments
                    if isinstance(seg, _GraphSegment)] or [0])

    def prepare(self):
        """Record all graphs of the executor now (the Simulator calls this once its plan
        list is complete), so that the first `run_steps` -- of any length -- only
        launches.  Does nothing for eager execution."""
        if self.profiling or not self.use_graph:
            return
        if self._segments is None:
            self._build_segments()
        for seg in self._segments:
            if isinstance(seg, _GraphSegment):
                seg.prepare()
        queue = self._queue()
        if queue is not None:
            queue.finish()

    def call_n_times(self, n):
        """Run the whole plan sequence ``n`` times and wait for it to finish."""
        self.enqueue_n_times(n)
        queue = self._queue()
        if queue is not None:
            queue.finish()
        if self.profiling:
            for p in self.plans:
                p.update_profiling()

    def enqueue_n_times(self, n):
        queue = self._queue()
        if self.profiling or not self.use_graph:
            # eager: one launch per plan, events around each when profiling
            for k in range(n):
                if k == n - 1:
                    for plan in self.before_last:
                        plan.enqueue() if hasattr(plan, "enqueue") else plan()
                for plan in self.plans:
                    if hasattr(plan, "enqueue"):
                        plan.enqueue(profiling=self.profiling)
                    else:
                        queue and queue.finish()
                        plan(profiling=self.profiling)
            return

        if self._segments is None:
            self._build_segments()
        if len(self._segments) == 1 and isinstance(self._segments[0], _GraphSegment):
            self._segments[0].launch(n)  # the common case: n replays, one C call
            return
        for k in range(n):
            if k == n - 1:
                for plan in self.before_last:
                    plan.enqueue()
            for seg in self._segments:
                if isinstance(seg, _GraphSegment):
                    seg.launch(1, tail=False)
                else:
                    queue and queue.finish()
                    seg()

    def close(self):
        for seg in self._segments or []:
            if isinstance(seg, _GraphSegment):
                seg.destroy()
        self._segments = None
