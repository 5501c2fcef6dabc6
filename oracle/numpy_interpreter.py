"""A model's operator list evaluated one operator at a time in numpy.  TEST INFRASTRUCTURE
(and, with ``blas=True``, the single-process NumPy leg of ``bench.py``'s CPU baseline); the
product never imports it.

Nothing here uses the simulator's operator rewrites, its planner, its view builder or its
plan_* layer: every base signal is one float32 array, a view is a strided window onto it,
the order of a step is a topological sort made here, and every operator is evaluated by
the formula of the reference kernel it maps to (file:line given per operator), in
float32 with the kernel's order of operations.  A simulator that merges, fuses, reorders
or batches operators must still produce these numbers.

The fused multiply-add of the GEMV partial sums is emulated in extended precision (the
product of two float32 is exact there; one rounding back to float32).

``NaiveInterpreter(model, blas=True)`` forms matrix-vector products with ``A @ x`` instead
(numpy's float32 product, its own summation order): the way a NumPy simulator of such a
model computes a step (one array expression per operator), which is what the CPU baseline
times.  Its results agree with the exact mode to rounding, not bit for bit.
"""

import heapq

import numpy as np

f32 = np.float32


def _fma(a, b, c):
    return (a.astype(np.longdouble) * np.longdouble(b) + c.astype(np.longdouble)).astype(f32)


class NaiveInterpreter:
    def __init__(self, model, blas=False):
        self.model = model
        self.blas = bool(blas)
        self.dt = model.dt
        self.ops = list(model.operators)
        self.mem = {}
        for op in self.ops:
            for sig in op.all_signals:
                if sig.base not in self.mem:
                    if getattr(sig.base, "sparse", False):  # a constant scipy CSR matrix
                        self.mem[sig.base] = sig.base.initial_value.astype(f32)
                    else:
                        self.mem[sig.base] = np.array(sig.base.initial_value, dtype=f32)
        self.order = self._step_order()
        self.tables = {}
        self.n_steps = 0
        self.samples = {p: [] for p in model.probes}

    # ------------------------------------------------------------ memory
    def view(self, sig):
        """Writable float32 window for `sig` onto its base array."""
        base = self.mem[sig.base]
        if sig.base is sig:
            return base
        flat = base.reshape(-1)
        strides = tuple(4 * s for s in sig.elemstrides)
        return np.lib.stride_tricks.as_strided(flat[sig.elemoffset:], shape=sig.shape,
                                               strides=strides, writeable=True)

    # ------------------------------------------------------------ order of a step
    def _step_order(self):
        """Per block of memory: all sets, then incs, then reads, then updates (nengo's
        step semantics, nengo/builder/operator.py as cited by planners.py:5-16 of the
        reference); among operators not ordered by that, the order of the model's list."""
        rank = {"sets": 0, "incs": 1, "reads": 2, "updates": 3}
        by_base = {}
        for i, op in enumerate(self.ops):
            for kind in rank:
                for sig in getattr(op, kind):
                    by_base.setdefault(sig.base, []).append((i, rank[kind], sig))
        after = {i: set() for i in range(len(self.ops))}
        for entries in by_base.values():
            ranked = [[e for e in entries if e[1] == r] for r in range(4)]
            for lo in range(4):  # only pairs of different kinds order each other
                for hi in range(lo + 1, 4):
                    for i, _, si in ranked[lo]:
                        for j, _, sj in ranked[hi]:
                            if i != j and (si is sj or si.may_share_memory(sj)):
                                after[j].add(i)
        indegree = {i: len(after[i]) for i in after}
        users = {i: [] for i in after}
        for j, before in after.items():
            for i in before:
                users[i].append(j)
        ready = [i for i, d in indegree.items() if d == 0]
        heapq.heapify(ready)
        order = []
        while ready:
            i = heapq.heappop(ready)
            order.append(i)
            for j in users[i]:
                indegree[j] -= 1
                if indegree[j] == 0:
                    heapq.heappush(ready, j)
        assert len(order) == len(self.ops), "cycle in the operator graph"
        return order

    # ------------------------------------------------------------ operators
    def _gemv_inc(self, A, x, y):
        """y += A @ x the way the reference's block GEMV adds it (clra_gemv.py:1043-1058,
        :1148-1153): per tile of 128 columns four strided partial sums, fused
        multiply-adds, (s0 + s2) + (s1 + s3); tiles added onto y one after the other."""
        if self.blas:
            y += A @ x
            return
        m, n = A.shape
        acc = y.copy()
        for c0 in range(0, n, 128):
            s = [np.zeros(m, dtype=f32) for _ in range(4)]
            for jj in range(min(128, n - c0)):
                s[jj & 3] = _fma(A[:, c0 + jj], x[c0 + jj], s[jj & 3])
            acc = acc + ((s[0] + s[2]) + (s[1] + s[3]))
        y[...] = acc

    def _DotInc(self, op):
        A, x, y = self.view(op.A), self.view(op.X).reshape(-1), self.view(op.Y)
        if A.size == 1:  # a scalar weight scales the vector (operators.py:175-177)
            y[...] = y + (x * A.reshape(-1)[0]).reshape(y.shape)
        else:
            self._gemv_inc(A.reshape(y.size, x.size), x, y.reshape(-1))

    def _SparseDotInc(self, op):
        """clra_gemv.py:1590-1623 (`sparsedot_inc`): y += A x with A in CSR form.  Only in
        the `blas` mode (scipy's product, its own summation order)."""
        if not self.blas:
            raise NotImplementedError("sparse products are not restated operation by operation")
        y = self.view(op.Y)
        y += (self.mem[op.A.base] @ self.view(op.X).reshape(-1)).reshape(y.shape)

    def _Reset(self, op):
        self.view(op.dst)[...] = f32(op.value)  # clra_nonlinearities.py:147-214

    def _Copy(self, op):
        """clra_nonlinearities.py:217-304 / :307-411."""
        src, dst = self.view(op.src), self.view(op.dst)
        s = src if op.src_slice is None else src[op.src_slice]
        if op.dst_slice is None:
            dst[...] = dst + s if op.inc else s
        else:
            dst[op.dst_slice] = dst[op.dst_slice] + s if op.inc else s

    def _ElementwiseInc(self, op):
        """clra_nonlinearities.py:449-525: y += (alpha * a) * x with alpha = 1."""
        a, x, y = self.view(op.A), self.view(op.X), self.view(op.Y)
        y[...] = y + np.broadcast_to((f32(1.0) * a) * x, y.shape)

    def _TimeUpdate(self, op):
        """clra_nonlinearities.py:119-133: a float32 counter, time = dt * step in double."""
        step, time = self.view(op.step), self.view(op.time)
        step[...] = step + f32(1.0)
        time[...] = f32(self.dt * float(step))

    def _SimNeurons(self, op):
        kind = type(op.neurons).__name__
        J, out = self.view(op.J), self.view(op.output)
        tau, ref, amp = f32(op.neurons.tau_rc), f32(op.neurons.tau_ref), f32(op.neurons.amplitude)
        if kind == "LIFRate":
            # clra_nonlinearities.py:1178-1180
            j = np.maximum(J - f32(1.0), f32(0.0))
            with np.errstate(divide="ignore"):
                out[...] = amp / (ref + tau * np.log1p((f32(1.0) / j).astype(np.float64)).astype(f32))
            return
        assert kind == "LIF", kind
        # clra_nonlinearities.py:1086-1133
        V, W = self.view(op.state["voltage"]), self.view(op.state["refractory_time"])
        dt, dt_inv = f32(self.dt), f32(1.0 / self.dt)
        w = W - dt
        delta_t = np.where(w > dt, f32(0.0), np.where(w < 0, dt, dt - w)).astype(f32)
        dv = -np.expm1((-delta_t / tau).astype(np.float64)).astype(f32) * (J - V)
        v = V + dv
        spiked = v > f32(1.0)
        with np.errstate(divide="ignore", invalid="ignore"):
            t_spike = dt + tau * np.log1p((-(v - f32(1.0)) / (J - f32(1.0))).astype(np.float64)).astype(f32)
        W[...] = np.where(spiked, ref + t_spike, w)
        V[...] = np.where(spiked | (v < 0), f32(0.0), v)
        out[...] = np.where(spiked, amp * dt_inv, f32(0.0))

    def _SimProcess(self, op):
        kind = type(op.process).__name__
        if hasattr(op.process, "table"):
            # table playback, clra_nonlinearities.py:1694-1730
            if op not in self.tables:
                rng = np.random.RandomState(op.process.seed)
                self.tables[op] = op.process.table(self.dt, op.output.size, rng).astype(f32)
            table = self.tables[op]
            step = int(self.mem[self.model.step])
            self.view(op.output)[...] = table[step % len(table)].reshape(op.output.shape)
            return
        assert kind in ("Lowpass", "LinearFilter"), kind
        num, den = op.process.discrete_tf(self.dt)
        x, y = self.view(op.input), self.view(op.output)
        if len(den) == 0 and len(num) == 1:
            y[...] = f32(num[0]) * x
        else:
            # first-order case of clra_nonlinearities.py:604-690: y = b0 x - a0 y
            assert len(den) == 1 and len(num) == 1, "general filters are not restated here"
            y[...] = f32(num[0]) * x - f32(den[0]) * y

    def _SimPyFunc(self, op):
        args = []
        if op.t is not None:
            args.append(float(self.view(op.t)))
        if op.x is not None:
            args.append(np.array(self.view(op.x), dtype=np.float64))
        value = op.fn(*args)
        if op.output is not None:
            self.view(op.output)[...] = np.asarray(value, dtype=np.float64).astype(f32).reshape(
                op.output.shape)

    def _SimPES(self, op):
        """simulator.py:1334-1345 of the reference: delta = (alpha * error) outer pre with
        alpha = -learning_rate * dt / n_pre, written (not added)."""
        pre, err, delta = self.view(op.pre_filtered), self.view(op.error), self.view(op.delta)
        alpha = f32(-op.learning_rate * self.dt / op.pre_filtered.shape[0])
        delta[...] = (alpha * err)[:, None] * pre[None, :]

    # ------------------------------------------------------------ running
    def step(self):
        for i in self.order:
            op = self.ops[i]
            getattr(self, "_" + type(op).__name__)(op)
        self.n_steps += 1
        for p in self.model.probes:
            period = 1 if p.sample_every is None else p.sample_every / self.dt
            if self.n_steps % period < 1:  # simulator.py:700-702 of the reference
                self.samples[p].append(np.array(self.view(self.model.sig[p]["in"])).reshape(-1))

    def run_steps(self, n):
        for _ in range(n):
            self.step()

    def data(self, probe):
        return np.array(self.samples[probe])
