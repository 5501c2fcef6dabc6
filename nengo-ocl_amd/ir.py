"""Operator-graph IR: signals, operators, neuron types, processes, model.

The reference consumes what nengo's builder produces: ``Signal`` objects with
views, and ``Operator`` objects that declare which signals they set / inc /
read / update (used at nengo_ocl/simulator.py:230-335, operators.py:19-194,
planners.py:9-95).  nengo itself is a third-party dependency
(``nengo>=3.1.0``, setup.py:31 of the reference) that may be absent, so this
module restates the small part of that interface the timestep path touches,
with nengo's attribute names (``op.dst``, ``op.A``, ``op.neurons.tau_rc``,
``op.state["voltage"]``, ``op.process`` ...).  The Simulator dispatches on
``type(op).__name__``, so graphs built by nengo and graphs built from these
classes take the same route.
"""

import numpy as np


# =============================================================== signals
class Signal:
    """A named block of simulator memory, or a view into another signal."""

    def __init__(self, initial_value=None, shape=None, name=None, base=None, readonly=False):
        if initial_value is None:
            initial_value = np.zeros(() if shape is None else shape)
        value = initial_value if base is not None else np.array(initial_value, copy=True)
        if value.dtype.kind not in "fiub":
            raise TypeError("signals hold numbers, got %s" % value.dtype)
        if base is None and value.dtype.kind in "iub":
            value = value.astype(np.float64)
        self._value = value
        self._value.setflags(write=False)
        self._base = base
        self.name = name
        self._readonly = bool(readonly)

    # --- identity and memory
    @property
    def base(self):
        return self if self._base is None else self._base

    @property
    def is_view(self):
        return self._base is not None

    @property
    def initial_value(self):
        return self._value

    @property
    def readonly(self):
        return self._readonly if self._base is None else self._base.readonly

    sparse = False

    @property
    def dtype(self):
        return self._value.dtype

    @property
    def shape(self):
        return self._value.shape

    @property
    def ndim(self):
        return self._value.ndim

    @property
    def size(self):
        return self._value.size

    @property
    def itemsize(self):
        return self._value.itemsize

    @property
    def offset(self):
        """Byte offset of this view from the start of its base."""
        a = self._value.__array_interface__["data"][0]
        b = self.base._value.__array_interface__["data"][0]
        return a - b

    @property
    def elemoffset(self):
        return self.offset // self.itemsize

    @property
    def strides(self):
        return self._value.strides

    @property
    def elemstrides(self):
        return tuple(s // self.itemsize for s in self._value.strides)

    def may_share_memory(self, other):
        return np.may_share_memory(self._value, other._value)

    # --- views
    def __getitem__(self, item):
        if item is Ellipsis or (isinstance(item, slice) and item == slice(None)):
            return self
        view = self._value[item]
        if not isinstance(view, np.ndarray) or (view.size and not np.may_share_memory(view, self._value)):
            raise ValueError("signals can only be sliced into views (no fancy indexing)")
        return Signal(view, name="%s[%s]" % (self.name, item), base=self.base)

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        view = self._value.reshape(shape)
        if view.size and not np.may_share_memory(view, self._value):
            raise ValueError("reshape would copy")
        return Signal(view, name="%s.reshape%s" % (self.name, (shape,)), base=self.base)

    def __repr__(self):
        return "Signal(name=%s, shape=%s)" % (self.name, self.shape)


class SparseSignal(Signal):
    """A constant sparse matrix (scipy CSR); never sliced or reshaped.  nengo's
    counterpart is a Signal whose initial value is a ``SparseMatrix`` (``sig.sparse``)."""

    sparse = True

    def __init__(self, matrix, name=None):
        import scipy.sparse

        self._csr = scipy.sparse.csr_matrix(matrix, dtype=np.float64)
        self._csr.sort_indices()
        self._base = None
        self.name = name
        self._readonly = True

    initial_value = property(lambda self: self._csr)
    dtype = property(lambda self: self._csr.dtype)
    shape = property(lambda self: self._csr.shape)
    ndim = property(lambda self: 2)
    size = property(lambda self: self._csr.nnz)

    def may_share_memory(self, other):
        return other is self

    def __getitem__(self, item):
        raise ValueError("sparse signals have no views")

    reshape = __getitem__


# ============================================================= operators
class Operator:
    """Base class: lists of signals set / incremented / read / updated this step.

    Within one step, per memory block: all sets, then incs, then reads, then
    updates (an update's result is first seen in the next step).
    """

    def __init__(self, tag=None):
        self.tag = tag
        self.sets, self.incs, self.reads, self.updates = [], [], [], []

    @property
    def all_signals(self):
        return list(self.sets) + list(self.incs) + list(self.reads) + list(self.updates)

    def init_signals(self, signals):
        for sig in self.all_signals:
            if sig.base not in signals:
                signals[sig.base] = np.array(sig.base.initial_value)

    def __repr__(self):
        return "<%s%s at 0x%x>" % (type(self).__name__, " %s" % self.tag if self.tag else "", id(self))


class TimeUpdate(Operator):
    def __init__(self, step, time, tag=None):
        super().__init__(tag)
        self.step, self.time = step, time
        self.sets = [step, time]


class Reset(Operator):
    def __init__(self, dst, value=0, tag=None):
        super().__init__(tag)
        self.dst, self.value = dst, float(value)
        self.sets = [dst]


class Copy(Operator):
    """``dst[dst_slice] (=|+=) src[src_slice]``."""

    def __init__(self, src, dst, src_slice=None, dst_slice=None, inc=False, tag=None):
        super().__init__(tag)
        self.src, self.dst = src, dst
        self.src_slice, self.dst_slice, self.inc = src_slice, dst_slice, bool(inc)
        # a basic slice writes / reads only that view, so copies into disjoint
        # slices of one signal do not order each other
        written = dst[dst_slice] if isinstance(dst_slice, slice) else dst
        self.reads = [src[src_slice] if isinstance(src_slice, slice) else src]
        if inc:
            self.incs = [written]
        else:
            self.sets = [written]


class DotInc(Operator):
    """``Y += A @ X``."""

    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        if X.ndim >= 2 and any(d > 1 for d in X.shape[1:]):
            raise ValueError("X must be a column vector")
        self.A, self.X, self.Y = A, X, Y
        self.reads = [A, X]
        self.incs = [Y]


class SparseDotInc(Operator):
    """``Y += A @ X`` with a sparse matrix signal A (nengo's SparseDotInc)."""

    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        if not getattr(A, "sparse", False):
            raise ValueError("A must be a sparse signal")
        if A.shape != (Y.size, X.size):
            raise ValueError("shape mismatch: %s @ %s -> %s" % (A.shape, X.shape, Y.shape))
        self.A, self.X, self.Y = A, X, Y
        self.incs, self.reads = [Y], [A, X]


class ElementwiseInc(Operator):
    """``Y += A * X`` with broadcasting."""

    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        self.A, self.X, self.Y = A, X, Y
        self.reads = [A, X]
        self.incs = [Y]


class SimPyFunc(Operator):
    """``output = fn(t, x)`` evaluated by a host function (or a translated kernel)."""

    def __init__(self, output, fn, t, x, tag=None):
        super().__init__(tag)
        self.output, self.fn, self.t, self.x = output, fn, t, x
        self.reads = [s for s in (t, x) if s is not None]
        self.sets = [] if output is None else [output]


class SimNeurons(Operator):
    def __init__(self, neurons, J, output, state=None, tag=None):
        super().__init__(tag)
        self.neurons, self.J, self.output = neurons, J, output
        self.state = {} if state is None else dict(state)
        self.reads = [J]
        self.sets = [output]
        self.updates = list(self.state.values())


class SimProcess(Operator):
    def __init__(self, process, input, output, t, mode="set", state=None, tag=None):
        super().__init__(tag)
        self.process, self.input, self.output, self.t, self.mode = process, input, output, t, mode
        self.state = {} if state is None else dict(state)
        self.reads = [t] + ([input] if input is not None else [])
        if output is not None:
            if mode == "update":
                self.updates = [output]
            elif mode == "inc":
                self.incs = [output]
            elif mode == "set":
                self.sets = [output]
            else:
                raise ValueError("unknown mode %r" % mode)
        self.updates = self.updates + list(self.state.values())


class SimPES(Operator):
    """``delta = -(learning_rate * dt / n_pre) * outer(error, pre_filtered)``."""

    def __init__(self, pre_filtered, error, delta, learning_rate, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.error, self.delta = pre_filtered, error, delta
        self.learning_rate = float(learning_rate)
        self.reads = [pre_filtered, error]
        self.updates = [delta]


class SimBCM(Operator):
    """``delta = learning_rate * dt * post_filtered * (post_filtered - theta) (outer) pre_filtered``."""

    def __init__(self, pre_filtered, post_filtered, theta, delta, learning_rate, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.post_filtered, self.theta = pre_filtered, post_filtered, theta
        self.delta, self.learning_rate = delta, float(learning_rate)
        self.reads = [pre_filtered, post_filtered, theta]
        self.updates = [delta]


class SimOja(Operator):
    """``delta = learning_rate * dt * post * (pre - beta * weights * post)`` (Hebbian term
    minus the forgetting term that bounds the weights)."""

    def __init__(self, pre_filtered, post_filtered, weights, delta, learning_rate, beta, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.post_filtered, self.weights = pre_filtered, post_filtered, weights
        self.delta, self.learning_rate, self.beta = delta, float(learning_rate), float(beta)
        self.reads = [pre_filtered, post_filtered, weights]
        self.updates = [delta]


class SimVoja(Operator):
    """``delta = learning_rate * dt * learning_signal * post_filtered *
    (scale * pre_decoded - scaled_encoders)``: encoders of active neurons move towards
    the decoded input."""

    def __init__(self, pre_decoded, post_filtered, scaled_encoders, delta, scale, learning_signal,
                 learning_rate, tag=None):
        super().__init__(tag)
        self.pre_decoded, self.post_filtered = pre_decoded, post_filtered
        self.scaled_encoders, self.delta = scaled_encoders, delta
        self.scale = np.asarray(scale, dtype=np.float64)
        self.learning_signal, self.learning_rate = learning_signal, float(learning_rate)
        self.reads = [pre_decoded, post_filtered, scaled_encoders, learning_signal]
        self.updates = [delta]


class ConvSpec:
    """Geometry of a convolution transform (what the operator's ``conv`` attribute holds
    in nengo: ``nengo.Convolution``)."""

    def __init__(self, n_filters, input_shape, kernel_size=(3, 3), strides=(1, 1),
                 padding="valid", channels_last=True):
        self.n_filters = int(n_filters)
        self.kernel_size = tuple(int(k) for k in kernel_size)
        self.strides = tuple(int(s) for s in strides)
        self.padding = padding
        self.channels_last = bool(channels_last)
        self.dimensions = len(self.kernel_size)
        self.input_shape = ImageShape(input_shape, channels_last)
        spatial = self.input_shape.spatial_shape
        if padding.lower() == "same":
            out = [-(-n // s) for n, s in zip(spatial, self.strides)]
        else:
            out = [(n - k) // s + 1 for n, k, s in zip(spatial, self.kernel_size, self.strides)]
        shape = tuple(out) + (self.n_filters,) if channels_last else (self.n_filters,) + tuple(out)
        self.output_shape = ImageShape(shape, channels_last)

    @property
    def kernel_shape(self):
        return self.kernel_size + (self.input_shape.n_channels, self.n_filters)


class ImageShape:
    def __init__(self, shape, channels_last=True):
        self.shape = tuple(int(s) for s in shape)
        self.channels_last = bool(channels_last)

    @property
    def spatial_shape(self):
        return self.shape[:-1] if self.channels_last else self.shape[1:]

    @property
    def n_channels(self):
        return self.shape[-1] if self.channels_last else self.shape[0]

    @property
    def size(self):
        return int(np.prod(self.shape))


class ConvInc(Operator):
    """``Y = conv(X, W)`` for one image signal (the reference's kernel sets Y,
    simulator.py:1290-1332)."""

    def __init__(self, W, X, Y, conv, tag=None):
        super().__init__(tag)
        self.W, self.X, self.Y, self.conv = W, X, Y, conv
        self.reads = [W, X]
        self.incs = [Y]


# =========================================================== neuron types
class LIFRate:
    def __init__(self, tau_rc=0.02, tau_ref=0.002, amplitude=1.0):
        self.tau_rc, self.tau_ref, self.amplitude = float(tau_rc), float(tau_ref), float(amplitude)

    def rates_from_current(self, J):
        """Steady-state rate for input current J (float64)."""
        J = np.asarray(J, dtype=np.float64)
        out = np.zeros_like(J)
        m = J > 1
        out[m] = self.amplitude / (self.tau_ref + self.tau_rc * np.log1p(1.0 / (J[m] - 1)))
        return out

    def gain_bias(self, max_rates, intercepts):
        """Gain and bias so that the neuron is silent at x = intercept and fires at
        max_rate at x = 1 (inverse of the rate curve)."""
        max_rates = np.asarray(max_rates, dtype=np.float64)
        intercepts = np.asarray(intercepts, dtype=np.float64)
        inv_tau_ref = 1.0 / self.tau_ref if self.tau_ref > 0 else np.inf
        if np.any(max_rates > inv_tau_ref):
            raise ValueError("max_rates must be below 1/tau_ref")
        x = 1.0 / (1 - np.exp((self.tau_ref - 1.0 / max_rates) / self.tau_rc))
        gain = (1 - x) / (intercepts - 1.0)
        bias = 1 - gain * intercepts
        return gain, bias

    def __eq__(self, other):
        return type(self) is type(other) and self.__dict__ == other.__dict__

    def __hash__(self):
        return hash((type(self).__name__,) + tuple(sorted(self.__dict__.items())))


class LIF(LIFRate):
    def __init__(self, tau_rc=0.02, tau_ref=0.002, min_voltage=0, amplitude=1.0):
        super().__init__(tau_rc, tau_ref, amplitude)
        self.min_voltage = min_voltage


class AdaptiveLIFRate(LIFRate):
    """LIF rate with an adaptation state N: J_eff = J - N, N += (dt/tau_n)(inc_n r - N)."""

    def __init__(self, tau_n=1.0, inc_n=0.01, tau_rc=0.02, tau_ref=0.002, amplitude=1.0):
        super().__init__(tau_rc, tau_ref, amplitude)
        self.tau_n, self.inc_n = float(tau_n), float(inc_n)


class AdaptiveLIF(LIF):
    def __init__(self, tau_n=1.0, inc_n=0.01, tau_rc=0.02, tau_ref=0.002, min_voltage=0,
                 amplitude=1.0):
        super().__init__(tau_rc, tau_ref, min_voltage, amplitude)
        self.tau_n, self.inc_n = float(tau_n), float(inc_n)


class RectifiedLinear(LIFRate):
    """r = amplitude * max(J, 0); silent at the intercept, max_rate at x = 1."""

    def __init__(self, amplitude=1.0):
        self.amplitude = float(amplitude)

    def rates_from_current(self, J):
        return self.amplitude * np.maximum(np.asarray(J, dtype=np.float64), 0.0)

    def gain_bias(self, max_rates, intercepts):
        max_rates = np.asarray(max_rates, dtype=np.float64)
        intercepts = np.asarray(intercepts, dtype=np.float64)
        gain = max_rates / (1 - intercepts)
        bias = -intercepts * gain
        return gain, bias


class SpikingRectifiedLinear(RectifiedLinear):
    """Integrates max(J, 0) and emits floor(V) spikes per step."""


class Sigmoid(LIFRate):
    """r = 1 / (tau_ref (1 + exp(-J))); the intercept is the inflection point."""

    def __init__(self, tau_ref=0.0025):
        self.tau_ref = float(tau_ref)
        self.amplitude = 1.0

    def rates_from_current(self, J):
        with np.errstate(over="ignore"):  # exp(-J) = inf for very negative J: a rate of 0
            return 1.0 / (self.tau_ref * (1.0 + np.exp(-np.asarray(J, dtype=np.float64))))

    def gain_bias(self, max_rates, intercepts):
        max_rates = np.asarray(max_rates, dtype=np.float64)
        intercepts = np.asarray(intercepts, dtype=np.float64)
        lim = 1.0 / self.tau_ref
        if np.any(max_rates >= lim):
            raise ValueError("max_rates must be below 1/tau_ref")
        inverse = -np.log(lim / max_rates - 1.0)
        gain = inverse / (1.0 - intercepts)
        bias = inverse - gain
        return gain, bias


# ============================================================== processes
class Process:
    seed = None


class LinearFilter(Process):
    """Continuous (``analog``) or discrete transfer function ``num / den``."""

    def __init__(self, num, den, analog=True):
        self.num = np.atleast_1d(np.asarray(num, dtype=np.float64))
        self.den = np.atleast_1d(np.asarray(den, dtype=np.float64))
        self.analog = analog

    def discrete_tf(self, dt):
        """(num, den) of the discrete filter as the filter kernel takes them:
        zero-order hold, normalised so den[0] = 1, then the leading zero of num and
        the leading one of den dropped (nengo_ocl/simulator.py:1214-1227)."""
        from scipy.signal import cont2discrete

        num, den = self.num, self.den
        if self.analog:
            if len(den) == 1:  # pure gain
                num, den = num / den[0], np.array([1.0])
            else:
                numd, dend, _ = cont2discrete((num, den), dt, method="zoh")
                num, den = numd.ravel(), dend
        num = num / den[0]
        den = den / den[0]
        num = num[1:] if (len(num) > 1 and num[0] == 0) else num
        return num, den[1:]


class Lowpass(LinearFilter):
    def __init__(self, tau):
        super().__init__([1.0], [tau, 1.0])
        self.tau = tau

    def discrete_tf(self, dt):
        if self.tau <= 0.03 * dt:  # effectively no filtering
            return np.array([1.0]), np.array([])
        a = np.exp(-dt / self.tau)
        return np.array([1.0 - a]), np.array([-a])


class Alpha(LinearFilter):
    def __init__(self, tau):
        super().__init__([1.0], [tau * tau, 2 * tau, 1.0])
        self.tau = tau


class WhiteSignal(Process):
    """Band-limited white noise of a given period, played back from a table."""

    def __init__(self, period, high, rms=0.5, seed=None):
        self.period, self.high, self.rms, self.seed = period, high, rms, seed

    def table(self, dt, size_out, rng):
        n = int(np.round(self.period / dt))
        n_coef = n // 2 + 1
        freqs = np.fft.rfftfreq(n, d=dt)
        coefs = rng.normal(size=(n_coef, size_out)) + 1j * rng.normal(size=(n_coef, size_out))
        coefs[0] = 0
        coefs[freqs > self.high] = 0
        sig = np.fft.irfft(coefs, n=n, axis=0)
        power = np.sqrt(np.mean(sig ** 2, axis=0))
        power[power == 0] = 1
        return sig * (self.rms / power)


class Uniform:
    def __init__(self, low, high):
        self.low, self.high = float(low), float(high)


class Gaussian:
    def __init__(self, mean, std):
        self.mean, self.std = float(mean), float(std)


class WhiteNoise(Process):
    """Independent samples of ``dist`` every step, times ``1/sqrt(dt)`` if ``scale``."""

    def __init__(self, dist=None, scale=True, seed=None):
        self.dist = Gaussian(0.0, 1.0) if dist is None else dist
        self.scale, self.seed = bool(scale), seed


class PresentInput(Process):
    def __init__(self, inputs, presentation_time):
        self.inputs = np.asarray(inputs, dtype=np.float64)
        self.presentation_time = float(presentation_time)


# ================================================================== model
class Probe:
    def __init__(self, target, sample_every=None, label=None):
        self.target, self.sample_every, self.label = target, sample_every, label


class Model:
    """What a build produces: operators, probes, named signals, dt."""

    def __init__(self, dt=0.001, label=None):
        self.dt = float(dt)
        self.label = label
        self.operators = []
        self.probes = []
        self.sig = {}
        self.params = {}
        self.seeds = {}
        self.step = Signal(np.array(0.0), name="step")
        self.time = Signal(np.array(0.0), name="time")
        self.add_op(TimeUpdate(self.step, self.time))

    def add_op(self, op):
        self.operators.append(op)
        return op

    def __str__(self):
        return "Model: %s" % self.label
