"""Minimal stand-ins for the parts of nengo that the simulator's nengo path touches.
TEST INFRASTRUCTURE: nengo cannot be installed here, so the branches of the simulator that
only run for operators, signals, processes and models *of nengo's family* are driven with
modules named like nengo's that expose the attribute names the reference's simulator reads
(`/root/reference/nengo_ocl/simulator.py`, cited per class).  These stand-ins recall
nengo 3.1's interfaces; they do not prove equality with a real nengo build.

`install(monkeypatch)` registers the modules in `sys.modules` for one test and returns the
namespace of classes.
"""

import sys
import types

import numpy as np

from nengo_ocl_amd import ir


def _module(name, **members):
    mod = types.ModuleType(name)
    for key, value in members.items():
        setattr(mod, key, value)
        if isinstance(value, type):
            value.__module__ = name
    return mod


# ------------------------------------------------------------------ signals
class SparseMatrix:
    """nengo.transforms.SparseMatrix: `indices` (nnz x 2), `data`, `shape`, `ndim`, `size`,
    `tocsr()`.  A Signal whose initial value is one has `sparse == True`."""

    def __init__(self, indices, data, shape):
        self.indices = np.asarray(indices, dtype=np.int64).reshape(-1, 2)
        self.data = np.asarray(data, dtype=np.float64)
        self.shape = tuple(shape)
        self.ndim = 2
        self.dtype = self.data.dtype

    @property
    def size(self):
        return len(self.data)

    def tocsr(self):
        import scipy.sparse

        m = scipy.sparse.csr_matrix((self.data, self.indices.T), shape=self.shape)
        m.sort_indices()
        return m


class Signal(ir.Signal):
    """nengo.builder.signal.Signal: `base`, `is_view`, `initial_value`, `readonly`, `shape`,
    `ndim`, `size`, `elemoffset`, `elemstrides`, `may_share_memory`, `name`, `sparse`
    (read at simulator.py:72-143, 266-300 of the reference).  With a `SparseMatrix` as its
    initial value it is a sparse signal (reference simulator.py:281-286, 321-324)."""

    def __init__(self, initial_value=None, **kwargs):
        if isinstance(initial_value, SparseMatrix):
            self._sparse_value = initial_value
            self._base = None
            self.name = kwargs.get("name")
            self._readonly = True
        else:
            super().__init__(initial_value, **kwargs)

    sparse = property(lambda self: hasattr(self, "_sparse_value"))

    def _dense_or(name):  # noqa: N805 (a helper evaluated in the class body)
        inherited = getattr(ir.Signal, name)

        def get(self):
            if self.sparse:
                return getattr(self._sparse_value, name) if name != "initial_value" \
                    else self._sparse_value
            return inherited.fget(self)

        return property(get)

    initial_value = _dense_or("initial_value")
    shape = _dense_or("shape")
    ndim = _dense_or("ndim")
    size = _dense_or("size")
    dtype = _dense_or("dtype")
    del _dense_or

    def may_share_memory(self, other):
        if self.sparse or getattr(other, "sparse", False):
            return other is self
        return super().may_share_memory(other)


class SignalDict(dict):
    """nengo.builder.signal.SignalDict as the reference uses it (simulator.py:273-276):
    `op.init_signals(sigdict)` fills it, `sigdict[base]` gives the initial array."""

    def init(self, signal):
        if signal.base not in self:
            base = signal.base
            value = base.initial_value.tocsr() if base.sparse else np.array(base.initial_value)
            dict.__setitem__(self, base, value)


# ------------------------------------------------------------------ operators
class Operator:
    """nengo.builder.operator.Operator: `sets`, `incs`, `reads`, `updates`, `all_signals`,
    `init_signals`, `tag`."""

    def __init__(self, tag=None):
        self.tag = tag
        self.sets, self.incs, self.reads, self.updates = [], [], [], []

    @property
    def all_signals(self):
        return self.sets + self.incs + self.reads + self.updates

    def init_signals(self, signals):
        for sig in self.all_signals:
            signals.init(sig)


class TimeUpdate(Operator):  # simulator.py:736-744: op.step, op.time
    def __init__(self, step, time, tag=None):
        super().__init__(tag)
        self.step, self.time = step, time
        self.sets = [step, time]


class Reset(Operator):  # simulator.py:818-832: op.dst, op.value
    def __init__(self, dst, value=0, tag=None):
        super().__init__(tag)
        self.dst, self.value = dst, float(value)
        self.sets = [dst]


class Copy(Operator):  # simulator.py:834-869: src, dst, src_slice, dst_slice, inc
    def __init__(self, src, dst, src_slice=None, dst_slice=None, inc=False, tag=None):
        super().__init__(tag)
        self.src, self.dst, self.src_slice, self.dst_slice, self.inc = (
            src, dst, src_slice, dst_slice, bool(inc))
        self.reads = [src]
        (self.incs if inc else self.sets).append(dst)


class DotInc(Operator):  # operators.py:51-66 of the reference: op.A, op.X, op.Y
    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        self.A, self.X, self.Y = A, X, Y
        self.reads, self.incs = [A, X], [Y]


class SparseDotInc(Operator):  # simulator.py:877-892 of the reference: op.A (sparse), op.X, op.Y
    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        assert A.sparse
        self.A, self.X, self.Y = A, X, Y
        self.reads, self.incs = [A, X], [Y]


class SimPES(Operator):  # simulator.py:1334-1345: pre_filtered, error, delta, learning_rate
    def __init__(self, pre_filtered, error, delta, learning_rate, encoders=None, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.error, self.delta = pre_filtered, error, delta
        self.learning_rate, self.encoders = learning_rate, encoders
        self.reads = [pre_filtered, error] + ([] if encoders is None else [encoders])
        self.updates = [delta]


class SimBCM(Operator):  # simulator.py:1347-1353: pre_filtered, post_filtered, theta, delta, learning_rate
    def __init__(self, pre_filtered, post_filtered, theta, delta, learning_rate, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.post_filtered, self.theta = pre_filtered, post_filtered, theta
        self.delta, self.learning_rate = delta, learning_rate
        self.reads, self.updates = [pre_filtered, post_filtered, theta], [delta]


class SimOja(Operator):  # simulator.py:1355-1365: ... weights, delta, learning_rate, beta
    def __init__(self, pre_filtered, post_filtered, weights, delta, learning_rate, beta, tag=None):
        super().__init__(tag)
        self.pre_filtered, self.post_filtered, self.weights = pre_filtered, post_filtered, weights
        self.delta, self.learning_rate, self.beta = delta, learning_rate, beta
        self.reads, self.updates = [pre_filtered, post_filtered, weights], [delta]


class SimVoja(Operator):  # simulator.py:1367-1386: pre_decoded, post_filtered, scaled_encoders, ...
    def __init__(self, pre_decoded, post_filtered, scaled_encoders, delta, scale, learning_signal,
                 learning_rate, tag=None):
        super().__init__(tag)
        self.pre_decoded, self.post_filtered = pre_decoded, post_filtered
        self.scaled_encoders, self.delta, self.scale = scaled_encoders, delta, scale
        self.learning_signal, self.learning_rate = learning_signal, learning_rate
        self.reads = [pre_decoded, post_filtered, scaled_encoders, learning_signal]
        self.updates = [delta]


class ChannelShape:  # nengo.transforms.ChannelShape as simulator.py:1290-1332 reads it
    def __init__(self, shape, channels_last=True):
        self.shape, self.channels_last = tuple(shape), channels_last
        self.spatial_shape = self.shape[:-1] if channels_last else self.shape[1:]
        self.n_channels = self.shape[-1] if channels_last else self.shape[0]
        self.size = int(np.prod(self.shape))
        self.dimensions = len(self.spatial_shape)


class Convolution:  # nengo.transforms.Convolution: the `conv` of a ConvInc (simulator.py:1290-1332)
    def __init__(self, n_filters, input_shape, kernel_size=(3, 3), strides=(1, 1), padding="valid",
                 channels_last=True):
        self.n_filters, self.kernel_size, self.strides = n_filters, tuple(kernel_size), tuple(strides)
        self.padding, self.channels_last = padding, channels_last
        self.input_shape = ChannelShape(input_shape, channels_last)
        self.dimensions = len(self.kernel_size)
        spatial = self.input_shape.spatial_shape
        if padding == "same":
            out = [-(-n // s) for n, s in zip(spatial, self.strides)]
        else:
            out = [(n - k) // s + 1 for n, k, s in zip(spatial, self.kernel_size, self.strides)]
        shape = tuple(out) + (n_filters,) if channels_last else (n_filters,) + tuple(out)
        self.output_shape = ChannelShape(shape, channels_last)


class ConvInc(Operator):  # simulator.py:1290-1332: op.W, op.X, op.Y, op.conv
    def __init__(self, W, X, Y, conv, tag=None):
        super().__init__(tag)
        self.W, self.X, self.Y, self.conv = W, X, Y, conv
        self.reads, self.incs = [W, X], [Y]


class ElementwiseInc(Operator):  # simulator.py:871-875: op.A, op.X, op.Y
    def __init__(self, A, X, Y, tag=None):
        super().__init__(tag)
        self.A, self.X, self.Y = A, X, Y
        self.reads, self.incs = [A, X], [Y]


class SimPyFunc(Operator):  # simulator.py:877-911: op.fn, op.t, op.x, op.output
    def __init__(self, output, fn, t, x, tag=None):
        super().__init__(tag)
        self.output, self.fn, self.t, self.x = output, fn, t, x
        self.reads = [s for s in (t, x) if s is not None]
        self.sets = [] if output is None else [output]


class SimNeurons(Operator):  # simulator.py:1035-1063: op.neurons, op.J, op.output, op.state[..]
    def __init__(self, neurons, J, output, state=None, tag=None):
        super().__init__(tag)
        self.neurons, self.J, self.output = neurons, J, output
        self.state = {} if state is None else dict(state)
        self.reads, self.sets = [J], [output]
        self.updates = list(self.state.values())


class SimProcess(Operator):  # simulator.py:1160-1191: op.process, input, output, t, mode
    def __init__(self, process, input, output, t, mode="set", state=None, tag=None):
        super().__init__(tag)
        self.process, self.input, self.output, self.t, self.mode = process, input, output, t, mode
        self.state = {} if state is None else dict(state)
        self.reads = [t] + ([input] if input is not None else [])
        if output is not None:
            {"update": self.updates, "inc": self.incs, "set": self.sets}[mode].append(output)
        self.updates = self.updates + list(self.state.values())


# ------------------------------------------------------------------ neurons, processes
class LIF:  # simulator.py:1046-1063: tau_rc, tau_ref, amplitude, min_voltage
    def __init__(self, tau_rc=0.02, tau_ref=0.002, min_voltage=0, amplitude=1.0):
        self.tau_rc, self.tau_ref, self.min_voltage, self.amplitude = (
            tau_rc, tau_ref, min_voltage, amplitude)


class AdaptiveLIF(LIF):  # clra_nonlinearities.py:1094-1132 through simulator.py:1080-1100
    def __init__(self, tau_n=1.0, inc_n=0.01, **kwargs):
        super().__init__(**kwargs)
        self.tau_n, self.inc_n = tau_n, inc_n


class LIFRate:  # simulator.py:1065-1078: tau_rc, tau_ref, amplitude
    def __init__(self, tau_rc=0.02, tau_ref=0.002, amplitude=1.0):
        self.tau_rc, self.tau_ref, self.amplitude = tau_rc, tau_ref, amplitude


class AdaptiveLIFRate(LIFRate):  # simulator.py:1102-1121: + tau_n, inc_n
    def __init__(self, tau_n=1.0, inc_n=0.01, **kwargs):
        super().__init__(**kwargs)
        self.tau_n, self.inc_n = tau_n, inc_n


class RectifiedLinear:  # simulator.py:1123-1130: amplitude
    def __init__(self, amplitude=1.0):
        self.amplitude = amplitude


class SpikingRectifiedLinear(RectifiedLinear):  # simulator.py:1132-1142: amplitude, state voltage
    pass


class Sigmoid:  # simulator.py:1144-1151: tau_ref
    def __init__(self, tau_ref=0.0025):
        self.tau_ref = tau_ref


class Gaussian:  # clra_nonlinearities.py:1486-1510 (get_dist_enums_params): mean, std
    def __init__(self, mean, std):
        self.mean, self.std = mean, std


class Uniform:  # the same: low, high
    def __init__(self, low, high):
        self.low, self.high = low, high


class Process:
    seed = None

    def get_rng(self, rng):  # simulator.py:1266
        seed = rng.randint(2 ** 31 - 1) if self.seed is None else self.seed
        return np.random.RandomState(seed)


class _StateSpaceStep:
    """What `LinearFilter.make_step` returns in nengo 3: an object with the discrete
    state-space matrices (simulator.py:1209-1216 of the reference reads f.A, f.B, f.C, f.D)."""

    def __init__(self, A, B, C, D):
        self.A, self.B, self.C, self.D = A, B, C, D


class LinearFilter(Process):
    def __init__(self, num, den, analog=True):
        self.num, self.den, self.analog = np.atleast_1d(num).astype(float), np.atleast_1d(
            den).astype(float), analog

    def make_state(self, shape_in, shape_out, dt, dtype=None):
        return {"X": np.zeros((len(self.den) - 1,) + tuple(shape_out))}

    def make_step(self, shape_in, shape_out, dt, rng, state):
        from scipy.signal import cont2discrete, tf2ss

        A, B, C, D = tf2ss(self.num, self.den)
        if self.analog and A.size:
            A, B, C, D, _ = cont2discrete((A, B, C, D), dt, method="zoh")
        return _StateSpaceStep(A, B, C, D)


class Lowpass(LinearFilter):
    def __init__(self, tau):
        super().__init__([1.0], [tau, 1.0])
        self.tau = tau


class WhiteSignal(Process):
    """Keeps its table in a variable named `signal` inside the step closure, which is where
    the reference looks for it (simulator.py:1263-1277, utils.py:40-41)."""

    def __init__(self, period, high, rms=0.5, seed=None):
        self._inner = ir.WhiteSignal(period, high, rms=rms, seed=seed)
        self.seed = seed

    def make_state(self, shape_in, shape_out, dt, dtype=None):
        return {}

    def make_step(self, shape_in, shape_out, dt, rng, state):
        signal = self._inner.table(dt, int(np.prod(shape_out)), rng)
        n = len(signal)

        def step_whitesignal(t):
            return signal[int(round(t / dt)) % n]

        return step_whitesignal


# ------------------------------------------------------------------ builder
class BuildError(Exception):
    pass


class Builder:
    """nengo.builder.Builder: a registry of build functions by object class."""

    builders = {}

    @classmethod
    def register(cls, nengo_class):
        def deco(fn):
            cls.builders[nengo_class] = fn
            return fn
        return deco

    @classmethod
    def build(cls, model, obj, *args, **kwargs):
        for c in type(obj).__mro__:
            if c in cls.builders:
                return cls.builders[c](model, obj, *args, **kwargs)
        raise BuildError("cannot build object of type %r" % type(obj).__name__)


class Model:
    """nengo.builder.Model as the reference constructs and reads it (simulator.py:230-243,
    248, 705-731): dt, label, decoder_cache, builder; operators, probes, sig, params, step,
    time; `build(network)`; `add_op`."""

    def __init__(self, dt=0.001, label=None, decoder_cache=None, builder=None):
        self.dt, self.label, self.decoder_cache = dt, label, decoder_cache
        self.builder = Builder() if builder is None else builder
        self.operators, self.probes, self.sig, self.params, self.seeds = [], [], {}, {}, {}
        self.step = Signal(np.array(0.0), name="step")
        self.time = Signal(np.array(0.0), name="time")
        self.add_op(TimeUpdate(self.step, self.time))

    def add_op(self, op):
        self.operators.append(op)
        return op

    def build(self, obj, *args, **kwargs):
        return self.builder.build(self, obj, *args, **kwargs)


class WhiteNoise(Process):  # simulator.py:1245-1258: dist, scale, seed
    def __init__(self, dist=None, scale=True, seed=None):
        self.dist = Gaussian(0.0, 1.0) if dist is None else dist
        self.scale, self.seed = scale, seed


class PresentInput(Process):  # simulator.py:1279-1288: inputs, presentation_time
    def __init__(self, inputs, presentation_time):
        self.inputs, self.presentation_time = np.asarray(inputs), presentation_time


def ss2tf(A, B, C, D):
    """nengo.utils.filter_design.ss2tf is scipy's routine of the same name."""
    from scipy.signal import ss2tf as scipy_ss2tf

    return scipy_ss2tf(A, B, C, D)


def install(monkeypatch):
    """Registers the stand-in modules for the duration of one test."""
    Builder.builders = {}
    mods = {
        "nengo": _module("nengo"),
        "nengo.builder": _module("nengo.builder", Model=Model, Builder=Builder),
        "nengo.builder.builder": _module("nengo.builder.builder", Model=Model),
        "nengo.builder.operator": _module(
            "nengo.builder.operator", Operator=Operator, TimeUpdate=TimeUpdate, Reset=Reset,
            Copy=Copy, DotInc=DotInc, ElementwiseInc=ElementwiseInc, SimPyFunc=SimPyFunc,
            SparseDotInc=SparseDotInc),
        "nengo.builder.learning_rules": _module("nengo.builder.learning_rules", SimPES=SimPES,
                                                SimBCM=SimBCM, SimOja=SimOja, SimVoja=SimVoja),
        "nengo.dists": _module("nengo.dists", Gaussian=Gaussian, Uniform=Uniform),
        "nengo.transforms": _module("nengo.transforms", SparseMatrix=SparseMatrix,
                                    Convolution=Convolution, ChannelShape=ChannelShape),
        "nengo.builder.transforms": _module("nengo.builder.transforms", ConvInc=ConvInc),
        "nengo.builder.neurons": _module("nengo.builder.neurons", SimNeurons=SimNeurons),
        "nengo.builder.processes": _module("nengo.builder.processes", SimProcess=SimProcess),
        "nengo.builder.signal": _module("nengo.builder.signal", Signal=Signal,
                                        SignalDict=SignalDict),
        "nengo.cache": _module("nengo.cache", get_default_decoder_cache=lambda: None),
        "nengo.exceptions": _module("nengo.exceptions", BuildError=BuildError),
        "nengo.neurons": _module("nengo.neurons", LIF=LIF, AdaptiveLIF=AdaptiveLIF, LIFRate=LIFRate,
                                 AdaptiveLIFRate=AdaptiveLIFRate, RectifiedLinear=RectifiedLinear,
                                 SpikingRectifiedLinear=SpikingRectifiedLinear, Sigmoid=Sigmoid),
        "nengo.synapses": _module("nengo.synapses", LinearFilter=LinearFilter, Lowpass=Lowpass),
        "nengo.processes": _module("nengo.processes", Process=Process, WhiteSignal=WhiteSignal,
                                   WhiteNoise=WhiteNoise, PresentInput=PresentInput),
        "nengo.utils": _module("nengo.utils"),
        "nengo.utils.filter_design": _module("nengo.utils.filter_design", ss2tf=ss2tf),
    }
    for name, mod in mods.items():
        monkeypatch.setitem(sys.modules, name, mod)
        parent, _, child = name.rpartition(".")
        if parent:
            setattr(mods[parent], child, mod)
    monkeypatch.delitem(sys.modules, "nengo_ocl_amd.builder", raising=False)
    return types.SimpleNamespace(
        Signal=Signal, Reset=Reset, Copy=Copy, DotInc=DotInc, ElementwiseInc=ElementwiseInc,
        SimPyFunc=SimPyFunc, SimNeurons=SimNeurons, SimProcess=SimProcess, LIF=LIF,
        Lowpass=Lowpass, WhiteSignal=WhiteSignal, Model=Model, Builder=Builder,
        BuildError=BuildError, SparseDotInc=SparseDotInc, SimPES=SimPES, AdaptiveLIF=AdaptiveLIF,
        SimBCM=SimBCM, SimOja=SimOja, SimVoja=SimVoja, LIFRate=LIFRate,
        AdaptiveLIFRate=AdaptiveLIFRate, RectifiedLinear=RectifiedLinear,
        SpikingRectifiedLinear=SpikingRectifiedLinear, Sigmoid=Sigmoid, WhiteNoise=WhiteNoise,
        Gaussian=Gaussian, Uniform=Uniform, ConvInc=ConvInc, conv_spec=Convolution,
        PresentInput=PresentInput,
        sparse_signal=lambda matrix, name=None: Signal(_as_sparse_matrix(matrix), name=name),
        family="nengo")


def _as_sparse_matrix(matrix):
    coo = matrix.tocoo()
    return SparseMatrix(np.stack([coo.row, coo.col], axis=1), coo.data, coo.shape)
