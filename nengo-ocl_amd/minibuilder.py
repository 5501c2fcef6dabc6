"""A small network front end that emits the operator graph nengo's builder emits.

nengo (``nengo>=3.1.0``, the reference's dependency, reference setup.py:31) is
what normally turns a ``Network`` into operators; it may be absent, so the
benchmark configurations and the parity tests are built with this module
instead.  It covers ensembles of LIF / LIFRate neurons, nodes (constant,
function of time, process, passthrough), decoded connections with functions,
transforms, slices and linear synapses, PES learning, and probes -- and emits,
per object, the operator pattern of nengo 3.1's builder as it is recalled here
(nengo's source is not available to check against, so equality with a real
nengo build of "the same" network is not claimed):

* ensemble:  ``Reset(in)``, ``Copy(bias -> J)``, ``DotInc(scaled_encoders, in, J)``,
  ``SimNeurons(J -> out; voltage, refractory_time)``
* decoded connection:  ``Reset(weighted)``, ``DotInc(transform @ decoders, out,
  weighted)``, ``SimProcess(synapse, weighted -> filtered, mode="update")``,
  ``Copy(filtered -> post.in[slice], inc=True)``
* node connection:  no-op / ``ElementwiseInc`` / ``DotInc`` for transform None /
  scalar / matrix, then the same synapse and copy
* PES:  ``SimProcess(pre_synapse, pre.out -> pre_filtered)``, ``Reset(error)``,
  ``SimPES(pre_filtered, error -> delta)``, ``Copy(delta -> weights, inc=True)``

Every connection gets its own weight signal, product and synapse, as nengo's builder
emits them; merging identical ones is the simulator's job
(`operators.merge_identical_chains`).  ``share_decoded=True`` makes the generator itself
let connections that leave one ensemble with the same function, transform and synapse
share one decoder matrix, one decoded signal and one filter (what a passthrough node
after the ensemble gives in nengo): the graph the rewrite must arrive at, kept for tests.
"""

import numpy as np

from . import ir
from .ir import (LIF, AdaptiveLIF, AdaptiveLIFRate, Alpha, Gaussian, LIFRate,  # noqa: F401
                 LinearFilter, Lowpass, PresentInput, RectifiedLinear, Sigmoid,
                 SpikingRectifiedLinear, Uniform, WhiteNoise, WhiteSignal)


class _Sliceable:
    def __getitem__(self, item):
        return ObjView(self, item)


class ObjView:
    def __init__(self, obj, item):
        self.obj, self.slice = obj, item


class Node(_Sliceable):
    def __init__(self, output=None, size_in=0, size_out=None, label=None):
        self.output, self.size_in, self.label = output, size_in, label
        if output is None:
            self.size_out = size_in  # passthrough
        elif callable(output) or isinstance(output, ir.Process):
            if size_out is None:
                size_out = 1 if callable(output) else None
            if size_out is None:
                raise ValueError("size_out is needed for process nodes")
            self.size_out = int(size_out)
        else:
            self.output = np.atleast_1d(np.asarray(output, dtype=np.float64))
            self.size_out = self.output.size


class Neurons(_Sliceable):
    def __init__(self, ensemble):
        self.ensemble = ensemble
        self.size_out = self.size_in = ensemble.n_neurons


class Ensemble(_Sliceable):
    def __init__(self, n_neurons, dimensions, radius=1.0, neuron_type=None, max_rates=(200, 400),
                 intercepts=(-1, 1), encoders=None, label=None, seed=None, noise=None):
        self.n_neurons, self.dimensions, self.radius = int(n_neurons), int(dimensions), radius
        self.neuron_type = LIF() if neuron_type is None else neuron_type
        self.max_rates, self.intercepts, self.encoders = max_rates, intercepts, encoders
        self.label, self.seed, self.noise = label, seed, noise
        self.neurons = Neurons(self)
        self.size_in = self.size_out = self.dimensions


class PES:
    def __init__(self, learning_rate=1e-4, pre_synapse=Lowpass(0.005)):
        self.learning_rate, self.pre_synapse = learning_rate, pre_synapse
        self.connection = None


class BCM:
    """Bienenstock-Cooper-Munro rule on weights between neurons."""

    def __init__(self, learning_rate=1e-9, pre_synapse=Lowpass(0.005), post_synapse=None,
                 theta_synapse=Lowpass(1.0)):
        self.learning_rate, self.pre_synapse = learning_rate, pre_synapse
        self.post_synapse = pre_synapse if post_synapse is None else post_synapse
        self.theta_synapse = theta_synapse
        self.connection = None
        self.size_in = 0


class Oja:
    """Oja's rule (Hebbian with a forgetting term) on weights between neurons."""

    def __init__(self, learning_rate=1e-6, pre_synapse=Lowpass(0.005), post_synapse=None,
                 beta=1.0):
        self.learning_rate, self.pre_synapse, self.beta = learning_rate, pre_synapse, beta
        self.post_synapse = pre_synapse if post_synapse is None else post_synapse
        self.connection = None
        self.size_in = 0


class Voja:
    """Vector Oja rule: moves the post ensemble's encoders towards the decoded input;
    its one-dimensional input scales the learning (0 switches it off)."""

    def __init__(self, learning_rate=1e-2, post_synapse=Lowpass(0.005)):
        self.learning_rate, self.post_synapse = learning_rate, post_synapse
        self.connection = None
        self.size_in = 1


class Convolution:
    """A convolution transform (nengo.Convolution): ``init`` has shape
    ``kernel_size + (input channels, n_filters)``."""

    def __init__(self, n_filters, input_shape, kernel_size=(3, 3), strides=(1, 1),
                 padding="valid", channels_last=True, init=None, seed=None):
        self.spec = ir.ConvSpec(n_filters, input_shape, kernel_size, strides, padding,
                                channels_last)
        if init is None:
            rng = np.random.RandomState(seed)
            fan_in = np.prod(self.spec.kernel_size) * self.spec.input_shape.n_channels
            init = rng.uniform(-1, 1, size=self.spec.kernel_shape) * np.sqrt(3.0 / fan_in)
        self.init = np.asarray(init, dtype=np.float64).reshape(self.spec.kernel_shape)
        self.size_in = self.spec.input_shape.size
        self.size_out = self.spec.output_shape.size


class Connection:
    def __init__(self, pre, post, function=None, transform=None, synapse=Lowpass(0.005),
                 learning_rule=None, reg=0.1, label=None):
        self.pre, self.post, self.function, self.transform = pre, post, function, transform
        self.synapse = Lowpass(synapse) if isinstance(synapse, (int, float)) else synapse
        self.learning_rule, self.reg, self.label = learning_rule, reg, label
        if learning_rule is not None:
            learning_rule.connection = self


class Probe(ir.Probe):
    def __init__(self, target, synapse=None, sample_every=None, label=None):
        super().__init__(target, sample_every=sample_every, label=label)
        self.synapse = Lowpass(synapse) if isinstance(synapse, (int, float)) else synapse


class Sparse:
    """A sparse transform (nengo.transforms.Sparse): ``shape`` and a scipy sparse ``init``."""

    def __init__(self, shape, init):
        import scipy.sparse

        self.shape = tuple(shape)
        self.init = scipy.sparse.csr_matrix(init)
        if self.init.shape != self.shape:
            raise ValueError("init has shape %s, not %s" % (self.init.shape, self.shape))


def _uniform(rng, spec, n):
    if np.ndim(spec) == 1 and len(spec) == 2 and not isinstance(spec, np.ndarray):
        return rng.uniform(spec[0], spec[1], size=n)
    return np.broadcast_to(np.asarray(spec, dtype=np.float64), (n,)).copy()


def sphere_surface(rng, n, d):
    x = rng.normal(size=(n, d))
    return x / np.linalg.norm(x, axis=1, keepdims=True)


def ball(rng, n, d):
    return sphere_surface(rng, n, d) * rng.uniform(size=(n, 1)) ** (1.0 / d)


def lstsq_l2(A, Y, reg=0.1):
    """Regularised least squares ``argmin |A D - Y|^2 + m sigma^2 |D|^2`` with
    ``sigma = reg * max(A)``; solved in whichever of the two Gram forms is smaller."""
    m, n = A.shape
    sigma = reg * A.max()
    lam = m * sigma * sigma
    if m >= n:
        G = A.T @ A
        G[np.diag_indices(n)] += lam
        return np.linalg.solve(G, A.T @ Y)
    G = A @ A.T
    G[np.diag_indices(m)] += lam
    return A.T @ np.linalg.solve(G, Y)


class Network:
    """Collects objects; ``build_model(dt)`` produces an `ir.Model`.

    ``solver``: "lstsq" solves decoders on sampled evaluation points;
    "surrogate" draws seeded random decoders of a plausible scale (for timing
    runs at sizes where hundreds of large solves would dominate start-up).
    """

    def __init__(self, seed=0, label=None, share_decoded=False, solver="lstsq",
                 n_eval_points=None):
        self.seed, self.label = seed, label
        self.share_decoded, self.solver, self.n_eval_points = share_decoded, solver, n_eval_points
        self.nodes, self.ensembles, self.connections, self.probes = [], [], [], []

    # --- object creation (returns the object, like nengo's constructors inside `with`)
    def Node(self, *args, **kwargs):
        obj = Node(*args, **kwargs)
        self.nodes.append(obj)
        return obj

    def Ensemble(self, *args, **kwargs):
        obj = Ensemble(*args, **kwargs)
        self.ensembles.append(obj)
        return obj

    def Connection(self, *args, **kwargs):
        obj = Connection(*args, **kwargs)
        self.connections.append(obj)
        return obj

    def Probe(self, *args, **kwargs):
        obj = Probe(*args, **kwargs)
        self.probes.append(obj)
        return obj

    @property
    def n_neurons(self):
        return sum(e.n_neurons for e in self.ensembles)

    def __str__(self):
        return "<minibuilder.Network %s>" % (self.label,)

    # ================================================================ build
    def build_model(self, dt=0.001):
        model = ir.Model(dt=dt, label="%s, dt=%f" % (self, dt))
        rng = np.random.RandomState(self.seed)
        self._decoded_cache = {}
        self._decoder_values = {}
        self._voja_targets = {(c.post.obj if isinstance(c.post, ObjView) else c.post)
                              for c in self.connections if isinstance(c.learning_rule, Voja)}
        for ens in self.ensembles:
            self._build_ensemble(model, ens, rng)
        for node in self.nodes:
            self._build_node(model, node, rng)
        # learning-rule error signals exist before connections target them
        for conn in self.connections:
            if conn.learning_rule is not None:
                rule = conn.learning_rule
                post_obj = conn.post.obj if isinstance(conn.post, ObjView) else conn.post
                if isinstance(rule, PES):
                    model.sig[rule] = {"in": ir.Signal(np.zeros(post_obj.size_in),
                                                       name="PES:error")}
                    model.add_op(ir.Reset(model.sig[rule]["in"]))
                elif isinstance(rule, Voja):  # learning signal: 1 unless something drives it
                    model.sig[rule] = {"in": ir.Signal(np.zeros(1), name="Voja:learning")}
                    model.add_op(ir.Reset(model.sig[rule]["in"], value=1.0))
                else:
                    model.sig[rule] = {"in": None}
        for conn in self.connections:
            self._build_connection(model, conn, rng)
        for probe in self.probes:
            self._build_probe(model, probe, rng)
        del self._decoded_cache, self._decoder_values
        return model

    def _build_ensemble(self, model, ens, rng):
        seed = ens.seed if ens.seed is not None else rng.randint(2 ** 31 - 1)
        erng = np.random.RandomState(seed)
        n, d = ens.n_neurons, ens.dimensions
        if ens.encoders is None:
            encoders = sphere_surface(erng, n, d)
        else:
            encoders = np.array(ens.encoders, dtype=np.float64).reshape(n, d)
            encoders /= np.linalg.norm(encoders, axis=1, keepdims=True)
        max_rates = _uniform(erng, ens.max_rates, n)
        intercepts = _uniform(erng, ens.intercepts, n)
        gain, bias = ens.neuron_type.gain_bias(max_rates, intercepts)
        scaled_encoders = encoders * (gain / ens.radius)[:, None]

        name = ens.label or "ens%d" % len(model.sig)
        sig = {
            "in": ir.Signal(np.zeros(d), name="%s.signal" % name),
            "encoders": ir.Signal(scaled_encoders, name="%s.scaled_encoders" % name,
                                  readonly=ens not in self._voja_targets),
        }
        nsig = {
            "in": ir.Signal(np.zeros(n), name="%s.neuron_in" % name),
            "out": ir.Signal(np.zeros(n), name="%s.neuron_out" % name),
            "bias": ir.Signal(bias, name="%s.bias" % name, readonly=True),
        }
        model.sig[ens], model.sig[ens.neurons] = sig, nsig
        model.params[ens] = dict(encoders=encoders, gain=gain, bias=bias, max_rates=max_rates,
                                 intercepts=intercepts, scaled_encoders=scaled_encoders, seed=seed)
        model.add_op(ir.Reset(sig["in"]))
        model.add_op(ir.Copy(nsig["bias"], nsig["in"]))
        model.add_op(ir.DotInc(sig["encoders"], sig["in"], nsig["in"], tag="%s encoding" % name))
        state_names = {"LIF": ("voltage", "refractory_time"),
                       "AdaptiveLIF": ("voltage", "refractory_time", "adaptation"),
                       "AdaptiveLIFRate": ("adaptation",),
                       "SpikingRectifiedLinear": ("voltage",)}
        state = {key: ir.Signal(np.zeros(n), name="%s.%s" % (name, key))
                 for key in state_names.get(type(ens.neuron_type).__name__, ())}
        if ens.noise is not None:  # injected into the input current
            model.add_op(ir.SimProcess(ens.noise, None, nsig["in"], model.time, mode="inc"))
        model.add_op(ir.SimNeurons(ens.neuron_type, nsig["in"], nsig["out"], state=state))

    def _build_node(self, model, node, rng):
        name = node.label or "node%d" % len(model.sig)
        if node.output is None:  # passthrough: in == out
            sig_in = ir.Signal(np.zeros(node.size_in), name="<Node %s>.in" % name)
            model.sig[node] = {"in": sig_in, "out": sig_in}
            model.add_op(ir.Reset(sig_in))
            return
        if node.size_in:  # out = f(t, in)
            if not callable(node.output) or isinstance(node.output, ir.Process):
                raise NotImplementedError("nodes with input need a function as output")
            sig_in = ir.Signal(np.zeros(node.size_in), name="<Node %s>.in" % name)
            out = ir.Signal(np.zeros(node.size_out), name="<Node %s>.out" % name)
            model.sig[node] = {"in": sig_in, "out": out}
            model.add_op(ir.Reset(sig_in))
            model.add_op(ir.SimPyFunc(out, node.output, model.time, sig_in))
            return
        if isinstance(node.output, np.ndarray):
            out = ir.Signal(node.output, name="<Node %s>.out" % name)
            model.sig[node] = {"in": None, "out": out}
            return
        out = ir.Signal(np.zeros(node.size_out), name="<Node %s>.out" % name)
        model.sig[node] = {"in": None, "out": out}
        if isinstance(node.output, ir.Process):
            if node.output.seed is None and hasattr(node.output, "table"):
                node.output.seed = int(rng.randint(2 ** 31 - 1))
            model.add_op(ir.SimProcess(node.output, None, out, model.time, mode="set"))
        else:
            model.add_op(ir.SimPyFunc(out, node.output, model.time, None))

    # --- decoders
    def _eval_activities(self, model, ens, rng):
        p = model.params[ens]
        n, d = ens.n_neurons, ens.dimensions
        m = self.n_eval_points
        if m is None:
            m = int(max(np.clip(500 * d, 750, 2500), 2 * n))
        pts = ball(rng, m, d) * ens.radius
        J = p["gain"] * (pts @ p["encoders"].T / ens.radius) + p["bias"]
        return pts, ens.neuron_type.rates_from_current(J)

    def _decoders(self, model, conn, ens, function, size_mid, rng):
        """Decoders (size_mid x n) for ``function`` of the ensemble's value.

        Solved values are cached per (ensemble, function): connections that do not
        share a decoded signal still get equal decoder *values* (nengo would sample
        new evaluation points per connection)."""
        n = ens.n_neurons
        key = (ens, function)
        if key in self._decoder_values:
            return self._decoder_values[key]
        if self.solver == "surrogate":
            # seeded random decoders of the magnitude real ones have (~ 1 / (n * rate));
            # a function that is identically zero keeps zero decoders
            probe = np.atleast_1d(function(rng.normal(size=ens.dimensions))) if function else None
            if probe is not None and not np.any(probe):
                dec = np.zeros((size_mid, n))
            else:
                dec = rng.normal(scale=2.0 / (100.0 * n), size=(size_mid, n))
        else:
            pts, acts = self._eval_activities(model, ens, rng)
            targets = pts if function is None else np.array(
                [np.atleast_1d(function(x)) for x in pts])
            dec = lstsq_l2(acts, targets, reg=conn.reg if conn is not None else 0.1).T
        self._decoder_values[key] = dec
        return dec

    # --- connections
    @staticmethod
    def _split(target):
        if isinstance(target, ObjView):
            return target.obj, target.slice
        return target, None

    def _apply_synapse(self, model, signal, synapse, name):
        if synapse is None:
            return signal
        filtered = ir.Signal(np.zeros(signal.shape), name="%s.filtered" % name)
        model.add_op(ir.SimProcess(synapse, signal, filtered, model.time, mode="update"))
        return filtered

    def _build_connection(self, model, conn, rng, into_signal=None):
        pre, pre_slice = self._split(conn.pre)
        post, post_slice = self._split(conn.post)
        crng = np.random.RandomState(rng.randint(2 ** 31 - 1))
        name = conn.label or "conn%d" % len(model.sig)
        sparse = conn.transform if isinstance(conn.transform, Sparse) else None
        convolution = conn.transform if isinstance(conn.transform, Convolution) else None
        transform = (None if conn.transform is None or sparse is not None or convolution is not None
                     else np.asarray(conn.transform, dtype=np.float64))
        rule = conn.learning_rule
        if convolution is not None and not isinstance(pre, (Neurons, Node)):
            raise NotImplementedError("convolution transforms on decoded connections")

        if isinstance(pre, Ensemble):
            if pre_slice is not None:
                sel = np.arange(pre.dimensions)[pre_slice]
                base_fn = conn.function
                function = (lambda x, f=base_fn, s=sel: (x if f is None else np.atleast_1d(f(x)))[s])
            else:
                function = conn.function
            learned = isinstance(rule, PES)
            if rule is not None and not isinstance(rule, (PES, Voja)):
                raise NotImplementedError("%s on a decoded connection" % type(rule).__name__)
            key = (pre, conn.function, None if transform is None else transform.tobytes(),
                   repr(pre_slice), self._synapse_key(conn.synapse))
            cached = self._decoded_cache.get(key) if (self.share_decoded and not learned) else None
            if cached is not None:
                signal = cached
            else:
                probe_x = np.zeros(pre.dimensions)
                size_mid = pre.dimensions if function is None else np.atleast_1d(function(probe_x)).size
                decoders = self._decoders(model, conn, pre, function, size_mid, crng)
                if transform is None:
                    weights = decoders
                elif transform.ndim == 0:
                    weights = transform * decoders
                elif transform.ndim == 1:
                    weights = transform[:, None] * decoders
                else:
                    weights = transform @ decoders
                wsig = ir.Signal(weights, name="%s.weights" % name, readonly=not learned)
                model.sig[conn] = {"weights": wsig}
                model.params[conn] = dict(weights=weights)
                weighted = ir.Signal(np.zeros(weights.shape[0]), name="%s.weighted" % name)
                model.add_op(ir.Reset(weighted))
                model.add_op(ir.DotInc(wsig, model.sig[pre.neurons]["out"], weighted,
                                       tag="%s.weights_dotinc" % name))
                signal = self._apply_synapse(model, weighted, conn.synapse, name)
                if self.share_decoded and not learned:
                    self._decoded_cache[key] = signal
                if learned:
                    self._build_pes(model, conn, pre, wsig, name)
            if isinstance(rule, Voja):
                self._build_voja(model, conn, post, signal, name)
        elif isinstance(pre, Neurons):
            signal = model.sig[pre]["out"]
            if pre_slice is not None:
                signal = signal[pre_slice]
            if rule is not None and not (isinstance(rule, (BCM, Oja)) and transform is not None
                                         and transform.ndim == 2 and isinstance(post, Neurons)
                                         and pre_slice is None and post_slice is None):
                raise NotImplementedError("%s needs full weights between two neuron "
                                          "populations" % type(rule).__name__)
            if convolution is not None:
                signal = self._build_convolution(model, convolution, signal, name)
            elif sparse is not None or (transform is not None and transform.ndim == 2):
                # weights between neurons: weighted = W @ activities, then the synapse
                n_out = sparse.shape[0] if sparse is not None else transform.shape[0]
                weighted = ir.Signal(np.zeros(n_out), name="%s.weighted" % name)
                model.add_op(ir.Reset(weighted))
                if sparse is not None:
                    wsig = ir.SparseSignal(sparse.init, name="%s.weights" % name)
                    model.add_op(ir.SparseDotInc(wsig, signal, weighted, tag="%s.weights" % name))
                else:
                    wsig = ir.Signal(transform, name="%s.weights" % name, readonly=rule is None)
                    model.add_op(ir.DotInc(wsig, signal, weighted, tag="%s.weights" % name))
                model.sig[conn] = {"weights": wsig}
                if rule is not None:
                    self._build_hebbian(model, conn, pre, post, wsig, name)
                signal = weighted
            elif transform is not None:
                raise NotImplementedError("scalar / diagonal transforms between neurons")
            signal = self._apply_synapse(model, signal, conn.synapse, name)
        elif isinstance(pre, Node):
            signal = model.sig[pre]["out"]
            if pre_slice is not None:
                signal = signal[pre_slice]
            if conn.function is not None:
                raise NotImplementedError("functions on node connections")
            if rule is not None:
                raise NotImplementedError("learning rules on connections from nodes")
            if convolution is not None:
                signal = self._build_convolution(model, convolution, signal, name)
            elif transform is not None:
                if transform.ndim == 0:
                    tsig = ir.Signal(transform, name="%s.transform" % name, readonly=True)
                    weighted = ir.Signal(np.zeros(signal.shape), name="%s.weighted" % name)
                    model.add_op(ir.Reset(weighted))
                    model.add_op(ir.ElementwiseInc(tsig, signal, weighted))
                else:
                    t2 = np.diag(transform) if transform.ndim == 1 else transform
                    tsig = ir.Signal(t2, name="%s.transform" % name, readonly=True)
                    weighted = ir.Signal(np.zeros(t2.shape[0]), name="%s.weighted" % name)
                    model.add_op(ir.Reset(weighted))
                    model.add_op(ir.DotInc(tsig, signal, weighted, tag="%s.transform" % name))
                signal = weighted
            signal = self._apply_synapse(model, signal, conn.synapse, name)
        else:
            raise TypeError("cannot connect from %r" % (pre,))

        # --- deliver
        if into_signal is not None:
            target = into_signal
        elif isinstance(post, Ensemble):
            target = model.sig[post]["in"]
        elif isinstance(post, Neurons):
            target = model.sig[post]["in"]
        elif isinstance(post, Node):
            if not post.size_in:
                raise ValueError("%s: the target node takes no input" % name)
            target = model.sig[post]["in"]
        elif isinstance(post, (PES, Voja)):
            target = model.sig[post]["in"]
        else:
            raise TypeError("cannot connect to %r" % (post,))
        n_target = target.size if post_slice is None else np.arange(target.size)[post_slice].size
        if signal.size != n_target:
            raise ValueError("%s: %d values into %d slots" % (name, signal.size, n_target))
        model.add_op(ir.Copy(signal, target, dst_slice=post_slice, inc=True, tag="%s" % name))

    @staticmethod
    def _synapse_key(synapse):
        if synapse is None:
            return None
        return (type(synapse).__name__, tuple(synapse.num), tuple(synapse.den), synapse.analog)

    def _build_pes(self, model, conn, pre, wsig, name):
        rule = conn.learning_rule
        acts = model.sig[pre.neurons]["out"]
        pre_filtered = self._apply_synapse(model, acts, rule.pre_synapse, "%s.pes_pre" % name)
        delta = ir.Signal(np.zeros(wsig.shape), name="%s.Delta" % name)
        model.add_op(ir.SimPES(pre_filtered, model.sig[rule]["in"], delta, rule.learning_rate))
        model.add_op(ir.Copy(delta, wsig, inc=True, tag="%s += delta" % name))
        model.sig[rule]["delta"] = delta

    def _build_hebbian(self, model, conn, pre, post, wsig, name):
        """BCM / Oja on weights between two neuron populations: filtered activities on
        both sides, the delta written by the rule, then added to the weights."""
        rule = conn.learning_rule
        pre_acts, post_acts = model.sig[pre]["out"], model.sig[post]["out"]
        pre_filtered = self._apply_synapse(model, pre_acts, rule.pre_synapse, "%s.rule_pre" % name)
        post_filtered = self._apply_synapse(model, post_acts, rule.post_synapse,
                                            "%s.rule_post" % name)
        delta = ir.Signal(np.zeros(wsig.shape), name="%s.Delta" % name)
        if isinstance(rule, BCM):
            theta = self._apply_synapse(model, post_acts, rule.theta_synapse, "%s.theta" % name)
            model.add_op(ir.SimBCM(pre_filtered, post_filtered, theta, delta, rule.learning_rate))
        else:
            model.add_op(ir.SimOja(pre_filtered, post_filtered, wsig, delta, rule.learning_rate,
                                   rule.beta))
        model.add_op(ir.Copy(delta, wsig, inc=True, tag="%s += delta" % name))
        model.sig[rule]["delta"] = delta

    def _build_voja(self, model, conn, post, pre_decoded, name):
        rule = conn.learning_rule
        if not isinstance(post, Ensemble):
            raise NotImplementedError("Voja needs an ensemble as the connection's target")
        if pre_decoded.size != post.dimensions:
            raise ValueError("Voja: the connection must deliver the ensemble's full input")
        post_filtered = self._apply_synapse(model, model.sig[post.neurons]["out"],
                                            rule.post_synapse, "%s.voja_post" % name)
        encoders = model.sig[post]["encoders"]
        delta = ir.Signal(np.zeros(encoders.shape), name="%s.Delta" % name)
        scale = model.params[post]["gain"] / post.radius
        model.add_op(ir.SimVoja(pre_decoded, post_filtered, encoders, delta, scale,
                                model.sig[rule]["in"], rule.learning_rate))
        model.add_op(ir.Copy(delta, encoders, inc=True, tag="%s encoders += delta" % name))
        model.sig[rule]["delta"] = delta

    def _build_convolution(self, model, convolution, signal, name):
        if signal.size != convolution.size_in:
            raise ValueError("%s: %d values into a convolution over %s" % (
                name, signal.size, convolution.spec.input_shape.shape))
        wsig = ir.Signal(convolution.init, name="%s.kernel" % name, readonly=True)
        weighted = ir.Signal(np.zeros(convolution.size_out), name="%s.weighted" % name)
        model.add_op(ir.Reset(weighted))
        model.add_op(ir.ConvInc(wsig, signal, weighted, convolution.spec, tag="%s.conv" % name))
        return weighted

    # --- probes
    def _build_probe(self, model, probe, rng):
        target, tslice = self._split(probe.target)
        if isinstance(target, Ensemble):
            sig_in = ir.Signal(np.zeros(target.dimensions if tslice is None else
                                        np.arange(target.dimensions)[tslice].size),
                               name="probe(%s)" % (target.label,))
            model.sig[probe] = {"in": sig_in}
            model.add_op(ir.Reset(sig_in))
            conn = Connection(probe.target, None, synapse=probe.synapse, label="probe_conn")
            self._build_connection(model, conn, rng, into_signal=sig_in)
        elif isinstance(target, (Node, Neurons)):
            src = model.sig[target]["out"]
            if tslice is not None:
                src = src[tslice]
            if probe.synapse is None:
                model.sig[probe] = {"in": src}
            else:
                filtered = self._apply_synapse(model, src, probe.synapse, "probe")
                model.sig[probe] = {"in": filtered}
        else:
            raise TypeError("cannot probe %r" % (target,))
        model.probes.append(probe)
