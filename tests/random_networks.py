"""Seeded random networks for the parity tests: ensembles of mixed sizes and dimensions
(small and large items, dimensions that are and are not multiples of four), several
connections into one ensemble, repeated connections out of one (duplicates to merge),
sliced targets, functions, a passthrough node, table and function inputs, probes of decoded
values, of spikes and of a connection-less ensemble.  TEST INFRASTRUCTURE.

``sliced=False`` leaves out connections into slices of an ensemble's input: an increment
into a view and the increments into the whole signal are separate operators whose order the
planner chooses (as in the reference, whose `compress` keys on the view), so a run is only
reproducible bit for bit by something that orders them the same way.

``rich=True`` draws the neuron type of every ensemble and the synapse of every connection at
random (spiking, rate, adaptive, rectified, sigmoid; first-order, second-order, none) and adds
learning (PES with an error ensemble, BCM / Oja between neurons, Voja on encoders), a sparse
and a dense transform between neurons, noise injected into an ensemble and a noise node."""

import numpy as np

from nengo_ocl_amd import minibuilder as mb


def _neuron_type(rng):
    kind = rng.randint(7)
    return [mb.LIF(), mb.LIF(tau_rc=0.03, tau_ref=0.001), mb.LIFRate(), mb.AdaptiveLIF(),
            mb.RectifiedLinear(), mb.SpikingRectifiedLinear(), mb.Sigmoid()][kind]


def _synapse(rng):
    kind = rng.randint(5)
    return [mb.Lowpass(0.005), mb.Lowpass(0.02), mb.Alpha(0.01), None, mb.Lowpass(0.003)][kind]


def random_network(seed, big=False, sliced=True, rich=False):
    rng = np.random.RandomState(seed)
    net = mb.Network(seed=seed, solver="lstsq", n_eval_points=300)
    dims_pool = [1, 2, 3, 4, 8, 16, 64] if not big else [4, 16, 32, 64, 64]
    n_ens = int(rng.randint(4, 9))
    ens = []
    for k in range(n_ens):
        d = int(rng.choice(dims_pool))
        n = int(rng.choice([30, 64, 100, 257] if not big else [512, 1024, 2048, 4096]))
        kwargs = {"neuron_type": _neuron_type(rng)} if rich else {}
        ens.append(net.Ensemble(n, d, label="e%d" % k, **kwargs))
    stim = net.Node(mb.WhiteSignal(period=0.3, high=8.0, seed=int(rng.randint(2 ** 31 - 1))),
                    size_out=3, label="stim")
    # a function whose float32 result is the same on host and device (one rounding either
    # way); transcendental functions differ in the last bits between the two
    wave = net.Node(lambda t: 1.0 - 4.0 * t, size_out=1, label="wave")
    relay = net.Node(None, size_in=2, label="relay")  # a passthrough
    probes = {}

    def fits(src_d, dst):
        """A transform taking src_d values into ensemble `dst`'s input."""
        return rng.normal(scale=0.6, size=(dst.dimensions, src_d))

    net.Connection(stim, ens[0], transform=fits(3, ens[0]), synapse=mb.Lowpass(0.005))
    if sliced:
        net.Connection(wave, ens[1][0:1], synapse=None)
    else:
        net.Connection(wave, ens[1], transform=np.ones((ens[1].dimensions, 1)), synapse=None)
    net.Connection(ens[0], relay, transform=fits(ens[0].dimensions, type("D", (), {"dimensions": 2})),
                   synapse=mb.Lowpass(0.01))
    net.Connection(relay, ens[2], transform=fits(2, ens[2]), synapse=None)
    for k in range(n_ens):
        # every ensemble sends to one to three others; some links repeat with the same
        # function / transform / synapse (identical products), some differ
        for j in rng.choice(n_ens, size=int(rng.randint(1, 4)), replace=False):
            if j == k:
                continue
            pre, post = ens[k], ens[int(j)]
            kind = rng.randint(4)
            syn = _synapse(rng) if rich else mb.Lowpass(0.005)
            if syn is None and not rich:
                syn = mb.Lowpass(0.005)
            if pre.dimensions == post.dimensions and kind < 2:
                tr = 0.5 if kind == 0 else None
                net.Connection(pre, post, transform=tr, synapse=syn if rich else mb.Lowpass(0.005))
            elif kind == 2 and post.dimensions >= 2 and sliced:
                net.Connection(pre, post[0:2], function=lambda x: [x[0] * x[0], -x[0]],
                               synapse=mb.Lowpass(0.02))
            else:
                net.Connection(pre, post, transform=fits(pre.dimensions, post),
                               synapse=syn if rich and syn is not None else mb.Lowpass(0.005))
    if rich:
        _learning_and_neuron_links(net, rng, ens, stim, probes, big)
    lonely = net.Ensemble(50, 2, label="lonely")  # no input at all
    for k in rng.choice(n_ens, size=3, replace=False):
        probes["e%d" % k] = net.Probe(ens[int(k)], synapse=0.01)
    probes["spikes"] = net.Probe(ens[0].neurons)
    probes["lonely"] = net.Probe(lonely.neurons, sample_every=0.004)
    probes["relay"] = net.Probe(relay)
    return net, probes


def _learning_and_neuron_links(net, rng, ens, stim, probes, big):
    import scipy.sparse

    n = 1024 if big else 60
    d = 16 if big else 2
    # PES: pre -> post learned, error = post - pre
    pre, post, err = (net.Ensemble(n, d, label="pes_%s" % k) for k in ("pre", "post", "err"))
    net.Connection(stim, pre, transform=rng.normal(scale=0.6, size=(d, 3)), synapse=mb.Lowpass(0.005))
    rule = mb.PES(learning_rate=float(rng.choice([1e-4, 3e-4])))
    net.Connection(pre, post, function=lambda x: np.zeros_like(x), learning_rule=rule,
                   synapse=mb.Lowpass(0.005))
    net.Connection(post, err, synapse=mb.Lowpass(0.005))
    net.Connection(pre, err, transform=-1.0, synapse=mb.Lowpass(0.005))
    net.Connection(err, rule, synapse=mb.Lowpass(0.005))
    probes["pes_post"] = net.Probe(post, synapse=0.01, sample_every=0.003)
    # Hebbian rules between neurons, a fixed dense and a sparse matrix between neurons
    a, b, c = (net.Ensemble(m, 2, label="heb_%s" % k) for k, m in (("a", 60), ("b", 40), ("c", 50)))
    net.Connection(stim[0:2], a, synapse=None)
    hebb = mb.BCM(learning_rate=1e-9) if rng.randint(2) else mb.Oja(learning_rate=1e-6)
    net.Connection(a.neurons, b.neurons, transform=rng.normal(scale=1e-3, size=(40, 60)),
                   learning_rule=hebb)
    net.Connection(b.neurons, c.neurons, transform=rng.normal(scale=2e-3, size=(50, 40)),
                   synapse=mb.Lowpass(0.01))
    weights = scipy.sparse.random(60, 50, density=0.1, random_state=rng, format="csr") * 1e-2
    net.Connection(c.neurons, a.neurons, transform=mb.Sparse((60, 50), weights),
                   synapse=mb.Lowpass(0.005))
    probes["heb_b"] = net.Probe(b.neurons)
    # Voja on the encoders of an ensemble with late intercepts
    va = net.Ensemble(50, 2, label="voja_pre")
    vb = net.Ensemble(80, 2, intercepts=(0.3, 0.9), label="voja_post")
    net.Connection(stim[1:3], va, synapse=None)
    net.Connection(va, vb, learning_rule=mb.Voja(learning_rate=5e-2), synapse=0.005)
    probes["voja"] = net.Probe(vb, synapse=0.01)
    # noise: into the neurons of an ensemble, and a node of its own (uniform: the Gaussian
    # transform uses the device's logarithm and cosine, equal to the host's to a bit only)
    noisy = net.Ensemble(50, 1, noise=mb.WhiteNoise(mb.Uniform(-0.2, 0.2), seed=int(rng.randint(1000))),
                         label="noisy")
    hiss = net.Node(mb.WhiteNoise(mb.Uniform(-1, 1), scale=False, seed=int(rng.randint(1000))),
                    size_out=1, label="hiss")
    net.Connection(hiss, noisy, synapse=mb.Lowpass(0.005))
    probes["noisy"] = net.Probe(noisy.neurons, sample_every=0.002)


def ensemble_array_network(probe_node=False):
    """Three ensembles whose filtered outputs a node collects, that node and the stimulus
    interleaved by two transforms into a second node, which drives an ensemble."""
    rng = np.random.RandomState(2)
    net = mb.Network(seed=5)
    stim = net.Node(mb.WhiteSignal(period=0.4, high=7.0, seed=2), size_out=3)
    parts = [net.Ensemble(60, 1, label="part%d" % k) for k in range(3)]
    out = net.Node(None, size_in=3, label="collect")
    mix = net.Node(None, size_in=6, label="interleave")
    for k, ens in enumerate(parts):
        net.Connection(stim[k:k + 1], ens, synapse=None)
        net.Connection(ens, out[k:k + 1], synapse=mb.Lowpass(0.005))
    net.Connection(out, mix[0::2], transform=rng.normal(size=(3, 3)), synapse=None)
    net.Connection(stim, mix[1::2], transform=rng.normal(size=(3, 3)), synapse=None)
    post = net.Ensemble(120, 6, label="post")
    net.Connection(mix, post, synapse=None)
    probes = {"post": net.Probe(post, synapse=0.01)}
    if probe_node:
        probes["collect"] = net.Probe(out)
    return net, probes
