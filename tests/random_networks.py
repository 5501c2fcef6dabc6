"""Seeded random networks for the parity tests: ensembles of mixed sizes and dimensions
(small and large items, dimensions that are and are not multiples of four), several
connections into one ensemble, repeated connections out of one (duplicates to merge),
sliced targets, functions, a passthrough node, table and function inputs, probes of decoded
values, of spikes and of a connection-less ensemble.  TEST INFRASTRUCTURE.

``sliced=False`` leaves out connections into slices of an ensemble's input: an increment
into a view and the increments into the whole signal are separate operators whose order the
planner chooses (as in the reference, whose `compress` keys on the view), so a run is only
reproducible bit for bit by something that orders them the same way."""

import numpy as np

from nengo_ocl_amd import minibuilder as mb


def random_network(seed, big=False, sliced=True):
    rng = np.random.RandomState(seed)
    net = mb.Network(seed=seed, solver="lstsq", n_eval_points=300)
    dims_pool = [1, 2, 3, 4, 8, 16, 64] if not big else [4, 16, 32, 64, 64]
    n_ens = int(rng.randint(4, 9))
    ens = []
    for k in range(n_ens):
        d = int(rng.choice(dims_pool))
        n = int(rng.choice([30, 64, 100, 257] if not big else [512, 1024, 2048, 4096]))
        ens.append(net.Ensemble(n, d, label="e%d" % k))
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
            if pre.dimensions == post.dimensions and kind < 2:
                tr = 0.5 if kind == 0 else None
                net.Connection(pre, post, transform=tr, synapse=mb.Lowpass(0.005))
            elif kind == 2 and post.dimensions >= 2 and sliced:
                net.Connection(pre, post[0:2], function=lambda x: [x[0] * x[0], -x[0]],
                               synapse=mb.Lowpass(0.02))
            else:
                net.Connection(pre, post, transform=fits(pre.dimensions, post),
                               synapse=mb.Lowpass(0.005))
    lonely = net.Ensemble(50, 2, label="lonely")  # no input at all
    for k in rng.choice(n_ens, size=3, replace=False):
        probes["e%d" % k] = net.Probe(ens[int(k)], synapse=0.01)
    probes["spikes"] = net.Probe(ens[0].neurons)
    probes["lonely"] = net.Probe(lonely.neurons, sample_every=0.004)
    probes["relay"] = net.Probe(relay)
    return net, probes
