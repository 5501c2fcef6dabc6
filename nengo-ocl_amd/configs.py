"""The five benchmark / parity configurations as seeded synthetic networks.

Each function returns ``(network, probes, info)`` built with `minibuilder`; sizes are
parameters so that parity tests can run reduced versions of the large ones.
Every array is drawn from seeded numpy generators, so the same call gives the
same operator graph for the CPU oracle and the GPU.

=====  ==========================================================================
name   network
=====  ==========================================================================
c0     the README example of the reference (README.rst:36-46): ``Node(np.sin)``
       -> a -> b with ``x**2``, two 100-neuron 1-D LIF ensembles, probes 0.01 s
c1     circular convolution of two unit vectors, D = 64: ``4*(D/2+1)`` 2-D product
       ensembles of 100 LIF neurons between dense DFT transforms
c2     Watts-Strogatz small world of 2048 1-D ensembles (k = 10, p = 0.1), every
       edge a decoded identity connection, 64 ensembles driven by 5 Hz noise
c3     256 ensembles x 4096 LIF x 64-D, four identity connections each: the
       bandwidth-bound case (1,048,576 neurons)
c4     PES learning: 64 (pre, post, error) triples of 2000-neuron 32-D ensembles
=====  ==========================================================================
"""

import numpy as np

from .minibuilder import LIF, PES, Lowpass, Network, Sparse, WhiteSignal


def c0_readme(seed=0, n_neurons=100, neuron_type=None):
    net = Network(seed=seed, label="c0-readme")
    stim = net.Node(np.sin, label="stim")
    kw = dict(neuron_type=neuron_type or LIF(tau_rc=0.02, tau_ref=0.002), max_rates=(200, 400),
              intercepts=(-1, 1))
    rng = np.random.RandomState(seed + 1000)
    enc = lambda: rng.choice([-1.0, 1.0], size=(n_neurons, 1))
    a = net.Ensemble(n_neurons, 1, encoders=enc(), label="a", **kw)
    b = net.Ensemble(n_neurons, 1, encoders=enc(), label="b", **kw)
    net.Connection(stim, a, synapse=Lowpass(0.005))
    net.Connection(a, b, function=lambda x: x ** 2, synapse=Lowpass(0.005))
    probes = dict(a=net.Probe(a, synapse=0.01), b=net.Probe(b, synapse=0.01))
    return net, probes, {}


def dft_half(n):
    x = np.arange(n)
    w = np.arange(n // 2 + 1)
    return np.exp((-2.0j * np.pi / n) * (w[:, None] * x[None, :]))


def circconv_transforms(dims):
    """Real matrices mapping a and b into the inputs of ``4*(dims/2+1)`` pairwise
    products, and the products back to ``circconv(a, b)`` (the construction used
    by nengo's CircularConvolution network: real and imaginary parts of the
    half spectrum, four products per frequency)."""
    dims2 = 4 * (dims // 2 + 1)
    tr = dft_half(dims)
    tr_a = np.zeros((dims2, dims))
    tr_b = np.zeros((dims2, dims))
    tr_a[0::4], tr_a[1::4], tr_a[2::4], tr_a[3::4] = tr.real, tr.real, tr.imag, tr.imag
    tr_b[0::4], tr_b[1::4], tr_b[2::4], tr_b[3::4] = tr.real, tr.imag, tr.real, tr.imag
    # inverse: real part from rr - ii, imaginary part from ri + ir
    half = np.zeros((dims // 2 + 1, 4, dims))
    idft = np.fft.irfft(np.eye(dims // 2 + 1), n=dims, axis=0)            # (dims, half) for real coefs
    idft_i = np.fft.irfft(1j * np.eye(dims // 2 + 1), n=dims, axis=0)     # for imaginary coefs
    half[:, 0, :] = idft.T
    half[:, 3, :] = -idft.T
    half[:, 1, :] = idft_i.T
    half[:, 2, :] = idft_i.T
    tr_out = half.reshape(dims2, dims).T
    return tr_a, tr_b, tr_out


def c1_circconv(seed=0, dims=64, n_per_dim=50, neuron_type=None):
    rng = np.random.RandomState(seed)
    a = rng.normal(size=dims)
    b = rng.normal(size=dims)
    a /= np.linalg.norm(a)
    b /= np.linalg.norm(b)
    tr_a, tr_b, tr_out = circconv_transforms(dims)
    n_prod = tr_a.shape[0]
    net = Network(seed=seed, label="c1-circconv-%d" % dims, share_decoded=False)
    in_a = net.Node(a, label="A")
    in_b = net.Node(b, label="B")
    prod_in = net.Node(size_in=2 * n_prod, label="product.input")
    prod_out = net.Node(size_in=n_prod, label="product.output")
    out = net.Node(size_in=dims, label="output")
    net.Connection(in_a, prod_in[0::2], transform=tr_a, synapse=None)
    net.Connection(in_b, prod_in[1::2], transform=tr_b, synapse=None)
    diag = np.array([[1, 1], [-1, 1], [1, -1], [-1, -1]], dtype=np.float64)
    radius = 2.0  # spectrum coefficients of unit vectors stay within about +-2
    for k in range(n_prod):
        erng = np.random.RandomState(seed * 7919 + k)
        ens = net.Ensemble(2 * n_per_dim, 2, radius=radius, label="product%d" % k,
                           encoders=diag[erng.randint(4, size=2 * n_per_dim)],
                           neuron_type=neuron_type or LIF())
        net.Connection(prod_in[2 * k:2 * k + 2], ens, synapse=None)
        net.Connection(ens, prod_out[k:k + 1], function=lambda x: x[0] * x[1],
                       synapse=Lowpass(0.005))
    net.Connection(prod_out, out, transform=tr_out, synapse=None)
    probes = dict(out=net.Probe(out, synapse=0.01))
    info = dict(a=a, b=b, expected=np.fft.irfft(np.fft.rfft(a) * np.fft.rfft(b), n=dims))
    return net, probes, info


def watts_strogatz_edges(n, k, p, rng):
    """Directed edge list of a ring lattice (k nearest neighbours, both directions)
    with each edge's target rewired with probability p (no self loops, no duplicates)."""
    targets = [set() for _ in range(n)]
    for i in range(n):
        for off in range(1, k // 2 + 1):
            targets[i].add((i + off) % n)
            targets[i].add((i - off) % n)
    edges = []
    for i in range(n):
        for j in sorted(targets[i]):
            if rng.uniform() < p:
                new = int(rng.randint(n))
                while new == i or new in targets[i]:
                    new = int(rng.randint(n))
                targets[i].discard(j)
                targets[i].add(new)
                j = new
            edges.append((i, j))
    return edges


def c2_watts_strogatz(seed=0, n_ens=2048, n_neurons=100, k=10, p=0.1, n_driven=64,
                      share_decoded=False):
    rng = np.random.RandomState(seed)
    net = Network(seed=seed, label="c2-watts-strogatz-%d" % n_ens, share_decoded=share_decoded,
                  n_eval_points=750)
    ens = [net.Ensemble(n_neurons, 1, label="e%d" % i,
                        encoders=rng.choice([-1.0, 1.0], size=(n_neurons, 1))) for i in range(n_ens)]
    edges = watts_strogatz_edges(n_ens, k, p, rng)
    in_degree = np.bincount([j for _, j in edges], minlength=n_ens)
    for i, j in edges:
        # scaled so that the summed input of a node stays within its radius
        net.Connection(ens[i], ens[j], transform=1.0 / max(in_degree[j], 1),
                       synapse=Lowpass(0.005))
    driven = rng.choice(n_ens, size=min(n_driven, n_ens), replace=False)
    for d in driven:
        node = net.Node(WhiteSignal(period=1.0, high=5.0, seed=int(rng.randint(2 ** 31 - 1))),
                        size_out=1, label="noise%d" % d)
        net.Connection(node, ens[int(d)], synapse=Lowpass(0.005))
    probed = [int(driven[0]), int((driven[0] + 1) % n_ens)]
    probes = {"e%d" % i: net.Probe(ens[i], synapse=0.01) for i in probed}
    return net, probes, dict(edges=edges, driven=driven)


def c3_large(seed=0, n_ens=256, n_neurons=4096, dims=64, fan_out=4, share_decoded=False,
             solver="surrogate", n_probes=2):
    """One decoder matrix, product and synapse per connection, as nengo builds separate
    connections (~1.3 GB of matrices at full size); the four connections that leave an
    ensemble carry equal decoders, which the simulator merges into one 64 x 4096 decoder
    per ensemble (~512 MB of matrices per step) unless told not to (``dedup=False``).
    ``share_decoded=True`` makes the generator emit the merged graph itself."""
    rng = np.random.RandomState(seed)
    net = Network(seed=seed, label="c3-large-%dx%d" % (n_ens, n_neurons),
                  share_decoded=share_decoded, solver=solver, n_eval_points=1024)
    ens = [net.Ensemble(n_neurons, dims, label="e%d" % i) for i in range(n_ens)]
    for i in range(n_ens):
        others = [j for j in range(n_ens) if j != i]
        for j in rng.choice(others, size=min(fan_out, len(others)), replace=False):
            net.Connection(ens[i], ens[int(j)], transform=1.0 / fan_out, synapse=Lowpass(0.005))
    drive = net.Node(WhiteSignal(period=1.0, high=5.0, seed=int(rng.randint(2 ** 31 - 1))),
                     size_out=dims, label="drive")
    net.Connection(drive, ens[0], synapse=Lowpass(0.005))
    probes = {"e%d" % i: net.Probe(ens[i], synapse=0.01) for i in range(min(n_probes, n_ens))}
    return net, probes, {}


def c4_pes(seed=0, n_triples=64, n_neurons=2000, dims=32, learning_rate=1e-4,
           solver="surrogate", sample_every=0.01):
    rng = np.random.RandomState(seed)
    net = Network(seed=seed, label="c4-pes-%dx%d" % (n_triples, n_neurons), solver=solver,
                  n_eval_points=1024)
    stim = net.Node(WhiteSignal(period=1.0, high=5.0, seed=int(rng.randint(2 ** 31 - 1))),
                    size_out=dims, label="stim")
    probes = {}
    for k in range(n_triples):
        pre = net.Ensemble(n_neurons, dims, label="pre%d" % k)
        post = net.Ensemble(n_neurons, dims, label="post%d" % k)
        err = net.Ensemble(n_neurons, dims, label="err%d" % k)
        net.Connection(stim, pre, synapse=Lowpass(0.005))
        rule = PES(learning_rate=learning_rate)
        net.Connection(pre, post, function=lambda x: np.zeros_like(x), learning_rule=rule,
                       synapse=Lowpass(0.005))
        net.Connection(post, err, synapse=Lowpass(0.005))
        net.Connection(pre, err, transform=-1.0, synapse=Lowpass(0.005))
        net.Connection(err, rule, synapse=Lowpass(0.005))
        if k < 2:
            probes["post%d" % k] = net.Probe(post, synapse=0.01, sample_every=sample_every)
    return net, probes, {}


def sparse_ring_weights(n, fan_outs, rewire_frac, rng, scale=1.0):
    """Sparse n x n weights of the shape the reference's sparse benchmark builds
    (examples/benchmark_wattsstrogatz.py:154-172): a directed ring in which every row
    holds `fan_outs` consecutive neighbours (wrapping around), a fraction of the column
    indices redrawn at random (duplicates inside a row may occur and stay separate
    entries); values normal(0, scale) instead of the reference's ones."""
    import scipy.sparse

    offsets = list(range(1, fan_outs + 1))
    offsets += [off - n for off in offsets]
    mat = scipy.sparse.diags(np.ones((len(offsets), n), dtype=np.float32), offsets=offsets,
                             shape=(n, n), format="csr")
    n_edges = mat.data.size
    rewire = np.nonzero(rng.random_sample(n_edges) < rewire_frac)[0]
    mat.indices[rewire] = rng.randint(n, size=rewire.size)
    mat.data[:] = rng.normal(scale=scale, size=n_edges)
    return mat


def c5_sparse_recurrent(seed=9, n_neurons=100000, fan_outs=100, rewire_frac=0.2,
                        weight_scale=2e-4, probe_neurons=64):
    """One population whose neurons are connected to each other through a sparse
    weight matrix (the reference's own sparse benchmark, examples/
    benchmark_wattsstrogatz.py:66-84): LIF with tau_ref 1 ms, recurrent synapse 0.1 s.
    The reference probes every neuron; here a slice of `probe_neurons` is probed."""
    rng = np.random.RandomState(seed)
    net = Network(seed=seed, label="c5-sparse-%d" % n_neurons)
    ens = net.Ensemble(n_neurons, 1, neuron_type=LIF(tau_ref=0.001), label="pop")
    weights = sparse_ring_weights(n_neurons, fan_outs, rewire_frac, rng, scale=weight_scale)
    net.Connection(ens.neurons, ens.neurons, transform=Sparse((n_neurons, n_neurons), weights),
                   synapse=Lowpass(0.1))
    probes = {"spikes": net.Probe(ens.neurons[:probe_neurons], synapse=0.03)}
    return net, probes, {"nnz": int(weights.nnz)}


CONFIGS = {
    "c0": c0_readme,
    "c1": c1_circconv,
    "c2": c2_watts_strogatz,
    "c3": c3_large,
    "c4": c4_pes,
    "c5": c5_sparse_recurrent,
}
