"""Learning rules, noise processes and convolution transforms through the mini-builder
and the whole simulator, on the CPU oracle backend: the operator graph the builder emits
does what the rule / process / transform is for.  (Device parity of the same networks is
in test_simulator_parity.py.)"""

import numpy as np
import pytest

from nengo_ocl_amd import ir
from nengo_ocl_amd import minibuilder as mb
from oracle.oracle_sim import OracleSimulator


def hebbian_network(rule, seed=3):
    net = mb.Network(seed=seed)
    node = net.Node(mb.WhiteSignal(1.0, 5.0, seed=1), size_out=2)
    a, b = net.Ensemble(60, 2), net.Ensemble(40, 2)
    net.Connection(node, a, synapse=None)
    W = np.random.RandomState(0).normal(scale=1e-3, size=(40, 60))
    conn = net.Connection(a.neurons, b.neurons, transform=W, learning_rule=rule)
    return net, conn, [net.Probe(a.neurons), net.Probe(b.neurons)]


def voja_network(gate=None, seed=3):
    net = mb.Network(seed=seed)
    node = net.Node(np.array([0.6, -0.8]))
    a = net.Ensemble(50, 2)
    b = net.Ensemble(80, 2, intercepts=(0.3, 0.9))
    net.Connection(node, a, synapse=None)
    rule = mb.Voja(learning_rate=5e-2)
    conn = net.Connection(a, b, learning_rule=rule, synapse=0.005)
    if gate is not None:  # the rule's input scales the learning; -1 on top of the default 1 stops it
        net.Connection(net.Node(np.array([gate])), rule, synapse=None)
    return net, conn, b, [net.Probe(b.neurons)]


def noise_network(seed=3):
    net = mb.Network(seed=seed)
    n1 = net.Node(mb.WhiteNoise(mb.Gaussian(0, 0.5), scale=True, seed=5), size_out=3)
    n2 = net.Node(mb.WhiteNoise(mb.Uniform(-1, 1), scale=False), size_out=2)
    ens = net.Ensemble(50, 1, noise=mb.WhiteNoise(mb.Gaussian(0, 0.1), seed=2))
    quiet = net.Ensemble(50, 1, seed=ens.seed)
    return net, [net.Probe(n1), net.Probe(n2), net.Probe(ens.neurons), net.Probe(quiet.neurons)]


def conv_network(channels_last=True, seed=3):
    net = mb.Network(seed=seed)
    shape = (8, 9, 2) if channels_last else (2, 8, 9)
    img = np.random.RandomState(1).uniform(0, 1, size=shape)
    node = net.Node(img.ravel())
    conv = mb.Convolution(4, shape, kernel_size=(3, 3), strides=(1, 2), padding="same",
                          channels_last=channels_last, seed=3)
    ens = net.Ensemble(conv.size_out, 1, neuron_type=mb.RectifiedLinear())
    net.Connection(node, ens.neurons, transform=conv, synapse=None)
    return net, conv, img, [net.Probe(ens.neurons)]


@pytest.mark.parametrize("rule_type", ["BCM", "Oja"])
def test_hebbian_rules_change_weights(rule_type):
    rule = mb.BCM(learning_rate=1e-9) if rule_type == "BCM" else mb.Oja(learning_rate=1e-6)
    net, conn, probes = hebbian_network(rule)
    with OracleSimulator(net, seed=1, learn_in_place=False) as sim:  # (the delta is read below)
        kinds = [type(op).__name__ for op in sim.model.operators]
        assert "Sim" + rule_type in kinds
        wsig = sim.model.sig[conn]["weights"]
        w0 = np.array(sim.signals[wsig])
        sim.run_steps(300)
        w1 = np.array(sim.signals[wsig])
        delta = np.array(sim.signals[sim.model.sig[rule]["delta"]])
    assert np.abs(w1 - w0).max() > 1e-3 and np.all(np.isfinite(w1))
    if rule_type == "Oja":
        # the Hebbian term dominates while weights are small: weights between neurons that
        # were active together grew
        pre = sim.data[probes[0]].mean(axis=0)
        post = sim.data[probes[1]].mean(axis=0)
        grown = (w1 - w0)[np.ix_(post > 20, pre > 20)]
        assert grown.mean() > 0
    assert np.abs(delta).max() > 0


def test_voja_moves_encoders_towards_the_input_and_can_be_gated():
    x = np.array([0.6, -0.8])
    results = {}
    for gate in (None, -1.0):
        net, conn, post, probes = voja_network(gate)
        with OracleSimulator(net, seed=1) as sim:
            enc = sim.model.sig[post]["encoders"]
            gain = sim.model.params[post]["gain"]
            e0 = np.array(sim.signals[enc]) / gain[:, None]
            sim.run_steps(500)
            e1 = np.array(sim.signals[enc]) / gain[:, None]
            active = sim.data[probes[0]].sum(axis=0) > 0
        results[gate] = (e0, e1, active)
    e0, e1, active = results[None]
    assert active.sum() >= 5
    # encoders of active neurons gather at the decoded input (a little shorter than x)
    target = e1[active].mean(axis=0)
    assert target @ x > 0.9 and np.linalg.norm(target) < 1.05
    before = np.linalg.norm(e0[active] - target, axis=1)
    after = np.linalg.norm(e1[active] - target, axis=1)
    assert after.max() < 0.5 * before.max() and after.mean() < 0.25 * before.mean()
    assert np.array_equal(e0[~active], e1[~active])  # silent neurons keep their encoders
    e0, e1, _ = results[-1.0]
    assert np.array_equal(e0, e1)  # learning signal 1 + (-1) = 0: nothing learned


def test_noise_nodes_and_neuron_noise():
    net, probes = noise_network()
    with OracleSimulator(net, seed=1) as sim:
        sim.run_steps(2000)
        g, u, noisy, quiet = (np.array(sim.data[p]) for p in probes)
        assert abs(g.std() / (0.5 / np.sqrt(1e-3)) - 1) < 0.05 and abs(g.mean()) < 1.5
        assert u.min() >= -1 and u.max() < 1 and abs(u.mean()) < 0.05
        assert abs(np.corrcoef(g[:, 0], g[:, 1])[0, 1]) < 0.1
        assert not np.array_equal(noisy, quiet)  # same ensemble parameters, different spikes
        sim.reset()
        sim.run_steps(2000)
        assert np.array_equal(g, sim.data[probes[0]]) and np.array_equal(noisy, sim.data[probes[2]])


@pytest.mark.parametrize("channels_last", [True, False])
def test_convolution_connection(channels_last):
    from scipy.signal import correlate2d

    net, conv, img, probes = conv_network(channels_last)
    with OracleSimulator(net, seed=1) as sim:
        assert any(isinstance(op, ir.ConvInc) for op in sim.model.operators)
        sim.run_steps(2)
        ens_out = sim.data[probes[0]][-1]
        J = np.array(sim.signals[[op for op in sim.model.operators
                                  if isinstance(op, ir.ConvInc)][0].Y])
    hwc = img if channels_last else img.transpose(1, 2, 0)
    padded = np.pad(hwc, ((1, 1), (1, 1), (0, 0)))
    want = np.stack([sum(correlate2d(padded[:, :, c], conv.init[:, :, c, k], mode="valid")
                         for c in range(2))[::1, ::2] for k in range(4)], axis=-1)
    if not channels_last:
        want = want.transpose(2, 0, 1)
    np.testing.assert_allclose(J.ravel(), want.ravel(), rtol=1e-5, atol=1e-5)
    assert ens_out.shape == (conv.size_out,) and ens_out.max() > 0


def test_unsupported_combinations_raise():
    net = mb.Network(seed=0)
    a, b = net.Ensemble(10, 1), net.Ensemble(10, 1)
    net.Connection(a, b, learning_rule=mb.BCM())
    with pytest.raises(NotImplementedError):
        net.build_model()
    net = mb.Network(seed=0)
    a, b = net.Ensemble(10, 1), net.Ensemble(10, 1)
    net.Connection(a.neurons, b, transform=np.ones((1, 10)), learning_rule=mb.Oja())
    with pytest.raises(NotImplementedError):
        net.build_model()


@pytest.mark.parametrize("rule_type", ["PES", "BCM", "Oja", "Voja"])
def test_learning_in_place_gives_the_same_simulation(rule_type):
    """`learn_in_place=True`: the rule adds its change to the learned matrix itself (no
    delta matrix, no copy).  Probe data of every step are bit-identical to the two-pass
    form.  In device memory the matrix is a step ahead of the two-pass one (it already holds
    the last step's change); what the host reads through `sim.signals` is the two-pass value
    all the same (a copy taken before the last step), the delta matrix is gone and says so,
    and a write to the matrix is refused."""
    from nengo_ocl_amd import configs

    def make():
        if rule_type == "PES":
            net, probes, _ = configs.c4_pes(n_triples=2, n_neurons=60, dims=3, solver="lstsq",
                                            learning_rate=3e-4, sample_every=None)
            return net, list(probes.values())
        if rule_type == "Voja":
            net, conn, post, probes = voja_network()
            return net, probes
        rule = mb.BCM(learning_rate=1e-9) if rule_type == "BCM" else mb.Oja(learning_rate=1e-6)
        net, conn, probes = hebbian_network(rule)
        return net, probes

    def learned(sim):
        """(learned matrix, delta matrix or None) per learning operator of the model."""
        rules = [op for op in sim.model.operators
                 if type(op).__name__ in ("SimPES", "SimBCM", "SimOja", "SimVoja")]
        copies = {op.src: op.dst for op in sim.model.operators if type(op).__name__ == "Copy"}
        return [(copies[op.delta], op.delta) for op in rules]

    (net_a, probes_a), (net_b, probes_b) = make(), make()
    with OracleSimulator(net_a, seed=1, learn_in_place=False) as two_pass, \
            OracleSimulator(net_b, seed=1, learn_in_place=True) as in_place:
        kinds = lambda sim: [type(op).__name__ for op in sim.operators]
        assert kinds(in_place).count("Copy") < kinds(two_pass).count("Copy")
        assert any(getattr(op, "apply_inc", False) for op in in_place.operators)
        for n in (1, 50, 150):
            two_pass.run_steps(n)
            in_place.run_steps(n)
            for (w_a, d_a), (w_b, d_b) in zip(learned(two_pass), learned(in_place)):
                assert np.array_equal(np.array(in_place.signals[w_b]),
                                      np.array(two_pass.signals[w_a]))
                ahead = np.array(two_pass.signals[w_a]) + np.array(two_pass.signals[d_a])
                assert np.array_equal(np.array(in_place.all_data[in_place.sidx[w_b]]), ahead)
                with pytest.raises(ValueError, match="not computed"):
                    in_place.signals[d_b]
                with pytest.raises(ValueError, match="updated in place"):
                    in_place.signals[w_b] = np.zeros(w_b.shape)
        in_place.reset()
        two_pass.reset()
        for (w_a, _), (w_b, _) in zip(learned(two_pass), learned(in_place)):
            assert np.array_equal(np.array(in_place.signals[w_b]), np.array(two_pass.signals[w_a]))
        two_pass.run_steps(7)
        in_place.run_steps(7)
        for (w_a, _), (w_b, _) in zip(learned(two_pass), learned(in_place)):
            assert np.array_equal(np.array(in_place.signals[w_b]), np.array(two_pass.signals[w_a]))
        for a, b in zip(probes_a, probes_b):
            assert np.array_equal(two_pass.data[a], in_place.data[b])
        assert any(np.abs(np.array(two_pass.signals[d])).max() > 0 for _, d in learned(two_pass))


def test_learning_in_place_leaves_probed_matrices_alone():
    rule = mb.Oja(learning_rate=1e-6)
    net, conn, probes = hebbian_network(rule)
    model = net.build_model()
    wsig = model.sig[conn]["weights"]
    probe = ir.Probe(None)
    model.probes.append(probe)
    model.sig[probe] = {"in": wsig}
    with OracleSimulator(None, model=model, seed=1, learn_in_place=True) as sim:
        assert not any(getattr(op, "apply_inc", False) for op in sim.operators)
