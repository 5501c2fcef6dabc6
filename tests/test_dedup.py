"""The operator rewrite that computes identical products and synapses once
(`operators.merge_identical_chains`), on the CPU oracle backend: what it merges, what it
must leave alone, and that every signal of the unmerged simulation keeps its values."""

import numpy as np
import pytest

from nengo_ocl_amd import configs, ir, minibuilder as mb
from nengo_ocl_amd import operators as ops_mod
from oracle.oracle_sim import OracleSimulator


def _pair(net, **kw):
    """Merged and unmerged simulators of ONE built model (same signal objects)."""
    model = net.build_model(dt=0.001)
    a = OracleSimulator(None, model=model, seed=1, dedup=True, **kw)
    b = OracleSimulator(None, model=model, seed=1, dedup=False, **kw)
    return model, a, b


def _same_everywhere(a, b, probes, steps):
    model = a.model
    a.run_steps(steps)
    b.run_steps(steps)
    for p in probes.values():
        assert np.array_equal(a.data[p], b.data[p])
        assert np.any(a.data[p] != 0)
    bases = {sig.base for op in model.operators for sig in op.all_signals
             if not getattr(sig, "sparse", False)}
    # signals a rewrite folded into another operator (deltas of rules that update in place,
    # vectors that were only copies) say so when read; which ones depends on the rewrites
    for sim in (a, b):
        for base in sim._not_computed:
            with pytest.raises(ValueError, match="not computed"):
                sim.signals[base]
    bases -= a._not_computed | b._not_computed
    assert bases <= set(b.all_bases)
    for base in bases:  # every signal of the model, dropped ones through their alias
        got, want = np.asarray(a.signals[base]), np.asarray(b.signals[base])
        assert got.shape == want.shape, base
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), base


def test_c3_per_connection_becomes_one_decoder_per_ensemble():
    kw = dict(n_ens=8, n_neurons=256, dims=16, fan_out=4, solver="lstsq")
    net, probes, _ = configs.c3_large(share_decoded=False, **kw)
    model, a, b = _pair(net)
    shared, _, _ = configs.c3_large(share_decoded=True, **kw)
    with a, b, OracleSimulator(shared, seed=1) as c:
        shape = lambda sim: [(t.__name__, len(ops)) for t, ops in sim.op_groups]
        assert shape(a) == shape(c) and shape(a) != shape(b)
        assert a.all_data.buf.size == c.all_data.buf.size < b.all_data.buf.size
        # 8 x 4 connections: 3 of every 4 weighted sums, synapse outputs and decoder
        # matrices are gone
        dropped = [s for s in a.signal_aliases if s not in a.all_bases]
        assert len(dropped) == 3 * 8 * 3
        assert [p.name for p in a._plans] == [p.name for p in c._plans]
        _same_everywhere(a, b, probes, 150)


def test_c2_edges_from_one_ensemble_share_their_decoders():
    net, probes, _ = configs.c2_watts_strogatz(n_ens=64, n_driven=8)
    model, a, b = _pair(net)
    with a, b:
        n_dots = lambda sim: sum(len(op.As) for op in sim.operators
                                 if isinstance(op, ops_mod.MultiDotInc))
        assert n_dots(a) < n_dots(b)
        _same_everywhere(a, b, probes, 100)


def test_learned_weights_are_left_alone():
    net, probes, _ = configs.c4_pes(n_triples=2, n_neurons=100, dims=4, solver="lstsq")
    model, a, b = _pair(net)
    with a, b:
        learned = [op.delta for op in model.operators if type(op).__name__ == "SimPES"]
        assert learned
        copies = [op for op in model.operators if type(op).__name__ == "Copy" and op.src in learned]
        for cp in copies:
            assert cp.dst not in a.signal_aliases and cp.dst in a.all_bases
        _same_everywhere(a, b, probes, 100)


def _fan(transforms, synapses, probe_conn=None, functions=None):
    """One ensemble connected to len(transforms) targets."""
    net = mb.Network(seed=5)
    stim = net.Node(lambda t: np.sin(6 * t), size_out=1)
    pre = net.Ensemble(60, 1)
    net.Connection(stim, pre, synapse=None)
    posts, conns = [], []
    for k, (tr, syn) in enumerate(zip(transforms, synapses)):
        post = net.Ensemble(40, 1)
        fn = None if functions is None else functions[k]
        conns.append(net.Connection(pre, post, transform=tr, synapse=syn, function=fn))
        posts.append(post)
    probes = {"p%d" % k: net.Probe(post, synapse=0.01) for k, post in enumerate(posts)}
    return net, probes, conns


def _n(sim, kind):
    return sum(len(ops) for t, ops in sim.op_groups if t.__name__ == kind)


def _n_dots(sim):
    return sum(len(op.As) for op in sim.operators if isinstance(op, ops_mod.MultiDotInc))


def test_what_merges_and_what_does_not():
    lp = lambda tau: mb.Lowpass(tau)
    # equal transforms and synapses: one product, one synapse
    net, probes, _ = _fan([0.5, 0.5, 0.5], [lp(0.005)] * 3)
    model, a, b = _pair(net)
    with a, b:
        assert _n_dots(b) - _n_dots(a) == 2
        assert _n(b, "SimProcess") - _n(a, "SimProcess") == 2
        _same_everywhere(a, b, probes, 100)
    # equal products behind different synapses: one product, every synapse stays
    net, probes, _ = _fan([0.5, 0.5, 0.5], [lp(0.005), lp(0.01), lp(0.02)])
    model, a, b = _pair(net)
    with a, b:
        assert _n_dots(b) - _n_dots(a) == 2
        assert _n(b, "SimProcess") == _n(a, "SimProcess")
        _same_everywhere(a, b, probes, 100)
    # different transforms or functions: different matrices, nothing merges
    for net, probes, _ in (_fan([0.5, 0.25, 1.0], [lp(0.005)] * 3),
                           _fan([1.0] * 2, [lp(0.005)] * 2, functions=[None, np.square])):
        model, a, b = _pair(net)
        with a, b:
            assert not a.signal_aliases
            assert _n_dots(b) == _n_dots(a)


def test_probed_and_written_signals_stay():
    # a probed weighted sum is kept as its own signal (its duplicate still merges into it
    # or stays; the probe reads the values it read before)
    x = ir.Signal(np.arange(3.0) + 1, name="x")
    W1 = ir.Signal(np.eye(3) * 2, name="W1", readonly=True)
    W2 = ir.Signal(np.eye(3) * 2, name="W2", readonly=True)
    W3 = ir.Signal(np.eye(3) * 2, name="W3", readonly=False)  # the host may change it
    ys = [ir.Signal(np.zeros(3), name="y%d" % k) for k in range(3)]
    out = ir.Signal(np.zeros(3), name="out")
    m = ir.Model(dt=0.001)
    m.operators.append(ir.TimeUpdate(m.step, m.time))
    for W, y in zip((W1, W2, W3), ys):
        m.operators += [ir.Reset(y), ir.DotInc(W, x, y)]
    m.operators.append(ir.Reset(out))
    for y in ys:
        m.operators.append(ir.Copy(y, out, inc=True))
    aliases = {}
    merged = ops_mod.merge_identical_chains(m.operators, aliases=aliases)
    assert aliases[ys[1]] is ys[0] and aliases[W2] is W1
    assert ys[2] not in aliases and W3 not in aliases
    assert len(merged) == len(m.operators) - 2
    assert sum(op.src is ys[0] for op in merged if type(op).__name__ == "Copy") == 2
    # the operators handed in are untouched
    assert sum(op.src is ys[0] for op in m.operators if type(op).__name__ == "Copy") == 1
    kept = ops_mod.merge_identical_chains(m.operators, keep=[ys[1]])
    assert len(kept) == len(m.operators)
    with OracleSimulator(None, model=m) as a, OracleSimulator(None, model=m, dedup=False) as b:
        a.run_steps(3)
        b.run_steps(3)
        assert np.array_equal(a.signals[out], b.signals[out])
        assert np.array_equal(a.signals[out], 3 * 2 * (np.arange(3.0) + 1))
        assert np.array_equal(a.signals[ys[1]], b.signals[ys[1]])  # through its alias


def test_a_view_or_second_writer_blocks_the_merge():
    x = ir.Signal(np.ones(4), name="x")
    W1 = ir.Signal(np.ones((4, 4)), name="W1", readonly=True)
    W2 = ir.Signal(np.ones((4, 4)), name="W2", readonly=True)
    y1, y2 = ir.Signal(np.zeros(4), name="y1"), ir.Signal(np.zeros(4), name="y2")
    z = ir.Signal(np.zeros(2), name="z")
    base = [ir.Reset(y1), ir.DotInc(W1, x, y1), ir.Reset(y2), ir.DotInc(W2, x, y2)]
    assert len(ops_mod.merge_identical_chains(base)) == 2
    viewed = base + [ir.Copy(y2[:2], z)]
    assert len(ops_mod.merge_identical_chains(viewed)) == len(viewed)
    extra = base + [ir.DotInc(W1, x, y2)]  # y2 gets one increment more than y1
    assert len(ops_mod.merge_identical_chains(extra)) == len(extra)


def test_host_writes_to_shared_signals_are_refused():
    """A write through `sim.signals` to a signal that merged connections share -- the dropped
    duplicate or the survivor -- would change every one of them where the reference changes
    one (reference accessor: simulator.py:451-463): it raises and names the switch; without
    the merge the write lands in the one connection."""
    kw = dict(n_ens=4, n_neurons=128, dims=8, fan_out=3, solver="lstsq")
    net, probes, _ = configs.c3_large(share_decoded=False, **kw)
    model, a, b = _pair(net)
    with a, b:
        decoders = [(dup, rep) for dup, rep in a.signal_aliases.items()
                    if dup.ndim == 2 and getattr(dup, "readonly", False)]
        assert decoders
        dup, rep = decoders[0]
        for sig in (dup, rep):
            with pytest.raises(ValueError, match="dedup=False"):
                a.signals[sig] = np.zeros(sig.shape)
        assert np.array_equal(np.asarray(a.signals[dup]), np.asarray(b.signals[dup]))  # reads are fine
        state = [d for d in a.signal_aliases if d.ndim == 1][0]
        with pytest.raises(ValueError, match="dedup=False"):
            a.signals[state] = np.zeros(state.shape)
        before = np.array(b.signals[rep])
        b.signals[dup] = np.zeros(dup.shape)  # unmerged: one connection changes
        assert not np.any(np.asarray(b.signals[dup]))
        assert np.array_equal(np.asarray(b.signals[rep]), before)
        b.run_steps(5)


@pytest.mark.parametrize("case", ["c1", "c4"])
def test_reference_host_state_keeps_every_signal(case):
    """`Simulator(reference_host_state=True)`: no rewrite that changes what lies in signal
    memory between two steps -- every signal of the model reads as the one-operator-at-a-time
    interpreter holds it, straight from the buffer, and every non-constant can be written."""
    from oracle.numpy_interpreter import NaiveInterpreter

    if case == "c1":
        net, probes, _ = configs.c1_circconv(dims=8, n_per_dim=20)
    else:
        net, probes, _ = configs.c4_pes(n_triples=2, n_neurons=60, dims=3, solver="lstsq")
    model = net.build_model(dt=0.001)
    naive = NaiveInterpreter(model)
    with OracleSimulator(None, model=model, seed=1, reference_host_state=True) as sim:
        assert not sim._not_computed and not sim._host_view and not sim.signal_aliases
        assert not sim._updated_in_place and not sim.signals_a_step_ahead
        sim.run_steps(60)
        naive.run_steps(60)
        for key, p in probes.items():
            assert np.array_equal(sim.data[p], naive.data(p)), key
        bases = {sig.base for op in model.operators for sig in op.all_signals}
        for base in bases:
            got = np.asarray(sim.all_data[sim.sidx[base]], dtype=np.float32).reshape(-1)
            assert np.array_equal(got, naive.mem[base].reshape(-1)), base
            sim.signals[base] = np.asarray(sim.signals[base])  # no signal refuses a write
