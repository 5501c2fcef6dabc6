"""Host logic above the plan_* boundary, run on the CPU oracle backend: operator
rewrites, dependency graph, planners, the Simulator's run / probe / reset logic.

Literal answers come from the reference's tests (tests/test_simulator.py:14-38,
tests/test_planners.py:13-47, tests/test_operators.py:30,54,82).
"""

import numpy as np
import pytest

from nengo_ocl_amd import configs, ir, minibuilder
from nengo_ocl_amd import operators as ops_mod
from nengo_ocl_amd.operators import MultiDotInc
from nengo_ocl_amd.planners import batching_planner, greedy_planner, operator_dependency_graph
from oracle.oracle_sim import OracleSimulator


def golden(name):
    import json
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                        "reference_test_vectors.json")
    with open(path) as f:
        return json.load(f)[name]


def literal_model():
    """The operator graph of the fixture multidotinc_compress (tests/test_simulator.py:14-38)."""
    g = golden("multidotinc_compress")
    sig = {name: ir.Signal(value, name=name) for name, value in g["signals"].items()}
    m = ir.Model(dt=0.001)
    for kind, *names in g["operators"]:
        m.operators.append(getattr(ir, kind)(*[sig[n] for n in names]))
    return m, sig["a"], sig["b"]


@pytest.mark.parametrize("fuse", [True, False])
def test_multidotinc_compress_literal(fuse):
    """tests/test_simulator.py:14-38: a = [4, -1]; b = [2, -1] then [4, -2]."""
    m, a, b = literal_model()
    with OracleSimulator(None, model=m, fuse=fuse) as sim:
        n_mdi = sum(isinstance(op, MultiDotInc) for op in sim.operators)
        assert n_mdi == 2  # four DotIncs folded onto two targets
        for expect in golden("multidotinc_compress")["expected_after_step"]:
            sim.step()
            assert np.allclose(sim.signals[a], expect["a"])
            assert np.allclose(sim.signals[b], expect["b"])


def test_get_views_scalar_swap_and_shapes():
    y = ir.Signal(np.zeros(5), name="y")
    x = ir.Signal(np.ones(5), name="x")
    a = ir.Signal(np.array(2.0), name="a")
    op = MultiDotInc(y, y, beta=1, gamma=0)
    op.add_AX(a, x)
    A_views, X_views, Y_view, Y_in_view, beta_view = op.get_views()
    assert A_views[0].shape == (5, 1) and X_views[0].shape == (1, 1)  # scalar A swapped with X
    assert Y_view.shape == (5, 1) and beta_view is None
    assert op.incs == [y] and op.sets == []
    bad = MultiDotInc(y, y, beta=1, gamma=0)
    bad.add_AX(ir.Signal(np.zeros((4, 5))), x)
    with pytest.raises(ValueError):
        bad.get_views()
    setter = MultiDotInc(y, x, beta=1, gamma=0)
    assert setter.sets == [y] and x in setter.reads


def feedforward_network(n=5):
    """The shape of tests/test_planners.py:22-38: n nodes -> n ensembles, probed."""
    net = minibuilder.Network(seed=0)
    probes = []
    for i in range(n):
        node = net.Node(minibuilder.WhiteSignal(1.0, 5.0, seed=i), size_out=1)
        ens = net.Ensemble(10, 1)
        net.Connection(node, ens, synapse=None)
        probes.append(net.Probe(ens, synapse=0.01))
    return net, probes


@pytest.mark.parametrize("planner", [greedy_planner, batching_planner])
@pytest.mark.parametrize("fuse", [True, False])
def test_planner_groups(planner, fuse):
    net, _ = feedforward_network()
    with OracleSimulator(net, planner=planner, fuse=fuse) as sim:
        names = [t.__name__ for t, _ in sim.op_groups]
        assert names.count("Reset") <= 1  # all resets planned together (test_planners.py:18)
        assert names.count("SimNeurons") == 1
        assert sum(len(ops) for _, ops in sim.op_groups) == len(sim.operators)
        # every op runs after all of its predecessors
        edges = operator_dependency_graph(sim.operators)
        position = {op: k for k, (_, ops) in enumerate(sim.op_groups) for op in ops}
        for pre, posts in edges.items():
            for post in posts:
                assert position[pre] < position[post]
        # no two ops of a group write overlapping memory
        for _, ops in sim.op_groups:
            written = [s for op in ops for s in list(op.sets) + list(op.incs) + list(op.updates)]
            for i, s in enumerate(written):
                for s2 in written[i + 1:]:
                    assert not (s is s2 or s.may_share_memory(s2))


def test_fusion_cuts_groups_and_keeps_results():
    make = lambda: configs.c2_watts_strogatz(n_ens=48, n_driven=6)
    sims = []
    for fuse in (True, False):
        net, probes, _ = make()
        sim = OracleSimulator(net, seed=1, fuse=fuse)
        sim.run_steps(200)
        sims.append((sim, probes))
    (fused, pf), (plain, pp) = sims
    assert len(fused.op_groups) < len(plain.op_groups) and len(fused.op_groups) <= 8
    for k in pf:
        assert np.array_equal(fused.data[pf[k]], plain.data[pp[k]])  # same additions, same order


def test_cycle_is_reported():
    a, b = ir.Signal(np.zeros(2), name="a"), ir.Signal(np.zeros(2), name="b")
    ops = [ir.Copy(a, b), ir.Copy(b, a)]  # a set-before-read cycle
    with pytest.raises(ValueError):
        greedy_planner(ops)


def test_simplifications_remove_ops():
    """remove_unmodified_resets drops 1 op, remove_zero_incs 1, both 2
    (tests/test_operators.py:30, :54, :82: an ensemble without input)."""
    def n_ops(simps):
        net = minibuilder.Network(seed=0)
        ens = net.Ensemble(10, 2)
        net.Probe(ens, synapse=0.01)
        model = net.build_model()
        old = ops_mod.simplifications
        ops_mod.simplifications = simps
        try:
            return len(ops_mod.simplify_operators(list(model.operators)))
        finally:
            ops_mod.simplifications = old

    base = n_ops([])
    assert n_ops([ops_mod.remove_unmodified_resets]) == base - 1
    assert n_ops([ops_mod.remove_zero_incs]) == base - 1
    assert n_ops([ops_mod.remove_unmodified_resets, ops_mod.remove_zero_incs]) == base - 2


def test_run_probe_reset_semantics():
    net, probes, _ = configs.c0_readme()
    with OracleSimulator(net, n_prealloc_probes=4, seed=1) as sim:
        assert sim._max_steps_between_probes == 4
        sim.run_steps(37)
        first = np.array(sim.data[probes["a"]])
        assert first.shape == (37, 1) and sim.n_steps == 37 and abs(sim.time - 0.037) < 1e-9
        assert np.allclose(sim.trange(), 0.001 * np.arange(1, 38))
        assert np.allclose(sim.trange(sample_every=0.005), 0.001 * np.arange(5, 38, 5))
        sim.reset()
        assert sim.n_steps == 0 and len(sim.data[probes["a"]]) == 0
        sim.run(0.0366)  # rounds to 37 steps
        assert np.array_equal(first, sim.data[probes["a"]])
        sim.clear_probes()
        sim.run_steps(5)
        assert len(sim.data[probes["a"]]) == 5 and sim.n_steps == 42
        with pytest.raises(ValueError):
            sim.run_steps(-1)
        with pytest.raises(ValueError):
            sim.run_steps(2 ** 24)
        with pytest.raises(ValueError):
            sim.run(-1.0)
        with pytest.raises(NotImplementedError):
            sim.reset(seed=3)
    from nengo_ocl_amd.simulator import SimulatorClosed

    with pytest.raises(SimulatorClosed):
        sim.run_steps(1)
    with pytest.raises(SimulatorClosed):
        sim.reset()
    with pytest.raises(NotImplementedError):
        sim.__getstate__()


def test_probe_sample_every():
    net, _, _ = configs.c4_pes(n_triples=1, n_neurons=50, dims=2, solver="lstsq", sample_every=0.01)
    p_fast = net.Probe(net.ensembles[0], synapse=0.01)
    p_slow = net.probes[0]
    with OracleSimulator(net, seed=1, n_prealloc_probes=32) as sim:
        assert sim._max_steps_between_probes == 32  # 32 buffer rows x the shortest period (1 step)
        sim.run_steps(95)
        assert len(sim.data[p_fast]) == 95 and len(sim.data[p_slow]) == 9
        assert len(sim.trange(sample_every=0.01)) == 9


def test_python_function_fallback_and_if_python_code():
    def make(fn):
        net = minibuilder.Network(seed=0)
        node = net.Node(fn, label="f")
        ens = net.Ensemble(20, 1)
        net.Connection(node, ens, synapse=None)
        return net, net.Probe(node)

    net, p = make(lambda t: np.cos(3 * t))
    with OracleSimulator(net) as sim:
        assert any(plan.name == "python_fn" for plan in sim._plans)
        sim.run_steps(20)
        t = sim.trange()
        assert np.allclose(sim.data[p][:, 0], np.cos(3 * t), atol=1e-6)
    with pytest.raises(RuntimeError):
        OracleSimulator(make(lambda t: t)[0], if_python_code="error")
    with pytest.warns(RuntimeWarning):
        OracleSimulator(make(lambda t: t)[0], if_python_code="warn").close()
    net, p = make(np.sin)  # in the unary table: no host callback
    with OracleSimulator(net, if_python_code="error") as sim:
        sim.run_steps(10)
        assert np.allclose(sim.data[p][:, 0], np.sin(sim.trange()), atol=1e-6)


def test_circconv_transforms_exact():
    for dims in (4, 16, 64):
        tr_a, tr_b, tr_out = configs.circconv_transforms(dims)
        rng = np.random.RandomState(dims)
        a, b = rng.normal(size=dims), rng.normal(size=dims)
        expect = np.fft.irfft(np.fft.rfft(a) * np.fft.rfft(b), n=dims)
        assert np.allclose(tr_out @ ((tr_a @ a) * (tr_b @ b)), expect)
        assert tr_a.shape == (4 * (dims // 2 + 1), dims)


def test_watts_strogatz_edges():
    rng = np.random.RandomState(0)
    edges = configs.watts_strogatz_edges(200, 10, 0.1, rng)
    assert len(edges) == 2000 and len(set(edges)) == 2000
    assert all(i != j for i, j in edges)
    lattice = sum(1 for i, j in edges if min((i - j) % 200, (j - i) % 200) <= 5)
    assert 0.8 * 2000 < lattice < 2000  # about 10 % rewired


def test_decoders_decode():
    """LstsqL2 decoders of the mini-builder reproduce x and x**2 from rate activities."""
    net = minibuilder.Network(seed=3)
    ens = net.Ensemble(200, 1)
    out = net.Node(size_in=2)
    net.Connection(ens, out[0:1], synapse=None)
    net.Connection(ens, out[1:2], function=lambda x: x ** 2, synapse=None)
    model = net.build_model()
    p = model.params[ens]
    xs = np.linspace(-1, 1, 21)[:, None]
    acts = ens.neuron_type.rates_from_current(p["gain"] * (xs @ p["encoders"].T) + p["bias"])
    ws = [model.params[c]["weights"] for c in net.connections]
    assert np.abs(acts @ ws[0].T - xs).max() < 0.05
    assert np.abs(acts @ ws[1].T - xs ** 2).max() < 0.05
    assert np.all(acts.max(axis=0) <= 400.5)


def test_plan_dependencies():
    """Conflicts order plans, independent plans stay unordered, edges implied by others
    are dropped, and a plan without memory sets is ordered against everything."""
    from nengo_ocl_amd.plan import plan_dependencies

    class P:
        def __init__(self, reads=None, writes=None):
            if reads is not None:
                self.reads_mem, self.writes_mem = set(reads), set(writes)

    plans = [P("", "t"),      # 0 clock
             P("a", "b"),     # 1 reads a, writes b
             P("b", "c"),     # 2 after 1 (read after write)
             P("t", "d"),     # 3 after 0 only
             P("c", "a"),     # 4 after 2 (c) and after 1 (write after read of a): 1 implied by 2
             P("dc", "")]     # 5 after 3 and 2; 4 does not write c or d
    assert plan_dependencies(plans) == [set(), set(), {1}, {0}, {2}, {2, 3}]
    plans.insert(3, P())      # unknown memory: a barrier
    deps = plan_dependencies(plans)
    assert deps[3] == {0, 2} and deps[4] == {3} and deps[5] == {3}
    plans = [P("", "x"), P("", "x"), P("x", "")]  # two writers of x stay in order
    assert plan_dependencies(plans) == [set(), {0}, {1}]


def test_small_plans_sink_and_merge(monkeypatch):
    """Short plans move behind unrelated long ones until they meet, runs of two or more
    are merged, conflicts and host callbacks stop the move, order of conflicting plans
    is kept."""
    from nengo_ocl_amd import hipra_sequence as hs

    class K:
        def __init__(self, name):
            self.__name__ = name

    class P:
        def __init__(self, label, kern, n_blocks, reads, writes):
            self.label, self.kern, self.name = label, K(kern), kern
            self.args = (None, n_blocks, 256, None, None) if kern == "nhip_copy" else ()
            self.reads_mem, self.writes_mem = set(reads), set(writes)
            self.queue = None

        def enqueue(self):
            pass

    class Host:  # a host callback plan: no enqueue
        label = "host"

    def small(label, reads, writes):
        return P(label, "nhip_copy", 1, reads, writes)

    def big(label, reads, writes):
        return P(label, "nhip_gemv", 0, reads, writes)

    monkeypatch.setattr(hs, "plan_sequence",
                        lambda queue, run: type("M", (), {"label": "+".join(p.label for p in run)})())
    plans = [small("clock", "", "t"), small("bias", "b", "j"), big("sum", "f", "x"),
             big("enc", "xj", "js"), big("dec", "s", "d"), small("input", "t", "n"),
             big("filter", "d", "f"), small("nfilter", "n", "m"), small("probe", "f", "")]
    labels = [p.label for p in hs.merge_small_plans(plans)]
    assert labels == ["sum", "clock+bias", "enc", "dec", "filter", "input+nfilter+probe"]
    # a copy of 5 blocks is not small; a host callback is never passed
    plans = [small("a", "", "p"), Host(), big("g", "q", "r"), small("b", "", "s"),
             P("wide", "nhip_copy", 5, "", "u"), small("c", "", "v")]
    labels = [p.label for p in hs.merge_small_plans(plans)]
    assert labels == ["a", "host", "g", "wide", "b+c"]
    # 1000 rows at one lane per row are four passes of a group: small; 100 rows at 64
    # lanes per row are 25 passes: not small; one pass in which a lane handles eight
    # elements one after the other: not small; more whole-group rows than are staged: not
    narrow, wider, deep, many = (P(k, "nhip_copy", 100, "", k) for k in "nwdm")
    narrow.args, wider.args = (None, 1000, 1, None, None), (None, 100, 64, None, None)
    deep.args, deep.row_iterations = (None, 1, 256, None, None), 8
    many.args = (None, 200, 256, None, None)
    assert hs.is_small(narrow)
    assert not hs.is_small(wider) and not hs.is_small(deep) and not hs.is_small(many)


def test_sequence_chains():
    """The operations of a sequence launch are sorted into chains: conflicting ones
    share a chain and keep their order, independent ones get chains of their own, and
    more chains than the launch has groups for are joined."""
    from nengo_ocl_amd import hipra_sequence as hs

    class P:
        def __init__(self, label, reads, writes):
            self.label, self.reads_mem, self.writes_mem = label, set(reads), set(writes)

    def labels(plans):
        return [[p.label for p in chain] for chain in hs.chains_of(plans)]

    clock, play, filt, probe = P("clock", "", "t"), P("play", "t", "n"), P("filter", "n", "m"), P("probe", "f", "p")
    assert labels([clock, play, filt, probe]) == [["clock", "play", "filter"], ["probe"]]
    # a later plan that touches two chains joins them; order inside the chain is the list's
    both = P("both", "mp", "z")
    assert labels([clock, probe, play, filt, both]) == [["clock", "probe", "play", "filter", "both"]]
    # readers of the same memory do not conflict; two writers do
    assert labels([P("a", "x", "u"), P("b", "x", "v"), P("c", "", "u")]) == [["a", "c"], ["b"]]
    # six independent plans: four chains at most, every plan still there exactly once
    many = [P(str(k), "", "abcdef"[k]) for k in range(6)]
    chains = labels(many)
    assert len(chains) == hs.MAX_CHAINS
    assert sorted(l for c in chains for l in c) == [str(k) for k in range(6)]
    assert all(c == sorted(c) for c in chains)
    # a plan without memory sets conflicts with everything
    class U:
        label = "unknown"
    assert labels([clock, U(), probe]) == [["clock", "unknown", "probe"]]


def test_neurons_without_input_read_their_bias():
    """An ensemble without incoming connections: the copy of its bias into J goes away
    (the neurons read the bias directly); spikes are unchanged."""
    def make():
        net = minibuilder.Network(seed=2)
        node = net.Node(minibuilder.WhiteSignal(1.0, 5.0, seed=0), size_out=1)
        driven, idle = net.Ensemble(40, 1), net.Ensemble(40, 1)
        net.Connection(node, driven, synapse=None)
        probes = [net.Probe(driven.neurons), net.Probe(idle.neurons)]
        return net, probes

    def n_copies(sim):
        return sum(type(op).__name__ == "Copy" for op in sim.operators)

    net, probes = make()
    plain = OracleSimulator(net, seed=1, fuse=False)
    net2, probes2 = make()
    fused = OracleSimulator(net2, seed=1, fuse=True)
    assert n_copies(fused) < n_copies(plain)
    idle_op = [op for op in fused.operators if type(op).__name__ == "SimNeurons"
               and "bias" in (op.J.name or "")]
    assert len(idle_op) == 1
    plain.run_steps(300)
    fused.run_steps(300)
    for a, b in zip(probes, probes2):
        assert np.array_equal(plain.data[a], fused.data[b])
    assert plain.data[probes[1]].sum() > 0


def test_vector_copies_are_propagated():
    """Chains of vector copies (passthrough nodes, ensembles with one unweighted input) are
    cut out of the step: the readers take the source, probe data stay equal to the
    unfused simulator's (a copy's only effect, -0.0 -> +0.0, compares equal), and copies
    that are probed, partial, weighted or read by other operators stay."""
    from nengo_ocl_amd.operators import MultiDotInc, propagate_vector_copies

    def is_copy(op):
        return (isinstance(op, MultiDotInc) and not op._incs_Y and op._float_beta == 0
                and op.gamma == 0 and len(op.As) == 1 and op.As[0].size == 1)

    for make, steps in ((lambda: configs.c1_circconv(dims=8, n_per_dim=30), 300),
                        (lambda: configs.c0_readme(n_neurons=50), 300)):
        sims = []
        for fuse in (True, False):
            net, probes, _ = make()
            sim = OracleSimulator(net, seed=1, fuse=fuse)
            sim.run_steps(steps)
            sims.append((sim, probes))
        (fused, pf), (plain, pp) = sims
        for k in pf:
            assert np.array_equal(fused.data[pf[k]], plain.data[pp[k]])
        # what is left of the copies in the fused graph is read by something other than a GEMV
        # (probes) or not a whole signal
        for op in fused.operators:
            if is_copy(op) and not op.Y.is_view and op.Xs[0].shape == op.Y.shape:
                users = [r for r in fused.operators if r is not op and any(s.base is op.Y.base for s in r.reads)]
                assert not users or not all(isinstance(r, MultiDotInc) for r in users)

    # unit cases on a hand-made graph: y = x feeds z = A @ y; a probed copy stays
    one = ir.Signal(np.array(1.0), name="one", readonly=True)
    x = ir.Signal(np.ones(3), name="x")
    y = ir.Signal(np.zeros(3), name="y")
    z = ir.Signal(np.zeros(2), name="z")
    A = ir.Signal(np.ones((2, 3)), name="A", readonly=True)

    def graph():
        copy = MultiDotInc(y, y, beta=0, gamma=0)
        copy.add_AX(one, x)
        user = MultiDotInc(z, z, beta=0, gamma=0)
        user.add_AX(A, y)
        return [copy, user]

    ops = propagate_vector_copies(graph())
    assert len(ops) == 1 and ops[0].Xs == [x]
    assert len(propagate_vector_copies(graph(), keep=[y])) == 2       # probed
    ops = graph()
    ops[0].gamma = 0.5                                                # not a plain copy
    assert len(propagate_vector_copies(ops)) == 2
    ops = graph() + [ir.Copy(y, ir.Signal(np.zeros(3), name="w"))]    # another kind of reader
    assert len(propagate_vector_copies(ops)) == 3
    two = ir.Signal(np.array(2.0), name="two", readonly=True)
    ops = graph()
    ops[0].As = [two]                                                 # a scaled copy
    assert len(propagate_vector_copies(ops)) == 2


def test_large_item_task_sizes():
    """Rows per task of the large-item GEMV: a launch of many groups takes the largest
    tasks (the start of a task is paid less often), a launch of few groups the size that
    spreads its groups evenly over the compute units, and a size that leaves too few
    tasks is not taken while another gives enough."""
    from types import SimpleNamespace

    from nengo_ocl_amd import hipra_gemv as g

    def tasks_of(n_items, rows, cols, max_rows, n_cu=256):
        prog = g.gemv_prog.__new__(g.gemv_prog)
        prog.queue = SimpleNamespace(lib=None, n_compute_units=n_cu)
        prog.geometry = [{"y_len": rows, "dots": [{"a_shape1": cols}]} for _ in range(n_items)]
        tasks = prog._tile_tasks(list(range(n_items)), max_rows, stream=True)
        # every row of every item exactly once, in order
        for b in range(n_items):
            mine = [(r0, n) for i, r0, n, _ in tasks if i == b]
            assert mine[0][0] == 0 and sum(n for _, n in mine) == rows
            assert all(mine[k][0] + mine[k][1] == mine[k + 1][0] for k in range(len(mine) - 1))
        return tasks

    # 584 matrices of 4096 x 28 (18,688 tasks of 128 rows): many groups per compute unit
    assert {n for _, _, n, _ in tasks_of(584, 4096, 28, 128)} == {128}
    # 256 matrices of 4096 x 64: 128 rows, 8 groups per compute unit
    assert {n for _, _, n, _ in tasks_of(256, 4096, 64, 128)} == {128}
    # 258 matrices of 64 x 4096 (blocks of 4 rows): 8-row tasks would leave 516 groups for
    # 256 compute units, 6-row tasks (the last of an item: 4) give 710 groups, under 3 each
    assert {n for _, _, n, _ in tasks_of(258, 64, 4096, 256)} == {6, 4}
    # 192 matrices of 2000 x 32 (blocks of 32 rows): 96-row tasks are 1008 groups, just under
    # 4 per compute unit; whole blocks rounded up instead, 128 rows (the last of an item:
    # 80), are 768 groups, 3 each, and fewer task starts
    assert {n for _, _, n, _ in tasks_of(192, 2000, 32, 128)} == {128, 80}
    # 64 x 4096 on a device of 64 compute units: 16-row tasks would be too few (1032)
    assert max(n for _, _, n, _ in tasks_of(258, 64, 4096, 256, n_cu=64)) < 16


def test_sparse_slice_window():
    """The run of X a wave keeps in LDS for a slice: centred on the median column, a
    multiple of 4, inside X; none for short or misaligned X, and none when it would hold
    less than a quarter of the slice's column indices."""
    from nengo_ocl_amd import hipra_spmv as h

    band = np.arange(5000, 5164).repeat(3)
    lo = h.slice_window(band, 100000, 64)
    assert lo % 4 == 0 and lo <= 5000 and lo + h.WINDOW >= 5164
    assert h.slice_window(band, 100000, 62) == -1            # X does not start on 16 bytes
    assert h.slice_window(np.arange(10), 500, 0) == -1       # X shorter than the window
    assert h.slice_window(np.zeros(0, dtype=np.int32), 100000, 0) == -1
    assert h.slice_window(np.arange(99990, 100000), 100000, 0) == 100000 - h.WINDOW
    assert h.slice_window(np.arange(0, 10), 100001, 0) == 0
    end = h.slice_window(np.arange(99995, 100001), 100001, 0)
    assert end % 4 == 0 and end + h.WINDOW <= 100001 and end <= 99995
    scattered = np.random.RandomState(0).randint(100000, size=6400)
    assert h.slice_window(scattered, 100000, 0) == -1
    mixed = np.sort(np.concatenate([band, scattered[:band.size // 4]]))  # four fifths in the band
    lo = h.slice_window(mixed, 100000, 0)
    assert lo >= 0 and lo <= 5000 and lo + h.WINDOW >= 5164


@pytest.mark.parametrize("seed", [2, 3])
def test_planning_is_reproducible(seed):
    """Two simulators of one model schedule the operators identically (by position in the
    operator list), also where several increments go into views that overlap and only the
    planner decides their order."""
    import gc

    from random_networks import random_network

    net, _ = random_network(seed, sliced=True)
    model = net.build_model(dt=0.001)
    schedules = []
    junk = []
    for k in range(3):
        junk.append([object() for _ in range(1000 * k + 17)])  # shifts later addresses
        with OracleSimulator(None, model=model, seed=1) as sim:
            where = {op: i for i, op in enumerate(sim.operators)}
            schedules.append([(t.__name__, [where[op] for op in ops]) for t, ops in sim.op_groups])
        gc.collect()
    assert schedules[0] == schedules[1] == schedules[2]


def test_sparse_product_sets_its_target():
    """Reset + one sparse product into a vector become a product that sets it (same bits,
    one operator group less); two products into one vector keep their Reset."""
    import scipy.sparse

    make = lambda: configs.c5_sparse_recurrent(n_neurons=2000, fan_outs=20, weight_scale=5e-4)
    runs = []
    for fuse in (True, False):
        net, probes, _ = make()
        with OracleSimulator(net, seed=1, fuse=fuse) as sim:
            kinds = [type(op).__name__ for op in sim.operators]
            assert ("SparseDotSet" in kinds) == fuse and ("SparseDotInc" in kinds) == (not fuse)
            if fuse:
                assert "Reset" not in kinds
            sim.run_steps(300)
            runs.append({k: np.array(sim.data[p]) for k, p in probes.items()})
            runs[-1]["signals"] = {b.name: np.array(sim.signals[b]) for b in sim.all_bases
                                   if b.name and b.name.endswith(".weighted")}
    assert np.any(runs[0]["spikes"] != 0)
    assert np.array_equal(runs[0]["spikes"], runs[1]["spikes"])
    for name, value in runs[0]["signals"].items():
        assert np.array_equal(value.view(np.uint32), runs[1]["signals"][name].view(np.uint32)), name

    from nengo_ocl_amd import ir, operators

    x, y = ir.Signal(np.ones(70), name="x"), ir.Signal(np.zeros(50), name="y")
    mats = [ir.SparseSignal(scipy.sparse.random(50, 70, density=0.2, random_state=k), name="w%d" % k)
            for k in range(2)]
    two = [ir.Reset(y), ir.SparseDotInc(mats[0], x, y), ir.SparseDotInc(mats[1], x, y)]
    assert operators.sparse_products_set_their_target(two) == two
    one = operators.sparse_products_set_their_target(two[:2])
    assert [type(op).__name__ for op in one] == ["SparseDotSet"]
    half = [ir.Reset(y, value=0.5), ir.SparseDotInc(mats[0], x, y)]  # not a reset to zero
    assert operators.sparse_products_set_their_target(half) == half


def test_synapses_write_the_node_input_they_feed():
    """An ensemble array: three ensembles whose filtered outputs are collected by a node, and
    two transforms interleaved into another node.  The synapses and the transforms write their
    part of the node's input themselves (no Reset, no copies); probes equal the
    operator-at-a-time interpreter bit for bit, and the collected input holds, between steps,
    what the next step reads.  A probed node input is left alone."""
    from oracle.numpy_interpreter import NaiveInterpreter
    from random_networks import ensemble_array_network as make

    net, probes = make(probe_node=False)
    model = net.build_model(dt=0.001)
    naive = NaiveInterpreter(model)
    with OracleSimulator(None, model=model, seed=1) as sim:
        names = {b.name for b in sim.signals_a_step_ahead}
        assert names == {"<Node collect>.in"}
        kinds = [type(op).__name__ for op in sim.operators]
        assert "Reset" not in kinds
        sim.run_steps(200)
        naive.run_steps(200)
        assert np.array_equal(sim.data[probes["post"]], naive.data(probes["post"]))
        assert np.any(sim.data[probes["post"]] != 0)
    net, probes = make(probe_node=True)
    model = net.build_model(dt=0.001)
    naive = NaiveInterpreter(model)
    with OracleSimulator(None, model=model, seed=1) as sim:
        assert not sim.signals_a_step_ahead
        sim.run_steps(100)
        naive.run_steps(100)
        for key, p in probes.items():
            assert np.array_equal(sim.data[p], naive.data(p)), key


def test_sparse_planner_choice_follows_the_reference_rule():
    """`spmv_algorithm_heuristic`: the cases of the reference's test_spmv_impl_heuristic
    (tests/test_clra_gemv.py:465-492) with their answers -- an identity matrix and one with a
    full column fit ELLPACK, one full row makes ELLPACK pad every row to the full width and
    CSR is chosen, a small matrix is ELLPACK whatever its shape -- for a device of 8 GB; and
    the planner names the reference's `algorithm` strings stand for."""
    import scipy.sparse

    from nengo_ocl_amd import hipra_spmv as sp

    class FakeQueue:
        global_mem_size = 8 << 30

    testing_limit = 1e-7
    bytes_limit = FakeQueue.global_mem_size * testing_limit
    size = int(3 * (8 * bytes_limit))
    best = scipy.sparse.eye(size, format="lil")
    bad = best.copy()
    bad[0, :] = 1
    ok = best.copy()
    ok[:, 0] = 1
    small = scipy.sparse.eye(10, format="lil")
    small[0, :] = 1
    for matrix, answer in ((best, "ELLPACK"), (ok, "ELLPACK"), (bad, "CSR"), (small, "ELLPACK")):
        hA = sp.HostSparseMatrix(matrix.tocsr())
        assert sp.spmv_algorithm_heuristic(FakeQueue, hA, footprint_soft_limit=testing_limit) == answer
    assert set(sp.algostr_to_planner) == {"ELLPACK", "ELLPACK-tree", "ELLPACK-twostep", "CSR"}
    for cls in sp.algostr_to_planner.values():
        assert issubclass(cls, sp.spmv_prog) and issubclass(cls, sp.plan_sparse_dot_inc)


def test_heavy_tasks_divide_evenly_over_the_dies():
    """Task records of a large-item launch are reordered so that every accelerator die (a
    contiguous range of the list, `nhip_xcd_remap`) gets the same number of tasks that stream
    a matrix; the light ones (no dot product) fill the ranges up.  Nothing is lost or
    duplicated; lists of equal tasks and short lists stay as they are."""
    from nengo_ocl_amd import hipra_gemv as g

    t = np.zeros((8194, 24), dtype=np.int32)
    t[:8064, 2], t[:8064, 9], t[:8064, 18] = 128, 1, 64
    t[:8064, 0], t[:8064, 1] = np.arange(8064) // 32, (np.arange(8064) % 32) * 128
    t[8064:, 2], t[8064:, 0] = 64, 300 + np.arange(130)
    out = g.spread_over_dies(t)
    assert sorted(map(tuple, out.tolist())) == sorted(map(tuple, t.tolist()))
    groups = -(-len(t) // 4)
    per, rem = divmod(groups, 8)
    pos, heavy = 0, []
    for x in range(8):
        size = (per + (1 if x < rem else 0)) * 4
        heavy.append(int((out[pos:pos + size, 9] > 0).sum()))
        pos += size
    assert heavy == [1008] * 8
    # heavy tasks keep their order (rows of one matrix stay neighbours)
    assert np.array_equal(out[out[:, 9] > 0], t[:8064])
    assert g.spread_over_dies(t[:8064]) is t[:8064] or np.array_equal(g.spread_over_dies(t[:8064]), t[:8064])
    assert np.array_equal(g.spread_over_dies(t[8000:8050]), t[8000:8050])  # 13 groups: left alone
    # few light tasks: ranges are filled with heavy ones, nothing is dropped
    few = np.concatenate([t[:8064], t[8064:8067]])
    out = g.spread_over_dies(few)
    assert sorted(map(tuple, out.tolist())) == sorted(map(tuple, few.tolist()))


def test_reset_restarts_the_random_streams_of_host_processes():
    """The reference's test_reset (tests/test_simulator.py:62-87): a node driven by a process
    whose step draws from the generator the simulator hands it gives the same samples again
    after `reset()`."""
    from nengo_ocl_amd import ir, minibuilder as mb
    from oracle.oracle_sim import OracleSimulator

    class CustomProcess(ir.Process):
        def get_rng(self, rng):
            return np.random.RandomState(rng.randint(2 ** 31 - 1) if self.seed is None else self.seed)

        def make_state(self, shape_in, shape_out, dt, dtype=None):
            return {}

        def make_step(self, shape_in, shape_out, dt, rng, state):
            return lambda t: rng.uniform(size=shape_out).ravel()

    net = mb.Network(seed=3)
    u = net.Node(CustomProcess(), size_out=2)
    up = net.Probe(u)
    with OracleSimulator(net, seed=3) as sim:
        sim.run_steps(10)
        ua = np.array(sim.data[up])
        sim.reset()
        sim.run_steps(10)
        ub = np.array(sim.data[up])
    assert ua.shape == (10, 2) and np.any(ua != 0) and len(np.unique(ua)) == 20
    assert np.array_equal(ua, ub)


def test_which_spikes_are_kept_as_bits():
    """`Simulator._store_spikes_as_bits` on stand-in plans: a population's spikes become bits
    when one large-item neuron launch writes them (tasks at multiples of 32 rows, one
    amplitude, one decay factor) and only whole-vector records of active-column launches
    read them; a probe or any other reader, a record over a part of the vector, a carried
    sequence that reads them, a host-visible copy, an initial value, an odd start or a
    per-neuron amplitude keep the floats.  The tables are updated accordingly: flag bit 11 in
    the population row, the value of a spike in word 15 of the reading records."""
    from types import SimpleNamespace as NS
    from nengo_ocl_amd import hipra_gemv as g
    from nengo_ocl_amd.simulator import Simulator

    class Table:
        def __init__(self):
            self.value = None

        def set(self, array):
            self.value = np.array(array)

    class Base:
        def __init__(self, name, size):
            self.name, self.size = name, size

    n_pops, n = 8, 200
    bases = [Base("s%d" % p, n) for p in range(n_pops)]
    starts = [1000 * p + (1 if p == 6 else 0) for p in range(n_pops)]  # population 6: odd start
    extra = Base("other", 10)
    amp_bits = int(np.array([2.0], dtype=np.float32).view(np.int32)[0])
    pops = np.zeros((n_pops, 8), dtype=np.int32)
    tasks = []
    for p in range(n_pops):
        pops[p] = (0, 0, starts[p], 1, 1, 1, amp_bits, 0x300 | (4 if p == 7 else 0))  # 7: amplitudes
        tasks += [(p, 0, 128, 0), (p, 128, n - 128, 0)]
    enc = NS(name="hipra_gemv.tile_lif", tag="enc", dev_pops=Table(), host_pops=pops,
             host_tasks=np.array(tasks, dtype=np.int32), reads_mem=set(), writes_mem=set(bases),
             bw_per_call=10 ** 6)
    records = np.zeros((n_pops + 1, 16), dtype=np.int32)
    for p in range(n_pops):
        records[p, 3], records[p, 4] = n, starts[p]
    records[n_pops, 3], records[n_pops, 4] = 100, starts[1] + 100  # a record over half of s1
    events = NS(name="hipra_gemv.events_filter", tag="ev", dev_event_table=Table(),
                event_table=records, reads_mem=set(bases), writes_mem={extra},
                carried=NS(reads_mem={bases[2]}))  # a carried gather reads s2
    probe = NS(name="hip_probes", reads_mem={bases[3]}, writes_mem=set())  # s3 is probed
    initial = np.zeros(10000, dtype=np.float32)
    initial[starts[4] + 5] = 1.0  # s4 starts with a spike
    sim = NS(reference_host_state=False, model=NS(dt=0.001), _initial_buf=initial,
             backend=NS(spikes_as_bits=True, store_spikes_as_bits=g.store_spikes_as_bits),
             all_bases=bases + [extra], sidx={b: i for i, b in enumerate(bases + [extra])},
             all_data=NS(starts=starts + [9000]), _host_view_index={bases[5]: 0})  # s5: host copy
    Simulator._store_spikes_as_bits(sim, [enc, events, probe])
    assert set(sim._spike_bits) == {bases[0]}
    start, size, value = sim._spike_bits[bases[0]]
    assert (start, size) == (0, n) and value == np.float32(2.0) * np.float32(1000.0)
    assert [int(f) & g.LIF_POP_BITS for f in pops[:, 7]] == [g.LIF_POP_BITS] + [0] * 7
    assert np.array_equal(enc.dev_pops.value.reshape(pops.shape), pops)
    value_bits = int(np.array([2000.0], dtype=np.float32).view(np.int32)[0])
    assert records[:, 15].tolist() == [value_bits] + [0] * n_pops
    assert np.array_equal(events.dev_event_table.value.reshape(records.shape), records)
    assert "spikes as bits" in enc.tag and enc.bw_per_call == 10 ** 6 - (4 * n - n // 8)

    # tasks that start between multiples of 32 rows, and the switches
    pops[:, 7] &= ~g.LIF_POP_BITS
    records[:, 15] = 0
    enc.host_tasks = np.array([(0, 0, 100, 0), (0, 100, 100, 0)], dtype=np.int32)
    Simulator._store_spikes_as_bits(sim, [enc, events, probe])
    assert not sim._spike_bits and not records[:, 15].any()
    enc.host_tasks = np.array(tasks, dtype=np.int32)
    for off in (dict(reference_host_state=True), dict(backend=NS(spikes_as_bits=False))):
        quiet = NS(**{**vars(sim), **off})
        Simulator._store_spikes_as_bits(quiet, [enc, events, probe])
        assert quiet._spike_bits == {} and not records[:, 15].any()
