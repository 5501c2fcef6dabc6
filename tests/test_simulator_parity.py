"""Whole-simulator parity: the HIP path against the CPU oracle on the same seeded
operator graph, through `Simulator.run`.

Criteria (stated by the task):
* rate neurons (LIFRate): decoded probe outputs within rtol 1e-4 / atol 1e-5;
* spiking LIF: at least 99.9 % of the per-neuron spike counts over the run are
  equal; the discrepancy is printed;
* step counter, time, probe sample counts: exact.

Both simulators share everything above the ``plan_*`` boundary (operator graph,
planner, ragged layout); below it one side is HIP kernels, the other the C
restatement of the reference kernels.  Configurations are the benchmark ones,
reduced where the full size would take the CPU oracle minutes.
"""

import numpy as np
import pytest

from helpers import assert_same_signals, buffer_differences

pytestmark = pytest.mark.gpu


def build_pair(make_net, **sim_kwargs):
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    net, probes, info = make_net()
    model = net.build_model(dt=0.001)
    gpu = Simulator(None, model=model, seed=1, **sim_kwargs)
    net2, probes2, _ = make_net()
    cpu = OracleSimulator(None, model=net2.build_model(dt=0.001), seed=1, dedup=False)
    return gpu, cpu, probes, probes2, info


def add_spike_probes(net, ensembles):
    return [net.Probe(e.neurons) for e in ensembles]


def spike_match(gpu_data, cpu_data, dt=0.001):
    g = np.round(np.asarray(gpu_data).sum(axis=0) * dt).astype(int)
    c = np.round(np.asarray(cpu_data).sum(axis=0) * dt).astype(int)
    return g, c


def check_spiking(gpu, cpu, spike_probes_g, spike_probes_c, steps, label):
    gpu.run_steps(steps)
    cpu.run_steps(steps)
    assert gpu.n_steps == cpu.n_steps == steps
    assert gpu.time == cpu.time
    n_total = n_equal = 0
    worst = 0
    for pg, pc in zip(spike_probes_g, spike_probes_c):
        g, c = spike_match(gpu.data[pg], cpu.data[pc])
        assert g.shape == c.shape
        n_total += g.size
        n_equal += int((g == c).sum())
        worst = max(worst, int(np.abs(g - c).max()))
    frac = n_equal / n_total
    print("%s: %d of %d per-neuron spike counts equal (%.4f %%), largest difference %d spikes, "
          "%d spikes in total" % (label, n_equal, n_total, 100 * frac, worst, int(c.sum())))
    assert frac >= 0.999
    return frac


def test_c0_readme_spiking_10s(queue):
    """The README network for 10 s (10,000 steps): spike counts of all 200 neurons."""
    from nengo_ocl_amd import configs

    def make():
        net, probes, info = configs.c0_readme()
        probes["spikes"] = add_spike_probes(net, net.ensembles)
        return net, probes, info

    gpu, cpu, pg, pc, _ = build_pair(make)
    with gpu, cpu:
        check_spiking(gpu, cpu, pg["spikes"], pc["spikes"], 10000, "c0")
        # decoded outputs are close too (filtered spike trains; not part of the criterion)
        for k in ("a", "b"):
            d = np.abs(gpu.data[pg[k]] - cpu.data[pc[k]])
            print("c0 decoded %s: max |gpu - oracle| = %.3g" % (k, d.max()))
        t = gpu.trange()
        assert np.abs(gpu.data[pg["a"]][:, 0] - np.sin(t)).mean() < 0.05


def test_c0_readme_rate(queue):
    """Same network with LIFRate neurons: decoded outputs rtol 1e-4 / atol 1e-5."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.ir import LIFRate

    gpu, cpu, pg, pc, _ = build_pair(lambda: configs.c0_readme(neuron_type=LIFRate()))
    with gpu, cpu:
        gpu.run(2.0)
        cpu.run(2.0)
        for k in ("a", "b"):
            g, c = gpu.data[pg[k]], cpu.data[pc[k]]
            assert g.shape == c.shape == (2000, 1)
            np.testing.assert_allclose(g, c, rtol=1e-4, atol=1e-5)
            print("c0 rate %s: max |gpu - oracle| = %.3g" % (k, np.abs(g - c).max()))


def test_c1_circconv_rate(queue):
    """D = 16 circular convolution with rate neurons: decoded output close to the
    oracle's, and both close to the true circular convolution."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.ir import LIFRate

    gpu, cpu, pg, pc, info = build_pair(
        lambda: configs.c1_circconv(dims=16, neuron_type=LIFRate()))
    with gpu, cpu:
        gpu.run(0.3)
        cpu.run(0.3)
        g, c = gpu.data[pg["out"]], cpu.data[pc["out"]]
        np.testing.assert_allclose(g, c, rtol=1e-4, atol=1e-5)
        err = np.linalg.norm(g[-1] - info["expected"]) / np.linalg.norm(info["expected"])
        print("c1 rate: relative error of the decoded convolution %.3f" % err)
        assert err < 0.3


def test_c1_circconv_spiking(queue):
    from nengo_ocl_amd import configs

    def make():
        net, probes, info = configs.c1_circconv(dims=64)
        probes["spikes"] = add_spike_probes(net, net.ensembles)
        return net, probes, info

    gpu, cpu, pg, pc, _ = build_pair(make)
    with gpu, cpu:
        check_spiking(gpu, cpu, pg["spikes"], pc["spikes"], 1000, "c1 (D=64, 13,200 neurons)")


def test_c2_watts_strogatz_spiking(queue):
    from nengo_ocl_amd import configs

    def make():
        net, probes, info = configs.c2_watts_strogatz(n_ens=256, n_driven=16)
        probes["spikes"] = add_spike_probes(net, net.ensembles)
        return net, probes, info

    gpu, cpu, pg, pc, _ = build_pair(make)
    with gpu, cpu:
        check_spiking(gpu, cpu, pg["spikes"], pc["spikes"], 1000, "c2 (256 ensembles, 25,600 neurons)")


@pytest.mark.parametrize("dedup", [True, False], ids=["merged-decoders", "per-connection"])
def test_c3_large_reduced_spiking(queue, dedup):
    """The GPU simulator with identical decoder products merged (or not) against the
    oracle simulator that keeps one product per connection."""
    from nengo_ocl_amd import configs

    def make():
        net, probes, info = configs.c3_large(n_ens=8, n_neurons=1024, dims=64, fan_out=4,
                                             solver="lstsq")
        probes["spikes"] = add_spike_probes(net, net.ensembles)
        return net, probes, info

    gpu, cpu, pg, pc, _ = build_pair(make, dedup=dedup)
    assert bool(gpu.signal_aliases) == dedup and not cpu.signal_aliases
    with gpu, cpu:
        # the neurons are updated by the GEMV that computes their input current
        assert any(p.name == "hipra_gemv.tile_lif" for p in gpu._plans)
        assert not any(p.name == "hip_lif" for p in gpu._plans)
        # and the synapse filters by the GEMV that decodes their input (the one that
        # visits only the columns of the neurons that spiked)
        assert any(p.name == "hipra_gemv.events_filter" for p in gpu._plans)
        check_spiking(gpu, cpu, pg["spikes"], pc["spikes"], 1000, "c3 reduced (8 x 1024 x 64-D)")


def test_c3_full_size_state_bit_exact(queue):
    """The benchmark network at its full size (256 ensembles x 4096 LIF x 64-D, the
    configuration the throughput is quoted on, surrogate decoders as in the benchmark):
    after 40 steps every signal -- currents, voltages, refractory times, spikes, decoded
    and filtered values -- and every probe sample is bit-identical to the oracle's, and
    the step runs as the two launches the benchmark times."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    net, probes, _ = configs.c3_large()  # one decoder matrix per connection; merged below
    net_o, probes_o, _ = configs.c3_large()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        assert len(gpu.signal_aliases) == 3 * 768
        names = [p.name for p in gpu._plans]
        # input sums + encoders + neurons; decoders + synapses, with clock / input / probes
        # riding in groups of their own
        assert sorted(names) == ["hipra_gemv.events_filter", "hipra_gemv.tile_lif"]
        assert [p.carried.name for p in gpu._plans if p.name == "hipra_gemv.events_filter"] == [
            "hip_sequence"]
        assert [p.input_sums for p in gpu._plans if p.name == "hipra_gemv.tile_lif"] == [254]
        classes = {p.name: p.kernel_class for p in gpu._plans if hasattr(p, "kernel_class")}
        assert classes["hipra_gemv.tile_lif"] == (3, 3, 4)     # compile-time shapes, narrow
        assert classes["hipra_gemv.events_filter"] == (4, 0, 4)  # columns of spiking neurons only
        gpu.run_steps(40)
        cpu.run_steps(40)
        for key in probes:
            assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]]), key
        assert np.asarray(gpu.all_data.buf).size > 140e6
        assert_same_signals(gpu, cpu)
        assert all(np.any(gpu.data[probes[key]] != 0) for key in probes)  # something happened


def _spike_reader(sim, signals):
    """A function that returns the current spike vector of every population, read in one
    device-to-host copy when the signals lie close together in the simulator's buffer."""
    idx = [int(sim.sidx[s]) for s in signals]
    starts = [int(sim.all_data.starts[i]) for i in idx]
    sizes = [int(s.size) for s in signals]
    lo, hi = min(starts), max(a + n for a, n in zip(starts, sizes))
    dev_buf = getattr(sim.all_data, "dev_buf", None)
    if dev_buf is None or hi - lo > 4 * sum(sizes):
        return lambda: np.concatenate([np.asarray(sim.signals[s]).ravel() for s in signals])

    as_bits = getattr(sim, "_spike_bits", {})  # populations whose spikes the device keeps as bits

    def part(span, s, a, n):
        if s not in as_bits:
            return span[a - lo: a - lo + n]
        words = np.ascontiguousarray(span[a - lo: a - lo + 2 * (-(-n // 64))])
        bits = np.unpackbits(words.view(np.uint8), bitorder="little")[:n]
        return bits.astype(np.float32) * as_bits[s][2]

    def read():
        span = dev_buf.get_span(lo, hi - lo)
        return np.concatenate([part(span, s, a, n) for s, a, n in zip(signals, starts, sizes)])
    return read


def test_c3_full_size_spike_counts_over_one_second(queue):
    """The acceptance criterion at the size the throughput is quoted on: 1000 steps (1 s) of
    the full benchmark network (1,048,576 LIF neurons, the two launches per step that the
    benchmark times, no extra probes), the spike vector of every population read after every
    step on both sides; at least 99.9 % of the per-neuron spike counts must be equal (they
    all are: the test prints the figures), and the final state is bit-identical."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    net, probes, _ = configs.c3_large()
    net_o, probes_o, _ = configs.c3_large()
    model, model_o = net.build_model(dt=0.001), net_o.build_model(dt=0.001)
    with Simulator(None, model=model, seed=1) as gpu, \
            OracleSimulator(None, model=model_o, seed=1) as cpu:
        assert sorted(p.name for p in gpu._plans) == ["hipra_gemv.events_filter",
                                                      "hipra_gemv.tile_lif"]
        spikes_g = [model.sig[e.neurons]["out"] for e in net.ensembles]
        spikes_c = [model_o.sig[e.neurons]["out"] for e in net_o.ensembles]
        read_g, read_c = _spike_reader(gpu, spikes_g), _spike_reader(cpu, spikes_c)
        n = sum(int(s.size) for s in spikes_g)
        assert n == 1048576
        counts_g, counts_c = np.zeros(n, dtype=np.int64), np.zeros(n, dtype=np.int64)
        steps_that_differ, first_difference = 0, None
        for step in range(1000):
            gpu.run_steps(1)
            cpu.run_steps(1)
            g, c = read_g() != 0, read_c() != 0
            counts_g += g
            counts_c += c
            if np.any(g != c):
                steps_that_differ += 1
                if first_difference is None:
                    first_difference = (step + 1, np.flatnonzero(g != c)[:8].tolist())
            if step % 100 == 99:
                print("step %d: %d spikes so far (oracle %d)" % (
                    step + 1, counts_g.sum(), counts_c.sum()), flush=True)
        equal = int((counts_g == counts_c).sum())
        print("c3 full size, 1 s: %d of %d per-neuron spike counts equal (%.4f %%), largest "
              "difference %d spikes, %d spikes in total (mean rate %.1f Hz), %d steps with any "
              "difference" % (equal, n, 100.0 * equal / n, int(np.abs(counts_g - counts_c).max()),
                              int(counts_c.sum()), counts_c.sum() / n, steps_that_differ))
        assert equal / n >= 0.999
        assert counts_c.sum() > 50 * n  # the network is active: tens of Hz per neuron
        # Beyond the criterion: so far every run has been bit-identical to the end.  That
        # rests on two implementations of expm1 / log1p rounding alike on every argument
        # met, which no test can promise for ever: a difference is reported with where it
        # began instead of failing a run that meets the criterion.
        diffs = buffer_differences(gpu, cpu)
        unequal = [k for k in probes if not np.array_equal(gpu.data[probes[k]], cpu.data[probes_o[k]])]
        if diffs or unequal:
            print("NOT bit-identical after 1 s: first step with a differing spike vector and "
                  "its neurons: %s; signals (name, elements, largest difference, first index): "
                  "%s; probes: %s" % (first_difference, diffs, unequal))
        else:
            print("final state and probe data bit-identical")


def test_merged_products_keep_every_signal(queue):
    """One built model (per-connection decoders, reduced c3) run on the GPU with identical
    products merged and without: every probe sample and every signal of the model --
    dropped duplicates through their alias -- bit-identical after 200 steps, and the
    merged step is the two launches of the benchmark."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    net, probes, _ = configs.c3_large(n_ens=8, n_neurons=1024, dims=64, fan_out=4)
    model = net.build_model(dt=0.001)
    with Simulator(None, model=model, seed=1) as a, \
            Simulator(None, model=model, seed=1, dedup=False) as b:
        assert sorted(p.name for p in a._plans) == ["hipra_gemv.events_filter", "hipra_gemv.tile_lif"]
        assert a.all_data.buf.size < b.all_data.buf.size
        a.run_steps(200)
        b.run_steps(200)
        for p in probes.values():
            assert np.array_equal(a.data[p], b.data[p]) and np.any(a.data[p] != 0)
        for base in {sig.base for op in model.operators for sig in op.all_signals}:
            got, want = np.asarray(a.signals[base]), np.asarray(b.signals[base])
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), base


def test_launch_fusions_change_nothing(queue, monkeypatch):
    """Input sums formed inside the encoder launch and the short operations of a step
    carried by the decoder launch, against the same model with each as a launch of its
    own, and decoders that visit only the columns of the neurons that spiked against decoders
    that multiply every column: four launches per step become two, every signal and probe
    sample stays bit-identical (eager and as a recorded graph), and a failed carry is
    reported."""
    from nengo_ocl_amd import _lib, configs
    from nengo_ocl_amd.simulator import Simulator

    net, probes, _ = configs.c3_large(n_ens=8, n_neurons=1024, dims=64, fan_out=4)
    model = net.build_model(dt=0.001)
    sims = []
    for sums, carry, graph, events in (("1", "1", True, "1"), ("1", "1", False, "1"),
                                       ("0", "0", True, "1"), ("1", "1", True, "0")):
        monkeypatch.setenv("NENGO_HIP_INPUT_SUMS", sums)
        monkeypatch.setenv("NENGO_HIP_CARRY_SEQUENCES", carry)
        monkeypatch.setenv("NENGO_HIP_EVENT_GEMV", events)
        sims.append(Simulator(None, model=model, seed=1, use_graph=graph))
    a, eager, plain, dense = sims
    with a, eager, plain, dense:
        assert [len(s._plans) for s in sims] == [2, 2, 4, 2]
        assert sorted(p.name for p in dense._plans) == ["hipra_gemv.tile_filter", "hipra_gemv.tile_lif"]
        for s in sims:
            s.run_steps(100)
        for other in (eager, plain, dense):
            for p in probes.values():
                assert np.array_equal(a.data[p], other.data[p]) and np.any(a.data[p] != 0)
            assert_same_signals(a, other)
        # a launch that cannot carry a sequence says so instead of dropping it
        lib = queue.lib
        carrier = [p for p in a._plans if getattr(p, "carried", None) is not None][0]
        fn, args = carrier.prelude
        _lib.check(fn(*args))
        small = [p for p in plain._plans if p.name == "hipra_gemv.wave_ref"][0]
        big = [p for p in plain._plans if p.name == "hipra_gemv.tile_lif"][0]
        assert lib.nhip_gemv_tile(queue.handle, *big.args[:7], 0, *big.args[8:12]) == -1
        _lib.check(fn(args[0], args[1], args[2], 0, 0))  # disarmed
        small()
        # the launch that visits active columns runs on half the registers of the others and
        # holds neither unary functions nor higher-order filters: a sequence said to need one
        # is refused by it (and the planner does not offer it one)
        from nengo_ocl_amd import hipra_sequence

        assert carrier.name == "hipra_gemv.events_filter" and args[4] == 0
        _lib.check(fn(args[0], args[1], args[2], args[3], 1))
        assert lib.nhip_gemv_events(queue.handle, *carrier.args) == -1
        bare = [p for p in plain._plans if p.name == "hipra_gemv.events_filter"][0]
        assert hipra_sequence._can_carry(bare, 0) and not hipra_sequence._can_carry(bare, 1)
        assert not hipra_sequence._can_carry(bare, 2)


def test_wide_populations_take_their_columns_in_runs(queue):
    """Ensembles of more than 4096 neurons: the launch that visits active columns takes their
    decoders 4096 columns at a time (its instance for such items, here with the step's short
    operations riding in it); 64-D and 20-D values (rows of the transposed matrices padded to
    16); every signal and probe sample equal the oracle simulator's bit for bit."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    for dims in (64, 20):
        make = lambda: configs.c3_large(n_ens=4, n_neurons=9000, dims=dims, fan_out=2)
        (net, probes, _), (net_o, probes_o, _) = make(), make()
        with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
            ev = [p for p in gpu._plans if p.name.startswith("hipra_gemv.events")]
            assert len(ev) == 1 and getattr(ev[0], "carried", None) is not None
            assert int(ev[0].event_table[:, 3].max()) == 9000
            for n in (1, 50, 49):
                gpu.run_steps(n)
                cpu.run_steps(n)
                assert_same_signals(gpu, cpu)
            for key in probes:
                assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]])
                assert np.any(gpu.data[probes[key]] != 0)


@pytest.mark.parametrize("case", ["c2", "c3-per-connection", "c4", "c5"])
def test_other_configurations_full_size_state_bit_exact(queue, case):
    """The other benchmark configurations at their full sizes (2048 ensembles on a
    small-world graph; the 1.37 GB variant of the large network; 64 PES-learning
    triples; one million neurons with sparse recurrent weights): every signal and
    every probe sample bit-identical to the oracle's after 30 steps."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = {"c2": configs.c2_watts_strogatz,
            "c3-per-connection": configs.c3_large,
            "c4": configs.c4_pes,
            "c5": lambda: configs.c5_sparse_recurrent(n_neurons=1000000)}[case]
    net, probes, _ = make()
    net_o, probes_o, _ = make()
    with Simulator(net, seed=1, dedup=False) as gpu, \
            OracleSimulator(net_o, seed=1, dedup=False) as cpu:
        if case == "c4":
            # the weight update rides in the launch that decodes with the learned matrices,
            # the filter of the activities it reads in the launch that updates the neurons
            names = [p.name for p in gpu._plans]
            assert names[:2] == ["hipra_gemv.tile_lif", "hipra_gemv.tile_filter"]
            assert "hip_outer_filter" not in names and "hip_elementwise_inc" not in names
            assert gpu._plans[1].learned_matrices == 64 and gpu._plans[0].deferred_filters == 64
        gpu.run_steps(30)
        cpu.run_steps(30)
        for key in probes:
            assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]]), key
        assert_same_signals(gpu, cpu)


@pytest.mark.parametrize("case", ["c2", "c4"])
def test_other_configurations_full_size_over_one_second(queue, case):
    """The small-world network and the PES-learning network at their full sizes over a
    simulated second (1000 steps, run in batches as `run` does): every probe sample and every
    signal -- the learned decoders included -- bit-identical to the oracle's at the end."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = {"c2": configs.c2_watts_strogatz, "c4": configs.c4_pes}[case]
    net, probes, _ = make()
    net_o, probes_o, _ = make()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        for _ in range(4):
            gpu.run_steps(250)
            cpu.run_steps(250)
        assert gpu.n_steps == cpu.n_steps == 1000 and gpu.time == cpu.time
        for key in probes:
            got, want = gpu.data[probes[key]], cpu.data[probes_o[key]]
            assert got.shape == want.shape and np.any(want != 0), key
            assert np.array_equal(got, want), key
        assert_same_signals(gpu, cpu)


def test_c4_pes_reduced(queue):
    """PES learning: weights after 1 s agree with the oracle's, and learning happened."""
    from nengo_ocl_amd import configs

    def make():
        net, probes, info = configs.c4_pes(n_triples=2, n_neurons=200, dims=4, solver="lstsq",
                                           learning_rate=1e-3)
        probes["spikes"] = add_spike_probes(net, net.ensembles)
        info["learned"] = [c for c in net.connections if c.learning_rule is not None]
        return net, probes, info

    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    net, pg, info = make()
    net2, pc, info2 = make()
    gpu = Simulator(net, seed=1)
    cpu = OracleSimulator(net2, seed=1)
    with gpu, cpu:
        check_spiking(gpu, cpu, pg["spikes"], pc["spikes"], 1000, "c4 reduced (2 triples x 200 x 4-D)")
        for conn_g, conn_c in zip(info["learned"], info2["learned"]):
            wg = gpu.signals[gpu.model.sig[conn_g]["weights"]]
            wc = cpu.signals[cpu.model.sig[conn_c]["weights"]]
            assert np.abs(wc).max() > 0, "no learning happened"
            rel = np.abs(wg - wc).max() / np.abs(wc).max()
            print("c4 learned weights: max relative difference %.3g" % rel)
            assert rel < 0.05
        assert len(gpu.data[pg["post0"]]) == len(cpu.data[pc["post0"]]) == 100  # every 10 steps


def test_run_steps_batches_and_reset(queue):
    """Probe draining across batches (n_prealloc_probes = 4), determinism after reset."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    net, probes, _ = configs.c0_readme()
    with Simulator(net, n_prealloc_probes=4, seed=1) as sim:
        sim.run_steps(37)
        first = np.array(sim.data[probes["a"]])
        assert first.shape == (37, 1) and sim.n_steps == 37
        assert np.allclose(sim.trange(), 0.001 * np.arange(1, 38))
        sim.reset()
        assert sim.n_steps == 0 and len(sim.data[probes["a"]]) == 0
        sim.run_steps(37)
        assert np.array_equal(first, sim.data[probes["a"]])
        sim.clear_probes()
        sim.run_steps(5)
        assert len(sim.data[probes["a"]]) == 5 and sim.n_steps == 42


def _graph_cases():
    from nengo_ocl_amd import configs

    return {
        "c2": lambda: configs.c2_watts_strogatz(n_ens=32, n_driven=4),
        "c1": lambda: configs.c1_circconv(dims=8, n_per_dim=30),
        "c4": lambda: configs.c4_pes(n_triples=3, n_neurons=100, dims=4),
        "c3": lambda: configs.c3_large(n_ens=6, n_neurons=256, dims=16, fan_out=2),
        "c5": lambda: configs.c5_sparse_recurrent(n_neurons=3000, fan_outs=30, weight_scale=5e-4),
    }


BRANCHES_OFF = ("recording a step as parallel graph branches is switched off: the call that "
                "ends such a multi-stream recording crashed inside the HIP runtime for the c4 "
                "step (host segmentation fault, no device fault); Simulator(branches=True) "
                "raises NotImplementedError")


@pytest.mark.parametrize("case", ["c2", "c1", "c4", "c3", "c5"])
@pytest.mark.parametrize("with_branches", [False, pytest.param(True, marks=pytest.mark.skip(
    reason=BRANCHES_OFF))], ids=["chain", "branches"])
def test_graph_replay_equals_eager(queue, case, with_branches):
    """The recorded graph -- one chain of kernels, short operations bound into sequence
    launches (and, when that mode is available, independent kernels as side-by-side
    branches) -- and the eager loop of one launch per operation give bit-identical
    state, also when the graph is replayed in several batches with host work in
    between."""
    from nengo_ocl_amd.simulator import Simulator

    results = []
    variants = [(True, False, True), (False, False, False)]
    if with_branches:
        variants.insert(0, (True, True, True))
    for use_graph, branches, merge in variants:
        net, probes, _ = _graph_cases()[case]()
        with Simulator(net, seed=1, use_graph=use_graph, branches=branches, merge_small=merge,
                       n_prealloc_probes=8) as sim:
            # short operations bound into a sequence, which is a launch or rides in one
            assert any(p.name == "hip_sequence" or getattr(p, "carried", None) is not None
                       for p in sim._plans) == merge
            for chunk in (3, 8, 21, 1, 40):
                sim.run_steps(chunk)
                _ = sim.signals[sim.model.time]
            if use_graph and branches:
                segs = [g for g in sim._plans._segments if hasattr(g, "n_streams_used")]
                assert segs and all(g.deps is not None for g in segs)
            results.append((np.array(sim.all_data.buf), {k: np.array(sim.data[p])
                                                         for k, p in probes.items()}))
    for other in results[1:]:
        assert np.array_equal(results[0][0], other[0])
        for k in results[0][1]:
            assert np.array_equal(results[0][1][k], other[1][k])


def test_step_counts_of_any_size_equal_the_eager_loop(queue):
    """`run_steps` calls of many different lengths (each a few launches of the recorded
    graphs of 2^k steps) with copies taken before the last step of every call (learned
    weights as the host reads them sit in the variant of the graph that holds the call's
    last step): state and probe data equal the eager loop's bit for bit after every call."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    make = lambda: configs.c4_pes(n_triples=2, n_neurons=300, dims=8, solver="lstsq",
                                  learning_rate=3e-4, sample_every=None)
    (net_a, probes_a, _), (net_b, probes_b, _) = make(), make()
    with Simulator(net_a, seed=1) as sim, Simulator(net_b, seed=1, use_graph=False) as eager:
        assert sim._host_view  # (the learned decoders are read from a copy)
        for n in (20, 20, 7, 5, 3, 64, 9, 16, 1, 1, 100, 33):
            sim.run_steps(n)
            eager.run_steps(n)
            assert_same_signals(sim, eager)
        for key in probes_a:
            assert np.array_equal(sim.data[probes_a[key]], eager.data[probes_b[key]])


def test_multidotinc_compress_literal(queue):
    """Literal answers of the reference's test_multidotinc_compress
    (tests/test_simulator.py:14-38): a = [4, -1]; b = [2, -1] then [4, -2]."""
    from nengo_ocl_amd import ir
    from nengo_ocl_amd.simulator import Simulator

    a = ir.Signal([0, 0], name="a")
    b = ir.Signal([0, 0], name="b")
    A = ir.Signal([[1, 2], [0, 1]], name="A")
    B = ir.Signal([[2, 1], [-1, 1]], name="B")
    x = ir.Signal([1, 1], name="x")
    y = ir.Signal([1, -1], name="y")
    m = ir.Model(dt=0.001)
    m.operators += [ir.Reset(a), ir.DotInc(A, x, a), ir.DotInc(B, y, a)]
    m.operators += [ir.DotInc(A, y, b), ir.DotInc(B, x, b)]
    with Simulator(None, model=m) as sim:
        sim.step()
        assert np.allclose(sim.signals[a], [4, -1])
        assert np.allclose(sim.signals[b], [2, -1])
        sim.step()
        assert np.allclose(sim.signals[a], [4, -1])
        assert np.allclose(sim.signals[b], [4, -2])


def test_guards(queue):
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator, SimulatorClosed

    net, _, _ = configs.c0_readme()
    sim = Simulator(net)
    with pytest.raises(ValueError):
        sim.run_steps(-1)
    with pytest.raises(ValueError):
        sim.run_steps(2 ** 24)
    with pytest.raises(ValueError):
        sim.run(-0.1)
    sim.close()
    with pytest.raises(SimulatorClosed):
        sim.run_steps(1)
    with pytest.raises(SimulatorClosed):
        sim.reset()


@pytest.mark.parametrize("kind", ["AdaptiveLIF", "AdaptiveLIFRate", "RectifiedLinear",
                                  "SpikingRectifiedLinear", "Sigmoid"])
def test_other_neuron_types(queue, kind):
    """A driven ensemble of every further neuron type, decoded and probed: all probe
    samples and every signal equal the oracle simulator's bit for bit."""
    from nengo_ocl_amd import minibuilder as mb
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    def make():
        kwargs = dict(tau_n=0.2, inc_n=0.05) if kind.startswith("Adaptive") else {}
        net = mb.Network(seed=4)
        node = net.Node(mb.WhiteSignal(1.0, 5.0, seed=1), size_out=2)
        ens = net.Ensemble(300, 2, neuron_type=getattr(mb, kind)(**kwargs))
        out = net.Ensemble(50, 2)
        net.Connection(node, ens, synapse=None)
        net.Connection(ens, out, synapse=0.01)
        return net, [net.Probe(ens.neurons), net.Probe(ens, synapse=0.02), net.Probe(out, synapse=0.02)]

    net, probes = make()
    net_o, probes_o = make()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        gpu.run_steps(400)
        cpu.run_steps(400)
        for a, b in zip(probes, probes_o):
            assert np.array_equal(gpu.data[a], cpu.data[b])
        assert_same_signals(gpu, cpu)
        assert gpu.data[probes[0]].sum() > 0


def test_sparse_recurrent_population(queue):
    """A population recurrently connected through a sparse weight matrix (the shape of
    the reference's sparse benchmark), 1 s: spikes and every signal bit-identical to the
    oracle simulator."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = lambda: configs.c5_sparse_recurrent(n_neurons=3000, fan_outs=30, weight_scale=5e-4,
                                               probe_neurons=3000)
    net, probes, info = make()
    net_o, probes_o, _ = make()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        # the product passes over zero operands (spikes) and steps the synapse behind its rows
        sparse = [p for p in gpu._plans if p.name == "hip_spmv_filter"]
        assert len(sparse) == 1 and sparse[0].skips_zero_x
        assert not any(p.name == "hip_reset" for p in gpu._plans)
        gpu.run_steps(1000)
        cpu.run_steps(1000)
        assert np.array_equal(gpu.data[probes["spikes"]], cpu.data[probes_o["spikes"]])
        assert_same_signals(gpu, cpu)
        rates = gpu.data[probes["spikes"]][-1]
        assert rates.max() > 50 and rates.std() > 10  # the recurrence shapes the activity


def test_profiling_and_plan_listing(queue, capsys):
    """`profiling=True` times every launch with events (one row per plan: calls, seconds,
    GF/s, GB/s), `print_plans` lists the launches of a step; results are unchanged."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    make = lambda: configs.c3_large(n_ens=4, n_neurons=512, dims=32, fan_out=2, solver="lstsq")
    net, probes, _ = make()
    net2, probes2, _ = make()
    with Simulator(net, seed=1, profiling=True) as prof, Simulator(net2, seed=1) as plain:
        prof.run_steps(40)
        plain.run_steps(40)
        for k in probes:
            assert np.array_equal(prof.data[probes[k]], plain.data[probes2[k]])
        table = prof.profiling_table()
        assert len(table) == len(prof._plans)
        assert all(row[0] == 40 and row[1] > 0 for row in table)
        gemv_rows = [row for row in table if "hipra_gemv.tile" in row[4]]
        assert gemv_rows and all(row[3] > 0 for row in gemv_rows)  # GB/s is reported
        prof.print_profiling(sort=1)
        prof.print_plans()
        out = capsys.readouterr().out
        assert "Profiling" in out and "hipra_gemv.tile_lif" in out and "totals:" in out


def _pair_equal(make, steps, check=None):
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    made_g, made_c = make(), make()
    with Simulator(made_g[0], seed=1) as gpu, OracleSimulator(made_c[0], seed=1) as cpu:
        gpu.run_steps(steps)
        cpu.run_steps(steps)
        for a, b in zip(made_g[-1], made_c[-1]):
            assert np.array_equal(gpu.data[a], cpu.data[b])
        assert_same_signals(gpu, cpu)
        if check is not None:
            check(gpu, made_g)
        return [p.name for p in gpu._plans]


@pytest.mark.parametrize("rule_type", ["BCM", "Oja"])
def test_hebbian_learning_network(queue, rule_type):
    """Weights between two populations learned with BCM / Oja for 400 steps: weights,
    deltas, spikes and every other signal bit-identical to the oracle simulator."""
    from nengo_ocl_amd import minibuilder as mb
    from test_builder_extras import hebbian_network

    make = lambda: hebbian_network(mb.BCM(learning_rate=1e-9) if rule_type == "BCM"
                                   else mb.Oja(learning_rate=1e-6))

    def check(gpu, made):
        w = np.array(gpu.signals[gpu.model.sig[made[1]]["weights"]])
        assert np.abs(w).max() > 5e-3  # started at ~3e-3: they were learned

    names = _pair_equal(make, 400, check)
    assert "hip_" + rule_type.lower() in names


def test_voja_learning_network(queue):
    from test_builder_extras import voja_network

    names = _pair_equal(lambda: voja_network(), 400)
    assert "hip_voja" in names


def test_noise_network(queue):
    """White-noise nodes and noise injected into neurons.  Uniform streams are equal bit
    for bit; Gaussian ones to the last bit except for rare rounding-boundary cases, and a
    single differing sample can move a spike, so this compares samples within one ulp and
    spike counts within the spiking criterion (99.9 %)."""
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator
    from test_builder_extras import noise_network

    (net, probes), (net_o, probes_o) = noise_network(), noise_network()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        assert "hip_whitenoise" in [p.name for p in gpu._plans]
        gpu.run_steps(1000)
        cpu.run_steps(1000)
        g = [np.array(gpu.data[p]) for p in probes]
        c = [np.array(cpu.data[p]) for p in probes_o]
        assert np.array_equal(g[1], c[1])                                 # uniform
        assert np.all(np.abs(g[0] - c[0]) <= np.spacing(np.abs(c[0])))    # Gaussian
        print("Gaussian samples equal: %.5f %%" % (100 * np.mean(g[0] == c[0])))
        counts_g, counts_c = g[2].sum(axis=0) * 1e-3, c[2].sum(axis=0) * 1e-3
        assert np.mean(np.round(counts_g) == np.round(counts_c)) >= 0.999
        assert np.array_equal(g[3], c[3])                                 # the quiet twin
        first = g[0]
        gpu.reset()
        gpu.run_steps(1000)
        assert np.array_equal(first, gpu.data[probes[0]])                 # streams restart


@pytest.mark.parametrize("channels_last", [True, False])
def test_convolution_network(queue, channels_last):
    from test_builder_extras import conv_network

    names = _pair_equal(lambda: conv_network(channels_last), 5)
    assert "hip_conv2d" in names


def function_node_network(seed=3):
    from nengo_ocl_amd import minibuilder as mb

    net = mb.Network(seed=seed)
    stim = net.Node(lambda t: [np.sin(6 * t), np.cos(3 * t) * np.exp(-t)], size_out=2)
    ens = net.Ensemble(200, 2, neuron_type=mb.LIFRate())
    net.Connection(stim, ens, synapse=None)
    # a node computing on decoded values: product, a rectification and a saturating gain
    calc = net.Node(lambda t, x: [x[0] * x[1], max(x[0], 0.0), np.tanh(3 * x[1]) if t > 0.1005 else 0.0],
                    size_in=2, size_out=3)
    net.Connection(ens, calc, synapse=0.01)
    out = net.Ensemble(100, 3, neuron_type=mb.LIFRate())
    net.Connection(calc, out, synapse=0.01)
    return net, [net.Probe(stim), net.Probe(calc), net.Probe(out, synapse=0.02)]


def test_function_nodes_run_on_the_device(queue):
    """Function nodes (of time, and of time and input) are compiled into the step: no host
    callback is left (`if_python_code="error"` would raise), the whole step is one graph,
    and the probes follow the oracle simulator, which calls the Python functions on the
    host, within the rate-neuron tolerance."""
    from nengo_ocl_amd.plan import PythonPlan
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    (net, probes), (net_o, probes_o) = function_node_network(), function_node_network()
    with Simulator(net, seed=1, if_python_code="error") as gpu, \
            OracleSimulator(net_o, seed=1) as cpu:
        assert not any(isinstance(p, PythonPlan) for p in gpu._plans)
        assert sum(p.name == "hip_direct_compiled" for p in gpu._plans) == 2
        assert any(isinstance(p, PythonPlan) for p in cpu._plans)
        gpu.run_steps(500)
        cpu.run_steps(500)
        for a, b in zip(probes, probes_o):
            np.testing.assert_allclose(gpu.data[a], cpu.data[b], rtol=1e-4, atol=1e-5)
        assert np.abs(gpu.data[probes[1]]).max() > 0.1


def test_c4_pes_learning_in_place(queue, monkeypatch):
    """The PES network with `learn_in_place=True` (the rule adds its change to the decoders
    in one pass): the device follows the oracle simulator bit for bit, and both reproduce
    the probe data of the two-pass form exactly."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = lambda: configs.c4_pes(n_triples=3, n_neurons=300, dims=8, solver="lstsq",
                                  learning_rate=3e-4, sample_every=None)
    nets = [make() for _ in range(4)]
    monkeypatch.setenv("NENGO_HIP_OUTER_FILTER", "0")
    apart = Simulator(nets[3][0], seed=1, learn_in_place=True)
    monkeypatch.delenv("NENGO_HIP_OUTER_FILTER")
    with Simulator(nets[0][0], seed=1, learn_in_place=True) as gpu, \
            OracleSimulator(nets[1][0], seed=1, learn_in_place=True) as cpu, \
            Simulator(nets[2][0], seed=1, learn_in_place=False) as two_pass, apart:
        assert sum(p.name == "hip_copy" for p in gpu._plans) < sum(
            p.name == "hip_copy" for p in two_pass._plans)
        # the weight update runs the filter of the activities it has read; switched off,
        # the two are launches of their own: one launch more, the same bits
        assert any(p.name == "hip_outer_filter" for p in gpu._plans)
        assert not any(p.name == "hip_outer_filter" for p in apart._plans)
        assert len(apart._plans) == len(gpu._plans) + 1
        for sim in (gpu, cpu, two_pass, apart):
            sim.run_steps(400)
        assert_same_signals(gpu, apart)
        for key in nets[0][1]:
            assert np.array_equal(gpu.data[nets[0][1][key]], cpu.data[nets[1][1][key]])
            assert np.array_equal(gpu.data[nets[0][1][key]], two_pass.data[nets[2][1][key]])
        assert_same_signals(gpu, cpu)
        assert np.abs(gpu.data[nets[0][1]["post0"]][-1]).max() > 0.05  # something was learned


@pytest.mark.parametrize("rule_type", ["BCM", "Oja", "Voja"])
def test_other_rules_learning_in_place(queue, rule_type):
    from nengo_ocl_amd import minibuilder as mb
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator
    from test_builder_extras import hebbian_network, voja_network

    def make():
        if rule_type == "Voja":
            return voja_network()
        return hebbian_network(mb.BCM(learning_rate=1e-9) if rule_type == "BCM"
                               else mb.Oja(learning_rate=1e-6))

    made_g, made_c = make(), make()
    with Simulator(made_g[0], seed=1, learn_in_place=True) as gpu, \
            OracleSimulator(made_c[0], seed=1, learn_in_place=True) as cpu:
        assert any(getattr(op, "apply_inc", False) for op in gpu.operators)
        gpu.run_steps(300)
        cpu.run_steps(300)
        for a, b in zip(made_g[-1], made_c[-1]):
            assert np.array_equal(gpu.data[a], cpu.data[b])
        assert_same_signals(gpu, cpu)


def test_graph_branches_are_switched_off(queue):
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    net, _, _ = configs.c0_readme(n_neurons=20)
    with pytest.raises(NotImplementedError, match="switched off"):
        Simulator(net, seed=1, branches=True)


@pytest.mark.gpu
def test_constants_with_a_transposed_copy_cannot_be_set(queue, monkeypatch):
    """Decoders that the device also keeps transposed (for the launch that visits only the
    columns of the neurons that spiked) refuse to be overwritten from the host; without that
    launch they can be."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    net, probes, _ = configs.c3_large(n_ens=4, n_neurons=1024, dims=16, fan_out=2)
    model = net.build_model(dt=0.001)
    # (dedup=False: every connection keeps its own matrix, so the only thing in the way of a
    # write is the transposed copy)
    with Simulator(None, model=model, seed=1, dedup=False) as sim:
        assert any(getattr(p, "event_driven", False) for p in sim._plans)
        weights = sorted(sim._copied_constants, key=lambda s: str(s.name))[0]
        with pytest.raises(ValueError, match="another layout"):
            sim.signals[weights] = np.zeros(weights.shape)
    monkeypatch.setenv("NENGO_HIP_EVENT_GEMV", "0")
    with Simulator(None, model=model, seed=1, dedup=False) as sim:
        assert not sim._copied_constants
        sim.signals[weights] = np.zeros(weights.shape)
        sim.run_steps(20)
        assert not np.any(np.asarray(sim.signals[weights]))


@pytest.mark.gpu
def test_constant_weights_between_neurons_visit_active_columns_only(queue):
    """A constant weight matrix from 1024 neurons onto 160 neurons (more than 64 rows: several
    groups of rows), with and without a synapse: the products read only the columns of the
    neurons that spiked, the neurons they drive are updated as usual, and everything equals
    the oracle simulator bit for bit."""
    from nengo_ocl_amd import minibuilder as mb
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    def make():
        rng = np.random.RandomState(4)
        net = mb.Network(seed=7)
        stim = net.Node(mb.WhiteSignal(period=0.5, high=6.0, seed=3), size_out=2)
        a = net.Ensemble(1024, 2, label="a")
        b = net.Ensemble(160, 1, label="b")
        c = net.Ensemble(96, 1, label="c")
        net.Connection(stim, a, synapse=None)
        net.Connection(a.neurons, b.neurons, transform=rng.normal(scale=2e-3, size=(160, 1024)),
                       synapse=None)
        net.Connection(a.neurons, c.neurons, transform=rng.normal(scale=2e-3, size=(96, 1024)),
                       synapse=mb.Lowpass(0.01))
        return net, [net.Probe(b.neurons), net.Probe(c.neurons), net.Probe(a, synapse=0.01)]

    (net, probes), (net_o, probes_o) = make(), make()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        events = [p for p in gpu._plans if getattr(p, "event_driven", False)]
        assert events and sum(p.n_tasks for p in events) >= 3 + 2  # 160 and 96 rows
        gpu.run_steps(300)
        cpu.run_steps(300)
        for p, q in zip(probes, probes_o):
            assert np.array_equal(gpu.data[p], cpu.data[q]) and np.any(gpu.data[p] != 0)
        assert_same_signals(gpu, cpu)


@pytest.mark.gpu
def test_host_reads_follow_the_reference_under_the_rewrites(queue):
    """What `sim.signals` returns between two steps, on the device, with every rewrite on:
    learned decoders that the rule updates in place read as the two-pass simulator holds
    them (device memory is a step ahead), node inputs that synapses write directly read as
    the unrewritten simulator holds them, deltas say that they are not computed, writes to
    in-place matrices are refused, and the copy behind this survives uneven `run_steps`
    lengths (graphs of several sizes), single steps and `reset`."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = lambda: configs.c4_pes(n_triples=3, n_neurons=300, dims=8, solver="lstsq",
                                  learning_rate=3e-4, sample_every=None)
    (net_g, _, _), (net_c, _, _) = make(), make()
    with Simulator(net_g, seed=1) as gpu, \
            OracleSimulator(net_c, seed=1, reference_host_state=True) as ref:
        assert gpu._updated_in_place and gpu._plans.before_last
        pairs = []  # (learned matrix, delta) of the device model / of the reference model
        for sim in (gpu, ref):
            rules = [op for op in sim.model.operators if type(op).__name__ == "SimPES"]
            copies = {op.src: op.dst for op in sim.model.operators if type(op).__name__ == "Copy"}
            pairs.append([(copies[op.delta], op.delta) for op in rules])

        def check():
            for (w_g, d_g), (w_r, d_r) in zip(*pairs):
                want = np.asarray(ref.signals[w_r])
                assert np.array_equal(np.asarray(gpu.signals[w_g]), want)
                ahead = want + np.asarray(ref.signals[d_r])
                assert np.array_equal(np.asarray(gpu.all_data[gpu.sidx[w_g]]), ahead)
                with pytest.raises(ValueError, match="not computed"):
                    gpu.signals[d_g]
                with pytest.raises(ValueError, match="updated in place"):
                    gpu.signals[w_g] = want

        check()  # nothing run yet: initial values
        for n in (1, 1, 37, 300, 2):
            gpu.run_steps(n)
            ref.run_steps(n)
            check()
        gpu.reset()
        ref.reset()
        check()
        gpu.run_steps(21)
        ref.run_steps(21)
        check()

    (net_g, probes_g, _), (net_c, probes_c, _) = (configs.c1_circconv(dims=16) for _ in range(2))
    model_g, model_c = net_g.build_model(dt=0.001), net_c.build_model(dt=0.001)
    with Simulator(None, model=model_g, seed=1) as gpu, \
            OracleSimulator(None, model=model_c, seed=1, reference_host_state=True) as ref:
        assert gpu.signals_a_step_ahead and not ref.signals_a_step_ahead
        by_name = {str(s.name): s for op in model_c.operators for s in op.all_signals}
        for n in (1, 50, 13):
            gpu.run_steps(n)
            ref.run_steps(n)
            for sig in gpu.signals_a_step_ahead:
                got, want = np.asarray(gpu.signals[sig]), np.asarray(ref.signals[by_name[str(sig.name)]])
                assert np.array_equal(got, want) and (n == 1 or np.any(want != 0)), sig
        for key in probes_g:
            assert np.array_equal(gpu.data[probes_g[key]], ref.data[probes_c[key]])


@pytest.mark.gpu
def test_writes_through_merged_signals_are_refused_on_the_device(queue):
    """Decoders that four connections share after the merge and that the device also keeps
    transposed: a write through the dropped duplicate or through the survivor raises (it
    would change all four connections, and the transposed copy would go stale); with
    `reference_host_state=True` the same write lands in one connection's matrix and the
    simulation uses it."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator

    net, probes, _ = configs.c3_large(n_ens=4, n_neurons=1024, dims=16, fan_out=2)
    model = net.build_model(dt=0.001)
    with Simulator(None, model=model, seed=1) as sim:
        assert any(getattr(p, "event_driven", False) for p in sim._plans)
        dups = [(d, r) for d, r in sim.signal_aliases.items() if d.ndim == 2]
        assert dups
        dup, rep = dups[0]
        assert rep.base in sim._copied_constants and dup.base not in sim._copied_constants
        for sig in (dup, rep):
            with pytest.raises(ValueError, match="dedup=False|another layout"):
                sim.signals[sig] = np.zeros(sig.shape)
        sim.run_steps(10)
        assert np.any(np.asarray(sim.signals[dup]))
    with Simulator(None, model=model, seed=1, reference_host_state=True) as sim:
        assert not sim.signal_aliases and not sim._copied_constants
        assert not any(getattr(p, "event_driven", False) for p in sim._plans)
        before = np.array(sim.signals[rep])
        sim.signals[dup] = np.zeros(dup.shape)
        sim.run_steps(10)
        assert not np.any(np.asarray(sim.signals[dup]))
        assert np.array_equal(np.asarray(sim.signals[rep]), before)


@pytest.mark.gpu
def test_currents_nobody_reads_are_not_stored_and_read_back_exact(queue, monkeypatch):
    """An input current that only the neuron update in the epilogue of its own launch reads
    is not written to memory (large and small populations); `sim.signals[J]` and
    `signal_buffer()` run the product again on demand and return the bits the launch would
    have stored (= the oracle's), before the first step the initial value, and a current
    that is probed is stored as before.  Switched off (`NENGO_HIP_SKIP_CURRENTS=0`) every
    current is stored."""
    from nengo_ocl_amd import configs, ir
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    def make():
        net, probes, _ = configs.c3_large(n_ens=4, n_neurons=1024, dims=32, fan_out=2, solver="lstsq")
        small = net.Ensemble(50, 2, label="small")
        net.Connection(net.ensembles[0], small, transform=np.ones((2, 32)) * 0.05)
        probes["small"] = net.Probe(small, synapse=0.01)
        model = net.build_model(dt=0.001)
        probe = ir.Probe(None)  # the input current of one population, probed
        model.probes.append(probe)
        model.sig[probe] = {"in": model.sig[net.ensembles[1].neurons]["in"]}
        probes["J1"] = probe
        return model, probes

    currents = lambda sim: [op.J for op in sim.model.operators if type(op).__name__ == "SimNeurons"]
    (model, probes), (model_o, probes_o) = make(), make()
    with Simulator(None, model=model, seed=1) as gpu, \
            OracleSimulator(None, model=model_o, seed=1) as cpu:
        lazy = set(gpu._lazy_currents)
        probed = model.sig[probes["J1"]]["in"].base
        assert len(lazy) == len(currents(gpu)) - 1 and probed not in lazy
        assert not cpu._lazy_currents
        for J in currents(gpu):  # before the first step: the initial value
            assert not np.any(np.asarray(gpu.signals[J]))
        for n in (1, 30, 7):
            gpu.run_steps(n)
            cpu.run_steps(n)
            in_memory = np.array(gpu.all_data[gpu.sidx[currents(gpu)[0]]]).ravel()
            assert not np.array_equal(in_memory, np.asarray(cpu.signals[currents(cpu)[0]]).ravel())
            for Jg, Jc in zip(currents(gpu), currents(cpu)):
                got, want = np.asarray(gpu.signals[Jg]), np.asarray(cpu.signals[Jc])
                assert np.array_equal(got, want) and np.any(want != 0)
            assert_same_signals(gpu, cpu)
        for key in probes:
            assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]]), key
        gpu.reset()
        cpu.reset()
        for J in currents(gpu):
            assert not np.any(np.asarray(gpu.signals[J]))
        gpu.run_steps(38)
        cpu.run_steps(38)
        assert_same_signals(gpu, cpu)
        monkeypatch.setenv("NENGO_HIP_SKIP_CURRENTS", "0")
        with Simulator(None, model=make()[0], seed=1) as stored:
            assert not stored._lazy_currents
            stored.run_steps(38)
            for Js, Jc in zip(currents(stored), currents(cpu)):
                in_memory = np.array(stored.all_data[stored.sidx[Js]]).ravel()
                assert np.array_equal(in_memory, np.asarray(cpu.signals[Jc]).ravel())


@pytest.mark.gpu
def test_spikes_only_event_launches_read_are_kept_as_bits(queue, monkeypatch):
    """Spikes that nothing but launches visiting active columns reads are left in device
    memory as one bit per neuron (populations whose size is no multiple of 64 included);
    `sim.signals[S]` and `signal_buffer()` give back the oracle's floats, before the first
    step zeros; writing them is refused; spikes that are probed stay floats; with
    `NENGO_HIP_SPIKE_BITS=0` (and with `reference_host_state`) every spike is a float; the
    probe data are the same bits either way."""
    from nengo_ocl_amd import configs, ir
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    def make():
        net, probes, _ = configs.c3_large(n_ens=4, n_neurons=1000, dims=32, fan_out=2, solver="lstsq")
        model = net.build_model(dt=0.001)
        probe = ir.Probe(None)  # the spikes of one population, probed
        model.probes.append(probe)
        model.sig[probe] = {"in": model.sig[net.ensembles[1].neurons]["out"]}
        probes["S1"] = probe
        return model, probes, [model.sig[e.neurons]["out"] for e in net.ensembles]

    (model, probes, spikes), (model_o, probes_o, spikes_o) = make(), make()
    with Simulator(None, model=model, seed=1) as gpu, \
            OracleSimulator(None, model=model_o, seed=1) as cpu:
        kept = gpu._spike_bits
        assert set(kept) == {s.base for s in spikes} - {spikes[1].base} and not cpu._spike_bits
        assert any("spikes as bits" in p.tag for p in gpu._plans)
        for s in spikes:  # before the first step: the initial value
            assert not np.any(np.asarray(gpu.signals[s]))
        for n in (1, 30, 7):
            gpu.run_steps(n)
            cpu.run_steps(n)
            total = 0
            for sg, sc in zip(spikes, spikes_o):
                got, want = np.asarray(gpu.signals[sg]), np.asarray(cpu.signals[sc])
                assert got.shape == want.shape and np.array_equal(got, want)
                total += np.count_nonzero(want)
                in_memory = np.array(gpu.all_data[gpu.sidx[sg]]).ravel()
                if sg.base in kept:  # sixteen words of bits, the rest never written
                    assert not np.any(in_memory[32:])
                else:
                    assert np.array_equal(in_memory, want.ravel())
            assert n == 1 or total > 0
            assert_same_signals(gpu, cpu)
        with pytest.raises(ValueError, match="one bit per neuron"):
            gpu.signals[spikes[0]] = np.zeros(spikes[0].shape, dtype=np.float32)
        gpu.signals[spikes[1]] = np.asarray(gpu.signals[spikes[1]])  # floats: as ever
        for key in probes:
            assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]]), key
        gpu.reset()
        cpu.reset()
        for s in spikes:
            assert not np.any(np.asarray(gpu.signals[s]))
        gpu.run_steps(38)
        cpu.run_steps(38)
        assert_same_signals(gpu, cpu)
        with Simulator(None, model=make()[0], seed=1, reference_host_state=True) as plain:
            assert not plain._spike_bits
        monkeypatch.setenv("NENGO_HIP_SPIKE_BITS", "0")
        model_f, probes_f, spikes_f = make()
        with Simulator(None, model=model_f, seed=1) as floats:
            assert not floats._spike_bits
            floats.run_steps(38)
            for sf, sc in zip(spikes_f, spikes_o):
                in_memory = np.array(floats.all_data[floats.sidx[sf]]).ravel()
                assert np.array_equal(in_memory, np.asarray(cpu.signals[sc]).ravel())
            for key in probes:
                assert np.array_equal(floats.data[probes_f[key]], gpu.data[probes[key]]), key


@pytest.mark.gpu
def test_populations_that_spike_densely_get_dense_products(queue):
    """The launch that visits only the columns of the neurons that spiked loses to the dense
    product when most neurons spike every step.  The constructor's calibration run sees a
    population spiking above a quarter of its neurons per step and plans its products dense;
    a population at ordinary rates keeps the launch; results equal the oracle simulator bit
    for bit either way, and the calibration leaves no trace in the simulation (time, probes,
    state)."""
    from nengo_ocl_amd import minibuilder as mb
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    def make():
        rng = np.random.RandomState(2)
        net = mb.Network(seed=9)
        stim = net.Node(mb.WhiteSignal(period=0.5, high=6.0, seed=3), size_out=2)
        hot = net.Ensemble(1024, 2, label="hot", max_rates=(470, 495), intercepts=(-1.0, -0.97),
                           neuron_type=mb.LIF(tau_rc=0.02, tau_ref=0.001))
        cool = net.Ensemble(1024, 2, label="cool")
        for ens in (hot, cool):
            net.Connection(stim, ens, synapse=None)
        targets = [net.Ensemble(128, 1, label="t%d" % k) for k in range(2)]
        for ens, target in zip((hot, cool), targets):
            net.Connection(ens.neurons, target.neurons, synapse=mb.Lowpass(0.01),
                           transform=rng.normal(scale=5e-5, size=(128, 1024)))
        return net, [net.Probe(t, synapse=0.01) for t in targets] + [net.Probe(hot.neurons)]

    (net, probes), (net_o, probes_o) = make(), make()
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu:
        report = gpu.event_calibration
        print("calibration:", report)
        # (hot, cool and the two target populations, whose probe decoders join the launch)
        assert report["populations"] == 4 and report["populations_switched_to_dense_products"] == 1
        assert report["largest_share_spiking_per_step"] > 0.25
        events = [p for p in gpu._plans if getattr(p, "event_driven", False)]
        # hot's product is dense now (next to that launch the few small products left are not
        # worth a launch of their own and may have joined it)
        n_event_tasks = sum(p.n_tasks for p in events)
        assert any(p.name.startswith("hipra_gemv.tile") for p in gpu._plans)
        assert gpu.n_steps == 0 and gpu.time == 0.0 and len(gpu.data[probes[0]]) == 0
        gpu.run_steps(200)
        cpu.run_steps(200)
        for p, q in zip(probes, probes_o):
            assert np.array_equal(gpu.data[p], cpu.data[q]) and np.any(gpu.data[p] != 0)
        share = np.count_nonzero(gpu.data[probes[2]]) / gpu.data[probes[2]].size
        assert share > 0.25, share
        assert_same_signals(gpu, cpu)
    with Simulator(make()[0], seed=1, event_calibration_steps=0) as uncalibrated:
        assert uncalibrated.event_calibration is None
        # hot's 128 rows (two groups of 64) are in the launch that visits active columns
        assert sum(p.n_tasks for p in uncalibrated._plans
                   if getattr(p, "event_driven", False)) >= n_event_tasks + 2
        assert not any(p.name.startswith("hipra_gemv.tile") for p in uncalibrated._plans)


@pytest.mark.gpu
def test_learning_rule_and_activity_filter_ride_in_the_two_launches(queue, monkeypatch):
    """A PES step at sizes that take the large-item kernels: the outer-product update is done
    by the launch that streams the learned decoders (each block written back with its change
    once it has gone into the sums), and the filter of the pre-synaptic activities by the next
    step's launch that updates the neurons (on the spikes it is about to replace).  Two
    launches per step instead of three; every probe sample and every signal as the host reads
    it -- the learned decoders, and the filtered activities whose last step is still pending
    in device memory -- equal the oracle simulator bit for bit, over uneven `run_steps`
    lengths, single steps and a reset; with the fold switched off the same numbers come from
    three launches.  Writes to what is pending are refused."""
    from nengo_ocl_amd import configs
    from nengo_ocl_amd.simulator import Simulator
    from oracle.oracle_sim import OracleSimulator

    make = lambda: configs.c4_pes(n_triples=3, n_neurons=1024, dims=32, solver="lstsq",
                                  learning_rate=3e-4, sample_every=None)
    (net, probes, _), (net_o, probes_o, _), (net_u, probes_u, _) = make(), make(), make()
    monkeypatch.setenv("NENGO_HIP_FOLD_LEARNING", "0")
    unfolded = Simulator(net_u, seed=1)
    monkeypatch.delenv("NENGO_HIP_FOLD_LEARNING")
    with Simulator(net, seed=1) as gpu, OracleSimulator(net_o, seed=1) as cpu, unfolded:
        assert [p.name for p in gpu._plans] == ["hipra_gemv.tile_lif", "hipra_gemv.tile_filter"]
        assert [p.name for p in unfolded._plans] == ["hipra_gemv.tile_lif", "hipra_gemv.tile_filter",
                                                     "hip_outer_filter"]
        assert gpu._plans[1].learned_matrices == 3 and gpu._plans[0].deferred_filters == 3
        assert len(gpu._pending_filters) == 3 and not unfolded._pending_filters
        pending = list(gpu._pending_filters)

        def check():
            assert_same_signals(gpu, cpu)
            assert_same_signals(gpu, unfolded)
            for f in pending:  # the two simulators lay their signals out in the same order
                same = cpu.all_bases[gpu.all_bases.index(f)]
                assert np.array_equal(np.asarray(gpu.signals[f]), np.asarray(cpu.signals[same]))

        check()  # before the first step
        for n in (1, 1, 37, 200, 2):
            for sim in (gpu, cpu, unfolded):
                sim.run_steps(n)
            check()
        f = pending[0]
        stored = np.asarray(gpu.all_data[gpu.sidx[f]]).ravel()
        assert np.any(np.asarray(gpu.signals[f]) != 0)
        assert not np.array_equal(stored, np.asarray(gpu.signals[f]).ravel())  # one step behind
        for sig in (f, gpu._pending_filters[f][0]):
            with pytest.raises(ValueError, match="pending"):
                gpu.signals[sig] = np.zeros(sig.shape)
        for sim in (gpu, cpu, unfolded):
            sim.reset()
        check()
        for sim in (gpu, cpu, unfolded):
            sim.run_steps(64)
        check()
        for key in probes:
            assert np.array_equal(gpu.data[probes[key]], cpu.data[probes_o[key]]), key
            assert np.array_equal(gpu.data[probes[key]], unfolded.data[probes_u[key]]), key
        assert np.abs(gpu.data[probes["post0"]][-1]).max() > 0.01  # something was learned
