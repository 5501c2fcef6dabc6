"""The simulator's front half (operator rewrites, planner, view builder, probe logic)
pinned without using any of it: an operator list evaluated one operator at a time by
`oracle.numpy_interpreter.NaiveInterpreter` must give the numbers `OracleSimulator` gives with
all of its merging, fusing and batching switched on.  Graph shapes follow the reference's
own fixtures (tests/test_operators.py:30,54,82, tests/test_planners.py:13-47) and the
benchmark configurations at reduced sizes."""

import numpy as np
import pytest

from helpers import assert_same_signals

from oracle.numpy_interpreter import NaiveInterpreter
from nengo_ocl_amd import configs, ir
from oracle.oracle_sim import OracleSimulator

CASES = {
    "c0": lambda: configs.c0_readme(),
    "c0-rate": lambda: configs.c0_readme(neuron_type=ir.LIFRate()),
    "c1": lambda: configs.c1_circconv(dims=8),
    "c2": lambda: configs.c2_watts_strogatz(n_ens=48, n_driven=6),
    "c3": lambda: configs.c3_large(n_ens=6, n_neurons=300, dims=16, fan_out=3, solver="lstsq"),
    "c4": lambda: configs.c4_pes(n_triples=2, n_neurons=150, dims=4, solver="lstsq"),
}


def _model_signals(model):
    return {sig.base for op in model.operators for sig in op.all_signals}


@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("options", [{}, {"learn_in_place": False}, {"fuse": False, "dedup": False}],
                         ids=["default", "two-pass-learning", "plain"])
def test_simulator_equals_one_operator_at_a_time(case, options):
    if "learn_in_place" in options and case != "c4":
        pytest.skip("no learning rule in this network")
    net, probes, _ = CASES[case]()
    model = net.build_model(dt=0.001)
    naive = NaiveInterpreter(model)
    steps = 100
    plain = options.get("fuse") is False
    with OracleSimulator(None, model=model, seed=1, **options) as sim:
        sim.run_steps(steps)
        naive.run_steps(steps)
        for key, p in probes.items():
            got, want = sim.data[p], naive.data(p)
            assert got.shape == want.shape, key
            assert np.any(want != 0), key
            if plain:
                np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
            else:
                assert np.array_equal(got, want), (key, np.abs(got - want).max())
        if plain:
            # without the fusion, increments into one target are separate operators that
            # the planner may run in another order than the model lists them (as in the
            # reference); sums then differ in the last bit, so no bit-for-bit sweep here
            return
        # every signal the simulator still computes, dropped duplicates through their alias
        skipped = 0
        for base in _model_signals(model):
            if base in sim._not_computed:
                # cut out of the graph by a rewrite (copies of other vectors, the delta
                # matrix of a rule that updates in place): reading it says so
                with pytest.raises(ValueError, match="not computed"):
                    sim.signals[base]
                skipped += 1
                continue
            # everything else reads as the interpreter (= the reference) holds it between
            # two steps: learned matrices updated in place and node inputs that synapses
            # write directly come from the copy taken before the last step
            got = np.asarray(sim.signals[base], dtype=np.float32).reshape(-1)
            assert np.array_equal(got, naive.mem[base].reshape(-1)), base
        if options.get("learn_in_place", True) and case == "c4":
            assert sim._updated_in_place and sim._host_view
        if case == "c1" and not options:
            assert sim.signals_a_step_ahead
        assert skipped < len(_model_signals(model)) // 4


def test_a_host_write_to_a_node_input_that_synapses_write_changes_no_step():
    """c1's product inputs are written by the synapses themselves at the end of a step
    (`signals_a_step_ahead`).  The reference resets and refills such an input at the start of
    every step, so a host write between two steps shows in a host read and nowhere else:
    same here."""
    net, probes, _ = CASES["c1"]()
    model = net.build_model(dt=0.001)
    with OracleSimulator(None, model=model, seed=1) as sim, \
            OracleSimulator(None, model=model, seed=1) as untouched:
        assert sim.signals_a_step_ahead
        sim.run_steps(20)
        untouched.run_steps(20)
        for sig in sim.signals_a_step_ahead:
            sim.signals[sig] = np.full(sig.shape, 7.0)
            assert np.all(np.asarray(sim.signals[sig]) == 7.0)
        sim.run_steps(20)
        untouched.run_steps(20)
        for p in probes.values():
            assert np.array_equal(sim.data[p], untouched.data[p])
        assert_same_signals(sim, untouched)
