"""The simulator's front half (operator rewrites, planner, view builder, probe logic)
pinned without using any of it: an operator list evaluated one operator at a time by
`naive_interpreter.NaiveInterpreter` must give the numbers `OracleSimulator` gives with
all of its merging, fusing and batching switched on.  Graph shapes follow the reference's
own fixtures (tests/test_operators.py:30,54,82, tests/test_planners.py:13-47) and the
benchmark configurations at reduced sizes."""

import numpy as np
import pytest

from naive_interpreter import NaiveInterpreter
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
        deltas = {op.delta.base for op in model.operators if type(op).__name__ == "SimPES"}
        in_place = deltas | {op.dst.base for op in model.operators
                             if type(op).__name__ == "Copy" and op.src.base in deltas}
        live = {sig.base for op in sim.operators for sig in op.all_signals}
        for base in _model_signals(model):
            if sim.signal_aliases.get(base, base) not in live:
                skipped += 1  # cut out of the graph by a rewrite (copies of other vectors)
                continue
            if options.get("learn_in_place", True) and base in in_place:
                continue  # deltas are not written in this mode and learned weights already
                #           hold the last step's change, by design
            if base in sim.signals_a_step_ahead:
                # a node input that synapses write directly: between steps it already
                # holds what the interpreter copies into it at the start of the next step
                ahead = naive.mem[base].copy().reshape(-1)
                for op in model.operators:
                    if (type(op).__name__ == "Copy" and op.dst.base is base and op.inc):
                        idx = np.arange(op.dst.size)
                        if op.dst_slice is not None:
                            idx = idx[op.dst_slice]
                        ahead[idx] = naive.mem[op.src.base].reshape(-1)
                got = np.asarray(sim.signals[base], dtype=np.float32).reshape(-1)
                assert np.array_equal(got, ahead), base
                continue
            got = np.asarray(sim.signals[base], dtype=np.float32).reshape(-1)
            assert np.array_equal(got, naive.mem[base].reshape(-1)), base
        assert skipped < len(_model_signals(model)) // 4
