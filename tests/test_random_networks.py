"""Randomly wired networks through every rewrite and launch fusion at once.

CPU: `OracleSimulator` (merging, fusing, planning on) against the operator-at-a-time
interpreter, bit for bit.  GPU: the device simulator against the oracle simulator (one product
per connection where no target is a slice), bit for bit, with small and with large ensembles (the small-
and the large-item kernels, input sums formed inside both, sequences carried by both)."""

import numpy as np
import pytest

from helpers import assert_same_signals

from oracle.numpy_interpreter import NaiveInterpreter
from oracle.oracle_sim import OracleSimulator
from random_networks import random_network


@pytest.mark.parametrize("seed,sliced", [(1, False), (2, False), (3, False), (4, False),
                                         (5, False), (6, False), (1, True), (2, True)])
def test_random_network_equals_one_operator_at_a_time(seed, sliced):
    net, probes = random_network(seed, sliced=sliced)
    model = net.build_model(dt=0.001)
    naive = NaiveInterpreter(model)
    with OracleSimulator(None, model=model, seed=1) as sim:
        sim.run_steps(80)
        naive.run_steps(80)
        assert any(np.any(naive.data(p) != 0) for p in probes.values())
        for key, p in probes.items():
            got, want = sim.data[p], naive.data(p)
            assert got.shape == want.shape, key
            if sliced:
                # increments into a slice and into the whole input are ordered by the
                # planner, not by the model's list: sums may differ in the last bit, and a
                # spike may then fall into the neighbouring step
                if key != "spikes":
                    np.testing.assert_allclose(got, want, rtol=1e-3, atol=2e-3)
            else:
                assert np.array_equal(got, want), (key, np.abs(got - want).max())
        if sliced:
            return
        live = {sig.base for op in sim.operators for sig in op.all_signals}
        for base in {sig.base for op in model.operators for sig in op.all_signals}:
            if sim.signal_aliases.get(base, base) in live and base not in sim.signals_a_step_ahead:
                got = np.asarray(sim.signals[base], dtype=np.float32).reshape(-1)
                assert np.array_equal(got, naive.mem[base].reshape(-1)), base


@pytest.mark.parametrize("seed", [31, 32, 33])
def test_rich_random_network_merged_equals_unmerged(seed):
    """Mixed neuron types, synapses of first and second order, learning rules, sparse and
    dense links between neurons, noise: with identical products merged every probe gives
    the numbers of the run that keeps one product per connection."""
    net, probes = random_network(seed, sliced=False, rich=True)
    model = net.build_model(dt=0.001)
    with OracleSimulator(None, model=model, seed=1) as a, \
            OracleSimulator(None, model=model, seed=1, dedup=False) as b:
        a.run_steps(120)
        b.run_steps(120)
        for key, p in probes.items():
            assert np.array_equal(a.data[p], b.data[p]), key
            assert np.all(np.isfinite(a.data[p])), key
        assert any(np.any(a.data[p] != 0) for p in probes.values())


@pytest.mark.gpu
@pytest.mark.parametrize("seed,big,sliced,rich", [
    (1, False, True, False), (2, False, True, False), (3, False, False, False),
    (4, False, False, False), (11, True, True, False), (12, True, False, False),
    (13, True, False, False), (21, False, True, True), (22, False, False, True),
    (23, False, False, True), (24, True, True, True), (25, True, False, True),
    (100, True, True, True), (101, False, False, True), (104, False, True, True),
    (105, True, False, False), (110, True, True, True), (115, True, False, True)])
def test_random_network_on_the_device(queue, seed, big, sliced, rich):
    """With slices among the targets the oracle simulator applies the same rewrites (the
    order of increments into overlapping views follows the operator list that is planned);
    without them it keeps one product per connection, so merging is checked as well."""
    from nengo_ocl_amd.simulator import Simulator

    net, probes = random_network(seed, big=big, sliced=sliced, rich=rich)
    model = net.build_model(dt=0.001)
    steps = 60 if big else 150
    with Simulator(None, model=model, seed=1) as gpu, \
            OracleSimulator(None, model=model, seed=1, dedup=sliced) as cpu:
        gpu.run_steps(steps)
        cpu.run_steps(steps)
        for key, p in probes.items():
            assert np.array_equal(gpu.data[p], cpu.data[p]), key
        assert any(np.any(cpu.data[p] != 0) for p in probes.values())
        live = {sig.base for op in gpu.operators for sig in op.all_signals}
        for base in {sig.base for op in model.operators for sig in op.all_signals}:
            if gpu.signal_aliases.get(base, base) in live and base in cpu.sidx:
                got = np.asarray(gpu.signals[base]).reshape(-1)
                want = np.asarray(cpu.signals[base]).reshape(-1)
                assert np.array_equal(got, want), base


@pytest.mark.gpu
@pytest.mark.parametrize("probe_node", [False, True])
def test_ensemble_array_on_the_device(queue, probe_node):
    """Synapses and transforms that write their part of a node's input (strided and
    one-element views as outputs of the GEMV and filter launches): the device equals the
    oracle simulator bit for bit, in every signal."""
    from nengo_ocl_amd.simulator import Simulator
    from random_networks import ensemble_array_network

    net, probes = ensemble_array_network(probe_node)
    model = net.build_model(dt=0.001)
    with Simulator(None, model=model, seed=1) as gpu, \
            OracleSimulator(None, model=model, seed=1) as cpu:
        assert bool(gpu.signals_a_step_ahead) == (not probe_node)
        gpu.run_steps(200)
        cpu.run_steps(200)
        for key, p in probes.items():
            assert np.array_equal(gpu.data[p], cpu.data[p]) and np.any(gpu.data[p] != 0), key
        assert_same_signals(gpu, cpu)
