#!/usr/bin/env python
"""Benchmark of the simulator timestep on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` builds the large
bandwidth-bound network (256 ensembles x 4096 LIF neurons x 64-D, 1,048,576
neurons; `nengo_ocl_amd.configs.c3_large`), runs W untimed steps, then times
exactly K steps of ``Simulator.run_steps`` (replays of a recorded graph that holds
16 steps; probe buffers are drained when full, here every 4096 steps) between
stream synchronisations and prints ONE JSON line:

* ``value``: simulator steps per second (inputs resident in HBM);
* ``roofline``: for the dominant kernel (the ragged gather-GEMV launch with the
  largest share of the step), algorithmic bytes per launch (the reference's own
  accounting: A + X per dot, Y_in, Y; plus the state its epilogue reads and
  writes) divided by its average duration, measured with HIP events on the
  simulator's stream in a separate eager pass over the same state, against the
  8 TB/s HBM peak; ``traffic`` is the HBM traffic per launch the hardware
  counters showed for that kernel (profiles/c3_shared_step.txt);
* ``cpu_baseline``: the CPU oracle (C restatement of the reference kernels,
  OpenMP) stepping the same network on the host cores for a bounded sample.

The network is built with one decoder matrix, product and synapse per connection, as a
model builder emits it; the simulator's operator rewrite (`operators.merge_identical_chains`)
computes identical ones once.  ``--no-dedup`` switches that off (c3 then reads 1.37 GB of
matrices per step).  Other configurations: ``--config c0|c1|c2|c4|c5``.

Next to ``value`` the line carries ``value_every_column`` (the same network with every
column of the matrices applied to spikes multiplied, timed by the same rule: ``value``
itself visits only the columns of the neurons that spiked, whose share is
``spiking_fraction``), a ``configs`` block with the other benchmark configurations (each
built, warmed up and timed for ``--config-steps`` steps with the same median rule: steps/s,
launches per step, GEMV bytes per step and their rate against the 8 TB/s peak) and, in
``cpu_baseline``, a second entry ``numpy``: the operator list of the same network evaluated
one operator at a time with numpy in this process (``oracle/numpy_interpreter.py``).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def make_network(config, variant, scale):
    from nengo_ocl_amd import configs

    if config == "c0":
        return configs.c0_readme(), "c0: README two-ensemble net, 200 LIF neurons"
    if config == "c1":
        dims = max(2, int(round(64 * scale)))  # (the reference's benchmark_circconv.py varies D)
        return (configs.c1_circconv(dims=dims),
                "c1: circular convolution D=%d, %d LIF neurons" % (dims, 100 * (2 * dims + 4)))
    if config == "c2":
        return (configs.c2_watts_strogatz(),
                "c2: Watts-Strogatz, 2048 ensembles x 100 LIF, 20,480 decoded edges")
    if config == "c3":
        # built the way a model builder emits it: one weight signal, one product and one
        # synapse per connection.  The simulator's operator rewrite computes identical ones
        # once (one decoder matrix per ensemble); `variant` "per-connection" switches that
        # rewrite off
        n_ens = max(2, int(round(256 * scale)))
        desc = ("c3: %d ensembles x 4096 LIF x 64-D, fan-out 4, %s, surrogate decoders"
                % (n_ens, "identical decoder products merged: one decoder matrix per ensemble "
                   "(~%d MB of matrices per step)" % (n_ens * 2) if variant == "shared" else
                   "one decoder matrix per connection (~%d MB of matrices per step)" % (n_ens * 5)))
        return configs.c3_large(n_ens=n_ens, share_decoded=False), desc
    if config == "c4":
        n = max(1, int(round(64 * scale)))
        return configs.c4_pes(n_triples=n), "c4: PES, %d triples x 2000 LIF x 32-D" % n
    if config == "c5":
        n = max(1000, int(round(1000000 * scale)))
        return (configs.c5_sparse_recurrent(n_neurons=n),
                "c5: %d LIF neurons, recurrent sparse weights, 100 per row" % n)
    raise SystemExit("unknown config %r" % config)


def gemv_summary(sim, profile_steps):
    """Per-plan average durations from an eager pass with HIP events around each launch."""
    plans = sim._plans
    plans.profiling = True
    for p in plans:
        p.atimes[:], p.btimes[:], p.ctimes[:] = [], [], []
        p.n_calls = 0
    sim.run_steps(profile_steps)  # run_steps drains the probe buffers between batches
    plans.profiling = False
    rows = []
    for p in plans:
        if p.n_calls:
            avg = sum(p.ctimes) / p.n_calls
            rows.append(dict(plan=str(p), name=p.name, avg_us=1e6 * avg,
                             bytes=p.bw_per_call,
                             gbs=(1e-9 * p.bw_per_call / avg) if p.bw_per_call and avg > 0 else None))
    return rows


def timed_steps(sim, steps, max_regions, reserve_steps=0):
    """Seconds of the median region of exactly `steps` steps of ``run_steps`` between stream
    synchronisations; a region shorter than 50 ms is timed up to `max_regions` times over.
    Returns (median, all regions)."""
    import torch

    def region():
        sim.queue.finish()
        t0 = time.perf_counter()
        sim.run_steps(steps)  # exactly K steps, probe buffers drained at the end
        sim.queue.finish()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    regions = [region()]
    while sum(regions) < 0.05 * len(regions) and len(regions) < max_regions and (
            sim.n_steps + steps + reserve_steps < 2 ** 24 - 1):
        regions.append(region())
    return sorted(regions)[len(regions) // 2], regions


def warm_up(sim, warmup):
    """W untimed steps, then one untimed launch of every recorded graph (2^k + ... + 2 + 1
    steps) so that no timed launch is a graph's first; the graphs themselves were recorded
    and uploaded when the Simulator was constructed."""
    import torch

    sim.run_steps(warmup)
    sim.run_steps(max(sim._plans.steps_of_every_graph(), 1))
    torch.cuda.synchronize()


def split_rows(sim, rows):
    """(GEMV rows with a rate, rows of launches that visit active columns only)."""
    event_plans = {str(p) for p in sim._plans if getattr(p, "event_driven", False)}
    event_rows = [r for r in rows if r["plan"] in event_plans]
    for r in event_rows:
        r["gbs"] = None
    gemv_rows = [r for r in rows if r["name"].startswith("hipra_gemv") and r["bytes"]
                 and r["plan"] not in event_plans]
    return gemv_rows, event_rows


def spiking_fraction(sim):
    """Share of the neurons of spiking populations that spiked in the last step."""
    import numpy as np

    spiking = [op.output for op in sim.operators if type(op).__name__ == "SimNeurons"]
    n = sum(int(np.asarray(sim.signals[s]).size) for s in spiking)
    nz = sum(int(np.count_nonzero(np.asarray(sim.signals[s]))) for s in spiking)
    return nz / max(n, 1)


def config_summary(config, steps, warmup, profile_steps, max_regions, cpu_budget=0.0,
                   numpy_budget=0.0):
    """One of the other benchmark configurations at its full size through the same protocol:
    built, warmed up, `steps` steps timed (median region), then an eager pass with events
    for the per-launch durations; with budgets, the two CPU legs on a short sample."""
    from nengo_ocl_amd.simulator import Simulator

    t0 = time.time()
    (net, probes, _), workload = make_network(config, "shared", 1.0)
    sim = Simulator(net, seed=1)
    build_s = time.time() - t0
    warm_up(sim, warmup)
    elapsed, regions = timed_steps(sim, steps, max_regions, reserve_steps=profile_steps)
    rows = gemv_summary(sim, profile_steps)
    gemv_rows, event_rows = split_rows(sim, rows)
    gemv_bytes = sum(r["bytes"] for r in gemv_rows)
    gemv_us = sum(r["avg_us"] for r in gemv_rows)
    sparse_rows = [r for r in rows if r["name"].startswith("hip_spmv") and r["bytes"]]
    out = {"workload": workload, "neurons": net.n_neurons, "steps": steps,
           "steps_per_s": steps / elapsed, "ms_per_step": 1e3 * elapsed / steps,
           "timed_regions": len(regions), "launches_per_step": len(sim._plans),
           "plans": [p.name for p in sim._plans],
           "kernel_us_per_step": sum(r["avg_us"] for r in rows),
           "gemv_bytes_per_step": gemv_bytes, "gemv_us_per_step": gemv_us,
           "gemv_gbs": 1e-3 * gemv_bytes / gemv_us if gemv_us else None,
           "gemv_frac_of_peak": 1e-3 * gemv_bytes / gemv_us / HBM_PEAK_GBS if gemv_us else None,
           "kernels": [{"plan": r["plan"], "avg_us": round(r["avg_us"], 2),
                        "gbs": None if r["gbs"] is None else round(r["gbs"], 1)} for r in rows],
           "build_s": build_s}
    if event_rows:
        out["launches_that_visit_active_columns_only"] = [r["plan"] for r in event_rows]
        out["spiking_fraction"] = spiking_fraction(sim)
    if sparse_rows:
        b, us = sum(r["bytes"] for r in sparse_rows), sum(r["avg_us"] for r in sparse_rows)
        out.update(sparse_bytes_per_step=b, sparse_gbs=1e-3 * b / us,
                   sparse_frac_of_peak=1e-3 * b / us / HBM_PEAK_GBS)
    out["n_prealloc_probes"] = sim.n_prealloc_probes
    sim.close()
    if cpu_budget > 0:
        out["cpu_baseline"] = cpu_baseline(config, "shared", 1.0, cpu_budget, elapsed / steps)
        if numpy_budget > 0:
            out["cpu_baseline"]["numpy"] = numpy_baseline(config, "shared", 1.0, numpy_budget)
    return out


KERNEL_SOURCES = ("gemv_tile.hip", "gemv_types.h", "gemv_rows.h", "neuron_math.h", "nhip_common.h",
                  "sequence_ops.h", "small_arg_math.h")


def kernel_sources_hash():
    """sha256 over the sources of the dominant kernel as they are in this tree."""
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "nengo-ocl_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(plan_name):
    """(bytes, source): HBM bytes per launch of the dominant kernel from the counter runs
    summarised in profiles/c3_shared_step.txt (FETCH_SIZE and WRITE_SIZE, scaled by what
    the same counters read for a plain copy of known size), and where the figure comes
    from.  The summary names the hash of the kernel sources it was taken with; when the
    sources in this tree hash differently the figure is stale and None is returned in its
    place.  (None, None) for other workloads."""
    kernel = {"hipra_gemv.tile_lif": "gemv_stream_kernel<1,0,0>",
              "hipra_gemv.tile_filter": "gemv_stream_kernel<2,4,0>"}.get(plan_name)
    rel = os.path.join("profiles", "c3_shared_step.txt")
    path = os.path.join(ROOT, rel)
    if kernel is None or not os.path.exists(path):
        return None, None
    value, profiled_hash = None, None
    for line in open(path):
        parts = line.split()
        if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == kernel:
            value = float(parts[2])
        if len(parts) == 2 and parts[0] == "kernel_sources_sha256":
            profiled_hash = parts[1]
    here = kernel_sources_hash()
    source = {"file": rel, "kernel": kernel, "kernel_sources_sha256_profiled": profiled_hash,
              "kernel_sources_sha256_tree": here, "current": profiled_hash == here,
              "method": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 256 MiB copy"}
    return (value if profiled_hash == here else None), source


def cpu_baseline(config, variant, scale, budget_s, dt_gpu_step):
    from oracle import oracle
    from oracle.oracle_sim import OracleSimulator

    (net, probes, _), _ = make_network(config, variant, scale)
    sim = OracleSimulator(net, seed=1, dedup=variant == "shared")
    sim.run_steps(2)  # warm caches, first-touch
    t0 = time.perf_counter()
    sim.run_steps(3)
    per_step = (time.perf_counter() - t0) / 3
    n = int(max(5, min(2000, budget_s / max(per_step, 1e-6))))
    t0 = time.perf_counter()
    sim.run_steps(n)
    elapsed = time.perf_counter() - t0
    sim.close()
    return dict(value=n / elapsed, unit="steps/s", cores=oracle.num_threads(), kind="port",
                sample="%d steps of the same network on the CPU oracle (C restatement of the "
                       "reference kernels, OpenMP over items), %.1f s" % (n, elapsed))


def numpy_baseline(config, variant, scale, budget_s):
    """The single-process NumPy leg: the operator list of the same network (one product per
    connection, as the builder emits it) evaluated one operator at a time, one numpy
    expression per operator, matrix-vector products through numpy's `@`."""
    from oracle.numpy_interpreter import NaiveInterpreter

    try:
        from threadpoolctl import threadpool_info

        threads = max([int(i.get("num_threads", 1)) for i in threadpool_info()
                       if i.get("user_api") == "blas"] or [1])
    except ImportError:
        threads = None
    (net, probes, _), _ = make_network(config, variant, scale)
    sim = NaiveInterpreter(net.build_model(dt=0.001), blas=True)
    sim.run_steps(1)
    t0 = time.perf_counter()
    sim.run_steps(2)
    per_step = (time.perf_counter() - t0) / 2
    n = int(max(3, min(2000, budget_s / max(per_step, 1e-6))))
    t0 = time.perf_counter()
    sim.run_steps(n)
    elapsed = time.perf_counter() - t0
    return dict(value=n / elapsed, unit="steps/s", cores=threads, kind="port",
                sample="%d steps of the same network, operator by operator in numpy (float32, "
                       "one process; matrix-vector products through numpy's BLAS, %s threads), "
                       "%.1f s" % (n, threads, elapsed))


def calibrate_copy(n_floats=64 * 1024 * 1024, repeats=20):
    """Plain device copy of a known size through the library's copy kernel: reads
    256 MiB and writes 256 MiB per launch.  Profiling this gives the scale of the
    FETCH_SIZE / WRITE_SIZE counters for a kernel whose traffic is known."""
    import numpy as np

    from nengo_ocl_amd.hipra_nonlinearities import plan_copy
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray, Queue
    from nengo_ocl_amd.raggedarray import RaggedArray

    queue = Queue(0)
    X = HIPRaggedArray(queue, RaggedArray([np.ones(n_floats, dtype=np.float32)]))
    Y = HIPRaggedArray(queue, RaggedArray([np.zeros(n_floats, dtype=np.float32)]))
    plan = plan_copy(queue, X, Y, np.zeros(1, dtype=np.int32))
    for _ in range(repeats):
        plan.enqueue()
    queue.finish()
    print(json.dumps({"kernel": "copy_kernel", "launches": repeats,
                      "read_bytes_per_launch": 4 * n_floats, "write_bytes_per_launch": 4 * n_floats}))


def traffic_floor(queue, n_rows, cols, n_reads=3, n_writes=4, repeats=60):
    """Duration (microseconds, events carried by the launches) of the library's calibration
    kernel on the traffic of a "GEMV + LIF" launch: `n_rows` x `cols` floats of matrix streamed
    once, `n_reads` state vectors read and `n_writes` written per row (bias, voltage and
    refractory time in; input current, voltage, refractory time and spikes out).  Two
    matrices are streamed in turn so that nothing is left in the caches.  Returns a dict with
    the duration without the writes, with ordinary and with non-temporal stores."""
    import ctypes

    import torch

    from nengo_ocl_amd import _lib

    lib = queue.lib
    n_rows -= n_rows % 128
    with torch.cuda.device(queue.device):
        mats = [torch.zeros(n_rows * cols, dtype=torch.float32, device=queue.device) for _ in range(2)]
        R = torch.zeros(max(n_reads, 1) * n_rows, dtype=torch.float32, device=queue.device)
        W = torch.zeros(max(n_writes, 1) * n_rows, dtype=torch.float32, device=queue.device)
    torch.cuda.synchronize()
    ev = [ctypes.c_void_p() for _ in range(2)]
    for e in ev:
        _lib.check(lib.nhip_event_create(ctypes.byref(e)))
    out = {}
    for key, writes, nt in (("reads_only_us", 0, 0), ("us", n_writes, 0),
                            ("nontemporal_stores_us", n_writes, 1)):
        total = 0.0
        for i in range(repeats + 4):
            timed = i >= 4
            if timed:
                _lib.check(lib.nhip_time_next_launch(ev[0], ev[1]))
            _lib.check(lib.nhip_calib_stream_mix(
                queue.handle, ctypes.c_void_p(mats[i & 1].data_ptr()), n_rows, cols,
                ctypes.c_void_p(R.data_ptr()), n_reads, ctypes.c_void_p(W.data_ptr()), writes, nt))
            if timed:
                ms = ctypes.c_float()
                _lib.check(lib.nhip_event_elapsed_ms(ev[0], ev[1], ctypes.byref(ms)))
                total += ms.value
        out[key] = 1e3 * total / repeats
    for e in ev:
        lib.nhip_event_destroy(e)
    queue.finish()
    out["bytes"] = 4 * n_rows * (cols + n_reads + n_writes)
    out["problem"] = "%d rows x %d columns, %d vectors read, %d written" % (n_rows, cols, n_reads, n_writes)
    return out


def event_driven_report(sim, event_rows, steps_per_s, make_sim, args):
    """What the launches that visit only the columns with x != 0 were given to do: the
    fraction of neurons that spiked in the last step, their algorithmic bytes (which they do
    not read), and the same simulation with every column multiplied, timed by the same rule
    as `value` (median of the same number of regions of K steps)."""
    out = {"plans": [r["plan"] for r in event_rows],
           "avg_us": sum(r["avg_us"] for r in event_rows),
           "algorithmic_bytes_per_step": sum(r["bytes"] for r in event_rows),
           "note": "these launches read only the columns of their matrices whose x is not zero "
                   "(results bit-identical to the dense product); their algorithmic bytes are "
                   "not traffic and are left out of gemv_all",
           "neurons_that_spiked_in_the_last_step": spiking_fraction(sim),
           # what the constructor's calibration run saw (populations that spike above the
           # threshold per step would have been given dense products)
           "calibration": sim.event_calibration}
    if args.no_dense_comparison:
        return out
    os.environ["NENGO_HIP_EVENT_GEMV"] = "0"
    try:
        dense = make_sim()
        warm_up(dense, args.warmup)
        elapsed, regions = timed_steps(dense, args.steps, args.max_regions)
        dense.close()
        out["every_column_multiplied"] = {
            "steps_per_s": args.steps / elapsed, "ms_per_step": 1e3 * elapsed / args.steps,
            "steps": args.steps, "timed_regions": len(regions), "reported": "median",
            "flag": "--dense-decoders"}
    finally:
        os.environ.pop("NENGO_HIP_EVENT_GEMV", None)
    out["speedup_over_every_column"] = steps_per_s / out["every_column_multiplied"]["steps_per_s"]
    return out


def micro_benchmarks(repeats=50):
    """Kernels that no benchmark network exercises, each on one representative problem:
    one JSON line per kernel with its average duration (start / stop events carried by
    the launch) and the rate of its algorithmic bytes."""
    import numpy as np

    from nengo_ocl_amd import fn_trace
    from nengo_ocl_amd import hipra_nonlinearities as nl
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray, Queue
    from nengo_ocl_amd.raggedarray import RaggedArray

    queue = Queue(0)
    rng = np.random.RandomState(0)
    dev = lambda arrays, **kw: HIPRaggedArray(queue, RaggedArray(arrays, dtype=np.float32, **kw))
    cases = []

    n_conn, m, n = 64, 2000, 2000  # 64 learned 2000 x 2000 weight matrices
    pre, post = dev([rng.rand(n) for _ in range(n_conn)]), dev([rng.rand(m) for _ in range(n_conn)])
    theta = dev([rng.rand(m) for _ in range(n_conn)])
    W, delta = (dev([rng.normal(size=(m, n)) for _ in range(n_conn)]) for _ in range(2))
    alpha, beta = np.full(n_conn, 1e-6, np.float32), np.ones(n_conn, np.float32)
    what = "%d x (%d x %d)" % (n_conn, m, n)
    cases.append(("bcm", what, nl.plan_bcm(queue, pre, post, theta, delta, alpha)))
    cases.append(("oja", what, nl.plan_oja(queue, pre, post, W, delta, alpha, beta)))
    cases.append(("oja, in place", what, nl.plan_oja(queue, pre, post, W, W, alpha, beta, inc=True)))
    err = dev([rng.rand(m) for _ in range(n_conn)])
    cases.append(("pes (outer product)", what,
                  nl.plan_elementwise_inc(queue, err, pre, delta, alpha=alpha, outer=True, inc=False)))

    for shape_in, nf, kernel, strides in (((28, 28, 1), 32, (3, 3), (1, 1)),
                                          ((26, 26, 32), 64, (3, 3), (2, 2)),
                                          ((224, 224, 3), 64, (7, 7), (2, 2))):
        nyi = (shape_in[0] - kernel[0]) // strides[0] + 1
        nyj = (shape_in[1] - kernel[1]) // strides[1] + 1
        data = dev([rng.rand(int(np.prod(shape_in))),
                    rng.normal(size=kernel[0] * kernel[1] * shape_in[2] * nf),
                    np.zeros(nyi * nyj * nf)])
        plan = nl.plan_conv2d(queue, data[[0]], data[[2]], data[[1]], shape_in, (nyi, nyj, nf), kernel,
                              strides=strides, channels_last=True)
        cases.append(("conv2d", "%s -> %s, kernel %s, stride %s" % (
            shape_in, (nyi, nyj, nf), kernel, strides), plan))

    Y = dev([np.zeros(1000000), np.zeros(64)])
    cases.append(("whitenoise (Gaussian)", "1,000,000 + 64 samples",
                  nl.plan_whitenoise(queue, Y, np.int32([1, 1]), np.float32([[0, 1], [0, 1]]),
                                     [1, 1], [0, 0], 1e-3, [1, 2])))
    n_nodes = 100000
    traced = fn_trace.trace(lambda t, x: [np.sin(t) * x[0] + x[1] ** 2, np.tanh(x[0] - x[1])],
                            True, 2, 2)
    T, X2, Y2 = dev([[0.5]] * n_nodes), dev([rng.rand(2) for _ in range(n_nodes)]), dev(
        [np.zeros(2)] * n_nodes)
    plan = nl.plan_direct(queue, traced.code, traced.init, traced.input_names, [T, X2], Y2)
    cases.append(("compiled function node", "%d instances of a 2 -> 2 function" % n_nodes, plan))

    gemv_micro(queue, rng, repeats)
    for name, what, plan in cases:
        for _ in range(3):
            plan()
        for _ in range(repeats):
            plan.enqueue(profiling=True)
        queue.finish()
        plan.update_profiling()
        avg = sum(plan.ctimes) / len(plan.ctimes)
        print(json.dumps({"kernel": name, "problem": what, "avg_us": round(1e6 * avg, 2),
                          "algorithmic_bytes": plan.bw_per_call,
                          "gbs": round(1e-9 * plan.bw_per_call / avg, 1) if plan.bw_per_call else None,
                          "gflops": round(1e-9 * plan.flops_per_call / avg, 1)
                          if plan.flops_per_call else None,
                          "timing": "events carried by the launch" if name != "compiled function node"
                          else "events around the launch"}), flush=True)


def gemv_micro(queue, rng, repeats):
    """The ragged GEMV alone on matrices of one shape: two sets of about 268 MB each
    (more than the caches hold), launched in turn; one JSON line per shape."""
    import numpy as np

    from nengo_ocl_amd import hipra_gemv
    from nengo_ocl_amd.hipraggedarray import HIPRaggedArray
    from nengo_ocl_amd.raggedarray import RaggedArray

    for m, n in ((4096, 8), (4096, 16), (4096, 28), (4096, 48), (4096, 64), (4096, 100),
                 (2048, 200), (64, 4096), (300, 9000), (4096, 10), (4096, 50)):
        n_items = max(1, int(round(268e6 / (4.0 * m * n))))
        progs = []
        for _ in range(2):
            block = rng.standard_normal(size=(m, n)).astype(np.float32)
            ra = lambda arrays: HIPRaggedArray(queue, RaggedArray(arrays, dtype=np.float32, align=True))
            A = ra([block] * n_items + [np.zeros(4, dtype=np.float32)])  # (readable behind the last)
            X = ra([rng.standard_normal(size=n).astype(np.float32)] * n_items)
            Y = ra([np.zeros(m, dtype=np.float32)] * n_items)
            js = [np.array([i], dtype=np.int32) for i in range(n_items)]
            progs.append(hipra_gemv.plan_block_gemv(queue, 1.0, A, js, X, js, 0.0, Y))
        plans = [p for prog in progs for p in prog.plans]
        for _ in range(3):
            for p in plans:
                p()
        for _ in range(repeats // 2):
            for p in plans:
                p.enqueue(profiling=True)
        queue.finish()
        total, calls, nbytes = 0.0, 0, 0
        for p in plans:
            p.update_profiling()
            total += sum(p.ctimes)
            calls += len(p.ctimes)
            nbytes += p.bw_per_call
        avg = total / calls * len(plans) / 2.0  # per set
        print(json.dumps({"kernel": "ragged GEMV, " + ", ".join(sorted({p.name for p in plans})),
                          "problem": "%d x (%d x %d), two sets in turn" % (n_items, m, n),
                          "class": sorted({str(p.kernel_class) for p in plans}),
                          "avg_us": round(1e6 * avg, 2), "algorithmic_bytes": nbytes // 2,
                          "gbs": round(1e-9 * (nbytes / 2.0) / avg, 1),
                          "timing": "events carried by the launch"}), flush=True)
        del progs, plans


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c3")
    ap.add_argument("--variant", default="shared", choices=["shared", "per-connection"],
                    help="c3: 'per-connection' is the same as --no-dedup")
    ap.add_argument("--no-dedup", action="store_true",
                    help="keep identical decoder products and synapses as the builder emitted "
                         "them, one per connection (c3: 1.37 GB of matrices per step)")
    ap.add_argument("--kernel-hash", action="store_true",
                    help="only print the hash of the dominant kernel's sources (the line a "
                         "counter summary under profiles/ carries)")
    ap.add_argument("--scale", type=float, default=1.0, help="fraction of the ensembles (c3, c4), of the dimensions (c1), of the neurons (c5)")
    ap.add_argument("--profile-steps", type=int, default=100)
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds; 0 skips the CPU leg")
    ap.add_argument("--dense-decoders", action="store_true",
                    help="multiply every column of the matrices applied to spike vectors "
                         "(default: only the columns of the neurons that spiked are visited)")
    ap.add_argument("--no-dense-comparison", action="store_true",
                    help="do not time the every-column variant next to the default one "
                         "(kernel traces then hold the default launches only)")
    ap.add_argument("--no-fuse", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--two-pass-learning", action="store_true",
                    help="learning rules write a delta matrix that a copy adds to the weights in "
                         "the next step, as the builder emits it (c4); default: one pass")
    ap.add_argument("--max-regions", type=int, default=25,
                    help="a timed region of K steps shorter than 50 ms is repeated up to this "
                         "many times; the median region is reported")
    ap.add_argument("--config-steps", type=int, default=1000,
                    help="timed steps of each of the other configurations in the `configs` "
                         "block (the benchmark runs of these networks are 1000 steps)")
    ap.add_argument("--other-configs", default="c0,c1,c2,c4,c5",
                    help="configurations reported in the `configs` block of a c3 run at full "
                         "size ('none' for none)")
    ap.add_argument("--config-cpu-budget", type=float, default=2.0,
                    help="seconds of each CPU leg for each of the other configurations")
    ap.add_argument("--numpy-budget", type=float, default=10.0,
                    help="seconds for the single-process NumPy leg of the CPU baseline; 0 skips it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run the plain copy kernel on 256 MiB (1 GiB of traffic per 2 "
                         "launches) 20 times: the known-size reference for HBM counters")
    ap.add_argument("--micro", action="store_true",
                    help="only time the kernels no benchmark network uses (learning rules, "
                         "convolution, noise, compiled function nodes), one JSON line each")
    args = ap.parse_args()
    if args.kernel_hash:
        return print("kernel_sources_sha256", kernel_sources_hash())
    if args.no_dedup:
        args.variant = "per-connection"
    if args.calibrate_copy:
        return calibrate_copy()
    if args.micro:
        return micro_benchmarks()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the timestep of one simulator runs on a single "
                         "MI355X and nothing here uses a second device (got --gpus %d)" % args.gpus)

    import torch

    from nengo_ocl_amd.simulator import Simulator

    if args.dense_decoders:
        os.environ["NENGO_HIP_EVENT_GEMV"] = "0"
    t0 = time.time()
    (net, probes, _), workload = make_network(args.config, args.variant, args.scale)
    make_sim = lambda: Simulator(net, seed=1, fuse=not args.no_fuse, use_graph=not args.no_graph,
                                 learn_in_place=not args.two_pass_learning,
                                 dedup=args.variant == "shared")
    sim = make_sim()
    build_s = time.time() - t0
    n_plans = len(sim._plans)

    warm_up(sim, args.warmup)
    # a region shorter than 50 ms is timed several times over (each region is exactly K
    # steps of the running simulation) and the median region is reported
    elapsed, regions = timed_steps(sim, args.steps, args.max_regions,
                                   reserve_steps=args.profile_steps)
    steps_per_s = args.steps / elapsed

    rows = gemv_summary(sim, args.profile_steps)
    # launches that visit only the columns of the neurons that spiked do not read their
    # algorithmic bytes: they are reported apart, without a rate
    gemv_rows, event_rows = split_rows(sim, rows)
    if event_rows:
        workload += ("; matrices applied to spikes are read only in the columns of the neurons "
                     "that spiked (--dense-decoders reads them whole)")
    dom = max(gemv_rows, key=lambda r: r["avg_us"]) if gemv_rows else None
    step_us_kernels = sum(r["avg_us"] for r in rows)
    gemv_bytes = sum(r["bytes"] for r in gemv_rows)
    gemv_us = sum(r["avg_us"] for r in gemv_rows)
    roofline = None
    if dom is not None:
        traffic, traffic_source = None, None
        if args.config == "c3" and args.variant == "shared" and args.scale == 1.0:
            traffic, traffic_source = measured_traffic(dom["name"])
        roofline = dict(bound="hbm", achieved=dom["gbs"], peak=HBM_PEAK_GBS, unit="GB/s",
                        frac=dom["gbs"] / HBM_PEAK_GBS, traffic=traffic,
                        traffic_source=traffic_source, kernel=dom["plan"],
                        avg_us=dom["avg_us"], bytes_per_launch=dom["bytes"])
        lif = next((p for p in sim._plans if str(p) == dom["plan"]
                    and p.name == "hipra_gemv.tile_lif"), None)
        if lif is not None:
            # the same traffic through a kernel that does nothing else: rows = neurons of the
            # launch, columns from its matrix bytes
            geo = [lif.prog.geometry[b] for b in lif.members]
            n_rows = sum(g["y_len"] for g in geo if g["dots"])
            cols = sum(g["y_len"] * d["a_shape1"] for g in geo for d in g["dots"]) // max(n_rows, 1)
            cols -= cols % 8
            if n_rows >= 128 and cols >= 8:
                # (input currents that only the launch's own epilogue reads are not stored)
                # and spikes that only launches visiting active columns read leave as a bit each
                n_writes = 3 if getattr(lif, "lazy_currents", None) else 4
                import numpy as np
                flags = np.asarray(lif.host_pops)[:, 7]
                if np.any(flags & 0x100) and np.array_equal((flags & 0x800) != 0, (flags & 0x100) != 0):
                    n_writes -= 1
                floor = traffic_floor(sim.queue, n_rows, cols, n_writes=n_writes)
                best = min(floor["us"], floor["nontemporal_stores_us"])
                roofline["plain_kernel_same_traffic"] = dict(
                    floor, frac_of_it=best / dom["avg_us"],
                    note="calibration kernel of the library: streams the matrix rows, reads 3 "
                         "and writes %d vectors per row, keeps no summation order and updates "
                         "no neurons" % n_writes)

    out = {
        "metric": "sim steps/sec + ragged-GEMV HBM GB/s (% peak), 1M-neuron LIF net, 1 MI355X",
        "value": steps_per_s,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": 1e3 * elapsed / args.steps,
        "timed_regions": {"count": len(regions), "reported": "median",
                          "ms_per_step_min": 1e3 * min(regions) / args.steps,
                          "ms_per_step_max": 1e3 * max(regions) / args.steps},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": workload, "neurons": net.n_neurons, "plans_per_step": n_plans,
                   "dt": 0.001, "graph": not args.no_graph,
                   "fused_copies": not args.no_fuse, "learn_in_place": not args.two_pass_learning,
                   "identical_products_merged": args.variant == "shared",
                   "n_prealloc_probes": sim.n_prealloc_probes,
                   "products_with_spikes_visit_active_columns_only": bool(event_rows)},
        "roofline": roofline,
        "gemv_all": {"bytes_per_step": gemv_bytes, "us_per_step": gemv_us,
                     "gbs": 1e-3 * gemv_bytes / gemv_us if gemv_us else None,
                     "frac_of_peak": (1e-3 * gemv_bytes / gemv_us / HBM_PEAK_GBS) if gemv_us else None},
        "event_driven": None,
        "kernels": [{"plan": r["plan"], "avg_us": round(r["avg_us"], 2),
                     "gbs": None if r["gbs"] is None else round(r["gbs"], 1)} for r in rows],
        "kernel_us_per_step": step_us_kernels,
        "build_s": build_s,
    }
    if event_rows:
        report = event_driven_report(sim, event_rows, steps_per_s, make_sim, args)
        out["event_driven"] = report
        # `value` depends on how many neurons spike; the figure that does not is the same
        # network with every column multiplied, timed by the same rule
        out["spiking_fraction"] = report["neurons_that_spiked_in_the_last_step"]
        dense = report.get("every_column_multiplied")
        out["value_every_column"] = dense["steps_per_s"] if dense else None
    elif args.dense_decoders:
        out["value_every_column"] = steps_per_s
        out["spiking_fraction"] = spiking_fraction(sim)
    sim.close()
    del sim
    full_size_default = (args.config == "c3" and args.variant == "shared" and args.scale == 1.0
                         and not (args.no_fuse or args.no_graph or args.two_pass_learning))
    if full_size_default and args.other_configs not in ("", "none"):
        out["configs"] = {}
        for name in args.other_configs.split(","):
            out["configs"][name] = config_summary(
                name, args.config_steps, args.warmup, args.profile_steps, args.max_regions,
                cpu_budget=min(args.cpu_budget, args.config_cpu_budget),
                numpy_budget=min(args.numpy_budget, args.config_cpu_budget))
    if args.cpu_budget > 0:
        out["cpu_baseline"] = cpu_baseline(args.config, args.variant, args.scale, args.cpu_budget,
                                           elapsed / args.steps)
        out["cpu_baseline"]["host_cpu_count"] = os.cpu_count()
        if args.numpy_budget > 0:
            out["cpu_baseline"]["numpy"] = numpy_baseline(args.config, args.variant, args.scale,
                                                          args.numpy_budget)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
