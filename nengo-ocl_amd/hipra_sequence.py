"""Runs of small plans of a timestep, bound into one launch each.

The reference launches every plan separately (plan.py:137-149).  On this device a
kernel that moves a few hundred floats costs what its launch and its first cold
memory accesses cost (4-5 us, strictly one after the other), so the clock update,
input playback, small copies and filters and the probe gather of a step cost more
than their work.  `merge_small_plans` moves such plans next to each other where the
memory they touch allows it and binds each run to one ``nhip_sequence`` launch, in
which a single work-group executes them in order -- the same device functions, the
same results.
"""

import ctypes

import numpy as np

from .hipraggedarray import to_device
from .plan import Plan

# kinds of include/nengo_hip.h
SEQ_RESET, SEQ_COPY, SEQ_SLICEDCOPY, SEQ_ELEMENTWISE_INC, SEQ_LINEARFILTER = 1, 2, 3, 4, 5
SEQ_TIMEUPDATE, SEQ_PRESENTINPUT, SEQ_DIRECT_UNARY, SEQ_PROBES = 6, 7, 8, 9

SEQ_OP_DTYPE = np.dtype([("kind", "<i4"), ("n_blocks", "<i4"), ("i0", "<i4"), ("lanes", "<i4"),
                         ("d0", "<f8"), ("p", "<u8", (8,))])
assert SEQ_OP_DTYPE.itemsize == 88

# one work-group runs the rows of an operation in passes of 256 / lanes rows, one pass
# after the other, and a lane its elements one after the other: only operations this
# short (passes x elements per lane), and only so many operations per launch and rows of
# whole-group operations (they are staged in LDS)
MAX_STEPS_PER_OP = 4
MAX_OPS = 16
MAX_STAGED_ROWS = 128


def _addr(pointer, byte_offset=0):
    if pointer is None:
        return 0
    value = pointer.value if isinstance(pointer, ctypes.c_void_p) else int(pointer)
    return (value or 0) + byte_offset


def sequence_op(plan):
    """(kind, n_rows, lanes, i0, d0, pointers) of a device plan, or None if its kernel has
    no counterpart in the sequence kernel."""
    name = getattr(getattr(plan, "kern", None), "__name__", None)
    a = getattr(plan, "args", ())
    if name == "nhip_reset":
        table, n, lanes, Y = a
        return SEQ_RESET, n, lanes, 0, 0.0, [table, Y]
    if name == "nhip_copy":
        desc, n, lanes, X, Y = a
        return SEQ_COPY, n, lanes, 0, 0.0, [desc, X, Y]
    if name == "nhip_slicedcopy":
        desc, n, lanes, X, Y, XI, YI = a
        return SEQ_SLICEDCOPY, n, lanes, 0, 0.0, [desc, X, Y, XI, YI]
    if name == "nhip_elementwise_inc":
        desc, n, lanes, A, X, Y = a
        return SEQ_ELEMENTWISE_INC, n, lanes, 0, 0.0, [desc, A, X, Y]
    if name == "nhip_linearfilter":
        desc, pos, n, lanes, X, Y, A, B, Xbuf, Ybuf = a
        return SEQ_LINEARFILTER, n, lanes, 0, 0.0, [desc, pos, X, Y, A, B, Xbuf, Ybuf]
    if name == "nhip_timeupdate":
        step, step_start, time, time_start, dt = a
        return SEQ_TIMEUPDATE, 1, 256, 0, float(dt), [_addr(step, 4 * step_start),
                                                      _addr(time, 4 * time_start)]
    if name == "nhip_presentinput":
        desc, n, lanes, dt, Y, T, S = a
        # the entry point takes dt as a float: round it the same way
        return SEQ_PRESENTINPUT, n, lanes, 0, float(np.float32(dt)), [desc, Y, T, S]
    if name == "nhip_direct_unary":
        opcode, desc, n, lanes, X, Y = a
        return SEQ_DIRECT_UNARY, n, lanes, int(opcode), 0.0, [desc, X, Y]
    if name == "nhip_probes":
        desc, n, lanes, countdowns, bufpositions, periods, X, Y = a
        return SEQ_PROBES, n, lanes, 0, 0.0, [desc, countdowns, bufpositions, periods, X, Y]
    return None


def _staged_rows(op):
    return op[1] if op[2] == 256 else 0


def is_small(plan):
    op = sequence_op(plan)
    if op is None:
        return False
    n_rows, lanes = op[1], op[2]
    passes = -(-n_rows // (256 // lanes))
    return (n_rows > 0 and passes * getattr(plan, "row_iterations", 1) <= MAX_STEPS_PER_OP
            and _staged_rows(op) <= MAX_STAGED_ROWS)


def _conflict(p, q):
    rp, wp = getattr(p, "reads_mem", None), getattr(p, "writes_mem", None)
    rq, wq = getattr(q, "reads_mem", None), getattr(q, "writes_mem", None)
    if rp is None or wp is None or rq is None or wq is None:
        return True
    return bool((wp & rq) or (wp & wq) or (rp & wq))


MAX_CHAINS = 4


def chains_of(plans):
    """`plans` sorted into chains: plans that conflict (one writes what the other reads
    or writes) share a chain and keep their order; chains are independent of each other
    and can run side by side.  At most MAX_CHAINS: the shortest ones are joined."""
    parent = list(range(len(plans)))

    def find(i):
        while parent[i] != i:
            parent[i] = parent[parent[i]]
            i = parent[i]
        return i

    for j in range(len(plans)):
        for i in range(j):
            if _conflict(plans[i], plans[j]):
                parent[find(j)] = find(i)
    groups = {}
    for i in range(len(plans)):
        groups.setdefault(find(i), []).append(i)
    chains = sorted(groups.values(), key=lambda c: c[0])
    while len(chains) > MAX_CHAINS:
        chains.sort(key=len)
        chains[0:2] = [sorted(chains[0] + chains[1])]
        chains.sort(key=lambda c: c[0])
    return [[plans[i] for i in chain] for chain in chains]


def sequence_needs(plans):
    """What not every kernel that can carry a sequence of `plans` holds (NHIP_SEQ_NEEDS_*):
    1 = a unary function, 2 = a linear filter of higher order (ring buffers)."""
    return (1 if any(sequence_op(p)[0] == SEQ_DIRECT_UNARY for p in plans) else 0) | (
        2 if any(getattr(p, "higher_order", False) for p in plans) else 0)


def plan_sequence(queue, plans):
    """One launch that runs `plans` (all small, see `is_small`): in order where they
    depend on each other, independent chains of them side by side (a group each)."""
    chains = chains_of(plans)
    plans = [p for chain in chains for p in chain]
    table = np.zeros(len(plans), dtype=SEQ_OP_DTYPE)
    for row, plan in zip(table, plans):
        kind, n, lanes, i0, d0, pointers = sequence_op(plan)
        row["kind"], row["n_blocks"], row["lanes"], row["i0"], row["d0"] = kind, n, lanes, i0, d0
        for k, ptr in enumerate(pointers):
            row["p"][k] = _addr(ptr)
    n_staged = int(table["n_blocks"][table["lanes"] == 256].sum())
    assert len(plans) <= MAX_OPS and n_staged <= MAX_STAGED_ROWS
    dev_table = to_device(queue, table.view(np.int32))
    chain_ops = (ctypes.c_int * len(chains))(*[len(c) for c in chains])
    chain_staged = (ctypes.c_int * len(chains))(
        *[sum(_staged_rows(sequence_op(p)) for p in c) for c in chains])
    merged = Plan(queue, queue.lib.nhip_sequence_chains,
                  (dev_table.ptr, chain_ops, chain_staged, len(chains)), gsize=(256 * len(chains),),
                  lsize=(256,), full_args=(dev_table, chain_ops, chain_staged) + tuple(plans),
                  name="hip_sequence",
                  tag=" | ".join("+".join(p.name.replace("hip_", "") for p in c) for c in chains))
    merged.members = list(plans)
    merged.needs = sequence_needs(plans)
    bws = [p.bw_per_call for p in plans if p.bw_per_call]
    merged.bw_per_call = sum(bws) if bws else None
    reads = [getattr(p, "reads_mem", None) for p in plans]
    writes = [getattr(p, "writes_mem", None) for p in plans]
    if all(r is not None for r in reads) and all(w is not None for w in writes):
        merged.reads_mem = set().union(*reads)
        merged.writes_mem = set().union(*writes)
    return merged


def merge_small_plans(plans):
    """The plan list with every run of two or more small plans bound into one launch.

    First every small plan sinks past the large plans behind it that touch different
    memory (the list order stays a valid execution order), so that small plans
    separated only by unrelated large ones meet; then runs are merged.
    """
    plans = list(plans)
    small = [hasattr(p, "enqueue") and is_small(p) for p in plans]
    for i in range(len(plans) - 2, -1, -1):
        if not small[i]:
            continue
        j = i
        while (j + 1 < len(plans) and not small[j + 1] and hasattr(plans[j + 1], "enqueue")
               and not _conflict(plans[j], plans[j + 1])):
            plans[j], plans[j + 1] = plans[j + 1], plans[j]
            small[j], small[j + 1] = small[j + 1], small[j]
            j += 1
    out, run = [], []

    def close():
        if len(run) >= 2:
            out.append(plan_sequence(run[0].queue, run))
        else:
            out.extend(run)
        del run[:]

    for plan, s in zip(plans, small):
        if s:
            rows = sum(_staged_rows(sequence_op(p)) for p in run + [plan])
            if len(run) == MAX_OPS or rows > MAX_STAGED_ROWS:
                close()
            run.append(plan)
        else:
            close()
            out.append(plan)
    close()
    return out


def _can_carry(plan, needs=0):
    """GEMV launches with an epilogue: the large-item kernel with compile-time shapes, the
    launch that visits only the columns with x != 0 (which runs on half the registers of the
    others and holds no unary functions and no higher-order filters: `needs`), the small-item
    kernel, and the sparse products."""
    cls = getattr(plan, "kernel_class", None)
    name = getattr(plan, "name", "")
    if name in ("hip_spmv", "hip_spmv_filter"):  # the sparse products (one or more slices)
        return getattr(plan, "prelude", None) is None and getattr(plan, "spmv", {}).get("n", 0) > 0
    if cls is None or getattr(plan, "prelude", None) is not None or getattr(plan, "n_tasks", 0) <= 0:
        return False
    if name in ("hipra_gemv.tile_lif", "hipra_gemv.tile_filter"):
        return cls[0] == 3 and cls[1] >= 2
    if name in ("hipra_gemv.events", "hipra_gemv.events_filter"):
        return cls[0] == 4 and needs == 0
    return name in ("hipra_gemv.wave_ref", "hipra_gemv.wave_ref_lif",
                    "hipra_gemv.wave_ref_filter") and cls[0] == 2


def carry_sequences(plans):
    """Sequence launches (and single small plans) next to a large-item GEMV launch that
    touches none of their memory ride in that launch, in work-groups of their own
    (``nhip_gemv_tile_carry``): the launch before them if it can take them, else the one
    after.  The plan list loses those launches; results are unchanged."""
    plans = list(plans)
    k = 0
    while k < len(plans):
        seq = plans[k]
        rides = getattr(seq, "name", "") == "hip_sequence" or (
            hasattr(seq, "enqueue") and is_small(seq))
        if not rides:
            k += 1
            continue
        needs = seq.needs if seq.name == "hip_sequence" else sequence_needs([seq])
        # the nearest launch that can take it, backwards then forwards, over plans that touch
        # none of its memory (moving past those changes nothing)
        j = None
        for step in (-1, 1):
            q = k + step
            while 0 <= q < len(plans) and hasattr(plans[q], "enqueue") and not _conflict(seq, plans[q]):
                if _can_carry(plans[q], needs):
                    j = q
                    break
                q += step
            if j is not None:
                break
        if j is None:
            k += 1
            continue
        if seq.name != "hip_sequence":
            seq = plan_sequence(seq.queue, [seq])
        carrier = plans[j]
        carrier.prelude = (seq.queue.lib.nhip_gemv_tile_carry, tuple(seq.args) + (seq.needs,))
        carrier.full_args = carrier.full_args + (seq,)
        carrier.carried = seq
        carrier.tag = "%s + %s" % (carrier.tag, seq.tag)
        carrier.gsize = (carrier.gsize[0] + seq.gsize[0],)
        if carrier.bw_per_call and seq.bw_per_call:
            carrier.bw_per_call += seq.bw_per_call
        carrier.reads_mem = carrier.reads_mem | seq.reads_mem
        carrier.writes_mem = carrier.writes_mem | seq.writes_mem
        del plans[k]  # (the same index now holds the next plan)
    return plans
