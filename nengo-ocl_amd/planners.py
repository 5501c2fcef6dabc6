"""Scheduling of one timestep: dependency graph and greedy grouping.

Counterpart of the reference's ``nengo_ocl/planners.py`` (``greedy_planner``
:9-95).  The reference takes the dependency graph from
``nengo.utils.simulator.operator_dependency_graph`` (third-party nengo); it is
restated here from nengo's documented rule so that the planner also runs on
graphs built without nengo: within one step and one memory block, every set
happens before every increment, sets and increments before every read, and
everything before every update -- also between different views that overlap.

The planner's output is a list of ``(operator type, [operators])`` groups; each
group becomes one (or a few) kernel launches, so the number of groups is the
number of launches per step.
"""

from collections import defaultdict

import numpy as np


def _share(a, b):
    """Do two signals have an element in common?  Views whose bounds overlap are looked at
    exactly: interleaved slices of one vector are disjoint."""
    if a is b:
        return True
    if not a.may_share_memory(b):
        return False
    try:
        return bool(np.shares_memory(a.initial_value, b.initial_value, max_work=100000))
    except Exception:  # too hard to decide, or a signal without a host array
        return True


def operator_dependency_graph(operators):
    """``{op: ops that must run after it}`` for one timestep.  The successors are kept in
    the order the rules below find them (a dict used as an ordered set): a hash-ordered
    set of operator objects would make the order in which operators become ready, and with
    it the order of increments into views that overlap, vary from one run to the next."""
    by_base = defaultdict(lambda: ({}, {}, {}, {}))  # base -> (sets, incs, reads, updates)
    for op in operators:
        for kind, sigs in enumerate((op.sets, op.incs, op.reads, op.updates)):
            for sig in sigs:
                by_base[sig.base][kind].setdefault(sig, []).append(op)

    edges = {op: {} for op in operators}

    def link(pre_table, post_table):
        for post_sig, post_ops in post_table.items():
            for pre_sig, pre_ops in pre_table.items():
                if _share(pre_sig, post_sig):
                    for pre in pre_ops:
                        for post in post_ops:
                            if pre is not post:
                                edges[pre][post] = None

    for sets, incs, reads, updates in by_base.values():
        link(sets, incs)
        link(sets, reads)
        link(incs, reads)
        link(sets, updates)
        link(incs, updates)
        link(reads, updates)
    return edges


def greedy_planner(operators):
    """The reference's rule (planners.py:39-91): among the ready types take the one
    with the most ready operators (ties: the type that became ready last)."""
    return _plan(operators, completing=False)


def batching_planner(operators):
    """Like `greedy_planner`, but a type all of whose remaining operators are ready is
    scheduled first (smallest such type first).

    Taking the largest ready set can split a type into several groups when a few
    of its operators sit behind a small group of another type (ensembles without
    input whose bias copy is the only Copy left, for instance): the large group
    goes first, the stragglers need a second launch of every later type.
    Finishing complete types first removes those splits and never adds a group
    for the type that is completed.  This is the Simulator's default.
    """
    return _plan(operators, completing=True)


def _plan(operators, completing):
    """Group operators by type into as few sequential groups as dependencies and
    write-overlap allow.

    Repeatedly: among operators whose predecessors are all scheduled, take the
    type with the most ready operators (ties: the type that became ready last),
    then greedily pick those of its operators whose written signals (sets
    against sets, incs against incs, updates against updates) do not overlap one
    another; they form one group.  Candidates are visited in the order they
    became ready, which follows the operator list alone, so the result is deterministic.
    """
    edges = operator_dependency_graph(operators)
    n_waiting = {op: 0 for op in operators}
    for op, posts in edges.items():
        for post in posts:
            n_waiting[post] += 1

    ready = {}  # type -> {op: None}, insertion ordered
    for op in operators:
        if n_waiting[op] == 0:
            ready.setdefault(type(op), {})[op] = None

    n_of_type = defaultdict(int)  # operators of each type not yet scheduled
    for op in operators:
        n_of_type[type(op)] += 1

    groups = []
    n_left = len(operators)
    while n_left > 0:
        if not ready:
            raise ValueError("Cycles in the op graph")
        chosen_type = sorted(ready.items(), key=lambda kv: len(kv[1]))[-1][0]
        if completing:
            complete = [t for t, ops in ready.items() if len(ops) == n_of_type[t]]
            if complete:
                chosen_type = min(complete, key=lambda t: n_of_type[t])

        written = (defaultdict(list), defaultdict(list), defaultdict(list))
        chosen = []
        for op in ready[chosen_type]:
            kinds = (op.sets, op.incs, op.updates)
            clash = any(_share(s, s2) for table, sigs in zip(written, kinds)
                        for s in sigs for s2 in table[s.base])
            if not clash:
                chosen.append(op)
                for table, sigs in zip(written, kinds):
                    for s in sigs:
                        table[s.base].append(s)

        assert chosen
        groups.append((chosen_type, chosen))
        for op in chosen:
            del ready[chosen_type][op]
        if not ready[chosen_type]:
            del ready[chosen_type]
        for op in chosen:
            for post in edges[op]:
                n_waiting[post] -= 1
                if n_waiting[post] == 0:
                    ready.setdefault(type(post), {})[post] = None
        n_left -= len(chosen)
        n_of_type[chosen_type] -= len(chosen)

    assert sum(len(ops) for _, ops in groups) == len(operators)
    return groups
