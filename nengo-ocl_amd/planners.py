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


def _share(a, b):
    return a is b or a.may_share_memory(b)


def operator_dependency_graph(operators):
    """``{op: set of ops that must run after it}`` for one timestep."""
    by_base = defaultdict(lambda: ({}, {}, {}, {}))  # base -> (sets, incs, reads, updates)
    for op in operators:
        for kind, sigs in enumerate((op.sets, op.incs, op.reads, op.updates)):
            for sig in sigs:
                by_base[sig.base][kind].setdefault(sig, []).append(op)

    edges = {op: set() for op in operators}

    def link(pre_table, post_table):
        for post_sig, post_ops in post_table.items():
            for pre_sig, pre_ops in pre_table.items():
                if _share(pre_sig, post_sig):
                    for pre in pre_ops:
                        for post in post_ops:
                            if pre is not post:
                                edges[pre].add(post)

    for sets, incs, reads, updates in by_base.values():
        link(sets, incs)
        link(sets, reads)
        link(incs, reads)
        link(sets, updates)
        link(incs, updates)
        link(reads, updates)
    return edges


def greedy_planner(operators):
    """Group operators by type into as few sequential groups as dependencies and
    write-overlap allow.

    Repeatedly: among operators whose predecessors are all scheduled, take the
    type with the most ready operators (ties: the type that became ready last),
    then greedily pick those of its operators whose written signals (sets
    against sets, incs against incs, updates against updates) do not overlap one
    another; they form one group.  Candidates are visited in the order they
    became ready, so the result is deterministic.
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

    groups = []
    n_left = len(operators)
    while n_left > 0:
        if not ready:
            raise ValueError("Cycles in the op graph")
        chosen_type = sorted(ready.items(), key=lambda kv: len(kv[1]))[-1][0]

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

    assert sum(len(ops) for _, ops in groups) == len(operators)
    return groups
