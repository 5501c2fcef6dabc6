"""The probe drain that allocates nothing (`nhip_probes_drain_static`) against the drain
that takes a caller's workspace (`nhip_probes_drain`), through the C-ABI: the blocks the
two hand to the host must be bit-identical, on two calls in a row of which the second
carries fewer rows, and sizes beyond the static block are refused."""

import ctypes

import numpy as np
import pytest

from helpers import RA, to_dev

pytestmark = pytest.mark.gpu

NHIP_E_TOOBIG = -4
STATIC_WORDS = 1 << 20


def _header(n):
    return (n + 2 + 63) // 64 * 64


class _Probed:
    """Three probed signals of widths 7, 24 and 300 with periods 1, 2.5 and 10 steps, a
    clock, and the tables both drains read."""

    def __init__(self, queue, n_buf):
        import torch

        from nengo_ocl_amd import hipra_nonlinearities as nl
        from nengo_ocl_amd.hipra_nonlinearities import ProbeDrain

        self.queue, self.torch = queue, torch
        self.src = RA([np.zeros(7), np.zeros(24), np.zeros(300), np.zeros(1), np.zeros(1)])
        self.d = to_dev(queue, self.src)
        Yh = RA([np.zeros((n_buf, 7)), np.zeros((n_buf, 24)), np.zeros((n_buf, 300))])
        self.dY = to_dev(queue, Yh)
        self.plan = nl.plan_probes(queue, [1.0, 2.5, 10.0], self.d[[0, 1, 2]], self.dY)
        self.drain = ProbeDrain(queue, self.plan, self.d, 3, 4)
        self.words_max = self.drain.words

    def step(self, rng, n):
        for k in range(n):
            vals = rng.normal(size=self.src.buf.size).astype(np.float32)
            self.d.dev_buf.set(vals)
            self.plan()

    def call(self, static, rows_bound, host):
        dr, p = self.drain, ctypes.c_void_p
        lib = self.queue.lib
        common = (self.queue.handle, dr.table.ptr, dr.n, dr.total_width, dr.max_width,
                  int(rows_bound), self.plan.dev_bufpositions.ptr, self.plan.Y.ptr, self.d.ptr,
                  dr.step_start, dr.time_start)
        if static:
            return lib.nhip_probes_drain_static(*common, p(host.data_ptr()))
        return lib.nhip_probes_drain(*common, p(dr.staging.data_ptr()), dr.words,
                                     p(host.data_ptr()))


def _both(m, rows_bound, marker):
    """Runs the workspace drain, restores the row counts, runs the static drain; returns
    the two host blocks (pinned, prefilled with `marker` beyond what a drain writes)."""
    torch = m.torch
    words = _header(3) + rows_bound * m.drain.total_width
    a = torch.full((words + 64,), marker, dtype=torch.float32).pin_memory()
    b = torch.full((words + 64,), marker, dtype=torch.float32).pin_memory()
    counts = m.plan.dev_bufpositions.get().copy()
    assert m.call(False, rows_bound, a) == 0
    assert not m.plan.dev_bufpositions.get().any()
    m.plan.dev_bufpositions.set(counts)
    assert m.call(True, rows_bound, b) == 0
    assert not m.plan.dev_bufpositions.get().any()
    return a.numpy(), b.numpy(), counts, words


def test_static_drain_equals_workspace_drain(queue, rng):
    m = _Probed(queue, n_buf=64)
    # first call: 50 steps -> 50, 20 and 5 rows; second call: 9 steps -> 9, 4 (or 3) and 1
    for steps, rows_bound, marker in ((50, 64, 7.5), (9, 12, -3.25)):
        m.step(rng, steps)
        a, b, counts, words = _both(m, rows_bound, marker)
        assert counts.max() == steps
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert (b[words:] == marker).all()  # nothing written beyond the block
        # and the block says what the buffers held
        got_counts = b[2:5].view(np.int32)
        assert np.array_equal(got_counts, counts)
        Y = m.dY
        for i in range(3):
            k = int(min(counts[i], rows_bound))
            w = int(m.drain.widths[i])
            at = _header(3) + rows_bound * int(m.drain.wprefix[i])
            assert np.array_equal(b[at:at + k * w].reshape(k, w), np.asarray(Y[i])[:k])
            assert not b[at + k * w:at + rows_bound * w].any()


def test_static_drain_rejects_blocks_beyond_its_array(queue, rng):
    m = _Probed(queue, n_buf=8)
    torch = m.torch
    host = torch.zeros(64, dtype=torch.float32).pin_memory()
    rows = (STATIC_WORDS - _header(3)) // m.drain.total_width + 1
    assert m.call(True, rows, host) == NHIP_E_TOOBIG
