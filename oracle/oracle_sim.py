"""The Simulator run on the CPU oracle.  TEST INFRASTRUCTURE ONLY.

``OracleSimulator`` is the product Simulator with the device side of the
``plan_*`` boundary replaced by `oracle.oracle` (host ragged arrays, C kernels):
same operator graph, same planner, same plan sequence, same probe logic, so a
difference between the two is a difference below the boundary.  Used by
``tests/`` and by ``bench.py``'s cpu_baseline leg; never by the product.
"""

import re

import numpy as np

from nengo_ocl_amd.simulator import Simulator

from . import oracle

_DIRECT_RE = re.compile(r"^\s*OUTPUT__\[0\]\s*=\s*([a-z]+)\(\s*(\w+)\[0\]\s*\)\s*;\s*$")


class OracleBackend:
    name = "oracle"
    queue = None

    def __init__(self):
        for name in ("plan_timeupdate", "plan_reset", "plan_copy", "plan_slicedcopy",
                     "plan_elementwise_inc", "plan_linearfilter", "plan_lif", "plan_lif_rate",
                     "plan_presentinput", "plan_block_gemv", "plan_rectified_linear",
                     "plan_spiking_rectified_linear", "plan_sigmoid", "plan_sparse_dot_inc",
                     "plan_bcm", "plan_oja", "plan_voja", "plan_conv2d", "plan_pool2d",
                     "plan_whitenoise"):
            setattr(self, name, getattr(oracle, name))

    @staticmethod
    def plan_probes(queue, periods, X, Y, tag=None):
        plan = oracle.plan_probes(queue, periods, X, Y, tag=tag)
        plan.dev_bufpositions = plan.bufpositions
        plan.dev_countdowns = plan.countdowns
        return plan

    @staticmethod
    def plan_direct(queue, code, init, input_names, inputs, output, tag=None):
        m = _DIRECT_RE.match(code or "")
        if m is None or m.group(1) not in oracle.UNARY_OPCODES:
            raise NotImplementedError(code)
        x = inputs[list(input_names).index(m.group(2))]
        return oracle.plan_direct_unary(queue, m.group(1), x, output, tag=tag)

    # host arrays stand in for device arrays
    def upload(self, host_ragged):
        return host_ragged

    def array(self, values, dtype=np.float32):
        return np.asarray(values, dtype=dtype)

    def finish(self):
        pass

    def read_rows(self, ragged, i, n_rows):
        return np.array(ragged[i][:n_rows])

    def write_all(self, ragged, host_buf):
        ragged.buf[...] = host_buf

    def get_array(self, arr):
        return np.array(arr)

    def fill_array(self, arr, value):
        arr[...] = value

    def set_array(self, arr, values):
        arr[...] = values


class OracleSimulator(Simulator):
    def __init__(self, network, **kwargs):
        kwargs.setdefault("backend", OracleBackend())
        kwargs.setdefault("use_graph", False)
        super().__init__(network, **kwargs)
