"""MI355X-native backend for Nengo models behind the ``nengo_ocl`` surface.

``Simulator(network)`` / ``Simulator(None, model=model)``, the ragged-array
signal layout, the ``plan_*`` builders, ``Plan`` / ``Plans`` and ``run_steps`` /
probe semantics follow the reference package (nengo_ocl/__init__.py:1-27
exports ``Simulator``); the kernels behind the ``plan_*`` boundary are
hand-written HIP for gfx950 in ``libnengo_hip.so``.
"""

import logging

from .version import version as __version__

ABI_VERSION = 1  # must equal NHIP_ABI_VERSION in include/nengo_hip.h

logging.getLogger(__name__).addHandler(logging.NullHandler())


def __getattr__(name):
    # the Simulator pulls in the whole host stack; import it on first use
    if name == "Simulator":
        from .simulator import Simulator

        return Simulator
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
