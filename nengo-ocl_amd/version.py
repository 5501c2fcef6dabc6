"""Version of this package and the nengo versions it is written against.

The reference keeps the same facts in nengo_ocl/version.py:20-48 and checks them when a
Simulator is constructed (simulator.py:195-206): versions of nengo it cannot work with are
refused, versions newer than the last one it was tested with get a warning.  This backend
reads operators, signals and processes the way nengo 3.1 lays them out (the reference
requires ``nengo>=3.1.0``, setup.py:31), so everything older is refused.
"""

version_info = (0, 1, 0)
version = ".".join(str(v) for v in version_info)

#: oldest nengo whose builder output this backend understands
minimum_nengo_version_info = (3, 1, 0)
minimum_nengo_version = ".".join(str(v) for v in minimum_nengo_version_info)

#: latest nengo at the time of writing (newer ones get a warning)
latest_nengo_version_info = (3, 1, 0)
latest_nengo_version = ".".join(str(v) for v in latest_nengo_version_info)


def check_nengo_version(nengo_module):
    """Raise for a nengo that is too old, warn for one newer than the tested one.  A module
    without version information passes (nothing to compare)."""
    import warnings

    info = getattr(getattr(nengo_module, "version", None), "version_info", None)
    if info is None:
        return
    info = tuple(info)[:3]
    text = getattr(nengo_module, "__version__", ".".join(str(v) for v in info))
    if info < minimum_nengo_version_info:
        raise ValueError(
            "This simulator does not support Nengo version %s (it needs %s or later). Upgrade "
            "with 'pip install --upgrade --no-deps nengo'." % (text, minimum_nengo_version))
    if info > latest_nengo_version_info:
        warnings.warn(
            "This backend has not been tested with your `nengo` version (%s). The latest "
            "fully supported version is %s" % (text, latest_nengo_version))
