"""ctypes binding of ``libnengo_hip.so`` (the C ABI declared in ``include/nengo_hip.h``).

The library is built in-tree by ``csrc/Makefile`` (``__graft_entry__.build()``
drives it).  There is no fallback: if the shared object is missing or lacks a
symbol, importing a device module raises, and every failed launch raises
``RuntimeError`` with the HIP error string.
"""

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# NENGO_HIP_LIBRARY points at an alternative build of the same ABI (kernel experiments)
LIB_PATH = os.environ.get("NENGO_HIP_LIBRARY") or os.path.join(_HERE, "libnengo_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

c_int = ctypes.c_int
c_void_p = ctypes.c_void_p
c_float = ctypes.c_float
c_double = ctypes.c_double
P = ctypes.c_void_p  # every device pointer crosses the boundary as void*

# name -> argument ctypes (all return int except where noted)
SIGNATURES = {
    "nhip_abi_version": [],
    "nhip_device_info": [P, P, P, ctypes.c_char_p, c_int],
    "nhip_gemv": [P, c_int, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P],
    "nhip_gemv_rows_per_task": [c_int, c_int, c_int, c_int],
    "nhip_gemv_rows_literal": [P, P, P, P, P, c_int, P, P, P, P],
    "nhip_gemv_tile": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P],
    "nhip_gemv_tile_lif": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P,
                           P, ctypes.c_double, c_int, P, P, P, P, P, P],
    "nhip_gemv_tile_lif_sums": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P,
                                P, ctypes.c_double, c_int, P, P, P, P, P, P, P],
    "nhip_gemv_tile_filter": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P, P, P, P],
    "nhip_gemv_tile_filter_learn": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P, P, P, P, P],
    "nhip_gemv_tile_lif_deferred": [P, c_int, c_int, c_int, P, P, P, P, c_int, P, P, P, P,
                                    P, ctypes.c_double, c_int, P, P, P, P, P, P, P, P, P],
    "nhip_gemv_tile_rows": [c_int, c_int],
    "nhip_gemv_rows_lif": [P, c_int, c_int, P, P, P, P, c_int, P, P, P, P,
                           P, ctypes.c_double, c_int, P, P, P, P, P, P],
    "nhip_gemv_rows_lif_sums": [P, c_int, c_int, P, P, P, P, c_int, P, P, P, P,
                                P, ctypes.c_double, c_int, P, P, P, P, P, P, P, P],
    "nhip_gemv_rows_filter": [P, c_int, c_int, P, P, P, P, c_int, P, P, P, P, P, P, P],
    "nhip_gemv_events": [P, P, c_int, P, P, P, P, P, P, c_int],
    "nhip_spmv_sell": [P, P, c_int, P, P, P, P, P],
    "nhip_spmv_sell_skip": [P, P, c_int, P, P, P, P, P, c_int, c_int, P],
    "nhip_spmv_sell_filter": [P, P, c_int, P, P, P, P, P, P, P, P, c_int, c_int, P],
    "nhip_lif": [P, P, c_int, c_double, c_int, P, P, P, P, P, P, P],
    "nhip_lif_rate": [P, P, c_int, P, P, P, P, P],
    "nhip_alif": [P, P, c_int, c_double, c_int, P, P, P, P, P, P, P, P, P, P],
    "nhip_alif_rate": [P, P, c_int, c_double, P, P, P, P, P, P, P, P],
    "nhip_relu": [P, P, c_int, P, P, P],
    "nhip_spiking_relu": [P, P, c_int, c_double, P, P, P, P],
    "nhip_sigmoid": [P, P, c_int, P, P, P],
    "nhip_linearfilter": [P, P, P, c_int, c_int, P, P, P, P, P, P],
    "nhip_elementwise_inc": [P, P, c_int, c_int, P, P, P],
    "nhip_outer_filter": [P, P, c_int, P, P, P, P, P],
    "nhip_learning_rule": [P, c_int, c_int, P, c_int, P, P, P, P, P, P],
    "nhip_conv2d": [P, P, P, P, P],
    "nhip_pool2d": [P, P, P, P],
    "nhip_whitenoise": [P, P, c_int, P, c_double, P],
    "nhip_philox4x32": [P, P, P, c_int],
    "nhip_rtc_compile": [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(c_void_p),
                         ctypes.c_char_p, c_int],
    "nhip_rtc_load": [P, ctypes.c_char_p, ctypes.POINTER(c_void_p)],
    "nhip_rtc_destroy": [P],
    "nhip_rtc_launch_direct": [P, P, c_int, P, P, P, P, P, P],
    "nhip_copy": [P, P, c_int, c_int, P, P],
    "nhip_slicedcopy": [P, P, c_int, c_int, P, P, P, P],
    "nhip_reset": [P, P, c_int, c_int, P],
    "nhip_timeupdate": [P, P, c_int, P, c_int, c_double],
    "nhip_presentinput": [P, P, c_int, c_int, c_float, P, P, P],
    "nhip_direct_unary": [P, c_int, P, c_int, c_int, P, P],
    "nhip_probes": [P, P, c_int, c_int, P, P, P, P, P],
    "nhip_probes_drain": [P, P, c_int, c_int, c_int, c_int, P, P, P, c_int, c_int, P,
                          ctypes.c_longlong, P],
    "nhip_probes_drain_static": [P, P, c_int, c_int, c_int, c_int, P, P, P, c_int, c_int, P],
    "nhip_fill_i32": [P, P, c_int, c_int],
    "nhip_sequence": [P, P, c_int, c_int],
    "nhip_sequence_chains": [P, P, P, P, c_int],
    "nhip_gemv_tile_carry": [P, P, P, c_int, c_int],
    "nhip_capture_begin": [P],
    "nhip_capture_end": [P, ctypes.POINTER(c_void_p)],
    "nhip_graph_upload": [P, P],
    "nhip_graph_launch": [P, P, c_int],
    "nhip_graph_destroy": [P],
    "nhip_stream_sync": [P],
    "nhip_time_next_launch": [P, P],
    "nhip_launch_events_pending": [],
    "nhip_event_create": [ctypes.POINTER(c_void_p)],
    "nhip_event_record": [P, P],
    "nhip_event_elapsed_ms": [P, P, ctypes.POINTER(c_float)],
    "nhip_event_destroy": [P],
    "nhip_calib_stream_mix": [P, P, ctypes.c_longlong, c_int, P, c_int, P, c_int, c_int],
}


class HipError(RuntimeError):
    pass


def build(verbose=False):
    """Compile the HIP sources for gfx950 into ``libnengo_hip.so`` (always recompiles)."""
    cmd = ["make", "-C", CSRC_DIR, "-B", "-j4"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError("building libnengo_hip.so failed (see output above)")
    return LIB_PATH


_lib = None


def lib():
    """The loaded library, with argument types set.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s not found: build it with `python -c 'import __graft_entry__ as g; "
            "g.build()'` or `make -C %s` (no CPU fallback exists)" % (LIB_PATH, CSRC_DIR)
        )
    handle = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(handle, name)  # AttributeError if the symbol is missing
        fn.argtypes = argtypes
        fn.restype = c_int
    handle.nhip_error_string.argtypes = [c_int]
    handle.nhip_error_string.restype = ctypes.c_char_p
    from . import ABI_VERSION

    if handle.nhip_abi_version() != ABI_VERSION:
        raise ImportError("libnengo_hip.so ABI %d != expected %d; rebuild it"
                          % (handle.nhip_abi_version(), ABI_VERSION))
    _lib = handle
    return _lib


def check(err, what=""):
    if err != 0:
        msg = lib().nhip_error_string(err)
        raise HipError("%s failed: %s (code %d)" % (what or "nengo_hip call",
                                                   msg.decode() if msg else "?", err))
