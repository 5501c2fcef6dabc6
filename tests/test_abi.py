"""The C ABI: the library loads and exports every entry point the header declares
(no GPU needed, no compute call is made)."""

import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nengo_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nhip_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for required in ("nhip_gemv", "nhip_lif", "nhip_lif_rate", "nhip_linearfilter",
                     "nhip_elementwise_inc", "nhip_copy", "nhip_slicedcopy", "nhip_reset",
                     "nhip_timeupdate", "nhip_presentinput", "nhip_probes", "nhip_capture_begin",
                     "nhip_graph_launch"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from nengo_ocl_amd import _lib

    assert os.path.exists(_lib.LIB_PATH), "build with __graft_entry__.build()"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), "%s declared in nengo_hip.h but not exported" % name


def test_binding_covers_header_and_versions_match():
    import nengo_ocl_amd
    from nengo_ocl_amd import _lib

    bound = set(_lib.SIGNATURES) | {"nhip_error_string"}
    assert bound == set(declared_symbols())
    lib = _lib.lib()
    assert lib.nhip_abi_version() == nengo_ocl_amd.ABI_VERSION
    assert b"bad argument" in lib.nhip_error_string(-1)
    assert lib.nhip_gemv_rows_per_task(0, 16, 4, 0) == 64
    assert lib.nhip_gemv_rows_per_task(0, 4, 4, 0) == 128
    assert lib.nhip_gemv_rows_per_task(0, 256, 4, 8) == 8
    assert lib.nhip_gemv_rows_per_task(0, 3, 4, 0) == 0


def test_product_does_not_import_the_oracle():
    """Nothing under the package may reach into oracle/ (the checker is not a fallback)."""
    pkg = os.path.join(ROOT, "nengo-ocl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f
                assert "liboracle" not in text, f


def test_no_device_no_fallback():
    """Without a HIP device the device layer raises instead of computing elsewhere."""
    import pytest
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from nengo_ocl_amd.hipraggedarray import Queue

    with pytest.raises(RuntimeError):
        Queue(0)


def test_bench_command_line_contract():
    """`bench.py --gpus N` with N above 1 exits with a message that says why (every box has one
    GPU); `--kernel-hash` prints the hash that `profiles/c3_shared_step.txt` is compared with."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    two = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert two.returncode != 0 and "one GPU" in (two.stdout + two.stderr)
    h = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--kernel-hash"],
                       capture_output=True, text=True, timeout=120)
    words = h.stdout.split()
    assert h.returncode == 0 and words[0] == "kernel_sources_sha256" and len(words[1]) == 64
