"""Runs the C++ host-layer test program (tests/host/host_tests.cpp): the add-on's DeviceInterface,
Search and BatchedSampler objects driven through the reference's virtual interface, checked against
the CPU oracle.  The program is built on the CPU (tests/host/Makefile) and only executed here."""
import ctypes
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
BIN = os.path.join(HERE, "host", "host_tests.bin")
ADDON = os.path.join(ROOT, "onnxruntime-genai_amd", "libmi355x_genai_hip.so")


def test_addon_exports_loader_entry_points():
    """The two symbols the reference's loader resolves (src/generators.cpp:321-356) exist and the
    version matches kDeviceInterfaceVersion (src/smartptrs.h:171).  No GPU call is made."""
    if not os.path.exists(ADDON):
        pytest.fail("add-on library not built: run `python __graft_entry__.py`")
    lib = ctypes.CDLL(ADDON)
    lib.GetInterfaceVersion.restype = ctypes.c_uint32
    assert lib.GetInterfaceVersion() == 1
    assert hasattr(lib, "GetInterface")


@pytest.mark.gpu
def test_host_layer_program():
    if not os.path.exists(BIN):
        pytest.fail("tests/host/host_tests.bin not built: run `python __graft_entry__.py`")
    print("running", BIN, flush=True)
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=110)
    print(proc.stdout[-6000:])
    print(proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert " 0 failed" in proc.stdout
