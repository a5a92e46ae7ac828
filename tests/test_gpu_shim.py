"""The C++ shim (behemoth-qtip_amd/csrc/quantizer.hpp: the reference's own C++ interface on top of the C ABI)
driven by a C++ caller that mirrors tests/test_gpu.cpp:301-372 of the reference."""
import os
import subprocess

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu


def test_cpp_shim_end_to_end():
    exe = os.path.join(ROOT, "tests", "cpp", "qtip_shim_test")
    assert os.path.exists(exe), "build it with __graft_entry__.build()"
    print("case: qtip_shim_test", flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "SHIM TEST PASSED" in r.stdout
