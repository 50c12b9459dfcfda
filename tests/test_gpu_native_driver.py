"""Runs the native C++ driver of the C ABI (tests/native/packdecode_driver.cpp) on the GPU.

The driver uses nothing but include/bitdecode.h, the HIP runtime and the C restatement of the oracle;
it is the counterpart of the reference's libtorch drivers test_single_packdecode.cu /
test_batch_packdecode.cu.  It is called in-process through its shared-library build."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_native_driver_passes_every_case(device):
    drv = os.path.join(_ROOT, "tests", "native", "libpackdecode_driver.so")
    lib = os.path.join(_ROOT, "bitladder_amd", "libbitdecode.so")
    ora = os.path.join(_ROOT, "oracle", "liboracle_c.so")
    for p in (drv, lib, ora):
        assert os.path.exists(p), f"{p} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`"
    run = ctypes.CDLL(drv).packdecode_driver_run
    run.restype = ctypes.c_int
    run.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    assert run(lib.encode(), ora.encode()) == 0
