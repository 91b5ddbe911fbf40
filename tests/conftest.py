import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; calls the HIP path through the C ABI")


@pytest.fixture(scope="session")
def ox():
    import oracle
    return oracle.load()


@pytest.fixture(scope="session")
def kxlib():
    """libkx.so on a machine with a GPU; fails (does not skip) when the library is missing."""
    import ctypes as C
    from blok_amd.lib import kx
    lib = kx()
    name = C.create_string_buffer(256)
    cus = C.c_int32()
    hbm = C.c_uint64()
    rc = lib.kx_device_info(name, 256, C.byref(cus), C.byref(hbm))
    if rc != 0:
        pytest.fail("no usable GPU: " + lib.kx_last_error().decode())
    print(f"\n[kx] device {name.value.decode()} CUs={cus.value} HBM={hbm.value / 1e9:.1f} GB", flush=True)
    return lib
