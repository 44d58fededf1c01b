"""The C ABI from a host that is not Python: ``tests/capi_host/host_check.cpp`` allocates its own
device memory with the HIP runtime, calls the library through ``include/steptron_moe.h`` only and
checks route plan, permute, grouped GEMM and the gathered weight gradient against loops on the host.  It is built (by
``__graft_entry__.build()``) as a one-function shared library so that it can run inside this
process; torch does not take part."""

import ctypes
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
LIB = Path(__file__).resolve().parent / "capi_host" / "libstm_host_check.so"


def test_c_host_drives_the_abi_without_torch():
    assert LIB.exists(), f"{LIB} is missing: run __graft_entry__.build() (or python -m steptronoss_amd.build)"
    lib = ctypes.CDLL(str(LIB))
    lib.stm_host_check.restype = ctypes.c_int
    lib.stm_host_check.argtypes = [ctypes.c_char_p, ctypes.c_int]
    msg = ctypes.create_string_buffer(512)
    status = lib.stm_host_check(msg, len(msg))
    assert status == 0, msg.value.decode()
    assert msg.value.decode().startswith("ok")
