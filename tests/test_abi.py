"""The C-ABI library loads without a GPU and exports every symbol include/fp6m.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fp6m.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp6m_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    import fp6_marlin
    names = _declared()
    assert "fp6m_mul" in names and len(names) >= 12
    lib = ctypes.CDLL(fp6_marlin.cabi.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), name


def test_argument_validation_needs_no_gpu():
    import fp6_marlin
    L = fp6_marlin.cabi.lib
    assert L.fp6m_abi_version() == 1
    assert L.fp6m_workspace_elems(4096, 16) == 512
    assert fp6_marlin.cabi.strerror(1).startswith("problem shape")
    z = ctypes.c_void_p(0)
    # shape errors are decided before any pointer or device is touched (fp6_marlin_cuda_kernel.cu:904-907)
    assert L.fp6m_mul(z, z, z, z, 16, 256, 64, z, 0, z, 128, 128, -1, 16, -1, -1) == 1    # k % thread_k
    assert L.fp6m_mul(z, z, z, z, 16, 256, 256, z, 0, z, 256, 256, -1, 16, -1, -1) == 2   # no such kernel
    assert L.fp6m_mul(z, z, z, z, 32, 256, 256, z, 0, z, 128, 128, -1, 16, -1, -1) == 2   # (128,128) needs m <= 16
    assert L.fp6m_mul(z, z, z, z, 0, 256, 256, z, 0, z, -1, -1, -1, 16, -1, -1) == 0      # empty problem
    assert L.fp6m_mul(z, z, z, z, 16, 256, 256, z, 0, z, -1, -1, -1, 16, -1, -1) == 5     # null pointers
