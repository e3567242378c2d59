"""The shared library loads and exports every entry point that include/hapmi.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hapmi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hapmi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(os.path.join(ROOT, "hap_amd", "libhapmi.so"))
    names = declared_symbols()
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_host_only_entry_points_work_without_a_gpu():
    lib = ctypes.CDLL(os.path.join(ROOT, "hap_amd", "libhapmi.so"))
    assert lib.hapmi_version() >= 1
    lib.hapmi_last_error.restype = ctypes.c_char_p
    out = (ctypes.c_int64 * 2)()
    rc = lib.hapmi_sharding_round(ctypes.c_int64(10), (ctypes.c_double * 2)(0.9, 0.9), ctypes.c_int64(2), out)
    assert rc == -1 and b"sharding_round" in lib.hapmi_last_error()


def test_product_refuses_cpu_tensors():
    import pytest
    import torch
    from hap_amd import ops
    from hap_amd._lib import HapmiError
    with pytest.raises(HapmiError):
        ops.add(torch.ones(4), torch.ones(4), torch.ones(4))
