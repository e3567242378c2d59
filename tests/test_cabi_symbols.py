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


def test_gemm_argument_checks_run_before_any_launch():
    """Pointer lists and the addend are validated on the host: these calls return an error without touching a device."""
    from hap_amd._lib import GemmArgs, _load, BF16, F32
    lib = _load()

    def args(**kw):
        a = GemmArgs()
        a.M, a.N, a.K, a.lda, a.ldb, a.ldc = 64, 64, 64, 64, 64, 64
        a.in_dtype, a.out_dtype, a.alpha, a.batch1, a.batch2 = BF16, F32, 1.0, 1, 1
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    ptrs = (ctypes.c_void_p * 17)(*([0x1000] * 17))
    lists = dict(A_list=ctypes.addressof(ptrs), B_list=ctypes.addressof(ptrs), C_list=ctypes.addressof(ptrs))
    cases = {
        b"go together": args(A_list=ctypes.addressof(ptrs), batch1=2),
        b"at most": args(batch1=17, **lists),
        b"must be NULL": args(A=0x1000, batch1=2, **lists),
        b"transA": args(a_rowsum_list=ctypes.addressof(ptrs), batch1=2, **lists),
        b"c_addend": args(A=0x1000, B=0x1000, C=0x1000, c_addend=0x1000),            # without accumulate
        b"null pointer": args(),
    }
    for needle, a in cases.items():
        rc = lib.hapmi_gemm(ctypes.byref(a), None)
        assert rc != 0 and needle in lib.hapmi_last_error(), (needle, rc, lib.hapmi_last_error())


def test_more_host_side_checks_without_a_gpu():
    """Argument checks that return before any device is touched: dropout in the GEMM epilogue refuses operands in
    pieces or with relu on load (it used to launch the piece-reading kernel without the dropout), the plan table knows
    twelve tile configurations, and the embedding backward accepts rows wider than one wave's 2048 columns."""
    from hap_amd._lib import GemmArgs, _load, BF16
    lib = _load()
    a = GemmArgs()
    a.M, a.N, a.K, a.lda, a.ldb, a.ldc = 64, 64, 64, 64, 64, 64
    a.in_dtype, a.out_dtype, a.alpha, a.batch1, a.batch2 = BF16, BF16, 1.0, 1, 1
    a.A, a.B, a.C, a.transA, a.transB = 0x1000, 0x1000, 0x1000, 0, 1
    a.drop_state, a.drop_stream_id, a.drop_p = 0x1000, 3, 0.1
    a.a_relu = 1
    rc = lib.hapmi_gemm(ctypes.byref(a), None)
    assert rc != 0 and b"no relu on an operand" in lib.hapmi_last_error(), lib.hapmi_last_error()

    i64 = ctypes.c_int64
    lib.hapmi_gemm_plan_set.argtypes = [i64, i64, i64, i64] + [ctypes.c_int] * 6
    assert lib.hapmi_gemm_plan_set(64, 64, 64, 1, 0, 1, 1, 1, 11, 1) == 0
    assert lib.hapmi_gemm_plan_set(64, 64, 64, 1, 0, 1, 1, 1, 12, 1) != 0          # no thirteenth configuration
    assert b"out of range" in lib.hapmi_last_error()
    assert lib.hapmi_gemm_plan_clear() == 0

    vp = ctypes.c_void_p
    lib.hapmi_embedding_bwd.argtypes = [vp, vp, vp, i64, i64, i64, ctypes.c_float, ctypes.c_int, vp]
    assert lib.hapmi_embedding_bwd(None, None, None, 0, 3 * 2048 + 8, 100, 1.0, 1, None) == 0    # nothing to do, no limit hit
    assert lib.hapmi_embedding_bwd(None, None, None, 0, 65536 * 2048, 100, 1.0, 1, None) == -5   # HAPMI_ELIMIT
