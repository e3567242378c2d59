"""ctypes binding of libhapmi.so.  There is no fallback: if the library is
missing or a call fails, an exception is raised."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "libhapmi.so")
_lib = None

F32, BF16 = 0, 1
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SIGMOID = 0, 1, 2, 3
MAX_RANKS = 64
GEMM_MAX_LIST = 16


class HapmiError(RuntimeError):
    pass


GEMM_MAX_SEGMENTS = 8


class GemmSegments(ctypes.Structure):
    _fields_ = [("n", ctypes.c_int), ("begin", ctypes.c_int64 * (GEMM_MAX_SEGMENTS + 1)),
                ("ld", ctypes.c_int64 * GEMM_MAX_SEGMENTS), ("base", ctypes.c_void_p * GEMM_MAX_SEGMENTS)]


class GemmArgs(ctypes.Structure):
    _fields_ = [
        ("A", ctypes.c_void_p), ("B", ctypes.c_void_p), ("C", ctypes.c_void_p), ("bias", ctypes.c_void_p),
        ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
        ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64),
        ("transA", ctypes.c_int), ("transB", ctypes.c_int),
        ("in_dtype", ctypes.c_int), ("out_dtype", ctypes.c_int),
        ("accumulate", ctypes.c_int), ("act", ctypes.c_int),
        ("alpha", ctypes.c_float),
        ("batch1", ctypes.c_int64), ("batch2", ctypes.c_int64),
        ("strideA1", ctypes.c_int64), ("strideA2", ctypes.c_int64),
        ("strideB1", ctypes.c_int64), ("strideB2", ctypes.c_int64),
        ("strideC1", ctypes.c_int64), ("strideC2", ctypes.c_int64),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("a_rowsum", ctypes.c_void_p),
        ("c_relu_mask", ctypes.c_void_p),
        ("c_addend", ctypes.c_void_p),
        ("A_list", ctypes.c_void_p), ("B_list", ctypes.c_void_p), ("C_list", ctypes.c_void_p),
        ("a_rowsum_list", ctypes.c_void_p),
        ("A_segments", ctypes.c_void_p), ("B_segments", ctypes.c_void_p), ("C_segments", ctypes.c_void_p),
        ("c_mask_segments", ctypes.c_void_p), ("B_segments_list", ctypes.c_void_p),
        ("a_relu", ctypes.c_int), ("b_relu", ctypes.c_int),
        ("drop_state", ctypes.c_void_p), ("drop_stream_id", ctypes.c_int64), ("drop_p", ctypes.c_float),
    ]


_HEADER = os.path.join(_HERE, "..", "include", "hapmi.h")
_SCALARS = {"int64_t": ctypes.c_int64, "int": ctypes.c_int, "float": ctypes.c_float, "double": ctypes.c_double,
            "hapmi_stream_t": ctypes.c_void_p}


def _prototypes():
    """(name, [ctypes argument types]) for every ``int hapmi_*(...)`` declared in include/hapmi.h.  Without
    explicit argument types ctypes would pass Python ints as 32-bit C ints, which is wrong for the int64_t
    parameters (those that travel on the stack keep garbage in their upper half)."""
    import re
    text = open(_HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = []
    for m in re.finditer(r"\bint\s+(hapmi_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        name, params = m.group(1), m.group(2).strip()
        types = []
        if params and params != "void":
            for prm in params.split(","):
                prm = " ".join(prm.split())
                if "*" in prm:
                    types.append(ctypes.c_void_p)
                else:
                    base = prm.rsplit(" ", 1)[0].replace("const ", "").strip()
                    types.append(_SCALARS[base])
        out.append((name, types))
    return out


class _Recorder:
    """Stands in for the library while a launch list is being recorded: every entry point behaves as usual and
    a successful call is appended to the list as (ctypes function, argument tuple).  The tuple keeps the
    argument blocks and host arrays of the call alive, so the list can be replayed call by call."""

    def __init__(self, handle, log):
        self._handle, self._log, self._wrapped = handle, log, {}

    def __getattr__(self, name):
        w = self._wrapped.get(name)
        if w is None:
            fn, log = getattr(self._handle, name), self._log

            def w(*args):
                rc = fn(*args)
                if rc == 0 and fn.restype is ctypes.c_int:
                    log.append((fn, args))
                return rc
            self._wrapped[name] = w
        return w


_recorder = None


def start_recording() -> None:
    """Record every library call made through ``lib()`` until ``stop_recording``."""
    global _recorder
    if _recorder is not None:
        raise HapmiError("a launch list is already being recorded")
    _recorder = _Recorder(_load(), [])


def stop_recording():
    global _recorder
    rec, _recorder = _recorder, None
    return rec._log if rec is not None else []


def host_call(fn) -> None:
    """Run ``fn()`` now and, while a launch list is being recorded, put it into the list as well: stream
    forks / joins (event record and wait) between the library calls of a phase replay in their place."""
    fn()
    if _recorder is not None:
        _recorder._log.append((fn, ()))


def replay(calls) -> None:
    for fn, args in calls:
        rc = fn(*args)
        if isinstance(rc, int) and rc != 0:                      # host calls (stream forks / joins) return nothing
            raise HapmiError(f"libhapmi error {rc} in {fn.__name__}: {_load().hapmi_last_error().decode()}")


def lib():
    return _recorder if _recorder is not None else _load()


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            raise HapmiError(f"{_PATH} is missing: build it with `python -m hap_amd.build` "
                             "(there is no fallback path)")
        handle = ctypes.CDLL(_PATH)
        handle.hapmi_last_error.restype = ctypes.c_char_p
        for name, types in _prototypes():
            fn = getattr(handle, name)
            fn.argtypes = types
            fn.restype = ctypes.c_int
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise HapmiError(f"libhapmi error {rc}: {_load().hapmi_last_error().decode()}")
