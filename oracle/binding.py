"""ctypes binding of ``libcortex_cpu_oracle.so`` (TEST INFRASTRUCTURE).

The oracle's entry points take the argument lists of ``include/cortex_hip.h``
without the leading stream and with host pointers.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

from cortex_amd import capi

ORACLE_DIR = Path(__file__).resolve().parent
ORACLE_LIB = ORACLE_DIR / "libcortex_cpu_oracle.so"

_DP = C.POINTER(capi.CtDims)


class OracleError(RuntimeError):
    pass


def build(force: bool = False) -> Path:
    """Compiles the oracle with g++ (see ``oracle/Makefile``)."""
    src = ORACLE_DIR / "cortex_cpu_oracle.cpp"
    stale = not ORACLE_LIB.exists() or (src.exists() and ORACLE_LIB.stat().st_mtime < src.stat().st_mtime)
    if force or stale:
        if force and ORACLE_LIB.exists():
            ORACLE_LIB.unlink()
        res = subprocess.run(["make", "-C", str(ORACLE_DIR)], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("oracle build failed:\n" + res.stdout + res.stderr)
    return ORACLE_LIB


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        handle = C.CDLL(str(build()))
        for name, argtypes in capi.PROTOTYPES.items():
            oname = "co_" + name[3:]
            if not hasattr(handle, oname):
                continue
            fn = getattr(handle, oname)
            fn.argtypes = argtypes[1:]  # the oracle takes no stream
            fn.restype = C.c_int
        handle.co_last_error.restype = C.c_char_p
        handle.co_elem_address.argtypes = [C.POINTER(_DP), C.c_int, C.c_int, C.c_int64, C.POINTER(C.c_int64),
                                           C.POINTER(C.c_int)]
        handle.co_elem_address.restype = C.c_int
        handle.co_num_threads.restype = C.c_int
        _lib = handle
    return _lib


def call(name: str, *args) -> None:
    """Calls ``co_<name>`` and raises :class:`OracleError` on failure."""
    handle = lib()
    rc = getattr(handle, "co_" + name)(*args)
    if rc != 0:
        raise OracleError(handle.co_last_error().decode())


def num_threads() -> int:
    return int(lib().co_num_threads())
