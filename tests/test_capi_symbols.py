"""The C-ABI library loads and exports every symbol include/cortex_hip.h
declares (no compute calls: this runs without a GPU)."""
import ctypes
import re
from pathlib import Path

from cortex_amd import capi

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "cortex_hip.h"


def declared_symbols():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ct_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_hot_path():
    names = declared_symbols()
    for required in ["ct_assign", "ct_assign_constant", "ct_unary_op", "ct_unary_accum", "ct_binary_op",
                     "ct_binary_op_constant", "ct_binary_accum", "ct_binary_accum_constant", "ct_ternary_op",
                     "ct_ternary_op_constant", "ct_ternary_op_constant_constant", "ct_unary_reduce", "ct_adam_step",
                     "ct_adadelta_step", "ct_memset", "ct_memcpy_async", "ct_last_error"]:
        assert required in names


def test_library_exports_every_declared_symbol():
    assert capi.LIB_PATH.exists(), "libcortex_hip.so has not been built (python -m cortex_amd.build)"
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_python_prototypes_cover_the_header():
    declared = set(declared_symbols())
    bound = set(capi.PROTOTYPES) | set(capi.STRING_FUNCTIONS)
    assert declared == bound, (declared - bound, bound - declared)


def test_error_reporting_without_a_device():
    # argument validation happens on the host before any device call
    lib = capi.load_library()
    rc = lib.ct_memcpy_async(None, None, 16, 99, None)
    assert rc != 0
    assert b"null pointer" in lib.ct_last_error() or b"unknown copy kind" in lib.ct_last_error()
    rc = lib.ct_memset(None, None, capi.F32, 0.0, -1)
    assert rc == 1 and b"negative" in lib.ct_last_error()
