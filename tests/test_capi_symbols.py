"""The C-ABI library loads without a GPU and exports every symbol that
include/torchrec_amd.h declares (no compute calls here)."""
import ctypes
import os
import re

from torchrec_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "torchrec_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tra_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    declared = _declared()
    assert declared == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name
    assert _lib.lib().tra_version() >= 1


def test_argument_errors_are_codes_not_crashes():
    l = _lib.lib()
    plan = ctypes.c_void_p()
    bad = (_lib.TableSpec * 1)()
    bad[0].dim, bad[0].dtype, bad[0].row_bytes, bad[0].rows = 6, _lib.INT4, 8, 10  # 6 nibbles: not whole dwords
    ftm = (ctypes.c_int32 * 1)(0)
    rc = l.tra_tbe_create(bad, 1, ftm, None, 1, ctypes.byref(plan))
    assert rc == -1 and b"dim" in l.tra_last_error()
    bad[0].dim, bad[0].dtype = 64, 9
    assert l.tra_tbe_create(bad, 1, ftm, None, 1, ctypes.byref(plan)) == -1
    assert l.tra_tbe_forward(None, None, None, None, 0, None, 1, 0, 0, 0, None, 0, None) == -1
    assert l.tra_cumsum(None, -1, 0, None, None, None) == -1
    assert l.tra_quantize_rows_sbhalf(None, 1, 8, 3, None, None) == -1
    assert l.tra_cumsum_workspace_bytes(10) == 0 and l.tra_cumsum_workspace_bytes(10**6) > 0
