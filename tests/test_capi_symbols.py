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


def test_more_argument_errors():
    """Entry points added after the first set: null and inconsistent arguments
    come back as codes with a message, before anything touches a device."""
    l = _lib.lib()
    i32, i64 = ctypes.c_int32, ctypes.c_int64
    # lengths entry
    assert l.tra_tbe_forward_lengths(None, None, None, None, 0, None, 1, 1, 0, 0, 0, None, 0, None, None) == -1
    assert b"null plan" in l.tra_last_error()
    ws = l.tra_tbe_forward_lengths_workspace_bytes
    assert ws(-1, 4, 0) == 0 and ws(26, 2048, 0) >= (26 * 2048 + 1) * 4 and ws(26, 2048, 1) > ws(26, 2048, 0)
    # position-weighted entry: the weight description is checked first
    one = (i32 * 1)(0)
    assert l.tra_tbe_forward_position_weighted(None, None, None, None, 0, 0, None, 0, one, one, 1, 1, 0, 0, 0,
                                               None, 0, None, None) == -1
    assert b"position weight" in l.tra_last_error()
    # per-key remap
    assert l.tra_mch_remap_keys(None, -1, None, 0, 1, 1, None, None, None, None, None, None) == -1
    assert l.tra_mch_remap_keys(None, 0, None, 0, 1, 1, None, None, None, None, None, None) == 0  # nothing to do
    assert l.tra_mch_remap_keys(None, 5, None, 0, 1, 1, None, None, None, None, None, None) == -1
    # copy: sizes and pointers in 16-byte units
    assert l.tra_copy_bytes(None, None, 24, None) == -1 and l.tra_copy_bytes(None, None, 0, None) == 0
    # launch description needs a plan and a buffer
    assert l.tra_tbe_launch_info(None, 1, 1, 0, 0, None, 0) == -1
    n = i64(0)
    assert l.tra_tbe_error_count(None, None, ctypes.byref(n)) == -1


def test_fastcall_module_binds_the_same_entry_point():
    """The extension module in front of tra_tbe_forward_lengths: built with the library, takes the
    entry point's address from Python, and refuses anything but fifteen integer arguments.  (No
    compute call here: that needs a GPU.)"""
    import ctypes

    from torchrec_amd import _fastcall

    lib = _lib.lib()
    address = ctypes.cast(lib.tra_tbe_forward_lengths, ctypes.c_void_p).value
    assert address
    fn = _lib.forward_lengths_entry()
    assert fn is _fastcall.forward_lengths
    import pytest

    with pytest.raises(TypeError):
        fn(1, 2, 3)
    with pytest.raises(TypeError):
        fn(*(["x"] * 15))
    # a null plan is refused by the entry point itself, with its usual code and message
    rc = fn(None, None, None, None, 0, None, 1, 1, 0, _lib.POOL_SUM, _lib.FP16, None, 0, None, None)
    assert rc < 0 and b"null plan" in lib.tra_last_error()
