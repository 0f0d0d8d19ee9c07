"""ctypes binding of ``libtorchrec_amd.so`` (the C ABI in include/torchrec_amd.h).

The library is built in-tree by ``torchrec_amd/csrc/Makefile`` (``build()`` in
``__graft_entry__.py`` or ``python -m torchrec_amd.build``).  There is no other
implementation behind these calls: if the library is missing, or there is no
gfx950 device, every entry point here raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtorchrec_amd.so")

# Names every build must export (checked by tests/test_capi_symbols.py).
EXPORTED_SYMBOLS = [
    "tra_version",
    "tra_last_error",
    "tra_device_arch",
    "tra_set_tuning",
    "tra_tbe_create",
    "tra_tbe_destroy",
    "tra_tbe_forward",
    "tra_tbe_forward_lengths_workspace_bytes",
    "tra_tbe_forward_lengths",
    "tra_tbe_forward_lengths_static_max_bytes",
    "tra_tbe_forward_lengths_static",
    "tra_tbe_forward_position_weighted",
    "tra_tbe_launch_info",
    "tra_tbe_set_bounds_check_mode",
    "tra_tbe_error_count",
    "tra_cumsum_workspace_bytes",
    "tra_cumsum",
    "tra_length_per_key",
    "tra_permute_2d_lengths",
    "tra_permute_2d_data",
    "tra_bucketize_workspace_bytes",
    "tra_bucketize_lengths",
    "tra_bucketize_scatter",
    "tra_quantize_rows",
    "tra_quantize_rows_sbhalf",
    "tra_offsets_range",
    "tra_position_weights",
    "tra_mch_remap",
    "tra_mch_remap_keys",
    "tra_regroup_columns",
    "tra_copy_bytes",
]

TRA_OK = 0
FP32, FP16, INT8, INT4, INT2 = 0, 1, 2, 3, 4
POOL_SUM, POOL_MEAN, POOL_NONE = 0, 1, 2


class TableSpec(ctypes.Structure):
    _fields_ = [
        ("offset", ctypes.c_int64),
        ("rows", ctypes.c_int64),
        ("dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("row_bytes", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class TorchrecAmdError(RuntimeError):
    pass


_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The loaded kernel library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TorchrecAmdError(
                f"{LIB_PATH} is missing: build it with `make -C torchrec_amd/csrc` "
                "(hipcc, --offload-arch=gfx950). torchrec_amd has no other backend."
            )
        l = ctypes.CDLL(LIB_PATH)
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
        l.tra_version.restype = ctypes.c_int
        l.tra_last_error.restype = ctypes.c_char_p
        l.tra_device_arch.argtypes = [ctypes.c_char_p, ctypes.c_int]
        l.tra_tbe_create.argtypes = [ctypes.POINTER(TableSpec), i32, ctypes.POINTER(i32), ctypes.POINTER(i32), i32, ctypes.POINTER(vp)]
        l.tra_tbe_destroy.argtypes = [vp]
        l.tra_tbe_forward.argtypes = [vp, vp, vp, vp, i32, vp, i32, i64, i32, i32, vp, i64, vp]
        l.tra_tbe_forward_lengths_workspace_bytes.argtypes = [i32, i32, i32]
        l.tra_tbe_forward_lengths_workspace_bytes.restype = i64
        l.tra_tbe_forward_lengths.argtypes = [vp, vp, vp, vp, i32, vp, i32, i32, i64, i32, i32, vp, i64, vp, vp]
        l.tra_tbe_forward_lengths_static_max_bytes.restype = i64
        l.tra_tbe_forward_lengths_static.argtypes = [vp, vp, vp, vp, i32, vp, i32, i32, i64, i32, i32, vp, i64, vp]
        l.tra_set_tuning.argtypes = [ctypes.c_char_p, i32]
        l.tra_tbe_forward_position_weighted.argtypes = [
            vp, vp, vp, vp, i32, i32, vp, i64, ctypes.POINTER(i32), ctypes.POINTER(i32), i32, i32, i64, i32, i32,
            vp, i64, vp, vp,
        ]
        l.tra_tbe_launch_info.argtypes = [vp, i32, i64, i32, i32, ctypes.c_char_p, i32]
        l.tra_tbe_set_bounds_check_mode.argtypes = [vp, i32]
        l.tra_tbe_error_count.argtypes = [vp, vp, ctypes.POINTER(i64)]
        l.tra_cumsum_workspace_bytes.argtypes = [i64]
        l.tra_cumsum_workspace_bytes.restype = i64
        l.tra_cumsum.argtypes = [vp, i64, i32, vp, vp, vp]
        l.tra_length_per_key.argtypes = [vp, i32, i32, i32, vp, vp]
        l.tra_permute_2d_lengths.argtypes = [vp, i32, i32, i32, vp, i32, vp, vp]
        l.tra_permute_2d_data.argtypes = [vp, i32, i32, vp, vp, i32, vp, i32, vp, vp, vp, vp]
        l.tra_bucketize_workspace_bytes.argtypes = [i32, i32, i32]
        l.tra_bucketize_workspace_bytes.restype = i64
        l.tra_bucketize_lengths.argtypes = [vp, vp, i32, vp, i32, i32, i32, vp, vp]
        l.tra_bucketize_scatter.argtypes = [vp, vp, i32, vp, vp, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp]
        l.tra_quantize_rows.argtypes = [vp, i64, i32, i32, vp, i32, vp]
        l.tra_quantize_rows_sbhalf.argtypes = [vp, i64, i32, i32, vp, vp]
        l.tra_offsets_range.argtypes = [vp, i64, i32, i64, vp, vp]
        l.tra_position_weights.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, vp]
        l.tra_mch_remap.argtypes = [vp, i64, i32, vp, vp, i64, i64, vp, vp]
        l.tra_mch_remap_keys.argtypes = [
            vp, i64, vp, i32, i32, i32, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(i64),
            ctypes.POINTER(i64), vp, vp,
        ]
        l.tra_regroup_columns.argtypes = [
            ctypes.POINTER(vp), ctypes.POINTER(i64), ctypes.POINTER(vp), ctypes.POINTER(i64), ctypes.POINTER(i32),
            i32, i64, i32, vp,
        ]
        l.tra_copy_bytes.argtypes = [vp, vp, i64, vp]
        _lib = l
    return _lib


def forward_lengths_entry():
    """``tra_tbe_forward_lengths`` as a callable of fifteen integers (addresses as ints, ``None`` for
    a null pointer) returning the entry point's code.  The in-tree extension module ``_fastcall``
    (built with the library; it reads the integers straight from the argument vector) when it is
    there, else the ctypes function: the same symbol of the same library either way."""
    l = lib()
    try:
        from torchrec_amd import _fastcall
    except ImportError:
        return l.tra_tbe_forward_lengths
    _fastcall.bind(ctypes.cast(l.tra_tbe_forward_lengths, ctypes.c_void_p).value)
    return _fastcall.forward_lengths


def check(rc: int) -> None:
    if rc != TRA_OK:
        msg = lib().tra_last_error().decode("utf-8", "replace")
        raise TorchrecAmdError(f"torchrec_amd error {rc}: {msg}")


def set_tuning(**knobs: Optional[int]) -> None:
    """Tuning overrides of the lookup (``balanced``, ``window``, ``unroll``, ``lds``, ``xcd``,
    ``cost_floor``, ``fused_scan``, ``cb``, ``fork``); ``None`` restores a knob's default.  For
    experiments and tests: process-wide, and not to be changed while lookups are in flight."""
    for name, value in knobs.items():
        check(lib().tra_set_tuning(name.encode(), -1 if value is None else int(value)))


def require_gpu(t: torch.Tensor, what: str) -> None:
    """The kernels run on MI355X only; there is no host implementation."""
    if t.device.type != "cuda":
        raise TorchrecAmdError(
            f"{what}: tensor is on {t.device}; torchrec_amd runs this on a gfx950 GPU only"
        )


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    """Device address of ``t`` as ctypes takes it for a ``void*`` argument (None = NULL)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> int:
    """The hipStream_t torch currently launches on for ``device`` (as an integer; 0 = null stream)."""
    if _raw_stream is not None:  # no Stream object is built on this route
        idx = device.index if device.index is not None else torch.cuda.current_device()
        return _raw_stream(idx)
    return torch.cuda.current_stream(device).cuda_stream
