"""TEST INFRASTRUCTURE — numpy/ctypes front end of the CPU oracle.

Loads ``libtbe_oracle.so`` (scalar C restatement, ``tbe_oracle.c``) and
``libfbgemm_shim.so`` (the real fbgemm kernels bundled in torch's
``libtorch_cpu.so``, ``fbgemm_shim.cpp``).  Nothing in ``torchrec_amd`` imports
this package: it exists for ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` only.

The packed-store builder below is an independent numpy restatement of the TBE
row layout the reference hands to fbgemm (header-first rows: fp16 scale, fp16
bias, payload, padding to ``row_alignment``; reference call sites
torchrec/quant/embedding_modules.py:273-276, 427-435 and
torch/include/fbgemm/FbgemmEmbedding.h:147-150).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

FP32, FP16, INT8, INT4, INT2 = 0, 1, 2, 3, 4
SUM, MEAN, NONE = 0, 1, 2
BITS = {FP32: 32, FP16: 16, INT8: 8, INT4: 4, INT2: 2}

_c_lib = None
_fb_lib = None


def build() -> None:
    """(Re)compile both oracle libraries with the Makefile next to this file."""
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)


def _load(name: str) -> ctypes.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        subprocess.run(["make", "-C", _HERE, name], check=True, capture_output=True)
    return ctypes.CDLL(path)


def c_lib() -> ctypes.CDLL:
    global _c_lib
    if _c_lib is None:
        lib = _load("libtbe_oracle.so")
        lib.oracle_tbe_forward.restype = ctypes.c_int64
        lib.oracle_permute_2d.restype = ctypes.c_int64
        lib.oracle_bucketize.restype = ctypes.c_int64
        lib.oracle_quantize_sbhalf.restype = ctypes.c_int
        lib.oracle_float_to_half.restype = ctypes.c_uint16
        lib.oracle_float_to_half.argtypes = [ctypes.c_float]
        lib.oracle_half_to_float.restype = ctypes.c_float
        lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        _c_lib = lib
    return _c_lib


def fbgemm_lib() -> ctypes.CDLL:
    global _fb_lib
    if _fb_lib is None:
        import torch  # noqa: F401  (makes libtorch_cpu.so resolvable)

        lib = _load("libfbgemm_shim.so")
        lib.fbgemm_tbe_forward.restype = ctypes.c_int64
        _fb_lib = lib
    return _fb_lib


def _p(a: Optional[np.ndarray]) -> ctypes.c_void_p:
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


# --------------------------------------------------------------------------
# quantization
# --------------------------------------------------------------------------
def quantize_sbhalf(w: np.ndarray, bits: int, impl: str = "c") -> np.ndarray:
    """fp32 [rows, D] -> uint8 [rows, D*bits/8 + 4] (payload, fp16 scale, fp16 bias)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, cols = w.shape
    out = np.zeros((rows, cols * bits // 8 + 4), dtype=np.uint8)
    if impl == "c":
        rc = c_lib().oracle_quantize_sbhalf(
            ctypes.c_int(bits), _p(w), ctypes.c_int64(rows), ctypes.c_int(cols), _p(out)
        )
        assert rc == 0, rc
    else:
        fbgemm_lib().fbgemm_quantize_sbhalf(
            ctypes.c_int(bits),
            _p(w),
            ctypes.c_int64(rows),
            ctypes.c_int(cols),
            _p(out),
            ctypes.c_int(1 if impl == "fbgemm_ref" else 0),
        )
    return out


# --------------------------------------------------------------------------
# packed TBE store
# --------------------------------------------------------------------------
def round_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


def row_bytes(dim: int, dtype: int, row_alignment: int) -> int:
    payload = dim * BITS[dtype] // 8
    header = 4 if dtype in (INT8, INT4, INT2) else 0
    return round_up(payload + header, row_alignment)


@dataclass
class Store:
    weights: np.ndarray  # uint8 flat
    table_offsets: np.ndarray  # int64 [T]
    table_rows: np.ndarray  # int64 [T]
    table_dims: np.ndarray  # int32 [T]
    table_dtypes: np.ndarray  # int32 [T]
    table_row_bytes: np.ndarray  # int32 [T]


def pack_store(
    tables: Sequence[Tuple[int, int, np.ndarray]],
    row_alignment: int = 16,
    table_alignment: int = 128,
) -> Store:
    """tables: (dtype, dim, data) where data is the fbgemm trailer-format uint8
    [rows, payload+4] for INT8/4/2, or a float16 / float32 [rows, dim] array."""
    offs, rows_l, dims, dts, rbs = [], [], [], [], []
    total = 0
    for dtype, dim, data in tables:
        rb = row_bytes(dim, dtype, row_alignment)
        offs.append(total)
        rows_l.append(data.shape[0])
        dims.append(dim)
        dts.append(dtype)
        rbs.append(rb)
        total = round_up(total + rb * data.shape[0], table_alignment)
    w = np.zeros(max(total, 1), dtype=np.uint8)
    for (dtype, dim, data), off, rb in zip(tables, offs, rbs):
        n = data.shape[0]
        view = w[off : off + n * rb].reshape(n, rb)
        if dtype in (INT8, INT4, INT2):
            payload = dim * BITS[dtype] // 8
            assert data.dtype == np.uint8 and data.shape[1] == payload + 4
            view[:, 0:4] = data[:, payload : payload + 4]
            view[:, 4 : 4 + payload] = data[:, :payload]
        elif dtype == FP16:
            view[:, : 2 * dim] = np.ascontiguousarray(data, dtype=np.float16).view(np.uint8)
        else:
            view[:, : 4 * dim] = np.ascontiguousarray(data, dtype=np.float32).view(np.uint8)
    return Store(
        w,
        np.asarray(offs, dtype=np.int64),
        np.asarray(rows_l, dtype=np.int64),
        np.asarray(dims, dtype=np.int32),
        np.asarray(dts, dtype=np.int32),
        np.asarray(rbs, dtype=np.int32),
    )


def tbe_forward(
    store: Store,
    feature_table_map: Sequence[int],
    B: int,
    indices: np.ndarray,
    offsets: np.ndarray,
    per_sample_weights: Optional[np.ndarray],
    pooling: int,
    out_dtype: int,
    impl: str = "c",
    nthreads: int = 1,
) -> np.ndarray:
    ftm = np.asarray(feature_table_map, dtype=np.int32)
    F = len(ftm)
    dims = store.table_dims[ftm]
    D_offsets = np.zeros(F + 1, dtype=np.int32)
    D_offsets[1:] = np.cumsum(dims)
    assert indices.dtype == offsets.dtype and indices.dtype in (np.int32, np.int64)
    is64 = int(indices.dtype == np.int64)
    indices = np.ascontiguousarray(indices)
    offsets = np.ascontiguousarray(offsets)
    assert offsets.shape[0] == F * B + 1
    L = int(offsets[-1])
    np_out = np.float32 if out_dtype == FP32 else np.float16
    if pooling == NONE:
        assert len(set(dims.tolist())) <= 1
        out = np.zeros((L, int(dims[0]) if F else 0), dtype=np_out)
    else:
        out = np.zeros((B, int(D_offsets[-1])), dtype=np_out)
    psw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=np.float32)
    args = [
        _p(store.weights),
        ctypes.c_int32(len(store.table_rows)),
        _p(store.table_offsets),
        _p(store.table_rows),
        _p(store.table_dims),
        _p(store.table_dtypes),
        _p(store.table_row_bytes),
        ctypes.c_int32(F),
        _p(ftm),
        _p(D_offsets),
        ctypes.c_int32(B),
        _p(indices),
        _p(offsets),
        ctypes.c_int32(is64),
        _p(psw),
        ctypes.c_int32(pooling),
        ctypes.c_int32(out_dtype),
        _p(out),
    ]
    if impl == "c":
        rc = c_lib().oracle_tbe_forward(*args)
    else:
        rc = fbgemm_lib().fbgemm_tbe_forward(*args, ctypes.c_int32(nthreads))
    if rc != 0:
        raise IndexError(f"embedding index out of range (oracle status {rc})")
    return out


# --------------------------------------------------------------------------
# index math
# --------------------------------------------------------------------------
def bounds_check_indices(rows_per_feature: Sequence[int], B: int, indices: np.ndarray, offsets: np.ndarray,
                         mode: str) -> Tuple[np.ndarray, int]:
    """What fbgemm_gpu's ``bounds_check_indices`` leaves of the ids before the lookup runs: in the
    WARNING and IGNORE modes an id outside [0, rows) of its feature's table, other than the pruned
    id -1, is rewritten to 0 (``"NONE"``: ids untouched).  Returns (ids, number of such ids).
    PARITY UNPINNED: fbgemm_gpu (unpinned dependency of the reference, requirements.txt:4) is not
    in this image and the reference holds no fixture for out-of-range ids; this restates the
    operator's documented behaviour at the call site that selects the mode
    (torchrec/distributed/quant_embedding_kernel.py:337-339).  Offsets are taken as valid."""
    ids = np.array(indices, copy=True)
    bad_total = 0
    for f, rows in enumerate(rows_per_feature):
        lo, hi = int(offsets[f * B]), int(offsets[(f + 1) * B])
        seg = ids[lo:hi]
        bad = ((seg < 0) | (seg >= rows)) & (seg != -1)
        bad_total += int(bad.sum())
        if mode in ("WARNING", "IGNORE"):
            seg[bad] = 0
    return ids, bad_total


def cumsum(lengths: np.ndarray) -> np.ndarray:
    lengths = np.ascontiguousarray(lengths)
    out = np.zeros(lengths.shape[0] + 1, dtype=lengths.dtype)
    c_lib().oracle_cumsum(
        _p(lengths), ctypes.c_int64(lengths.shape[0]), ctypes.c_int(lengths.dtype == np.int64), _p(out)
    )
    return out


def permute_2d(
    permute: Sequence[int],
    lengths: np.ndarray,  # [T, B]
    values: np.ndarray,
    weights: Optional[np.ndarray] = None,
) -> Tuple[np.ndarray, np.ndarray, Optional[np.ndarray]]:
    perm = np.asarray(permute, dtype=np.int32)
    lengths = np.ascontiguousarray(lengths)
    T, B = lengths.shape
    values = np.ascontiguousarray(values)
    per_feature = lengths.sum(axis=1)
    total = int(per_feature[perm].sum()) if len(perm) else 0
    out_l = np.zeros((len(perm), B), dtype=lengths.dtype)
    out_v = np.zeros(total, dtype=values.dtype)
    w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32)
    out_w = None if w is None else np.zeros(total, dtype=np.float32)
    n = c_lib().oracle_permute_2d(
        _p(perm),
        ctypes.c_int32(len(perm)),
        ctypes.c_int32(T),
        ctypes.c_int32(B),
        _p(lengths),
        ctypes.c_int(lengths.dtype == np.int64),
        _p(values),
        ctypes.c_int(values.dtype.itemsize),
        _p(w),
        _p(out_l),
        _p(out_v),
        _p(out_w),
    )
    assert n == total
    return out_l, out_v, out_w


def bucketize(
    lengths: np.ndarray,  # [F*B]
    indices: np.ndarray,
    block_sizes: Sequence[int],  # [F]
    W: int,
    weights: Optional[np.ndarray] = None,
    keep_orig_idx: bool = False,
    return_permute: bool = False,
):
    lengths = np.ascontiguousarray(lengths)
    indices = np.ascontiguousarray(indices)
    assert lengths.dtype == indices.dtype
    F = len(block_sizes)
    B = lengths.shape[0] // F if F else 0
    bs = np.asarray(block_sizes, dtype=np.int64)
    new_l = np.zeros(W * F * B, dtype=lengths.dtype)
    new_i = np.zeros(indices.shape[0], dtype=indices.dtype)
    w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32)
    new_w = None if w is None else np.zeros(indices.shape[0], dtype=np.float32)
    perm = np.zeros(indices.shape[0], dtype=np.int64) if return_permute else None
    scratch = np.zeros(W * F * B + 1, dtype=np.int64)
    n = c_lib().oracle_bucketize(
        _p(lengths),
        _p(indices),
        ctypes.c_int(lengths.dtype == np.int64),
        _p(w),
        _p(bs),
        ctypes.c_int32(F),
        ctypes.c_int32(B),
        ctypes.c_int32(W),
        ctypes.c_int(int(keep_orig_idx)),
        _p(new_l),
        _p(new_i),
        _p(new_w),
        _p(perm),
        _p(scratch),
    )
    new_i = new_i[:n]
    if new_w is not None:
        new_w = new_w[:n]
    return new_l, new_i, new_w, perm
