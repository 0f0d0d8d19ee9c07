"""Shared builders for the parity tests: the same seeded tables and ids are
handed to the HIP path (torch tensors) and to the CPU oracle (numpy)."""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np

import oracle as O

SPARSE_NAMES = {O.FP32: "FP32", O.FP16: "FP16", O.INT8: "INT8", O.INT4: "INT4", O.INT2: "INT2"}


def make_table(rng: np.random.Generator, dtype: int, rows: int, dim: int) -> np.ndarray:
    """Oracle-side table data: fbgemm trailer rows for int types, else a float array."""
    w = rng.normal(0, 0.1, (rows, dim)).astype(np.float32)
    if dtype in (O.INT8, O.INT4, O.INT2):
        return O.quantize_sbhalf(w, O.BITS[dtype])
    return w.astype(np.float16) if dtype == O.FP16 else w


def weight_pair(dtype: int, data: np.ndarray):
    """(payload bytes, scale_bias bytes or None) as numpy, the TBE's weight_lists entry."""
    if dtype in (O.INT8, O.INT4, O.INT2):
        return data[:, :-4], data[:, -4:]
    return data.view(np.uint8).reshape(data.shape[0], -1), None


def make_bags(
    rng: np.random.Generator,
    rows_per_feature: Sequence[int],
    B: int,
    max_len: int,
    idx_dtype=np.int32,
    empty_frac: float = 0.1,
    fixed_len: Optional[int] = None,
):
    F = len(rows_per_feature)
    if fixed_len is not None:
        lengths = np.full(F * B, fixed_len, dtype=np.int64)
    else:
        lengths = rng.integers(0, max_len + 1, F * B)
        lengths[rng.random(F * B) < empty_frac] = 0
    offsets = np.zeros(F * B + 1, dtype=idx_dtype)
    offsets[1:] = np.cumsum(lengths)
    per_feature = lengths.reshape(F, B).sum(axis=1)
    ids = np.concatenate(
        [rng.integers(0, rows_per_feature[f], int(per_feature[f])) for f in range(F)]
    ).astype(idx_dtype) if F else np.zeros(0, dtype=idx_dtype)
    return lengths.astype(idx_dtype), offsets, ids


def bits_equal(a: np.ndarray, b: np.ndarray) -> int:
    """Number of elements whose bit patterns differ."""
    assert a.shape == b.shape and a.dtype == b.dtype, (a.shape, b.shape, a.dtype, b.dtype)
    v = np.uint16 if a.dtype == np.float16 else np.uint32
    return int((a.view(v) != b.view(v)).sum())


def bucketize_python(lengths, ids, weights, block_sizes, W, keep):
    """Independent pure-Python statement of block bucketization (the same rule as
    block_bucketize_ref in the reference's torchrec/distributed/tests/test_utils.py:299-466)."""
    F = len(block_sizes)
    n = len(lengths)
    B = n // F
    buckets = [[[] for _ in range(n)] for _ in range(W)]
    unb = [-1] * len(ids)
    j = 0
    for i in range(n):
        bs = block_sizes[i // B]
        for _ in range(lengths[i]):
            p = ids[j] // bs
            if p < W:
                buckets[p][i].append((ids[j] if keep else ids[j] % bs, None if weights is None else weights[j], j))
            j += 1
    new_l, new_i, new_w = [], [], []
    for p in range(W):
        for i in range(n):
            new_l.append(len(buckets[p][i]))
            for v, w, src in buckets[p][i]:
                unb[src] = len(new_i)
                new_i.append(v)
                new_w.append(w)
    return new_l, new_i, new_w, unb
