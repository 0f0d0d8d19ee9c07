"""Registers the handful of ``torch.ops.fbgemm.*`` operators that TorchRec's
quantized inference path calls by name, backed by the kernels of this
package, so that unmodified TorchRec code finds them:

* ``asynchronous_complete_cumsum`` (torchrec/sparse/jagged_tensor.py:79-80)
* ``permute_2D_sparse_data`` (torchrec/sparse/jagged_tensor.py:2573-2583)
* ``offsets_range`` (torchrec/modules/feature_processor_.py:82-84)
* ``block_bucketize_sparse_features`` (torchrec/distributed/embedding_sharding.py:263-289)
* ``FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf`` (torchrec/quant/embedding_modules.py:261-265)

``import torchrec_amd.fbgemm_ops`` (or ``register()``) is a no-op for every
operator that another library (fbgemm_gpu) has already defined.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from torchrec_amd import ops

_SCHEMAS = {
    "asynchronous_complete_cumsum": "(Tensor t_in) -> Tensor",
    "permute_2D_sparse_data": (
        "(Tensor permute, Tensor lengths, Tensor values, Tensor? weights=None, "
        "SymInt? permuted_lengths_sum=None) -> (Tensor, Tensor, Tensor?)"
    ),
    "offsets_range": "(Tensor offsets, SymInt range_size) -> Tensor",
    "block_bucketize_sparse_features": (
        "(Tensor lengths, Tensor indices, bool bucketize_pos, bool sequence, Tensor block_sizes, "
        "SymInt my_size, Tensor? weights=None, Tensor? batch_size_per_feature=None, SymInt max_B=-1, "
        "Tensor[]? block_bucketize_pos=None, bool keep_orig_idx=False, Tensor? total_num_blocks=None) "
        "-> (Tensor, Tensor, Tensor?, Tensor?, Tensor?)"
    ),
    "FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf": "(Tensor input, int bit_rate) -> Tensor",
}


def _permute(permute, lengths, values, weights=None, permuted_lengths_sum=None):
    return ops.permute_2D_sparse_data(permute, lengths, values, weights, permuted_lengths_sum)


def _bucketize(lengths, indices, bucketize_pos, sequence, block_sizes, my_size, weights=None,
               batch_size_per_feature=None, max_B=-1, block_bucketize_pos=None, keep_orig_idx=False,
               total_num_blocks=None):
    if batch_size_per_feature is not None or block_bucketize_pos is not None or total_num_blocks is not None:
        raise NotImplementedError(
            "variable batch sizes, uneven shard boundaries and two-level bucketization are not supported"
        )
    return ops.block_bucketize_sparse_features(
        lengths, indices, bucketize_pos, sequence, block_sizes, my_size, weights, keep_orig_idx
    )


_IMPLS: dict = {
    "asynchronous_complete_cumsum": ops.asynchronous_complete_cumsum,
    "permute_2D_sparse_data": _permute,
    "offsets_range": ops.offsets_range,
    "block_bucketize_sparse_features": _bucketize,
    "FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf": ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf,
}

_library: Optional[torch.library.Library] = None
_registered: List[str] = []


def _exists(name: str) -> bool:
    try:
        getattr(torch.ops.fbgemm, name)
        return True
    except (AttributeError, RuntimeError):
        return False


def register() -> List[str]:
    """Defines the missing operators; returns the names this call (or an earlier one) registered."""
    global _library
    for name, schema in _SCHEMAS.items():
        if name in _registered or _exists(name):
            continue
        if _library is None:
            _library = torch.library.Library("fbgemm", "FRAGMENT")
        _library.define(name + schema)
        # One implementation for every device: the front ends in ops.py pick the
        # HIP kernel for device tensors themselves.
        _library.impl(name, _IMPLS[name], "CompositeExplicitAutograd")
        _registered.append(name)
    return list(_registered)


register()
