"""KeyedJaggedTensor-level block bucketization: the index step of row-wise
sharding (torchrec/distributed/embedding_sharding.py:219-388).  Ids of feature
``f`` go to bucket ``id // block_sizes[f]`` (dropped when that is
``>= num_buckets``) and become ``id % block_sizes[f]`` unless the original ids
are kept; the result is a KJT with ``num_buckets`` copies of the keys,
bucket-major, order inside a bag preserved.  One GPU runs no all-to-all after
it; the functions exist so that callers of the reference's helpers find them.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from torchrec_amd import ops
from torchrec_amd.sparse.jagged_tensor import KeyedJaggedTensor


def _bucketize(
    kjt: KeyedJaggedTensor,
    num_buckets: int,
    block_sizes: torch.Tensor,
    sequence: bool,
    bucketize_pos: bool,
    block_bucketize_row_pos: Optional[List[torch.Tensor]],
    keep_original_indices: bool,
):
    assert block_sizes.numel() == len(kjt.keys()), (
        f"Expecting block sizes for {len(kjt.keys())} features, but {block_sizes.numel()} received."
    )
    if block_bucketize_row_pos is not None:
        raise NotImplementedError("uneven shard sizes (block_bucketize_row_pos) are not supported")
    return ops.block_bucketize_sparse_features(
        kjt.lengths().view(-1),
        kjt.values(),
        bucketize_pos=bucketize_pos,
        sequence=sequence,
        block_sizes=block_sizes.to(device=kjt.values().device, dtype=kjt.values().dtype),
        my_size=num_buckets,
        weights=kjt.weights_or_none(),
        keep_orig_idx=keep_original_indices,
    )


def bucketize_kjt_before_all2all(
    kjt: KeyedJaggedTensor,
    num_buckets: int,
    block_sizes: torch.Tensor,
    total_num_blocks: Optional[torch.Tensor] = None,
    output_permute: bool = False,
    bucketize_pos: bool = False,
    block_bucketize_row_pos: Optional[List[torch.Tensor]] = None,
    keep_original_indices: bool = False,
) -> Tuple[KeyedJaggedTensor, Optional[torch.Tensor]]:
    """Returns (bucketized KJT, unbucketize permute when ``output_permute``)."""
    if total_num_blocks is not None:
        raise NotImplementedError("two-level bucketization (total_num_blocks) is not supported")
    lengths, indices, weights, pos, unbucketize = _bucketize(
        kjt, num_buckets, block_sizes, output_permute, bucketize_pos, block_bucketize_row_pos, keep_original_indices
    )
    return (
        KeyedJaggedTensor(
            keys=list(kjt.keys()) * num_buckets,  # duplicates are told apart by position
            values=indices,
            weights=pos if bucketize_pos else weights,
            lengths=lengths.view(-1),
            stride=kjt.stride(),
        ),
        unbucketize,
    )


def bucketize_kjt_inference(
    kjt: KeyedJaggedTensor,
    num_buckets: int,
    block_sizes: torch.Tensor,
    total_num_buckets: Optional[torch.Tensor] = None,
    bucketize_pos: bool = False,
    block_bucketize_row_pos: Optional[List[torch.Tensor]] = None,
    is_sequence: bool = False,
    keep_original_indices: bool = False,
) -> Tuple[KeyedJaggedTensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Returns (bucketized KJT, unbucketize permute, bucket of every input id); the
    last two only for sequence features."""
    if total_num_buckets is not None:
        raise NotImplementedError("two-level bucketization (total_num_buckets) is not supported")
    lengths, indices, weights, pos, unbucketize = _bucketize(
        kjt, num_buckets, block_sizes, is_sequence, bucketize_pos, block_bucketize_row_pos, keep_original_indices
    )
    bucket_mapping = None
    if is_sequence:
        values = kjt.values()
        per_key = kjt.lengths().view(len(kjt.keys()), -1).sum(dim=1)
        per_id_block = torch.repeat_interleave(
            block_sizes.to(device=values.device, dtype=values.dtype), per_key, output_size=values.numel()
        )
        bucket_mapping = torch.div(values, per_id_block, rounding_mode="floor")
    return (
        KeyedJaggedTensor(
            keys=[k for _ in range(num_buckets) for k in kjt.keys()],
            values=indices,
            weights=pos if bucketize_pos else weights,
            lengths=lengths.view(-1),
            stride=kjt.stride(),
        ),
        unbucketize,
        bucket_mapping,
    )
