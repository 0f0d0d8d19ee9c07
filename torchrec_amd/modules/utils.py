"""Helpers that turn the flat sequence-lookup output into per-feature
JaggedTensors (torchrec/modules/utils.py:41-51, 301-348, 414-417)."""
from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Optional

import torch

from torchrec_amd import ops
from torchrec_amd.sparse.jagged_tensor import JaggedTensor


@torch.fx.wrap
def _fx_to_list(tensor: torch.Tensor) -> List[int]:
    return tensor.long().tolist()


@torch.fx.wrap
def _slice_1d_tensor(tensor: torch.Tensor, start: int, end: int) -> torch.Tensor:
    if tensor.numel() == 0:
        return tensor
    return tensor[start:end]


@torch.fx.wrap
def _get_batching_hinted_output(lengths: torch.Tensor, output: torch.Tensor) -> torch.Tensor:
    # Identity; kept as a graph marker for batching-aware serving stacks.
    return output


def _permute_indices(indices: List[int], permute: List[int]) -> List[int]:
    return [indices[p] for p in permute]


def construct_jagged_tensors_inference(
    embeddings: torch.Tensor,
    lengths: torch.Tensor,
    values: torch.Tensor,
    embedding_names: List[str],
    need_indices: bool = False,
    features_to_permute_indices: Optional[Dict[str, List[int]]] = None,
    reverse_indices: Optional[torch.Tensor] = None,
    remove_padding: bool = False,
) -> Dict[str, JaggedTensor]:
    """``embeddings`` [L, D], ``lengths`` [F, B] -> {name: JaggedTensor}.

    Each JaggedTensor's values are a row range (view) of ``embeddings``; a name
    that occurs several times (column-wise shards of one feature) gets its row
    ranges concatenated along dim 1, in the order ``features_to_permute_indices``
    gives.  The per-feature row counts are reduced on the device and fetched
    with a single F-element copy.
    """
    with torch.profiler.record_function("## construct_jagged_tensors_inference ##"):
        if reverse_indices is not None:
            embeddings = torch.index_select(embeddings, 0, reverse_indices.to(torch.int32))
        elif remove_padding:
            embeddings = _slice_1d_tensor(embeddings, 0, int(lengths.sum().item()))
        num_features, batch = lengths.shape
        rows_per_feature: List[int] = ops.length_per_key(lengths.reshape(-1), num_features, batch)
        row_ranges = torch.split(embeddings, rows_per_feature, dim=0)
        id_ranges = torch.split(values, rows_per_feature) if need_indices else None
        positions: Dict[str, List[int]] = defaultdict(list)
        for pos, name in enumerate(embedding_names):
            positions[name].append(pos)
        out: Dict[str, JaggedTensor] = {}
        for name, where in positions.items():
            if features_to_permute_indices and name in features_to_permute_indices:
                where = _permute_indices(where, features_to_permute_indices[name])
            first = where[0]
            rows = row_ranges[first] if len(where) == 1 else torch.cat([row_ranges[w] for w in where], dim=1)
            out[name] = JaggedTensor(
                values=rows, lengths=lengths[first], weights=None if id_ranges is None else id_ranges[first]
            )
        return out
