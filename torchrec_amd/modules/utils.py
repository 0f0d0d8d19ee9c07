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
    permuted = [0] * len(indices)
    for i, p in enumerate(permute):
        permuted[i] = indices[p]
    return permuted


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

    Each JaggedTensor's values are a row range (view) of ``embeddings``.  The
    per-feature row counts are reduced on the device and fetched with a single
    F-element copy.
    """
    with torch.profiler.record_function("## construct_jagged_tensors_inference ##"):
        if reverse_indices is not None:
            embeddings = torch.index_select(embeddings, 0, reverse_indices.to(torch.int32))
        elif remove_padding:
            embeddings = _slice_1d_tensor(embeddings, 0, int(lengths.sum().item()))
        F, B = lengths.shape
        length_per_key: List[int] = ops.length_per_key(lengths.reshape(-1), F, B)
        lengths_tuple = torch.unbind(lengths, dim=0)
        embeddings_list = torch.split(embeddings, length_per_key, dim=0)
        values_list = torch.split(values, length_per_key) if need_indices else None
        key_indices = defaultdict(list)
        for i, key in enumerate(embedding_names):
            key_indices[key].append(i)
        ret: Dict[str, JaggedTensor] = {}
        for key, indices in key_indices.items():
            if features_to_permute_indices and key in features_to_permute_indices:
                indices = _permute_indices(indices, features_to_permute_indices[key])
            ret[key] = JaggedTensor(
                lengths=lengths_tuple[indices[0]],
                values=(
                    embeddings_list[indices[0]]
                    if len(indices) == 1
                    else torch.cat([embeddings_list[i] for i in indices], dim=1)
                ),
                weights=values_list[indices[0]] if values_list is not None else None,
            )
        return ret
