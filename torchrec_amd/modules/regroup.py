"""``KTRegroupAsDict``: the module form of ``KeyedTensor.regroup_as_dict``
(torchrec/modules/regroup.py:129-242).  Where each block of each group comes
from is worked out on the first batch and kept; ``clear_cache()`` forgets it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from torchrec_amd.modules.embedding_configs import data_type_to_dtype
from torchrec_amd.sparse.jagged_tensor import KeyedTensor, _regroup_plan, regroup_kts
from torchrec_amd.types import DataType


class KTRegroupAsDict(torch.nn.Module):
    """``forward(List[KeyedTensor]) -> {keys[i]: blocks of groups[i] side by side}``.

    ``emb_dtype`` casts the inputs first; ``multi_device`` is accepted for
    signature parity (nothing here lives on a fixed device).  A key held by two
    of the KeyedTensors is an error, as in the reference."""

    def __init__(self, groups: List[List[str]], keys: List[str], emb_dtype: Optional[DataType] = None,
                 multi_device: bool = False) -> None:
        super().__init__()
        torch._C._log_api_usage_once(f"torchrec.modules.{self.__class__.__name__}")
        assert len(groups) == len(keys), "Groups and keys should have same length"
        self._groups = groups
        self._keys = keys
        self._emb_dtype = emb_dtype
        self._multi_device = multi_device
        self._is_inited = False
        self._plan = None

    def embedding_cast(self, embs: List[torch.Tensor]) -> List[torch.Tensor]:
        if self._emb_dtype is None:
            return embs
        dtype = data_type_to_dtype(self._emb_dtype)
        return [emb.to(dtype=dtype) for emb in embs]

    def forward(self, keyed_tensors: List[KeyedTensor]) -> Dict[str, torch.Tensor]:
        if not self._is_inited:
            seen = set()
            for kt in keyed_tensors:
                for key in kt.keys():
                    if key in seen:
                        raise RuntimeError(f"Duplicate key {key} found in KeyedTensors, undefined behavior")
                    seen.add(key)
            self._plan = _regroup_plan(keyed_tensors, self._groups)
            self._is_inited = True
        if self._emb_dtype is not None:
            keyed_tensors = [
                KeyedTensor(keys=kt.keys(), length_per_key=kt.length_per_key(), values=v, key_dim=kt.key_dim())
                for kt, v in zip(keyed_tensors, self.embedding_cast([kt.values() for kt in keyed_tensors]))
            ]
        return dict(zip(self._keys, regroup_kts(keyed_tensors, self._groups, plan=self._plan)))

    def clear_cache(self) -> None:
        self._is_inited = False
        self._plan = None
