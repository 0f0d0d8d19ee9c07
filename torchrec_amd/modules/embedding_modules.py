"""Unquantized EmbeddingBagCollection / EmbeddingCollection.

These are the float modules ``from_float`` of the quantized collections
consumes (torchrec/modules/embedding_modules.py:97-301, 335-543).  Their
forward is plain PyTorch (``nn.EmbeddingBag`` / ``nn.Embedding``); they carry
the table configs, the ``feature@table`` naming rule and the
``embedding_bags.<table>.weight`` state-dict layout.
"""
from __future__ import annotations

import abc
from typing import Dict, List, Optional, Union

import torch
import torch.nn as nn

from torchrec_amd.modules.embedding_configs import (
    DataType,
    EmbeddingBagConfig,
    EmbeddingConfig,
    pooling_type_to_str,
)
from torchrec_amd.sparse.jagged_tensor import JaggedTensor, KeyedJaggedTensor, KeyedTensor


def get_embedding_names_by_table(
    tables: Union[List[EmbeddingBagConfig], List[EmbeddingConfig]],
) -> List[List[str]]:
    """Output names per table: ``feature``, or ``feature@table`` when the feature
    feeds more than one table (torchrec/modules/embedding_modules.py:75-94)."""
    seen: Dict[str, int] = {}
    for config in tables:
        for feature_name in config.feature_names:
            seen[feature_name] = seen.get(feature_name, 0) + 1
    return [
        [f if seen[f] == 1 else f + "@" + config.name for f in config.feature_names]
        for config in tables
    ]


class EmbeddingBagCollectionInterface(abc.ABC, nn.Module):
    @abc.abstractmethod
    def forward(self, features: KeyedJaggedTensor) -> KeyedTensor: ...

    @abc.abstractmethod
    def embedding_bag_configs(self) -> List[EmbeddingBagConfig]: ...

    @abc.abstractmethod
    def is_weighted(self) -> bool: ...


class EmbeddingBagCollection(EmbeddingBagCollectionInterface):
    """Pooled embeddings of several tables; output ``KeyedTensor`` [B, sum(dims)]."""

    def __init__(
        self,
        tables: List[EmbeddingBagConfig],
        is_weighted: bool = False,
        device: Optional[torch.device] = None,
    ) -> None:
        super().__init__()
        self._is_weighted = is_weighted
        self.embedding_bags: nn.ModuleDict = nn.ModuleDict()
        self._embedding_bag_configs = tables
        self._lengths_per_embedding: List[int] = []
        names = set()
        for config in tables:
            if config.name in names:
                raise ValueError(f"Duplicate table name {config.name}")
            names.add(config.name)
            dtype = torch.float32 if config.data_type == DataType.FP32 else torch.float16
            self.embedding_bags[config.name] = nn.EmbeddingBag(
                num_embeddings=config.num_embeddings,
                embedding_dim=config.embedding_dim,
                mode=pooling_type_to_str(config.pooling),
                device=device,
                include_last_offset=True,
                dtype=dtype,
            )
            if device is None:
                device = self.embedding_bags[config.name].weight.device
            if not config.feature_names:
                config.feature_names = [config.name]
            self._lengths_per_embedding.extend(len(config.feature_names) * [config.embedding_dim])
        self._device: torch.device = device or torch.device("cpu")
        self._embedding_names: List[str] = [
            n for per_table in get_embedding_names_by_table(tables) for n in per_table
        ]
        self._feature_names: List[List[str]] = [t.feature_names for t in tables]
        self.reset_parameters()

    def forward(self, features: KeyedJaggedTensor) -> KeyedTensor:
        pooled: List[torch.Tensor] = []
        feature_dict = features.to_dict()
        for i, bag in enumerate(self.embedding_bags.values()):
            for feature_name in self._feature_names[i]:
                f = feature_dict[feature_name]
                pooled.append(
                    bag(
                        input=f.values(),
                        offsets=f.offsets(),
                        per_sample_weights=f.weights() if self._is_weighted else None,
                    ).float()
                )
        return KeyedTensor(
            keys=self._embedding_names,
            values=torch.cat(pooled, dim=1),
            length_per_key=self._lengths_per_embedding,
        )

    def is_weighted(self) -> bool:
        return self._is_weighted

    def embedding_bag_configs(self) -> List[EmbeddingBagConfig]:
        return self._embedding_bag_configs

    @property
    def device(self) -> torch.device:
        return self._device

    def reset_parameters(self) -> None:
        if torch.device(self._device).type == "meta":
            return
        for config in self._embedding_bag_configs:
            assert config.init_fn is not None
            config.init_fn(self.embedding_bags[config.name].weight)


class EmbeddingCollectionInterface(abc.ABC, nn.Module):
    @abc.abstractmethod
    def forward(self, features: KeyedJaggedTensor) -> Dict[str, JaggedTensor]: ...

    @abc.abstractmethod
    def embedding_configs(self) -> List[EmbeddingConfig]: ...

    @abc.abstractmethod
    def need_indices(self) -> bool: ...

    @abc.abstractmethod
    def embedding_dim(self) -> int: ...

    @abc.abstractmethod
    def embedding_names_by_table(self) -> List[List[str]]: ...


class EmbeddingCollection(EmbeddingCollectionInterface):
    """Per-id (sequence) embeddings; output one ``JaggedTensor`` per feature."""

    def __init__(
        self,
        tables: List[EmbeddingConfig],
        device: Optional[torch.device] = None,
        need_indices: bool = False,
    ) -> None:
        super().__init__()
        self.embeddings: nn.ModuleDict = nn.ModuleDict()
        self._embedding_configs = tables
        self._embedding_dim: int = -1
        self._need_indices: bool = need_indices
        self._device: torch.device = device if device is not None else torch.device("cpu")
        names = set()
        for config in tables:
            if config.name in names:
                raise ValueError(f"Duplicate table name {config.name}")
            names.add(config.name)
            self._embedding_dim = config.embedding_dim if self._embedding_dim < 0 else self._embedding_dim
            if self._embedding_dim != config.embedding_dim:
                raise ValueError(
                    "All tables in a EmbeddingCollection are required to have same embedding dimension."
                    + f" Violating case: {config.name}'s embedding_dim {config.embedding_dim} !="
                    + f" {self._embedding_dim}"
                )
            dtype = torch.float32 if config.data_type == DataType.FP32 else torch.float16
            self.embeddings[config.name] = nn.Embedding(
                num_embeddings=config.num_embeddings,
                embedding_dim=config.embedding_dim,
                device=device,
                dtype=dtype,
            )
            if config.init_fn is not None and torch.device(self._device).type != "meta":
                config.init_fn(self.embeddings[config.name].weight)
            if not config.feature_names:
                config.feature_names = [config.name]
        self._embedding_names_by_table: List[List[str]] = get_embedding_names_by_table(tables)
        self._feature_names: List[List[str]] = [t.feature_names for t in tables]

    def forward(self, features: KeyedJaggedTensor) -> Dict[str, JaggedTensor]:
        out: Dict[str, JaggedTensor] = {}
        jt_dict = features.to_dict()
        for i, emb in enumerate(self.embeddings.values()):
            names = self._embedding_names_by_table[i]
            for j, feature_name in enumerate(self._feature_names[i]):
                f = jt_dict[feature_name]
                out[names[j]] = JaggedTensor(
                    values=emb(f.values()).float(),
                    lengths=f.lengths(),
                    weights=f.values() if self._need_indices else None,
                )
        return out

    def need_indices(self) -> bool:
        return self._need_indices

    def embedding_dim(self) -> int:
        return self._embedding_dim

    def embedding_configs(self) -> List[EmbeddingConfig]:
        return self._embedding_configs

    def embedding_names_by_table(self) -> List[List[str]]:
        return self._embedding_names_by_table

    @property
    def device(self) -> torch.device:
        return self._device
