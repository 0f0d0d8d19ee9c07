"""Embedding collections behind managed-collision id remapping
(torchrec/modules/mc_embedding_modules.py:30-171): the KJT's ids are first
remapped by the ManagedCollisionCollection, then looked up."""
from __future__ import annotations

from typing import Dict, Optional, Tuple, Union

import torch.nn as nn

from torchrec_amd.modules.embedding_modules import EmbeddingBagCollection, EmbeddingCollection
from torchrec_amd.modules.mc_modules import ManagedCollisionCollection
from torchrec_amd.sparse.jagged_tensor import JaggedTensor, KeyedJaggedTensor, KeyedTensor


class BaseManagedCollisionEmbeddingCollection(nn.Module):
    def __init__(
        self,
        embedding_module: Union[EmbeddingBagCollection, EmbeddingCollection],
        managed_collision_collection: ManagedCollisionCollection,
        return_remapped_features: bool = False,
        allow_in_place_embed_weight_update: bool = False,
    ) -> None:
        super().__init__()
        self._managed_collision_collection = managed_collision_collection
        self._return_remapped_features = return_remapped_features
        self._allow_in_place_embed_weight_update = allow_in_place_embed_weight_update
        self._embedding_module = embedding_module
        configs = (
            embedding_module.embedding_bag_configs()
            if isinstance(embedding_module, EmbeddingBagCollection)
            else embedding_module.embedding_configs()
        )
        assert (
            configs == managed_collision_collection.embedding_configs()
        ), "Embedding Collection and Managed Collision Collection must contain the same Embedding Configs"

    def forward(
        self, features: KeyedJaggedTensor
    ) -> Tuple[Union[KeyedTensor, Dict[str, JaggedTensor]], Optional[KeyedJaggedTensor]]:
        features = self._managed_collision_collection(features)
        res = self._embedding_module(features)
        return (res, features) if self._return_remapped_features else (res, None)


class ManagedCollisionEmbeddingCollection(BaseManagedCollisionEmbeddingCollection):
    def __init__(
        self,
        embedding_collection: EmbeddingCollection,
        managed_collision_collection: ManagedCollisionCollection,
        return_remapped_features: bool = False,
        allow_in_place_embed_weight_update: bool = False,
    ) -> None:
        super().__init__(
            embedding_collection, managed_collision_collection, return_remapped_features,
            allow_in_place_embed_weight_update,
        )

    @property
    def _embedding_collection(self) -> EmbeddingCollection:
        return self._embedding_module  # type: ignore[return-value]


class ManagedCollisionEmbeddingBagCollection(BaseManagedCollisionEmbeddingCollection):
    def __init__(
        self,
        embedding_bag_collection: EmbeddingBagCollection,
        managed_collision_collection: ManagedCollisionCollection,
        return_remapped_features: bool = False,
        allow_in_place_embed_weight_update: bool = False,
    ) -> None:
        super().__init__(
            embedding_bag_collection, managed_collision_collection, return_remapped_features,
            allow_in_place_embed_weight_update,
        )

    @property
    def _embedding_bag_collection(self) -> EmbeddingBagCollection:
        return self._embedding_module  # type: ignore[return-value]
