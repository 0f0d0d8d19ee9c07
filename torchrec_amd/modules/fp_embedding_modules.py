"""EmbeddingBagCollection behind feature processors
(torchrec/modules/fp_embedding_modules.py:20-220): the KJT first gets its
per-id weights from the processors, then goes through the weighted collection.
"""
from __future__ import annotations

from typing import Dict, List, Tuple, Union

import torch
import torch.nn as nn

from torchrec_amd.modules.embedding_modules import EmbeddingBagCollection
from torchrec_amd.modules.feature_processor_ import FeatureProcessor, FeatureProcessorsCollection
from torchrec_amd.sparse.jagged_tensor import KeyedJaggedTensor, KeyedTensor


def apply_feature_processors_to_kjt(features: KeyedJaggedTensor,
                                    feature_processors: Dict[str, nn.Module]) -> KeyedJaggedTensor:
    """Weights of every key from its processor (1 for keys without one); ids and
    lengths are passed through unchanged."""
    per_key = features.to_dict()
    weights: List[torch.Tensor] = []
    for key in features.keys():
        jt = per_key[key]
        processor = feature_processors[key] if key in feature_processors else None
        if processor is None:
            weights.append(torch.ones(jt.values().shape[0], device=jt.values().device))
        else:
            weights.append(processor(jt).weights())
    return KeyedJaggedTensor(keys=features.keys(), values=features.values(),
                             weights=torch.cat(weights) if weights else features.weights_or_none(),
                             lengths=features.lengths(), offsets=features.offsets_or_none(), stride=features.stride())


class FeatureProcessorDictWrapper(FeatureProcessorsCollection):
    """A dict of per-feature processors presented as one collection."""

    def __init__(self, feature_processors: nn.ModuleDict) -> None:
        super().__init__()
        self._feature_processors = feature_processors

    def forward(self, features: KeyedJaggedTensor) -> KeyedJaggedTensor:
        return apply_feature_processors_to_kjt(features, self._feature_processors)


class FeatureProcessedEmbeddingBagCollection(nn.Module):
    """``feature_processors``: one ``FeatureProcessor`` per feature name, or one
    ``FeatureProcessorsCollection`` for the whole KJT.  The wrapped collection
    must be weighted."""

    def __init__(self, embedding_bag_collection: EmbeddingBagCollection,
                 feature_processors: Union[Dict[str, FeatureProcessor], FeatureProcessorsCollection]) -> None:
        super().__init__()
        table_features = [n for c in embedding_bag_collection.embedding_bag_configs() for n in c.feature_names]
        self._embedding_bag_collection = embedding_bag_collection
        self._feature_processors: Union[nn.ModuleDict, FeatureProcessorsCollection]
        if isinstance(feature_processors, FeatureProcessorsCollection):
            self._feature_processors = feature_processors
        else:
            assert set(table_features) == set(
                feature_processors.keys()
            ), "Passed in feature processors do not match feature names of embedding bag"
            self._feature_processors = nn.ModuleDict(feature_processors)
        assert (
            embedding_bag_collection.is_weighted()
        ), "EmbeddingBagCollection must accept weighted inputs for feature processor"
        self._feature_names: List[str] = list(dict.fromkeys(table_features))  # distinct, table order

    def split(self) -> Tuple[FeatureProcessorsCollection, EmbeddingBagCollection]:
        processors = self._feature_processors
        if isinstance(processors, nn.ModuleDict):
            processors = FeatureProcessorDictWrapper(processors)
        return processors, self._embedding_bag_collection

    def is_weighted(self) -> bool:
        return self._embedding_bag_collection.is_weighted()

    def forward(self, features: KeyedJaggedTensor) -> KeyedTensor:
        processors = self._feature_processors
        if isinstance(processors, FeatureProcessorsCollection):
            return self._embedding_bag_collection(processors(features))
        per_key = features.to_dict()
        processed = [processors[key](per_key[key]) for key in self._feature_names]
        return self._embedding_bag_collection(
            KeyedJaggedTensor(
                keys=self._feature_names,
                values=torch.cat([jt.values() for jt in processed]),
                lengths=torch.cat([jt.lengths() for jt in processed]),
                weights=torch.cat([jt.weights() for jt in processed]),
            )
        )
