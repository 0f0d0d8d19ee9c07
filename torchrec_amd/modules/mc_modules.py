"""Managed-collision (zero-collision hashing) id remapping, inference side
(torchrec/modules/mc_modules.py).

A managed-collision module maps raw feature ids to rows of a table of
``zch_size`` rows: ids present in its sorted id table go to the row recorded
for them, every other id to the last row.  Training fills and evicts that
table; this build loads it (``load_state_dict``; buffer names are the
reference's, :1059-1095) and serves lookups.  Profiling / eviction (training
mode) is not built and raises.  On the GPU the remap is one binary-search
kernel per table (``tra_mch_remap``) instead of the reference's searchsorted +
gather + two masked writes (:959-989).
"""
from __future__ import annotations

import abc
from typing import Callable, Dict, List, Optional, Sequence

import torch
import torch.nn as nn

from torchrec_amd import ops
from torchrec_amd.modules.embedding_configs import BaseEmbeddingConfig
from torchrec_amd.sparse.jagged_tensor import JaggedTensor, KeyedJaggedTensor


class ManagedCollisionModule(nn.Module):
    """Dict[str, JaggedTensor] -> same with ids remapped into ``[0, output_size())``."""

    def __init__(self, device: torch.device) -> None:
        super().__init__()
        self._device = device

    @property
    def device(self) -> torch.device:
        return self._device

    @abc.abstractmethod
    def preprocess(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]: ...

    @abc.abstractmethod
    def remap(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]: ...

    @abc.abstractmethod
    def profile(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]: ...

    @abc.abstractmethod
    def output_size(self) -> int: ...

    @abc.abstractmethod
    def input_size(self) -> int: ...

    def evict(self) -> Optional[torch.Tensor]:
        return None

    def reset_inference_mode(self) -> None:
        pass


class MCHManagedCollisionModule(ManagedCollisionModule):
    """Sorted-table remap (:992-1432, inference subset).

    ``_mch_sorted_raw_ids`` [zch_size] int64, ascending, unused slots and the last
    entry hold int64 max; ``_mch_remapped_ids_mapping`` [zch_size] int64, the row of
    each sorted id.  A miss maps to ``output_global_offset + zch_size - 1``.
    ``eviction_policy`` / ``eviction_interval`` are accepted for signature
    compatibility and unused.
    """

    def __init__(
        self,
        zch_size: int,
        device: torch.device,
        eviction_policy: object = None,
        eviction_interval: int = 1,
        input_hash_size: int = (2**63) - 1,
        input_hash_func: Optional[Callable[[torch.Tensor, int], torch.Tensor]] = None,
        name: Optional[str] = None,
        output_global_offset: int = 0,
    ) -> None:
        super().__init__(device)
        assert zch_size > 0, "zch_size must be > 0"
        self._zch_size = zch_size
        self._name = name
        self._input_hash_size = input_hash_size
        self._input_hash_func = input_hash_func
        self._output_global_offset = output_global_offset
        self._eviction_policy = eviction_policy
        self._eviction_interval = eviction_interval
        imax = torch.iinfo(torch.int64).max
        self.register_buffer(
            "_mch_sorted_raw_ids", torch.full((zch_size,), imax, dtype=torch.int64, device=device)
        )
        self.register_buffer(
            "_mch_remapped_ids_mapping",
            torch.arange(output_global_offset, output_global_offset + zch_size, dtype=torch.int64, device=device),
        )

    def set_id_table(self, raw_ids: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """Fills the table from a set of distinct raw ids (at most ``zch_size - 1``):
        id ``raw_ids[i]`` is served by row ``rows[i]`` (default: ``output_global_offset + i``)."""
        raw_ids = raw_ids.to(torch.int64).reshape(-1)
        n = raw_ids.numel()
        assert n <= self._zch_size - 1, "the last slot is the delimiter / miss row"
        if rows is None:
            rows = torch.arange(self._output_global_offset, self._output_global_offset + n, dtype=torch.int64)
        order = torch.argsort(raw_ids)
        dev = self._mch_sorted_raw_ids.device
        self._mch_sorted_raw_ids.fill_(torch.iinfo(torch.int64).max)
        self._mch_sorted_raw_ids[:n] = raw_ids[order].to(dev)
        self._mch_remapped_ids_mapping[:n] = rows.to(torch.int64).reshape(-1)[order].to(dev)

    def preprocess(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]:
        if self._input_hash_func is None:
            return features
        return {
            name: JaggedTensor(
                values=self._input_hash_func(f.values(), self._input_hash_size),
                lengths=f.lengths(),
                offsets=f.offsets(),
                weights=f.weights_or_none(),
            )
            for name, f in features.items()
        }

    def profile(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]:
        if self.training:
            raise NotImplementedError(
                "managed-collision profiling and eviction (training) are not part of the inference build; call .eval()"
            )
        return features

    def remap(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]:
        miss = self._output_global_offset + self._zch_size - 1
        return {
            name: JaggedTensor(
                values=ops.mch_remap(f.values(), self._mch_sorted_raw_ids, self._mch_remapped_ids_mapping, miss),
                lengths=f.lengths(),
                offsets=f.offsets(),
                weights=f.weights_or_none(),
            )
            for name, f in features.items()
        }

    def forward(self, features: Dict[str, JaggedTensor]) -> Dict[str, JaggedTensor]:
        return self.remap(self.profile(self.preprocess(features)))

    def output_size(self) -> int:
        return self._zch_size

    def input_size(self) -> int:
        return self._input_hash_size


class ManagedCollisionCollection(nn.Module):
    """One managed-collision module per table; ``forward`` remaps a KJT whose keys
    are (a permutation of) the tables' features and returns it in table order
    (:323-430)."""

    def __init__(
        self,
        managed_collision_modules: Dict[str, ManagedCollisionModule],
        embedding_configs: Sequence[BaseEmbeddingConfig],
        need_preprocess: bool = True,
    ) -> None:
        super().__init__()
        self._managed_collision_modules = nn.ModuleDict(managed_collision_modules)
        self._embedding_configs = embedding_configs
        self.need_preprocess = need_preprocess
        self._table_to_features: Dict[str, List[str]] = {c.name: c.feature_names for c in embedding_configs}
        self._table_feature_splits: List[int] = [len(f) for f in self._table_to_features.values()]
        for config in embedding_configs:
            if config.name not in managed_collision_modules:
                raise ValueError(f"Table {config.name} is not present in managed_collision_modules")
            assert managed_collision_modules[config.name].output_size() == config.num_embeddings, (
                f"max_output_id in managed collision module for {config.name} must match {config.num_embeddings}"
            )
        self._feature_names: List[str] = [f for c in embedding_configs for f in c.feature_names]

    def embedding_configs(self) -> Sequence[BaseEmbeddingConfig]:
        return self._embedding_configs

    def _one_launch_tables(self, features: KeyedJaggedTensor):
        """Per key of ``features`` (already in table order) the sorted-id table, row
        mapping and miss row of its module, when every module is an inference-mode
        MCH module without an input hash and the ids are on the GPU; else None."""
        if features.values().device.type != "cuda" or not features.keys():
            return None
        sorted_ids, mappings, miss = [], [], []
        for config in self._embedding_configs:
            module = self._managed_collision_modules[config.name]
            if (
                type(module) is not MCHManagedCollisionModule
                or module.training
                or module._input_hash_func is not None
                or module._mch_sorted_raw_ids.device != features.values().device
            ):
                return None
            for _ in config.feature_names:
                sorted_ids.append(module._mch_sorted_raw_ids)
                mappings.append(module._mch_remapped_ids_mapping)
                miss.append(module._output_global_offset + module._zch_size - 1)
        return sorted_ids, mappings, miss

    def forward(self, features: KeyedJaggedTensor) -> KeyedJaggedTensor:
        order = [features.keys().index(f) for f in self._feature_names]
        if order != list(range(len(features.keys()))):
            features = features.permute(order)
        tables = self._one_launch_tables(features)
        if tables is not None:
            # all keys in one launch: no split per table, no host read of the
            # per-key id counts, no concatenation
            return KeyedJaggedTensor(
                keys=features.keys(),
                values=ops.mch_remap_keys(features.values(), features.offsets(), features.stride(), *tables),
                lengths=features.lengths(),
                offsets=features.offsets(),
                weights=features.weights_or_none(),
                stride=features.stride(),
            )
        splits = features.split(self._table_feature_splits)
        values: List[torch.Tensor] = []
        # modules are visited in table (config) order, which is the order of the splits
        for config, kjt in zip(self._embedding_configs, splits):
            module = self._managed_collision_modules[config.name]
            out = module({config.name: JaggedTensor(values=kjt.values(), lengths=kjt.lengths())})
            values.append(out[config.name].values())
        return KeyedJaggedTensor(
            keys=features.keys(),
            values=torch.cat(values) if values else features.values(),
            lengths=features.lengths(),
            weights=features.weights_or_none(),
        )

    def evict(self) -> Dict[str, Optional[torch.Tensor]]:
        return {name: None for name in self._managed_collision_modules.keys()}
