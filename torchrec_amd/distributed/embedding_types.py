"""Config types of one group of (possibly sharded) tables behind one lookup
operator: names, fields and helper methods as in
torchrec/distributed/embedding_types.py:76-119 (EmbeddingComputeKernel and its
mapping to a memory location) and :214-307 (ShardedEmbeddingTable,
GroupedEmbeddingConfig), and torchrec/modules/embedding_configs.py:403-407
(EmbeddingTableConfig)."""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, unique
from typing import Any, Dict, List, Optional

from torch.distributed._shard.metadata import ShardMetadata
from torch.distributed._shard.sharded_tensor.metadata import ShardedTensorMetadata

from torchrec_amd.modules.embedding_configs import BaseEmbeddingConfig, PoolingType
from torchrec_amd.tbe.enums import EmbeddingLocation
from torchrec_amd.types import DataType


@unique
class EmbeddingComputeKernel(Enum):
    DENSE = "dense"
    FUSED = "fused"
    FUSED_UVM = "fused_uvm"
    FUSED_UVM_CACHING = "fused_uvm_caching"
    QUANT = "quant"
    QUANT_UVM = "quant_uvm"
    QUANT_UVM_CACHING = "quant_uvm_caching"
    KEY_VALUE = "key_value"
    CUSTOMIZED_KERNEL = "customized_kernel"
    SSD_VIRTUAL_TABLE = "ssd_virtual_table"
    DRAM_VIRTUAL_TABLE = "dram_virtual_table"


_LOCATION_OF_KERNEL: Dict[EmbeddingComputeKernel, EmbeddingLocation] = {
    EmbeddingComputeKernel.DENSE: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.FUSED: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.QUANT: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.KEY_VALUE: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.SSD_VIRTUAL_TABLE: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.DRAM_VIRTUAL_TABLE: EmbeddingLocation.DEVICE,
    EmbeddingComputeKernel.FUSED_UVM: EmbeddingLocation.MANAGED,
    EmbeddingComputeKernel.QUANT_UVM: EmbeddingLocation.MANAGED,
    EmbeddingComputeKernel.FUSED_UVM_CACHING: EmbeddingLocation.MANAGED_CACHING,
    EmbeddingComputeKernel.QUANT_UVM_CACHING: EmbeddingLocation.MANAGED_CACHING,
}


def compute_kernel_to_embedding_location(compute_kernel: EmbeddingComputeKernel) -> EmbeddingLocation:
    try:
        return _LOCATION_OF_KERNEL[compute_kernel]
    except KeyError:
        raise ValueError(f"Invalid EmbeddingComputeKernel {compute_kernel}") from None


@dataclass
class EmbeddingTableConfig(BaseEmbeddingConfig):
    pooling: PoolingType = PoolingType.SUM
    is_weighted: bool = False
    has_feature_processor: bool = False
    embedding_names: List[str] = field(default_factory=list)


@dataclass
class ShardedConfig:
    local_rows: int = 0
    local_cols: int = 0


@dataclass
class ShardedMetaConfig(ShardedConfig):
    local_metadata: Optional[ShardMetadata] = None
    global_metadata: Optional[ShardedTensorMetadata] = None
    dtensor_metadata: Optional[Any] = None


@dataclass
class EmbeddingAttributes:
    compute_kernel: EmbeddingComputeKernel = EmbeddingComputeKernel.DENSE


@dataclass
class ShardedEmbeddingTable(ShardedMetaConfig, EmbeddingAttributes, EmbeddingTableConfig):
    """One table's local shard: ``local_rows`` x ``local_cols`` of the
    ``num_embeddings`` x ``embedding_dim`` table, at ``local_metadata.shard_offsets``."""

    fused_params: Optional[Dict[str, Any]] = None


@dataclass
class GroupedEmbeddingConfig:
    """Tables that share one lookup operator."""

    data_type: DataType
    pooling: PoolingType
    is_weighted: bool
    has_feature_processor: bool
    compute_kernel: EmbeddingComputeKernel
    embedding_tables: List[ShardedEmbeddingTable]
    fused_params: Optional[Dict[str, Any]] = None
    enable_embedding_update: bool = False

    def _per_feature(self, of_table) -> list:
        return [x for t in self.embedding_tables for x in of_table(t)]

    def feature_hash_sizes(self) -> List[int]:
        return self._per_feature(lambda t: [t.num_embeddings] * t.num_features())

    def num_features(self) -> int:
        return sum(t.num_features() for t in self.embedding_tables)

    def dim_sum(self) -> int:
        return sum(t.num_features() * t.local_cols for t in self.embedding_tables)

    def table_names(self) -> List[str]:
        return [t.name for t in self.embedding_tables]

    def feature_names(self) -> List[str]:
        return self._per_feature(lambda t: t.feature_names)

    def embedding_dims(self) -> List[int]:
        return self._per_feature(lambda t: [t.local_cols] * t.num_features())

    def embedding_names(self) -> List[str]:
        return self._per_feature(lambda t: t.embedding_names)

    def embedding_shard_metadata(self) -> List[Optional[ShardMetadata]]:
        return self._per_feature(lambda t: [t.local_metadata] * t.num_features())

    def is_using_virtual_table(self) -> bool:
        return any(t.use_virtual_table for t in self.embedding_tables)
