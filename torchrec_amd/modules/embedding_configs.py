"""Table configs and dtype plumbing of the quantized embedding modules.

Same names, fields and mapping rules as torchrec/modules/embedding_configs.py
(PoolingType :23-36, DATA_TYPE_NUM_BITS :61-70, dtype_to_data_type :73-95,
pooling_type_to_pooling_mode :98-115, data_type_to_sparse_type :127-143,
BaseEmbeddingConfig :329-396, EmbeddingBagConfig :410-420, EmbeddingConfig
:423-430, QuantConfig :433-436), with this package's own SparseType /
PoolingMode enums standing in for fbgemm_gpu's.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, unique
from functools import partial
from math import sqrt
from typing import Any, Callable, Dict, List, NamedTuple, Optional

import torch

from torchrec_amd.tbe.enums import PoolingMode, SparseType
from torchrec_amd.types import DataType


@unique
class PoolingType(Enum):
    SUM = "SUM"
    MEAN = "MEAN"
    NONE = "NONE"


DATA_TYPE_NUM_BITS: Dict[DataType, int] = {
    DataType.FP32: 32,
    DataType.FP16: 16,
    DataType.BF16: 16,
    DataType.INT8: 8,
    DataType.UINT8: 8,
    DataType.NFP8: 8,
    DataType.INT4: 4,
    DataType.INT2: 2,
}

_DTYPE_TO_DATA_TYPE = {
    torch.float32: DataType.FP32,
    torch.float16: DataType.FP16,
    torch.bfloat16: DataType.BF16,
    torch.int32: DataType.INT32,
    torch.int64: DataType.INT64,
    torch.quint8: DataType.INT8,
    torch.qint8: DataType.INT8,
    torch.int8: DataType.INT8,
    torch.uint8: DataType.UINT8,
    torch.quint4x2: DataType.INT4,
    torch.quint2x4: DataType.INT2,
    torch.float8_e4m3fn: DataType.NFP8,
}

_DATA_TYPE_TO_DTYPE = {
    DataType.FP32: torch.float32,
    DataType.FP16: torch.float16,
    DataType.BF16: torch.bfloat16,
    DataType.NFP8: torch.float8_e4m3fn,
    DataType.INT64: torch.int64,
    DataType.INT32: torch.int32,
    DataType.INT8: torch.int8,
    DataType.UINT8: torch.uint8,
    DataType.INT4: torch.quint4x2,
    DataType.INT2: torch.quint2x4,
}

_DATA_TYPE_TO_SPARSE_TYPE = {
    DataType.FP32: SparseType.FP32,
    DataType.FP16: SparseType.FP16,
    DataType.BF16: SparseType.BF16,
    DataType.INT8: SparseType.INT8,
    DataType.UINT8: SparseType.INT8,
    DataType.INT4: SparseType.INT4,
    DataType.INT2: SparseType.INT2,
    DataType.NFP8: SparseType.FP8,
}


def dtype_to_data_type(dtype: torch.dtype) -> DataType:
    try:
        return _DTYPE_TO_DATA_TYPE[dtype]
    except KeyError:
        raise Exception(f"Invalid data type {dtype}") from None


def data_type_to_dtype(data_type: DataType) -> torch.dtype:
    try:
        return _DATA_TYPE_TO_DTYPE[data_type]
    except KeyError:
        raise ValueError(f"DataType {data_type} cannot be converted to dtype") from None


def data_type_to_sparse_type(data_type: DataType) -> SparseType:
    try:
        return _DATA_TYPE_TO_SPARSE_TYPE[data_type]
    except KeyError:
        raise ValueError(f"Invalid DataType {data_type}") from None


def pooling_type_to_pooling_mode(pooling_type: PoolingType, sharding_type: Any = None) -> PoolingMode:
    name = pooling_type.value
    if name == PoolingType.SUM.value:
        return PoolingMode.SUM
    if name == PoolingType.MEAN.value:
        # Row-wise shardings pool partial sums and divide afterwards.
        if sharding_type is not None and getattr(sharding_type, "value", sharding_type) in (
            "row_wise",
            "table_row_wise",
        ):
            return PoolingMode.SUM
        return PoolingMode.MEAN
    if name == PoolingType.NONE.value:
        return PoolingMode.NONE
    raise Exception(f"Invalid pooling type {pooling_type}")


def pooling_type_to_str(pooling_type: PoolingType) -> str:
    if pooling_type.value == PoolingType.SUM.value:
        return "sum"
    if pooling_type.value == PoolingType.MEAN.value:
        return "mean"
    raise ValueError(f"Unsupported pooling type {pooling_type}")


@dataclass
class BaseEmbeddingConfig:
    """One embedding table (torchrec/modules/embedding_configs.py:329-396)."""

    num_embeddings: int
    embedding_dim: int
    name: str = ""
    data_type: DataType = DataType.FP32
    feature_names: List[str] = field(default_factory=list)
    weight_init_max: Optional[float] = None
    weight_init_min: Optional[float] = None
    num_embeddings_post_pruning: Optional[int] = None
    init_fn: Optional[Callable[[torch.Tensor], Optional[torch.Tensor]]] = None
    need_pos: bool = False
    input_dim: Optional[int] = None
    total_num_buckets: Optional[int] = None
    use_virtual_table: bool = False
    virtual_table_eviction_policy: Optional[Any] = None
    enable_embedding_update: bool = False

    def get_weight_init_max(self) -> float:
        if self.weight_init_max is None:
            return sqrt(1 / self.num_embeddings)
        return self.weight_init_max

    def get_weight_init_min(self) -> float:
        if self.weight_init_min is None:
            return -sqrt(1 / self.num_embeddings)
        return self.weight_init_min

    def num_features(self) -> int:
        return len(self.feature_names)

    def __post_init__(self) -> None:
        if self.init_fn is None:
            self.init_fn = partial(
                torch.nn.init.uniform_, a=self.get_weight_init_min(), b=self.get_weight_init_max()
            )


@dataclass
class EmbeddingBagConfig(BaseEmbeddingConfig):
    """A table whose lookups are pooled per bag."""

    pooling: PoolingType = PoolingType.SUM


@dataclass
class EmbeddingConfig(BaseEmbeddingConfig):
    """A table whose lookups are returned per id (sequence embeddings)."""


class QuantConfig(NamedTuple):
    activation: Any  # torch.quantization.PlaceholderObserver partial
    weight: Any
    per_table_weight_dtype: Optional[Dict[str, torch.dtype]] = None
