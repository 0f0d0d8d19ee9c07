"""Enums of the table-batched-embedding operator boundary.

Names and integer codes follow fbgemm_gpu's SparseType / PoolingMode /
EmbeddingLocation, which the reference imports at
torchrec/quant/embedding_modules.py:28-32 and
torchrec/modules/embedding_configs.py:18-19.
"""
from __future__ import annotations

import enum

import torch


@enum.unique
class SparseType(enum.Enum):
    FP32 = "fp32"
    FP16 = "fp16"
    FP8 = "fp8"
    INT8 = "int8"
    INT4 = "int4"
    INT2 = "int2"
    BF16 = "bf16"

    def __str__(self) -> str:
        return self.value

    def as_int(self) -> int:
        return {
            SparseType.FP32: 0,
            SparseType.FP16: 1,
            SparseType.INT8: 2,
            SparseType.INT4: 3,
            SparseType.INT2: 4,
            SparseType.BF16: 5,
            SparseType.FP8: 6,
        }[self]

    @staticmethod
    def from_int(ty: int) -> "SparseType":
        for t in SparseType:
            if t.as_int() == ty:
                return t
        raise ValueError(f"Unsupported sparse type: {ty}")

    def bit_rate(self) -> int:
        return {
            SparseType.FP32: 32,
            SparseType.FP16: 16,
            SparseType.BF16: 16,
            SparseType.FP8: 8,
            SparseType.INT8: 8,
            SparseType.INT4: 4,
            SparseType.INT2: 2,
        }[self]

    def is_float(self) -> bool:
        return self in (SparseType.FP32, SparseType.FP16, SparseType.FP8, SparseType.BF16)

    def as_dtype(self) -> torch.dtype:
        return {
            SparseType.FP32: torch.float32,
            SparseType.FP16: torch.float16,
            SparseType.BF16: torch.bfloat16,
            SparseType.FP8: torch.uint8,
            SparseType.INT8: torch.uint8,
            SparseType.INT4: torch.quint4x2,
            SparseType.INT2: torch.quint2x4,
        }[self]

    @staticmethod
    def from_dtype(dtype: torch.dtype) -> "SparseType":
        if dtype == torch.float32:
            return SparseType.FP32
        if dtype == torch.float16:
            return SparseType.FP16
        if dtype == torch.bfloat16:
            return SparseType.BF16
        if dtype in (torch.int8, torch.uint8, torch.quint8, torch.qint8):
            return SparseType.INT8
        if dtype == torch.quint4x2:
            return SparseType.INT4
        if dtype == torch.quint2x4:
            return SparseType.INT2
        raise ValueError(f"Unsupported sparse dtype: {dtype}")


class PoolingMode(enum.IntEnum):
    SUM = 0
    MEAN = 1
    NONE = 2


class EmbeddingLocation(enum.IntEnum):
    DEVICE = 0
    MANAGED = 1
    MANAGED_CACHING = 2
    HOST = 3
    MTIA = 4


class BoundsCheckMode(enum.IntEnum):
    """What the lookup does about an id outside its table (fbgemm_gpu's codes;
    the reference re-exports the enum as torchrec.distributed.types.BoundsCheckMode)."""

    FATAL = 0    # raise
    WARNING = 1  # report and go on
    IGNORE = 2   # go on silently
    NONE = 3     # no check
