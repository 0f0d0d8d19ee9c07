"""Value types shared by the table configs (mirrors torchrec/types.py:17-71)."""
from __future__ import annotations

from enum import Enum, unique

import torch
import torch.nn as nn


class CopyMixIn:
    """Lets a module decide what DistributedModelParallel-style ``copy(device)`` does."""

    def copy(self, device: torch.device) -> nn.Module:  # pragma: no cover - interface
        raise NotImplementedError


class ModuleCopyMixin(CopyMixIn):
    def copy(self, device: torch.device) -> nn.Module:
        return self.to(device)  # type: ignore[attr-defined]


class ModuleNoCopyMixin(CopyMixIn):
    """The quantized modules own device buffers that must not be duplicated."""

    def copy(self, device: torch.device) -> nn.Module:
        return self  # type: ignore[return-value]


@unique
class DataType(Enum):
    """Element type of an embedding table (torchrec/types.py:53-71)."""

    FP32 = "FP32"
    FP16 = "FP16"
    BF16 = "BF16"
    INT64 = "INT64"
    INT32 = "INT32"
    INT8 = "INT8"
    UINT8 = "UINT8"
    INT4 = "INT4"
    INT2 = "INT2"
    NFP8 = "NFP8"

    def __str__(self) -> str:
        return self.value
