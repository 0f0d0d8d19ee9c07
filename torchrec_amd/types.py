"""Value types shared by the table configs (same names and values as
torchrec/types.py:17-71)."""
from __future__ import annotations

from enum import Enum

import torch
import torch.nn as nn


class CopyMixIn:
    """Lets a module decide what a DistributedModelParallel-style ``copy(device)`` does."""

    def copy(self, device: torch.device) -> nn.Module:  # pragma: no cover - interface
        raise NotImplementedError


class ModuleCopyMixin(CopyMixIn):
    """``copy`` moves the module."""

    def copy(self, device: torch.device) -> nn.Module:
        moved: nn.Module = self.to(device)  # type: ignore[attr-defined]
        return moved


class ModuleNoCopyMixin(CopyMixIn):
    """``copy`` is the identity: the quantized modules own device buffers that
    must not be duplicated."""

    def copy(self, device: torch.device) -> nn.Module:
        same: nn.Module = self  # type: ignore[assignment]
        return same


class _NamedEnum(Enum):
    def __str__(self) -> str:
        return str(self.value)


# Element type of an embedding table: every member's value is its own name.
DataType = _NamedEnum(  # type: ignore[misc]
    "DataType",
    [(n, n) for n in ("FP32", "FP16", "BF16", "INT64", "INT32", "INT8", "UINT8", "INT4", "INT2", "NFP8")],
    module=__name__,
)
