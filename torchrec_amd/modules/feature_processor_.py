"""Feature processors: modules that attach per-id weights to sparse features
before an embedding lookup (torchrec/modules/feature_processor_.py).

``PositionWeightedModule`` (one feature, :46-103) and
``PositionWeightedModuleCollection`` (a whole KeyedJaggedTensor, :161-260) give
the id at position ``p`` of its bag the learned weight ``position_weight[p]``.
On the GPU the collection computes all weights of a KJT in one kernel launch
(``tra_position_weights``), with no per-key split and no host round trip;
tensors on the host use plain torch index arithmetic.
"""
from __future__ import annotations

import abc
from typing import Dict, List, Mapping, Optional

import torch
from torch import nn

from torchrec_amd import ops
from torchrec_amd.sparse.jagged_tensor import JaggedTensor, KeyedJaggedTensor
from torchrec_amd.types import CopyMixIn


class FeatureProcessor(nn.Module):
    """JaggedTensor -> JaggedTensor with ``weights`` populated."""

    @abc.abstractmethod
    def forward(self, features: JaggedTensor) -> JaggedTensor: ...


class FeatureProcessorsCollection(nn.Module):
    """KeyedJaggedTensor -> KeyedJaggedTensor with ``weights`` populated."""

    @abc.abstractmethod
    def forward(self, features: KeyedJaggedTensor) -> KeyedJaggedTensor: ...


def _positions(offsets: torch.Tensor, num_values: int) -> torch.Tensor:
    return ops.offsets_range(offsets.long(), num_values)


class PositionWeightedModule(FeatureProcessor):
    """Position weights of one id-list feature; ``max_feature_length`` is the
    truncation size of the feature and the length of the weight vector."""

    def __init__(self, max_feature_length: int, device: Optional[torch.device] = None) -> None:
        super().__init__()
        self.position_weight = nn.Parameter(torch.empty([max_feature_length], device=device), requires_grad=True)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        with torch.no_grad():
            self.position_weight.fill_(1.0)

    def forward(self, features: JaggedTensor) -> JaggedTensor:
        seq = _positions(features.offsets(), features.values().numel())
        return JaggedTensor(
            values=features.values(),
            lengths=features.lengths(),
            offsets=features.offsets(),
            weights=torch.gather(self.position_weight, dim=0, index=seq),
        )


class PositionWeightedModuleCollection(FeatureProcessorsCollection, CopyMixIn):
    """Position weights for the keys named in ``max_feature_lengths``; other
    keys of the KJT get weight 1."""

    def __init__(self, max_feature_lengths: Dict[str, int], device: Optional[torch.device] = None) -> None:
        super().__init__()
        self.max_feature_lengths = max_feature_lengths
        for length in max_feature_lengths.values():
            if length <= 0:
                raise ValueError("max feature lengths must be positive")
        self.position_weights: nn.ParameterDict = nn.ParameterDict()
        self.position_weights_dict: Dict[str, nn.Parameter] = {}
        for key, length in max_feature_lengths.items():
            self.position_weights[key] = nn.Parameter(torch.empty([length], device=device))
            self.position_weights_dict[key] = self.position_weights[key]
        # (keys, device) -> (key_start, key_len) index tensors of the fused GPU path
        self._layout_cache: Dict[object, object] = {}
        self._table_cache = None  # (stamp of the parameters, concatenated fp32 table)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        with torch.no_grad():
            for key in self.max_feature_lengths:
                self.position_weights[key].fill_(1.0)
                self.position_weights_dict[key] = self.position_weights[key]

    def _resync(self) -> None:
        for k, p in self.position_weights.items():
            self.position_weights_dict[k] = p
        self._layout_cache = {}
        self._table_cache = None

    def _layout(self, keys: List[str], dev: torch.device):
        """For a key order: where each key's weight vector sits in the
        concatenation of the vectors of the keys that have one (start, length;
        length 0 = weight 1), as host lists and as device tensors."""
        ck = (tuple(keys), dev)
        layout = self._layout_cache.get(ck)
        if layout is None:
            starts, lens, pos = [], [], 0
            for k in keys:
                if k in self.position_weights_dict:
                    n = self.position_weights_dict[k].numel()
                    starts.append(pos)
                    lens.append(n)
                    pos += n
                else:
                    starts.append(0)
                    lens.append(0)
            layout = (
                torch.tensor(starts, dtype=torch.int32, device=dev),
                torch.tensor(lens, dtype=torch.int32, device=dev),
                starts,
                lens,
            )
            self._layout_cache[ck] = layout
        return layout

    def _table(self, keys: List[str], dev: torch.device) -> torch.Tensor:
        """The weight vectors of ``keys`` in one fp32 tensor.  Rebuilt only when a
        parameter was replaced or written to since the last call (its version
        counter moved; a write through ``.data`` does not move it: call
        ``_resync()`` after one)."""
        present = [self.position_weights_dict[k] for k in keys if k in self.position_weights_dict]
        stamp = (tuple(keys), dev, tuple((id(p), p._version) for p in present))
        if self._table_cache is None or self._table_cache[0] != stamp:
            table = (
                torch.cat([p.detach().float().to(dev) for p in present])
                if present
                else torch.zeros(1, dtype=torch.float32, device=dev)
            )
            self._table_cache = (stamp, table)
        return self._table_cache[1]

    def kernel_layout(self, keys: List[str], dev: torch.device):
        """``(table, key_start, key_len)`` as the lookup operator's
        ``position_weights`` argument takes them."""
        layout = self._layout(keys, dev)
        return self._table(keys, dev), layout[2], layout[3]

    def _weights_gpu(self, features: KeyedJaggedTensor) -> torch.Tensor:
        keys = features.keys()
        dev = features.values().device
        layout = self._layout(keys, dev)
        return ops.position_weights(
            features.offsets(), len(keys), features.stride(), layout[0], layout[1], self._table(keys, dev),
            features.values().numel(),
        )

    def forward(self, features: KeyedJaggedTensor) -> KeyedJaggedTensor:
        if not features.keys():
            weights = features.weights_or_none()
        elif features.values().device.type == "cuda":
            weights = self._weights_gpu(features)
        else:
            cat_seq = _positions(features.offsets(), features.values().numel())
            parts: List[torch.Tensor] = []
            for key, seq in zip(features.keys(), torch.split(cat_seq, features.length_per_key())):
                if key in self.position_weights_dict:
                    parts.append(torch.gather(self.position_weights_dict[key], dim=0, index=seq))
                else:
                    parts.append(torch.ones(seq.shape[0], device=features.values().device))
            weights = torch.cat(parts)
        return KeyedJaggedTensor(
            keys=features.keys(),
            values=features.values(),
            weights=weights,
            lengths=features.lengths(),
            offsets=features.offsets(),
            stride=features.stride(),
        )

    def copy(self, device: torch.device) -> nn.Module:
        self.position_weights = self.position_weights.to(device=device)
        self._resync()
        return self

    def _apply(self, *args, **kwargs) -> nn.Module:  # keep the plain dict in step with the ParameterDict
        super()._apply(*args, **kwargs)
        self._resync()
        return self

    def load_state_dict(self, state_dict: Mapping[str, torch.Tensor], strict: bool = True, assign: bool = False):
        result = super().load_state_dict(state_dict, strict, assign)
        self._resync()
        return result
