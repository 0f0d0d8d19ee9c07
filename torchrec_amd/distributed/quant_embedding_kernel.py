"""One lookup operator per group of table shards.

``QuantBatchedEmbeddingBag`` (pooled) and ``QuantBatchedEmbedding`` (one row
per id) are what the inference sharders of the reference instantiate per
shard (torchrec/distributed/quant_embedding_kernel.py:248-477, 480-663): they
turn a ``GroupedEmbeddingConfig`` into one table-batched lookup over the
shards' ``local_rows`` x ``local_cols`` and feed it the ids of a
KeyedJaggedTensor whose keys are already the group's features, in order.
``fused_params`` carries the knobs the sharders set: whether the state dict
shows scale and bias apart from the payload, the bounds-check mode, whether
the operator is called as a registered submodule, and whether it is handed
lengths instead of offsets.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, Iterator, List, Optional, Tuple

import torch
import torch.nn as nn

from torchrec_amd import ops
from torchrec_amd.distributed.embedding_types import (
    GroupedEmbeddingConfig,
    compute_kernel_to_embedding_location,
)
from torchrec_amd.distributed.fused_params import (
    TBEToRegisterMixIn,
    fused_param_bounds_check_mode,
    fused_param_lengths_to_offsets_lookup,
    is_fused_param_quant_state_dict_split_scale_bias,
    is_fused_param_register_tbe,
    tbe_fused_params,
)
from torchrec_amd.modules.embedding_configs import (
    DATA_TYPE_NUM_BITS,
    data_type_to_sparse_type,
    dtype_to_data_type,
    pooling_type_to_pooling_mode,
)
from torchrec_amd.sparse.jagged_tensor import KeyedJaggedTensor
from torchrec_amd.tbe.enums import BoundsCheckMode, EmbeddingLocation, PoolingMode, SparseType
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen,
    rounded_row_size_in_bytes,
)
from torchrec_amd.types import DataType

SplitWeights = Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]


def _row_alignment(device_type: str) -> int:
    # Rows of a GPU table start on 16-byte boundaries (one dwordx4 load never
    # straddles two rows); host tables are packed.
    return 16 if device_type == "cuda" else 1


def _copy_config(original: GroupedEmbeddingConfig, data_type: DataType, sparse_type: SparseType,
                 device: torch.device) -> GroupedEmbeddingConfig:
    """The quantized counterpart of a float group's config: ``local_cols`` and the
    shard metadata's second size become the packed row size in bytes
    (quant_embedding_kernel.py:57-97).  Like the reference's, this describes
    whole-width shards only.  Every table's own ``data_type`` is set as well
    (the reference sets the group's only): the operator is built from the
    tables' types, and a float group's tables still say FP32."""
    config = copy.deepcopy(original)
    config.data_type = data_type
    align = _row_alignment(device.type)

    def packed(cols: int) -> int:
        return rounded_row_size_in_bytes(cols, sparse_type, align)

    for table in config.embedding_tables:
        table.data_type = data_type
        table.local_cols = packed(table.local_cols)
        if table.local_metadata is not None:
            table.local_metadata.shard_sizes = [table.local_rows, table.local_cols]
        meta = table.global_metadata
        if meta is None:
            continue
        for shard in meta.shards_metadata:
            if shard != table.local_metadata:
                shard.shard_sizes = [shard.shard_sizes[0], packed(shard.shard_sizes[1])]
        meta.size = torch.Size([meta.size[0], sum(s.shard_sizes[1] for s in meta.shards_metadata)])
    return config


def _quantize_weight(state_dict: Dict[str, torch.Tensor],
                     data_type: DataType) -> List[Tuple[torch.Tensor, Optional[torch.Tensor]]]:
    """Row-wise quantization of every tensor of ``state_dict`` to
    (payload, 4-byte fp16 scale/bias) pairs (quant_embedding_kernel.py:100-120)."""
    pairs: List[Tuple[torch.Tensor, Optional[torch.Tensor]]] = []
    for weight in state_dict.values():
        if weight.dtype not in (torch.float, torch.float16):
            raise Exception(f"Unsupported dtype: {weight.dtype}")
        fused = ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(weight, DATA_TYPE_NUM_BITS[data_type])
        pairs.append((fused[:, :-4], fused[:, -4:]))
    return pairs


def _get_runtime_device(device: Optional[torch.device], config: GroupedEmbeddingConfig,
                        shard_index: Optional[int] = None) -> torch.device:
    """Where the lookups will run: ``device`` unless it is absent or meta, in
    which case the shards' placements decide (quant_embedding_kernel.py:147-178)."""
    if device is not None and device.type != "meta":
        return device
    which = shard_index or 0

    def on_cpu(table) -> bool:
        local = table.local_metadata
        if local is not None and local.placement is not None and local.placement.device().type == "cpu":
            return True
        meta = table.global_metadata
        if meta is None or not len(meta.shards_metadata):
            return False
        placement = meta.shards_metadata[which].placement
        return placement is not None and placement.device().type == "cpu"

    return torch.device("cpu") if all(on_cpu(t) for t in config.embedding_tables) else torch.device("cuda")


@torch.fx.wrap
def _unwrap_kjt(features: KeyedJaggedTensor) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    # GPU rule of the reference (:181-192): ids and offsets as int32.
    return features.values().int(), features.offsets().int(), features.weights_or_none()


def _unwrap_kjt_for_cpu(features: KeyedJaggedTensor,
                        weighted: bool) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    ids = features.values()
    return ids, features.offsets().type(ids.dtype), features.weights() if weighted else None


@torch.fx.wrap
def _unwrap_kjt_lengths(features: KeyedJaggedTensor) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    return features.values().int(), features.lengths().int(), features.weights_or_none()


@torch.fx.wrap
def _unwrap_optional_tensor(tensor: Optional[torch.Tensor]) -> torch.Tensor:
    assert tensor is not None
    return tensor


class IntNBitTableBatchedEmbeddingBagsCodegenWithLength(IntNBitTableBatchedEmbeddingBagsCodegen):
    """The lookup operator called with the KJT's lengths in place of offsets
    (quant_embedding_kernel.py:228-245).  The reference runs a cumulative sum
    first; here the lookup kernel derives the bag starts itself."""

    def forward(self, indices: torch.Tensor, lengths: torch.Tensor,  # type: ignore[override]
                per_sample_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
        num_features = len(self.feature_table_map)
        assert num_features > 0 and lengths.numel() % num_features == 0, "lengths must have F * B entries"
        return super().forward(indices, None, per_sample_weights,
                               batch_size=lengths.numel() // num_features, lengths=lengths)


class _QuantShardLookup(nn.Module, TBEToRegisterMixIn):
    """What the pooled and the sequence module share: the operator built from
    the group's shards, its state-dict view and weight accessors."""

    def __init__(self, config: GroupedEmbeddingConfig, device: Optional[torch.device],
                 fused_params: Optional[Dict[str, Any]], shard_index: Optional[int],
                 pooling_mode: PoolingMode, with_lengths: bool, pass_bounds_check: bool) -> None:
        super().__init__()
        torch._C._log_api_usage_once(f"torchrec.distributed.{self.__class__.__name__}")
        self._config: GroupedEmbeddingConfig = config
        tables = config.embedding_tables
        if any(t.use_virtual_table for t in tables):
            raise NotImplementedError("virtual (key-value backed) tables are not supported")
        self._local_rows: List[int] = [t.local_rows for t in tables]
        self._local_cols: List[int] = [t.local_cols for t in tables]
        self._num_embeddings: List[int] = [t.num_embeddings for t in tables]
        self._embedding_dims: List[int] = [t.embedding_dim for t in tables]
        self._feature_table_map: List[int] = [i for i, t in enumerate(tables) for _ in range(t.num_features())]
        self._emb_module_registered: bool = is_fused_param_register_tbe(fused_params)
        self._quant_state_dict_split_scale_bias: bool = is_fused_param_quant_state_dict_split_scale_bias(fused_params)
        self._runtime_device: torch.device = _get_runtime_device(device, config, shard_index)
        self._tbe_row_alignment: int = _row_alignment(self._runtime_device.type)

        on_gpu = device is not None and device.type == "cuda"
        specs = []
        for table, rows, cols in zip(tables, self._local_rows, self._local_cols):
            location = compute_kernel_to_embedding_location(table.compute_kernel) if on_gpu else EmbeddingLocation.HOST
            # With scale and bias split off, local_cols counts elements of the shard;
            # otherwise the shard is the whole row and the table's own width applies.
            dim = cols if self._quant_state_dict_split_scale_bias else table.embedding_dim
            specs.append((table.name, rows, dim, data_type_to_sparse_type(table.data_type), location))

        operator = IntNBitTableBatchedEmbeddingBagsCodegenWithLength if with_lengths else IntNBitTableBatchedEmbeddingBagsCodegen
        extra: Dict[str, Any] = dict(tbe_fused_params(fused_params) or {})
        if pass_bounds_check:
            extra["bounds_check_mode"] = fused_param_bounds_check_mode(fused_params) or BoundsCheckMode.WARNING
        self._emb_module: IntNBitTableBatchedEmbeddingBagsCodegen = operator(
            embedding_specs=specs, device=device, pooling_mode=pooling_mode,
            feature_table_map=self._feature_table_map, row_alignment=self._tbe_row_alignment,
            uvm_host_mapped=True, feature_names_per_table=[t.feature_names for t in tables], **extra,
        )
        if device is not None:
            self._emb_module.initialize_weights()

    @property
    def emb_module(self) -> IntNBitTableBatchedEmbeddingBagsCodegen:
        return self._emb_module

    @property
    def config(self) -> GroupedEmbeddingConfig:
        return self._config

    def get_tbes_to_register(self) -> Dict[IntNBitTableBatchedEmbeddingBagsCodegen, GroupedEmbeddingConfig]:
        return {self._emb_module: self._config}

    def _call_operator(self, **kwargs: Any) -> torch.Tensor:
        # A registered operator is called as a submodule, so that a tracer
        # records a call_module node and keeps the operator in the graph module.
        return self._emb_module(**kwargs) if self._emb_module_registered else self._emb_module.forward(**kwargs)

    def split_embedding_weights(self) -> List[SplitWeights]:
        mode = 2 if self._quant_state_dict_split_scale_bias else 0
        return list(self._emb_module.split_embedding_weights_with_scale_bias(split_scale_bias_mode=mode))

    def named_buffers(self, prefix: str = "", recurse: bool = True,
                      remove_duplicate: bool = True) -> Iterator[Tuple[str, torch.Tensor]]:
        """``<table>.weight`` (and ``.weight_qscale`` / ``.weight_qbias`` when split):
        views of the operator's packed store, not copies."""
        assert remove_duplicate, f"remove_duplicate=False not supported in {type(self).__name__}.named_buffers"
        head = prefix + "." if prefix else ""
        for table, (weight, qscale, qbias) in zip(self._config.embedding_tables, self.split_embedding_weights()):
            yield f"{head}{table.name}.weight", weight
            if self._quant_state_dict_split_scale_bias:
                yield f"{head}{table.name}.weight_qscale", qscale  # type: ignore[misc]
                yield f"{head}{table.name}.weight_qbias", qbias  # type: ignore[misc]

    @classmethod
    def from_float(cls, module: nn.Module, use_precomputed_fake_quant: bool = False):
        """Quantizes the float module's tables (its ``config`` is the group, its
        parameters the tables in order) to ``module.qconfig.weight().dtype``."""
        assert hasattr(module, "qconfig"), "BaseEmbedding input float module must have qconfig defined"
        data_type = dtype_to_data_type(module.qconfig.weight().dtype)
        split = getattr(module, "named_split_embedding_weights", None)
        state_dict = dict(split()) if split is not None else dict(module.named_parameters())
        device = next(iter(state_dict.values())).device
        config = _copy_config(module.config, data_type, data_type_to_sparse_type(data_type), device)
        quantized = cls(config=config, device=device)
        quantized.emb_module.assign_embedding_weights(_quantize_weight(state_dict, data_type))
        return quantized


class QuantBatchedEmbeddingBag(_QuantShardLookup):
    """Pooled lookup over one group of shards; ``forward(kjt) -> [B, sum of dims]``."""

    def __init__(self, config: GroupedEmbeddingConfig, pg: Optional[Any] = None,
                 device: Optional[torch.device] = None, fused_params: Optional[Dict[str, Any]] = None,
                 shard_index: Optional[int] = None) -> None:
        lengths_to_tbe = fused_param_lengths_to_offsets_lookup(fused_params)
        super().__init__(config, device, fused_params, shard_index,
                         pooling_mode=pooling_type_to_pooling_mode(config.pooling),
                         with_lengths=lengths_to_tbe, pass_bounds_check=True)
        self._pg = pg
        self._pooling: PoolingMode = self._emb_module.pooling_mode
        self._is_weighted: Optional[bool] = config.is_weighted
        self.lengths_to_tbe: bool = lengths_to_tbe

    def init_parameters(self) -> None:
        pass

    def _emb_module_forward(self, indices: torch.Tensor, lengths_or_offsets: torch.Tensor,
                            weights: Optional[torch.Tensor]) -> torch.Tensor:
        kwargs: Dict[str, Any] = {"indices": indices}
        kwargs["lengths" if self.lengths_to_tbe else "offsets"] = lengths_or_offsets
        if self._is_weighted:
            kwargs["per_sample_weights"] = _unwrap_optional_tensor(weights)
        return self._call_operator(**kwargs)

    def forward(self, features: KeyedJaggedTensor) -> torch.Tensor:
        if self.lengths_to_tbe:
            indices, bags, weights = _unwrap_kjt_lengths(features)
        elif self._runtime_device.type == "cpu":
            indices, bags, weights = _unwrap_kjt_for_cpu(features, self._config.is_weighted)
        else:
            indices, bags, weights = _unwrap_kjt(features)
        return self._emb_module_forward(indices, bags, weights)


class QuantBatchedEmbedding(_QuantShardLookup):
    """Sequence lookup over one group of shards; ``forward(kjt) -> [ids, dim]``."""

    def __init__(self, config: GroupedEmbeddingConfig, pg: Optional[Any] = None,
                 device: Optional[torch.device] = None, fused_params: Optional[Dict[str, Any]] = None,
                 shard_index: Optional[int] = None) -> None:
        super().__init__(config, device, fused_params, shard_index, pooling_mode=PoolingMode.NONE,
                         with_lengths=False, pass_bounds_check=False)
        self._pg = pg

    def forward(self, features: KeyedJaggedTensor) -> torch.Tensor:
        if self._runtime_device.type == "cpu":
            values, offsets, _ = _unwrap_kjt_for_cpu(features, weighted=self._config.is_weighted)
        else:
            values, offsets, _ = _unwrap_kjt(features)
        return self._call_operator(indices=values, offsets=offsets)
