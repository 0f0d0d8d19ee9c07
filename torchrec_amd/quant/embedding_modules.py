"""Quantized EmbeddingBagCollection / EmbeddingCollection for MI355X.

Drop-in for ``torchrec.quant.embedding_modules`` (constructor and ``forward``
signatures: torchrec/quant/embedding_modules.py:343-356, 501-504, 745-758,
893-896; ``from_float`` :569-615, :964-1004; accessors :617-630, :1009-1026;
prep helpers :161-202; ``quantize_state_dict`` :205-280).  Table grouping, key
order, ``feature@table`` naming, output dtypes and ``state_dict`` layout follow
the reference; the execution differs:

* the KeyedJaggedTensor is never permuted or split.  Each lookup kernel reads
  bag ``(f, b)`` at ``offsets[pos(f) * B + b]`` where ``pos(f)`` is the
  position of feature ``f`` among the input keys, so a different key order, an
  unused key or a feature shared by two tables costs nothing and needs no
  host round trip;
* all table groups write straight into one ``[B, sum(dims)]`` output (no
  ``torch.cat``);
* the pooled path issues no device-to-host copy.  The sequence path needs the
  per-feature row counts as Python ints to slice its output and fetches them
  with one F-element copy.
"""
from __future__ import annotations

import copy
import itertools
from collections import defaultdict
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple, Type, Union

import torch
import torch.nn as nn
from torch import Tensor

from torchrec_amd import ops
from torchrec_amd.modules.embedding_configs import (
    BaseEmbeddingConfig,
    DATA_TYPE_NUM_BITS,
    data_type_to_sparse_type,
    DataType,
    dtype_to_data_type,
    EmbeddingBagConfig,
    EmbeddingConfig,
    pooling_type_to_pooling_mode,
    PoolingType,
    QuantConfig,
)
from torchrec_amd.modules.embedding_modules import (
    EmbeddingBagCollection as OriginalEmbeddingBagCollection,
    EmbeddingBagCollectionInterface,
    EmbeddingCollection as OriginalEmbeddingCollection,
    EmbeddingCollectionInterface,
    get_embedding_names_by_table,
)
from torchrec_amd.modules.feature_processor_ import FeatureProcessorsCollection, PositionWeightedModuleCollection
from torchrec_amd.modules.fp_embedding_modules import (
    FeatureProcessedEmbeddingBagCollection as OriginalFeatureProcessedEmbeddingBagCollection,
)
from torchrec_amd.modules.mc_embedding_modules import (
    ManagedCollisionEmbeddingCollection as OriginalManagedCollisionEmbeddingCollection,
)
from torchrec_amd.modules.mc_modules import ManagedCollisionCollection
from torchrec_amd.modules.utils import _get_batching_hinted_output
from torchrec_amd.sparse.jagged_tensor import (
    ComputeKJTToJTDict,
    JaggedTensor,
    KeyedJaggedTensor,
    KeyedTensor,
)
from torchrec_amd.tbe.enums import EmbeddingLocation, PoolingMode
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen,
)
from torchrec_amd.tensor_types import UInt2Tensor, UInt4Tensor
from torchrec_amd.types import ModuleNoCopyMixin

MODULE_ATTR_REGISTER_TBES_BOOL: str = "__register_tbes_in_named_modules"
MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS: str = "__quant_state_dict_split_scale_bias"
MODULE_ATTR_ROW_ALIGNMENT_INT: str = "__register_row_alignment_in_named_modules"
MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT: str = "__emb_name_to_num_rows_post_pruning"
MODULE_ATTR_REMOVE_STBE_PADDING_BOOL: str = "__remove_stbe_padding"
MODULE_ATTR_USE_UNFLATTENED_LENGTHS_FOR_BATCHING: str = "__use_unflattened_lengths_for_batching"
MODULE_ATTR_USE_BATCHING_HINTED_OUTPUT: str = "__use_batching_hinted_output"
MODULE_ATTR_CACHE_FEATURES_ORDER: str = "__cache_features_order"

DEFAULT_ROW_ALIGNMENT = 16


# ---------------------------------------------------------------------------
# small graph-friendly helpers (same names as the reference's fx.wrap'd ones)
# ---------------------------------------------------------------------------
@torch.fx.wrap
def _get_feature_length(feature: KeyedJaggedTensor) -> Tensor:
    return feature.lengths()


@torch.fx.wrap
def _get_kjt_keys(feature: KeyedJaggedTensor) -> List[str]:
    return feature.keys()


@torch.fx.wrap
def _permute_kjt(
    features: KeyedJaggedTensor,
    permute_order: List[int],
    permute_order_tensor: Optional[Tensor] = None,
) -> KeyedJaggedTensor:
    """Materialized reorder of a KJT (kept for callers; forward() does not need it)."""
    if permute_order == list(range(len(permute_order))):
        return features.flatten_lengths()
    return features.permute(permute_order, permute_order_tensor)


@torch.fx.wrap
def _cat_embeddings(embeddings: List[Tensor]) -> Tensor:
    return embeddings[0] if len(embeddings) == 1 else torch.cat(embeddings, dim=1)


@torch.fx.wrap
def _get_unflattened_lengths(lengths: torch.Tensor, num_features: int) -> torch.Tensor:
    return lengths.view(num_features, -1)


@torch.fx.wrap
def _fx_trec_unwrap_kjt(kjt: KeyedJaggedTensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(indices, offsets) with the dtype rule of the reference (:315-329): host
    keeps the index dtype and casts offsets to it; device tensors become int32."""
    indices = kjt.values()
    offsets = kjt.offsets()
    if kjt.device().type == "cpu":
        return indices, offsets.type(dtype=indices.dtype)
    return indices.int(), offsets.int()


def for_each_module_of_type_do(
    module: nn.Module,
    module_types: List[Type[torch.nn.Module]],
    op: Callable[[torch.nn.Module], None],
) -> None:
    for m in module.modules():
        if any(isinstance(m, t) for t in module_types):
            op(m)


def quant_prep_enable_quant_state_dict_split_scale_bias(module: nn.Module) -> None:
    setattr(module, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, True)


def quant_prep_enable_quant_state_dict_split_scale_bias_for_types(
    module: nn.Module, module_types: List[Type[torch.nn.Module]]
) -> None:
    for_each_module_of_type_do(
        module, module_types, lambda m: setattr(m, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, True)
    )


def quant_prep_enable_register_tbes(module: nn.Module, module_types: List[Type[torch.nn.Module]]) -> None:
    for_each_module_of_type_do(
        module, module_types, lambda m: setattr(m, MODULE_ATTR_REGISTER_TBES_BOOL, True)
    )


def quant_prep_customize_row_alignment(
    module: nn.Module, module_types: List[Type[torch.nn.Module]], row_alignment: int
) -> None:
    for_each_module_of_type_do(
        module, module_types, lambda m: setattr(m, MODULE_ATTR_ROW_ALIGNMENT_INT, row_alignment)
    )


def quant_prep_enable_cache_features_order(
    module: nn.Module, module_types: List[Type[torch.nn.Module]]
) -> None:
    for_each_module_of_type_do(
        module, module_types, lambda m: setattr(m, MODULE_ATTR_CACHE_FEATURES_ORDER, True)
    )


# ---------------------------------------------------------------------------
# weight quantization (setup time)
# ---------------------------------------------------------------------------
_INT_TYPES = (DataType.INT8, DataType.INT4, DataType.INT2)


def quantize_state_dict(
    module: nn.Module,
    table_name_to_quantized_weights: Dict[str, Tuple[Tensor, Tensor]],
    table_name_to_data_type: Dict[str, DataType],
    table_name_to_num_embeddings_post_pruning: Optional[Dict[str, int]] = None,
) -> torch.device:
    """Fills ``table_name_to_quantized_weights[table] = (payload, scale_bias)``.

    INT8/INT4/INT2: row-wise quantization on the GPU (same bytes as
    FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf), trailer split off as a
    ``[rows, 4]`` uint8 tensor.  FP16/FP32: the raw bytes, no scale_bias.
    """
    device = torch.device("cpu")
    post_pruning = table_name_to_num_embeddings_post_pruning or {}
    for key, tensor in module.state_dict().items():
        splits = key.split(".")
        assert splits[-1] == "weight"
        table_name = splits[-2]
        data_type = table_name_to_data_type[table_name]
        num_rows = post_pruning.get(table_name, tensor.shape[0])
        device = tensor.device
        num_bits = DATA_TYPE_NUM_BITS[data_type]
        scale_shift: Optional[Tensor]
        if tensor.is_meta:
            quant_weight = torch.empty(
                (num_rows, (tensor.shape[1] * num_bits) // 8), device="meta", dtype=torch.uint8
            )
            scale_shift = (
                torch.empty((num_rows, 4), device="meta", dtype=torch.uint8)
                if data_type in _INT_TYPES
                else None
            )
        else:
            if num_rows != tensor.shape[0]:
                tensor = tensor[:num_rows, :]
            if tensor.dtype not in (torch.float, torch.float16):
                raise Exception(f"Unsupported dtype: {tensor.dtype}")
            if data_type == DataType.FP16:
                quant_weight, scale_shift = tensor.half().contiguous().view(torch.uint8), None
            elif data_type == DataType.FP32:
                quant_weight, scale_shift = tensor.float().contiguous().view(torch.uint8), None
            elif data_type in _INT_TYPES:
                quant_res = ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(tensor, num_bits)
                quant_weight, scale_shift = quant_res[:, :-4], quant_res[:, -4:]
            else:
                raise NotImplementedError(f"quantization to {data_type}")
        table_name_to_quantized_weights[table_name] = (quant_weight, scale_shift)
    return device


def _get_device(module: nn.Module) -> torch.device:
    for _, tensor in module.state_dict().items():
        return tensor.device
    return torch.device("cpu")


def _update_embedding_configs(
    embedding_configs: Sequence[BaseEmbeddingConfig],
    quant_config: Union[QuantConfig, Any],
    tables_to_rows_post_pruning: Optional[Dict[str, int]] = None,
) -> None:
    per_table = (
        quant_config.per_table_weight_dtype
        if isinstance(quant_config, QuantConfig) and quant_config.per_table_weight_dtype
        else {}
    )
    for config in embedding_configs:
        config.data_type = dtype_to_data_type(
            per_table[config.name] if config.name in per_table else quant_config.weight().dtype
        )
        if tables_to_rows_post_pruning and config.name in tables_to_rows_post_pruning:
            config.num_embeddings_post_pruning = tables_to_rows_post_pruning[config.name]


def _build_tbe(
    emb_configs: Sequence[BaseEmbeddingConfig],
    pooling_mode: PoolingMode,
    device: torch.device,
    output_dtype: torch.dtype,
    row_alignment: int,
    table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]],
    use_post_pruning_rows: bool,
) -> IntNBitTableBatchedEmbeddingBagsCodegen:
    location = EmbeddingLocation.HOST if device.type == "cpu" else EmbeddingLocation.DEVICE
    embedding_specs = []
    weight_lists: Optional[List[Tuple[Tensor, Optional[Tensor]]]] = (
        [] if table_name_to_quantized_weights else None
    )
    feature_table_map: List[int] = []
    for idx, table in enumerate(emb_configs):
        rows = table.num_embeddings
        if use_post_pruning_rows and getattr(table, "num_embeddings_post_pruning", None) is not None:
            rows = table.num_embeddings_post_pruning
        embedding_specs.append(
            (table.name, rows, table.embedding_dim, data_type_to_sparse_type(table.data_type), location)
        )
        if weight_lists is not None:
            weight_lists.append(table_name_to_quantized_weights[table.name])  # type: ignore[index]
        feature_table_map.extend([idx] * table.num_features())
    emb_module = IntNBitTableBatchedEmbeddingBagsCodegen(
        embedding_specs=embedding_specs,
        pooling_mode=pooling_mode,
        weight_lists=weight_lists,
        device=device,
        output_dtype=data_type_to_sparse_type(dtype_to_data_type(output_dtype)),
        row_alignment=row_alignment,
        feature_table_map=feature_table_map,
    )
    if weight_lists is None:
        emb_module.initialize_weights()
    return emb_module


def _register_table_buffers(
    holder: nn.ModuleDict,
    tables: Sequence[BaseEmbeddingConfig],
    emb_module: IntNBitTableBatchedEmbeddingBagsCodegen,
    split_scale_bias: bool,
) -> None:
    """state_dict entries ``<table>.weight[/weight_qscale/weight_qbias]`` that alias TBE storage."""
    views = emb_module.split_embedding_weights_with_scale_bias(
        split_scale_bias_mode=2 if split_scale_bias else 0
    )
    for config, (weight, qscale, qbias) in zip(tables, views):
        holder[config.name] = torch.nn.Module()
        if config.data_type == DataType.INT4:
            weight = UInt4Tensor(weight)
        elif config.data_type == DataType.INT2:
            weight = UInt2Tensor(weight)
        holder[config.name].register_buffer("weight", weight)
        if split_scale_bias:
            holder[config.name].register_buffer("weight_qscale", qscale)
            holder[config.name].register_buffer("weight_qbias", qbias)


class _FeatureOrderMixin:
    """Resolves where each module feature sits among the input keys."""

    _feature_names: List[str]
    _features_order: Optional[List[int]]

    def _resolve_order(self, kjt_keys: List[str]) -> List[int]:
        if getattr(self, MODULE_ATTR_CACHE_FEATURES_ORDER, False):
            # the reference's contract for this flag: the first key order seen is kept
            if self._features_order is None:
                self._features_order = [kjt_keys.index(k) for k in self._feature_names]
            return self._features_order
        # otherwise resolved per key order, remembered so that a repeated order costs one dict lookup
        cache = self.__dict__.setdefault("_order_by_keys", {})
        ck = tuple(kjt_keys)
        order = cache.get(ck)
        if order is None:
            order = [kjt_keys.index(k) for k in self._feature_names]
            if len(cache) < 64:
                cache[ck] = order
        return order

    def _group_positions(self, order: List[int]) -> List[tuple]:
        """``order`` cut into one tuple per lookup operator (cached per order object)."""
        cache = self.__dict__.setdefault("_positions_by_order", {})
        hit = cache.get(id(order))
        if hit is not None and hit[0] is order:
            return hit[1]
        groups, f0 = [], 0
        for n_feat in self._feature_splits:
            groups.append(tuple(order[f0 : f0 + n_feat]))
            f0 += n_feat
        if len(cache) < 64:
            cache[id(order)] = (order, groups)
        return groups


# ---------------------------------------------------------------------------
# pooled
# ---------------------------------------------------------------------------
class EmbeddingBagCollection(EmbeddingBagCollectionInterface, ModuleNoCopyMixin, _FeatureOrderMixin):
    """Quantized pooled embeddings: ``forward(KeyedJaggedTensor) -> KeyedTensor``.

    Tables are grouped by ``(pooling, use_virtual_table)`` into one
    table-batched operator each; a group may mix INT8/INT4/INT2/FP16/FP32
    tables and embedding dims.
    """

    def __init__(
        self,
        tables: List[EmbeddingBagConfig],
        is_weighted: bool,
        device: torch.device,
        output_dtype: torch.dtype = torch.float,
        table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = None,
        register_tbes: bool = False,
        quant_state_dict_split_scale_bias: bool = False,
        row_alignment: int = DEFAULT_ROW_ALIGNMENT,
        cache_features_order: bool = False,
    ) -> None:
        super().__init__()
        self._is_weighted = is_weighted
        self._embedding_bag_configs: List[EmbeddingBagConfig] = tables
        self._key_to_tables: Dict[Tuple[PoolingType, bool], List[EmbeddingBagConfig]] = defaultdict(list)
        self._feature_names: List[str] = []
        self._feature_splits: List[int] = []
        self._length_per_key: List[int] = []
        self._features_order: Optional[List[int]] = None
        # Kept in a plain list: their state is exposed through self.embedding_bags.
        self._emb_modules: List[nn.Module] = []
        self._output_dtype = output_dtype
        self._device: torch.device = torch.device(device)
        self._table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = None
        self.row_alignment = row_alignment
        self._kjt_to_jt_dict = ComputeKJTToJTDict()

        table_names = set()
        for table in self._embedding_bag_configs:
            if table.name in table_names:
                raise ValueError(f"Duplicate table name {table.name}")
            table_names.add(table.name)
            if getattr(table, "use_virtual_table", False):
                raise NotImplementedError("virtual (KV-backed) tables are not supported")
            self._key_to_tables[(table.pooling, False)].append(table)

        for (pooling, _virtual), emb_configs in self._key_to_tables.items():
            self._emb_modules.append(
                _build_tbe(
                    emb_configs,
                    pooling_type_to_pooling_mode(pooling),
                    self._device,
                    output_dtype,
                    row_alignment,
                    table_name_to_quantized_weights,
                    use_post_pruning_rows=True,
                )
            )
            for table in emb_configs:
                self._feature_names.extend(table.feature_names)
            self._feature_splits.append(sum(table.num_features() for table in emb_configs))

        ordered_tables = list(itertools.chain(*self._key_to_tables.values()))
        self._embedding_names: List[str] = list(
            itertools.chain(*get_embedding_names_by_table(ordered_tables))
        )
        for table in ordered_tables:
            self._length_per_key.extend([table.embedding_dim] * len(table.feature_names))
        self._total_D: int = sum(self._length_per_key)

        self.embedding_bags: nn.ModuleDict = nn.ModuleDict()
        for (_key, group_tables), emb_module in zip(self._key_to_tables.items(), self._emb_modules):
            _register_table_buffers(
                self.embedding_bags, group_tables, emb_module, quant_state_dict_split_scale_bias
            )

        setattr(self, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, quant_state_dict_split_scale_bias)
        setattr(self, MODULE_ATTR_REGISTER_TBES_BOOL, register_tbes)
        self.register_tbes = register_tbes
        if register_tbes:
            self.tbes: torch.nn.ModuleList = torch.nn.ModuleList(self._emb_modules)
        setattr(self, MODULE_ATTR_CACHE_FEATURES_ORDER, cache_features_order)

    def forward(
        self,
        features: KeyedJaggedTensor,
        position_weights: Optional[Tuple[Tensor, List[int], List[int]]] = None,
    ) -> KeyedTensor:
        """``features``: KJT of shape [F x B x jagged] -> KeyedTensor [B, sum(dims)].

        ``position_weights`` (not an argument of the reference; the
        feature-processed subclass passes it) weighs every id by its position
        in its bag inside the lookup kernel, see the operator's ``forward``."""
        # The common serving call first: one lookup operator, no weights, a KJT
        # built from lengths whose keys are this module's features in order.
        # Everything the general route below would establish is checked here
        # in a few attribute reads, and the operator is launched directly.
        ops_ = self._emb_modules
        if (
            len(ops_) == 1
            and not self._is_weighted
            and position_weights is None
            and features._offsets is None
            and not self.register_tbes  # (registered operators are called as modules, below)
        ):
            op = ops_[0]
            v, ln, keys = features._values, features._lengths, features._keys
            # (devices are compared by index: get_device() is -1 for a host tensor, and the
            # operator's device always carries an index)
            dev = op.current_device
            di = dev.index if dev.type == "cuda" else -2
            vdt = v.dtype
            if (
                ln is not None
                and (keys is self._feature_names or keys == self._feature_names)
                and v.get_device() == di
                and ln.get_device() == di
                and (vdt is torch.int64 or vdt is torch.int32)
                and ln.dtype is vdt
                and ln.dim() == 1
                and v.is_contiguous()
                and ln.is_contiguous()
                and op._weights_initialized
                and op._buffers["weights_dev"].get_device() == di
                and not getattr(self, MODULE_ATTR_CACHE_FEATURES_ORDER, False)
            ):
                K = len(keys)
                n_len = ln.numel()
                B = n_len // K if K else 0
                # (a feature that feeds two tables appears twice among the module's feature names: its
                # bags are then read twice from one key, which the general route below resolves)
                unique = self.__dict__.get("_feature_names_are_unique")
                if unique is None:
                    unique = self._feature_names_unique()
                if (
                    B > 0
                    and n_len == K * B
                    and features._stride in (None, B)
                    and features._stride_per_key is None
                    and unique
                ):
                    out = torch.empty(B, self._total_D, dtype=self._output_dtype, device=dev)
                    op._launch_from_lengths(
                        None, v, ln, int(v.dtype is torch.int64), None, B, K, v.numel(), out.data_ptr(), out.stride(0)
                    )
                    return KeyedTensor(keys=self._embedding_names, values=out, length_per_key=self._length_per_key)
        order = self._resolve_order(_get_kjt_keys(features))
        B = features.stride()
        indices = features.values()
        # A KJT that was built from lengths and has not had its offsets asked
        # for goes to a single operator as it is: the operator derives the
        # offsets itself (inside the lookup kernel when the call is large).
        lengths = None
        if (
            len(self._emb_modules) == 1
            and features.offsets_or_none() is None
            and features.lengths_or_none() is not None
            and B > 0
        ):
            offsets, lengths = None, features.lengths()
        else:
            offsets = features.offsets()
        psw = features.weights() if self._is_weighted and position_weights is None else None
        out = torch.empty((B, self._total_D), dtype=self._output_dtype, device=indices.device)
        col = 0
        for emb_op, positions in zip(self._emb_modules, self._group_positions(order)):
            # An operator registered as a submodule (register_tbes) is called as a module, so that
            # hooks and leaf-module tracing see the call (torchrec/quant/embedding_modules.py:546-557).
            call = emb_op if self.register_tbes else emb_op.forward
            call(  # type: ignore[operator]
                indices=indices,
                offsets=offsets,
                lengths=lengths,
                per_sample_weights=psw,
                feature_positions=positions,
                batch_size=B,
                out=out,
                out_col=col,
                position_weights=position_weights,
            )
            col += emb_op.total_D  # type: ignore[union-attr]
        return KeyedTensor(keys=self._embedding_names, values=out, length_per_key=self._length_per_key)

    def _feature_names_unique(self) -> bool:
        unique = getattr(self, "_feature_names_are_unique", None)
        if unique is None:
            unique = self._feature_names_are_unique = len(set(self._feature_names)) == len(self._feature_names)
        return unique

    def _get_name(self) -> str:
        return "QuantizedEmbeddingBagCollection"

    @classmethod
    def from_float(
        cls, module: OriginalEmbeddingBagCollection, use_precomputed_fake_quant: bool = False
    ) -> "EmbeddingBagCollection":
        assert hasattr(module, "qconfig"), "EmbeddingBagCollection input float module must have qconfig defined"
        pruning_dict: Dict[str, int] = getattr(
            module, MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT, {}
        )
        embedding_bag_configs = copy.deepcopy(module.embedding_bag_configs())
        _update_embedding_configs(embedding_bag_configs, module.qconfig, pruning_dict)
        table_name_to_quantized_weights: Dict[str, Tuple[Tensor, Tensor]] = {}
        device = quantize_state_dict(
            module,
            table_name_to_quantized_weights,
            {table.name: table.data_type for table in embedding_bag_configs},
            pruning_dict,
        )
        return cls(
            embedding_bag_configs,
            module.is_weighted(),
            device=device,
            output_dtype=module.qconfig.activation().dtype,
            table_name_to_quantized_weights=table_name_to_quantized_weights,
            register_tbes=getattr(module, MODULE_ATTR_REGISTER_TBES_BOOL, False),
            quant_state_dict_split_scale_bias=getattr(
                module, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, False
            ),
            row_alignment=getattr(module, MODULE_ATTR_ROW_ALIGNMENT_INT, DEFAULT_ROW_ALIGNMENT),
            cache_features_order=getattr(module, MODULE_ATTR_CACHE_FEATURES_ORDER, False),
        )

    def embedding_bag_configs(self) -> List[EmbeddingBagConfig]:
        return self._embedding_bag_configs

    def is_weighted(self) -> bool:
        return self._is_weighted

    def output_dtype(self) -> torch.dtype:
        return self._output_dtype

    @property
    def device(self) -> torch.device:
        return self._device


# The lookup kernel keeps the position-weight layout of a launch in its launch
# arguments: at most this many features per operator.
_MAX_FUSED_POSITION_FEATURES = 128


class FeatureProcessedEmbeddingBagCollection(EmbeddingBagCollection):
    """Quantized collection behind a feature processor
    (torchrec/quant/embedding_modules.py:633-731): ``forward`` first lets
    ``feature_processor`` attach per-id weights to the KJT, then runs the
    weighted lookup."""

    def __init__(
        self,
        tables: List[EmbeddingBagConfig],
        is_weighted: bool,
        device: torch.device,
        output_dtype: torch.dtype = torch.float,
        table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = None,
        register_tbes: bool = False,
        quant_state_dict_split_scale_bias: bool = False,
        row_alignment: int = DEFAULT_ROW_ALIGNMENT,
        # Optional only because it is the last positional argument; without a
        # feature processor use EmbeddingBagCollection.
        feature_processor: Optional[FeatureProcessorsCollection] = None,
        cache_features_order: bool = False,
    ) -> None:
        super().__init__(
            tables,
            is_weighted,
            device,
            output_dtype,
            table_name_to_quantized_weights,
            register_tbes,
            quant_state_dict_split_scale_bias,
            row_alignment,
            cache_features_order,
        )
        assert feature_processor is not None, "Use EmbeddingBagCollection for no feature_processor"
        self.feature_processor: FeatureProcessorsCollection = feature_processor

    def forward(self, features: KeyedJaggedTensor) -> KeyedTensor:  # type: ignore[override]
        # Position weights on the GPU are looked up inside the lookup kernel: no
        # weight tensor is written and read back, and no weighted KJT is built.
        fp = self.feature_processor
        if (
            isinstance(fp, PositionWeightedModuleCollection)
            and features.values().device.type == "cuda"
            and features.keys()
            and all(len(op.feature_table_map) <= _MAX_FUSED_POSITION_FEATURES for op in self._emb_modules)
        ):
            return super().forward(features, position_weights=fp.kernel_layout(features.keys(), features.values().device))
        return super().forward(fp(features))

    def _get_name(self) -> str:
        return "QuantFeatureProcessedEmbeddingBagCollection"

    @classmethod
    def from_float(  # type: ignore[override]
        cls, module: OriginalFeatureProcessedEmbeddingBagCollection, use_precomputed_fake_quant: bool = False
    ) -> "FeatureProcessedEmbeddingBagCollection":
        assert hasattr(
            module, "qconfig"
        ), "FeatureProcessedEmbeddingBagCollection input float module must have qconfig defined"
        ebc = module._embedding_bag_collection
        qconfig = module.qconfig
        pruning_dict: Dict[str, int] = getattr(
            module, MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT, {}
        )
        embedding_bag_configs = copy.deepcopy(ebc.embedding_bag_configs())
        _update_embedding_configs(embedding_bag_configs, qconfig, pruning_dict)
        table_name_to_quantized_weights: Dict[str, Tuple[Tensor, Tensor]] = {}
        device = quantize_state_dict(
            ebc,
            table_name_to_quantized_weights,
            {table.name: table.data_type for table in embedding_bag_configs},
            pruning_dict,
        )
        feature_processor, _ = module.split()  # a per-feature dict is wrapped into a collection
        return cls(
            embedding_bag_configs,
            ebc.is_weighted(),
            device=device,
            output_dtype=qconfig.activation().dtype,
            table_name_to_quantized_weights=table_name_to_quantized_weights,
            register_tbes=getattr(module, MODULE_ATTR_REGISTER_TBES_BOOL, False),
            quant_state_dict_split_scale_bias=getattr(ebc, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, False),
            row_alignment=getattr(ebc, MODULE_ATTR_ROW_ALIGNMENT_INT, DEFAULT_ROW_ALIGNMENT),
            feature_processor=feature_processor,
            cache_features_order=getattr(module, MODULE_ATTR_CACHE_FEATURES_ORDER, False),
        )


# ---------------------------------------------------------------------------
# sequence
# ---------------------------------------------------------------------------
class EmbeddingCollection(EmbeddingCollectionInterface, ModuleNoCopyMixin, _FeatureOrderMixin):
    """Quantized per-id embeddings: ``forward(KeyedJaggedTensor) -> Dict[str, JaggedTensor]``.

    Tables are grouped by ``(data_type, use_virtual_table)``; all share one dim.
    """

    def __init__(  # noqa C901
        self,
        tables: List[EmbeddingConfig],
        device: torch.device,
        need_indices: bool = False,
        output_dtype: torch.dtype = torch.float,
        table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = None,
        register_tbes: bool = False,
        quant_state_dict_split_scale_bias: bool = False,
        row_alignment: int = DEFAULT_ROW_ALIGNMENT,
        cache_features_order: bool = False,
    ) -> None:
        super().__init__()
        self._emb_modules: List[IntNBitTableBatchedEmbeddingBagsCodegen] = []
        self._embedding_configs = tables
        self._embedding_dim: int = -1
        self._need_indices: bool = need_indices
        self._output_dtype = output_dtype
        self._device = torch.device(device)
        self.row_alignment = row_alignment
        self._key_to_tables: Dict[Tuple[DataType, bool], List[EmbeddingConfig]] = defaultdict(list)
        self._feature_names: List[str] = []
        self._features_order: Optional[List[int]] = None
        self._table_name_to_quantized_weights = table_name_to_quantized_weights

        table_names = set()
        for table in self._embedding_configs:
            if table.name in table_names:
                raise ValueError(f"Duplicate table name {table.name}")
            table_names.add(table.name)
            self._embedding_dim = table.embedding_dim if self._embedding_dim < 0 else self._embedding_dim
            if self._embedding_dim != table.embedding_dim:
                raise ValueError(
                    "All tables in a EmbeddingCollection are required to have same embedding dimension."
                    + f" Violating case: {table.name}'s embedding_dim {table.embedding_dim} !="
                    + f" {self._embedding_dim}"
                )
            if getattr(table, "use_virtual_table", False):
                raise NotImplementedError("virtual (KV-backed) tables are not supported")
            self._key_to_tables[(table.data_type, False)].append(table)

        self._feature_splits: List[int] = []
        for (_data_type, _virtual), emb_configs in self._key_to_tables.items():
            self._emb_modules.append(
                _build_tbe(
                    emb_configs,
                    PoolingMode.NONE,
                    self._device,
                    output_dtype,
                    row_alignment,
                    table_name_to_quantized_weights,
                    use_post_pruning_rows=False,
                )
            )
            for table in emb_configs:
                self._feature_names.extend(table.feature_names)
            self._feature_splits.append(sum(table.num_features() for table in emb_configs))

        self.embeddings: nn.ModuleDict = nn.ModuleDict()
        for (_key, group_tables), emb_module in zip(self._key_to_tables.items(), self._emb_modules):
            _register_table_buffers(
                self.embeddings, group_tables, emb_module, quant_state_dict_split_scale_bias
            )

        self._embedding_names_by_batched_tables: Dict[Tuple[DataType, bool], List[str]] = {
            key: list(itertools.chain(*get_embedding_names_by_table(group)))
            for key, group in self._key_to_tables.items()
        }
        self._embedding_names_by_table: List[List[str]] = get_embedding_names_by_table(
            self._embedding_configs
        )
        setattr(self, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, quant_state_dict_split_scale_bias)
        setattr(self, MODULE_ATTR_REGISTER_TBES_BOOL, register_tbes)
        self.register_tbes = register_tbes
        if register_tbes:
            self.tbes: torch.nn.ModuleList = torch.nn.ModuleList(self._emb_modules)
        setattr(self, MODULE_ATTR_CACHE_FEATURES_ORDER, cache_features_order)

    def forward(self, features: KeyedJaggedTensor) -> Dict[str, JaggedTensor]:
        """Each feature's JaggedTensor is a row range (view) of one ``[L, D]`` lookup buffer."""
        kjt_keys = _get_kjt_keys(features)
        order = self._resolve_order(kjt_keys)
        if len(set(order)) != len(order):
            # A feature feeding two tables needs two distinct row ranges in the
            # output: materialize the repeated ids once.
            features = features.permute(order)
            kjt_keys = features.keys()
            order = list(range(len(order)))
        B = features.stride()
        indices = features.values()
        offsets = features.offsets()
        lengths = features.lengths()
        L = indices.numel()
        # Row ranges of the input keys: one small device-to-host copy.  Where the
        # KJT does not carry the per-key counts, their reduction and copy are
        # queued in front of the lookup and waited for behind its launch: the
        # host then waits for work that is already queued and builds the output
        # views while the lookup runs, and the lookup never waits for the host.
        counts_later = None
        if (
            features.length_per_key_or_none() is None
            and features.offset_per_key_or_none() is None
            and indices.is_cuda
            and kjt_keys
            and L > 0
            and B > 0
        ):
            counts_later = ops.length_per_key_async(features.lengths(), len(kjt_keys), B)
        else:
            offset_per_key = features.offset_per_key()
        lookup = torch.empty((L, self._embedding_dim), dtype=self._output_dtype, device=indices.device)
        try:
            f0 = 0
            for emb_module, n_feat in zip(self._emb_modules, self._feature_splits):
                # (a registered operator is called as a module, torchrec/quant/embedding_modules.py:938-942)
                call = emb_module if self.register_tbes else emb_module.forward
                call(
                    indices=indices,
                    offsets=offsets,
                    feature_positions=order[f0 : f0 + n_feat],
                    batch_size=B,
                    out=lookup,
                )
                f0 += n_feat
        finally:
            # The reduction queued on the side stream reads the KJT's lengths: it is waited for
            # also when a lookup raises, before anything of this call is released.
            if counts_later is not None:
                features._length_per_key = counts_later()  # the KJT remembers them, as length_per_key() would
        if counts_later is not None:
            offset_per_key = features.offset_per_key()
        # The batching hint sees the flattened lengths by default and the [F, B] lengths when the
        # module is prepared for it (torchrec/quant/embedding_modules.py:943-950); here the lengths
        # are those of the whole KJT, because all operators write one buffer.
        if getattr(self, MODULE_ATTR_USE_UNFLATTENED_LENGTHS_FOR_BATCHING, False):
            if kjt_keys:
                lengths = _get_unflattened_lengths(features.lengths(), len(kjt_keys))
            lookup = _get_batching_hinted_output(lengths=lengths, output=lookup)
        else:
            if getattr(self, MODULE_ATTR_USE_BATCHING_HINTED_OUTPUT, True):
                lookup = _get_batching_hinted_output(lengths=features.lengths(), output=lookup)
            if kjt_keys:
                lengths = _get_unflattened_lengths(features.lengths(), len(kjt_keys))
        if getattr(self, MODULE_ATTR_REMOVE_STBE_PADDING_BOOL, False):
            # Rows past the last id that belongs to a bag (a padded values tensor) are dropped
            # (construct_jagged_tensors_inference(remove_padding=True), torchrec/modules/utils.py:315-316).
            lookup = lookup[: offset_per_key[-1]]
        lengths_rows = torch.unbind(lengths, dim=0) if kjt_keys else ()
        feature_embeddings: Dict[str, JaggedTensor] = {}
        f = 0
        for key in self._key_to_tables.keys():
            for embedding_name in self._embedding_names_by_batched_tables[key]:
                pos = order[f]
                start, end = offset_per_key[pos], offset_per_key[pos + 1]
                rows = self._rows_for(lookup, f, start, end)
                feature_embeddings[embedding_name] = JaggedTensor(
                    values=rows,
                    lengths=lengths_rows[pos],
                    weights=indices[start:end] if self._need_indices else None,
                )
                f += 1
        return feature_embeddings

    def _rows_for(self, lookup: Tensor, f: int, start: int, end: int) -> Tensor:
        return lookup[start:end]

    @classmethod
    def from_float(
        cls, module: OriginalEmbeddingCollection, use_precomputed_fake_quant: bool = False
    ) -> "EmbeddingCollection":
        assert hasattr(module, "qconfig"), "EmbeddingCollection input float module must have qconfig defined"
        embedding_configs = copy.deepcopy(module.embedding_configs())
        _update_embedding_configs(embedding_configs, module.qconfig)
        table_name_to_quantized_weights: Dict[str, Tuple[Tensor, Tensor]] = {}
        device = quantize_state_dict(
            module,
            table_name_to_quantized_weights,
            {table.name: table.data_type for table in embedding_configs},
        )
        return cls(
            embedding_configs,
            device=device,
            need_indices=module.need_indices(),
            output_dtype=module.qconfig.activation().dtype,
            table_name_to_quantized_weights=table_name_to_quantized_weights,
            register_tbes=getattr(module, MODULE_ATTR_REGISTER_TBES_BOOL, False),
            quant_state_dict_split_scale_bias=getattr(
                module, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, False
            ),
            row_alignment=getattr(module, MODULE_ATTR_ROW_ALIGNMENT_INT, DEFAULT_ROW_ALIGNMENT),
            cache_features_order=getattr(module, MODULE_ATTR_CACHE_FEATURES_ORDER, False),
        )

    def _get_name(self) -> str:
        return "QuantizedEmbeddingCollection"

    def need_indices(self) -> bool:
        return self._need_indices

    def embedding_dim(self) -> int:
        return self._embedding_dim

    def embedding_configs(self) -> List[EmbeddingConfig]:
        return self._embedding_configs

    def embedding_names_by_table(self) -> List[List[str]]:
        return self._embedding_names_by_table

    def output_dtype(self) -> torch.dtype:
        return self._output_dtype

    @property
    def device(self) -> torch.device:
        return self._device


class QuantManagedCollisionEmbeddingCollection(EmbeddingCollection):
    """Quantized sequence collection behind managed-collision id remapping
    (torchrec/quant/embedding_modules.py:1029-1177): ``forward`` remaps the
    KJT's ids with ``managed_collision_collection`` and returns
    ``(embeddings, remapped features)``."""

    def __init__(
        self,
        tables: List[EmbeddingConfig],
        device: torch.device,
        need_indices: bool = False,
        output_dtype: torch.dtype = torch.float,
        table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = None,
        register_tbes: bool = False,
        quant_state_dict_split_scale_bias: bool = False,
        row_alignment: int = DEFAULT_ROW_ALIGNMENT,
        managed_collision_collection: Optional[ManagedCollisionCollection] = None,
        return_remapped_features: bool = False,
        cache_features_order: bool = False,
    ) -> None:
        super().__init__(
            tables,
            device,
            need_indices,
            output_dtype,
            table_name_to_quantized_weights,
            register_tbes,
            quant_state_dict_split_scale_bias,
            row_alignment,
            cache_features_order,
        )
        assert managed_collision_collection, "Managed collision collection cannot be None"
        self._managed_collision_collection: ManagedCollisionCollection = managed_collision_collection
        self._return_remapped_features = return_remapped_features
        assert str(self.embedding_configs()) == str(
            self._managed_collision_collection.embedding_configs()
        ), "Embedding Collection and Managed Collision Collection must contain the same Embedding Configs"
        # the quantized form serves inference only
        for mc_module in self._managed_collision_collection._managed_collision_modules.values():
            mc_module.reset_inference_mode()
            mc_module.eval()

    def forward(  # type: ignore[override]
        self, features: KeyedJaggedTensor
    ) -> Tuple[Dict[str, JaggedTensor], Optional[KeyedJaggedTensor]]:
        features = self._managed_collision_collection(features)
        return (super().forward(features), features)

    def _get_name(self) -> str:
        return "QuantManagedCollisionEmbeddingCollection"

    @classmethod
    def from_float(  # type: ignore[override]
        cls, module: OriginalManagedCollisionEmbeddingCollection, return_remapped_features: bool = False
    ) -> "QuantManagedCollisionEmbeddingCollection":
        assert hasattr(
            module, "qconfig"
        ), "QuantManagedCollisionEmbeddingCollection input float module must have qconfig defined"
        ec = module._embedding_module
        qconfig = module.qconfig
        embedding_configs = copy.deepcopy(ec.embedding_configs())
        _update_embedding_configs(embedding_configs, qconfig)
        _update_embedding_configs(module._managed_collision_collection._embedding_configs, qconfig)
        # The reference takes weights only from a precomputed dict on the float
        # module (else the tables are filled later from a state_dict); here the
        # float weights are quantized when they exist.
        table_name_to_quantized_weights: Optional[Dict[str, Tuple[Tensor, Tensor]]] = getattr(
            ec, "_table_name_to_quantized_weights", None
        )
        device = _get_device(ec)
        if table_name_to_quantized_weights is None and device.type != "meta":
            table_name_to_quantized_weights = {}
            quantize_state_dict(
                ec, table_name_to_quantized_weights, {t.name: t.data_type for t in embedding_configs}
            )
        return cls(
            embedding_configs,
            device=device,
            output_dtype=qconfig.activation().dtype,
            table_name_to_quantized_weights=table_name_to_quantized_weights,
            register_tbes=getattr(module, MODULE_ATTR_REGISTER_TBES_BOOL, False),
            quant_state_dict_split_scale_bias=getattr(ec, MODULE_ATTR_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, False),
            row_alignment=getattr(ec, MODULE_ATTR_ROW_ALIGNMENT_INT, DEFAULT_ROW_ALIGNMENT),
            managed_collision_collection=module._managed_collision_collection,
            return_remapped_features=module._return_remapped_features,
            cache_features_order=getattr(ec, MODULE_ATTR_CACHE_FEATURES_ORDER, False),
        )

