"""Entry points that turn a float model into its quantized inference form
(torchrec/inference/modules.py): ``quantize_embeddings`` :139-169,
``quantize_dense`` :318-343, ``set_pruning_data`` :357-373,
``quantize_inference_model`` :376-490, ``get_table_to_weights_from_tbe`` /
``assign_weights_to_tbe`` :628-655.  The swap itself is
``torch.quantization.quantize_dynamic`` with the ``from_float`` constructors of
``torchrec_amd.quant``; sharding a quantized model over several GPUs
(``shard_quant_model`` :493-625) is not part of this one-GPU build.
"""
from __future__ import annotations

import abc
import logging
from typing import Any, Dict, List, Optional, Tuple, Type

import torch
import torch.nn as nn
import torch.quantization as quant

from torchrec_amd import quant as trec_quant
from torchrec_amd.modules.embedding_configs import QuantConfig
from torchrec_amd.modules.embedding_modules import (
    EmbeddingBagCollection,
    EmbeddingBagCollectionInterface,
    EmbeddingCollection,
    EmbeddingCollectionInterface,
)
from torchrec_amd.modules.fp_embedding_modules import FeatureProcessedEmbeddingBagCollection
from torchrec_amd.quant.embedding_modules import (
    EmbeddingBagCollection as QuantEmbeddingBagCollection,
    EmbeddingCollection as QuantEmbeddingCollection,
    FeatureProcessedEmbeddingBagCollection as QuantFeatureProcessedEmbeddingBagCollection,
    MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT,
    quant_prep_enable_cache_features_order,
    quant_prep_enable_register_tbes,
)
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen,
)

logger: logging.Logger = logging.getLogger(__name__)


def trim_torch_package_prefix_from_typename(typename: str) -> str:
    if typename.startswith("<torch_package_"):
        typename = ".".join(typename.split(".")[1:])
    return typename


DEFAULT_QUANT_MAPPING: Dict[str, Type[torch.nn.Module]] = {
    trim_torch_package_prefix_from_typename(torch.typename(EmbeddingBagCollection)): QuantEmbeddingBagCollection,
    trim_torch_package_prefix_from_typename(torch.typename(EmbeddingCollection)): QuantEmbeddingCollection,
}
DEFAULT_QUANTIZATION_DTYPE: torch.dtype = torch.int8
FEATURE_PROCESSED_EBC_TYPE: str = trim_torch_package_prefix_from_typename(
    torch.typename(FeatureProcessedEmbeddingBagCollection)
)


def quantize_feature(module: torch.nn.Module, inputs: Tuple[torch.Tensor, ...]) -> Tuple[torch.Tensor, ...]:
    """Forward pre-hook of fp16-lowered dense modules: float inputs become half."""
    return tuple(
        i.half() if isinstance(i, torch.Tensor) and i.dtype in (torch.float32, torch.float64) else i for i in inputs
    )


def quantize_embeddings(
    module: nn.Module,
    dtype: torch.dtype,
    inplace: bool,
    additional_qconfig_spec_keys: Optional[List[Type[nn.Module]]] = None,
    additional_mapping: Optional[Dict[Type[nn.Module], Type[nn.Module]]] = None,
    output_dtype: torch.dtype = torch.float,
    per_table_weight_dtype: Optional[Dict[str, torch.dtype]] = None,
) -> nn.Module:
    """Swaps every EmbeddingBagCollection (and the additional module types) for
    its quantized counterpart; ``dtype`` is the weight type (torch.qint8 / int8,
    quint4x2, quint2x4, half), ``per_table_weight_dtype`` overrides it per table."""
    qconfig = QuantConfig(
        activation=quant.PlaceholderObserver.with_args(dtype=output_dtype),
        weight=quant.PlaceholderObserver.with_args(dtype=dtype),
        per_table_weight_dtype=per_table_weight_dtype,
    )
    qconfig_spec: Dict[Type[nn.Module], QuantConfig] = {EmbeddingBagCollection: qconfig}
    mapping: Dict[Type[nn.Module], Type[nn.Module]] = {EmbeddingBagCollection: trec_quant.EmbeddingBagCollection}
    for t in additional_qconfig_spec_keys or []:
        qconfig_spec[t] = qconfig
    if additional_mapping is not None:
        mapping.update(additional_mapping)
    return quant.quantize_dynamic(module, qconfig_spec=qconfig_spec, mapping=mapping, inplace=inplace)


class PredictModule(nn.Module):
    """Serving wrapper: subclasses turn a dict of input tensors into the wrapped
    module's arguments in ``predict_forward``; ``forward`` runs it under
    ``torch.inference_mode`` (torchrec/inference/modules.py:262-315)."""

    def __init__(self, module: nn.Module, device: Optional[str] = None) -> None:
        super().__init__()
        self._module: nn.Module = module
        self._device: Optional[torch.device] = torch.device(device) if device else None
        self._module.eval()

    @property
    def predict_module(self) -> nn.Module:
        return self._module

    @abc.abstractmethod
    def predict_forward(self, batch: Dict[str, torch.Tensor]) -> Any: ...

    def forward(self, batch: Dict[str, torch.Tensor]) -> Any:
        if self._device is None:
            self._device = torch.device("cuda", torch.cuda.current_device())
        with torch.inference_mode():
            return self.predict_forward(batch)

    def state_dict(self, destination=None, prefix: str = "", keep_vars: bool = False) -> Dict[str, Any]:  # type: ignore[override]
        return self._module.state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)


def quantize_dense(
    predict_module: PredictModule, dtype: torch.dtype, additional_embedding_module_type: List[Type[nn.Module]] = []
) -> nn.Module:
    """Lowers every child that is not an embedding collection to fp16."""
    module = predict_module.predict_module
    reassign = {}
    for name, mod in module.named_children():
        if not (
            isinstance(mod, (EmbeddingBagCollectionInterface, EmbeddingCollectionInterface))
            or any(type(mod) is clazz for clazz in additional_embedding_module_type)
        ):
            if dtype != torch.half:
                raise NotImplementedError("only fp16 is supported for non-embedding module lowering")
            new_mod = mod.half()
            new_mod.register_forward_pre_hook(quantize_feature)
            reassign[name] = new_mod
    for key, value in reassign.items():
        module._modules[key] = value
    return predict_module


def set_pruning_data(
    model: torch.nn.Module,
    tables_to_rows_post_pruning: Dict[str, int],
    module_types: Optional[List[Type[nn.Module]]] = None,
) -> torch.nn.Module:
    """Marks the collections so that quantization keeps only the first
    ``tables_to_rows_post_pruning[table]`` rows of each listed table."""
    if module_types is None:
        module_types = [EmbeddingBagCollection, FeatureProcessedEmbeddingBagCollection]
    for _, module in model.named_modules():
        if type(module) in module_types:
            setattr(module, MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT, tables_to_rows_post_pruning)
    return model


def _get_submodule_parent(model: nn.Module, fqn: str) -> Tuple[nn.Module, str]:
    parent_fqn, _, name = fqn.rpartition(".")
    return (model.get_submodule(parent_fqn) if parent_fqn else model), name


def quantize_inference_model(
    model: torch.nn.Module,
    quantization_mapping: Optional[Dict[str, Type[torch.nn.Module]]] = None,
    per_table_weight_dtype: Optional[Dict[str, torch.dtype]] = None,
    fp_weight_dtype: torch.dtype = DEFAULT_QUANTIZATION_DTYPE,
    quantization_dtype: torch.dtype = DEFAULT_QUANTIZATION_DTYPE,
    output_dtype: torch.dtype = torch.float,
) -> torch.nn.Module:
    """Module-swaps the float collections of ``model`` for the quantized ones, in
    place: EmbeddingBagCollection -> QuantEmbeddingBagCollection,
    EmbeddingCollection -> QuantEmbeddingCollection (or ``quantization_mapping``,
    keyed by type name), FeatureProcessedEmbeddingBagCollection -> its quantized
    form with ``fp_weight_dtype`` tables."""
    if quantization_mapping is None:
        quantization_mapping = DEFAULT_QUANT_MAPPING

    additional_qconfig_spec_keys: List[Type[nn.Module]] = []
    additional_mapping: Dict[Type[nn.Module], Type[nn.Module]] = {}
    fp_modules: List[Tuple[str, FeatureProcessedEmbeddingBagCollection]] = []
    for n, m in model.named_modules():
        typename = trim_torch_package_prefix_from_typename(torch.typename(m))
        if typename in quantization_mapping:
            additional_qconfig_spec_keys.append(type(m))
            additional_mapping[type(m)] = quantization_mapping[typename]
        elif typename == FEATURE_PROCESSED_EBC_TYPE:
            fp_modules.append((n, m))  # type: ignore[arg-type]

    # Feature-processed collections are swapped directly (their tables live in
    # the wrapped collection, which must not be swapped on its own afterwards).
    for fqn, fp_module in fp_modules:
        quant_prep_enable_register_tbes(model, [FeatureProcessedEmbeddingBagCollection])
        quant_prep_enable_cache_features_order(model, [FeatureProcessedEmbeddingBagCollection])
        fp_module.qconfig = QuantConfig(  # type: ignore[assignment]
            activation=quant.PlaceholderObserver.with_args(dtype=output_dtype),
            weight=quant.PlaceholderObserver.with_args(dtype=fp_weight_dtype),
            per_table_weight_dtype=per_table_weight_dtype,
        )
        parent, name = _get_submodule_parent(model, fqn)
        parent.register_module(name, QuantFeatureProcessedEmbeddingBagCollection.from_float(fp_module))

    quant_prep_enable_register_tbes(model, list(additional_mapping.keys()))
    quant_prep_enable_cache_features_order(model, [EmbeddingBagCollection, EmbeddingCollection])
    quantize_embeddings(
        model,
        dtype=quantization_dtype,
        additional_qconfig_spec_keys=additional_qconfig_spec_keys,
        additional_mapping=additional_mapping,
        inplace=True,
        per_table_weight_dtype=per_table_weight_dtype,
        output_dtype=output_dtype,
    )
    logger.info(f"Default quantization dtype is {quantization_dtype}, {per_table_weight_dtype=}.")
    return model


def shard_quant_model(*args: Any, **kwargs: Any) -> Any:
    raise NotImplementedError(
        "shard_quant_model places table shards on several GPUs; this build runs the quantized path on one GPU"
    )


def get_table_to_weights_from_tbe(
    model: torch.nn.Module,
) -> Dict[str, Tuple[torch.Tensor, Optional[torch.Tensor]]]:
    """table name -> (payload bytes, scale_bias bytes or None) of every lookup operator in ``model``."""
    table_to_weight = {}
    for module in model.modules():
        if isinstance(module, IntNBitTableBatchedEmbeddingBagsCodegen):
            weights = module.split_embedding_weights()
            for i, spec in enumerate(module.embedding_specs):
                table_to_weight[spec[0]] = weights[i]
    return table_to_weight


def assign_weights_to_tbe(
    model: torch.nn.Module, table_to_weight: Dict[str, Tuple[torch.Tensor, Optional[torch.Tensor]]]
) -> None:
    """Copies ``table_to_weight`` (as returned above) into the operators of ``model``."""
    for module in model.modules():
        if isinstance(module, IntNBitTableBatchedEmbeddingBagsCodegen):
            q_weights = []
            for spec in module.embedding_specs:
                assert spec[0] in table_to_weight, f"{spec[0]} not in table_to_weight"
                q_weights.append(table_to_weight[spec[0]])
            module.assign_embedding_weights(q_weights)
