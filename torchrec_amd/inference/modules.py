"""Entry points that turn a float model into its quantized inference form.

Same names and arguments as torchrec/inference/modules.py:
``quantize_embeddings`` (:139-169), ``quantize_dense`` (:318-343),
``set_pruning_data`` (:357-373), ``quantize_inference_model`` (:376-490),
``get_table_to_weights_from_tbe`` / ``assign_weights_to_tbe`` (:628-655),
``PredictModule`` (:262-315).  The swap itself is torch's
``quantize_dynamic`` driving the ``from_float`` constructors of
``torchrec_amd.quant``.  ``shard_quant_model`` (:493-625) spreads tables over
several GPUs and is refused here: this build runs on one.
"""
from __future__ import annotations

import abc
import logging
from typing import Any, Dict, Iterator, List, Optional, Tuple, Type

import torch
import torch.nn as nn
from torch.quantization import PlaceholderObserver, quantize_dynamic

from torchrec_amd.modules import embedding_modules as float_modules
from torchrec_amd.modules.embedding_configs import QuantConfig
from torchrec_amd.modules.fp_embedding_modules import FeatureProcessedEmbeddingBagCollection
from torchrec_amd.quant import embedding_modules as quant_modules
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen,
)

logger: logging.Logger = logging.getLogger(__name__)

EmbeddingBagCollection = float_modules.EmbeddingBagCollection
EmbeddingCollection = float_modules.EmbeddingCollection
QuantEmbeddingBagCollection = quant_modules.EmbeddingBagCollection
QuantEmbeddingCollection = quant_modules.EmbeddingCollection
QuantFeatureProcessedEmbeddingBagCollection = quant_modules.FeatureProcessedEmbeddingBagCollection


def trim_torch_package_prefix_from_typename(typename: str) -> str:
    """``<torch_package_3>.a.b.C`` -> ``a.b.C`` (type names of packaged models)."""
    head, _, rest = typename.partition(".")
    return rest if head.startswith("<torch_package_") else typename


def _typename(obj: Any) -> str:
    return trim_torch_package_prefix_from_typename(torch.typename(obj))


DEFAULT_QUANTIZATION_DTYPE: torch.dtype = torch.int8
DEFAULT_QUANT_MAPPING: Dict[str, Type[torch.nn.Module]] = {
    _typename(EmbeddingBagCollection): QuantEmbeddingBagCollection,
    _typename(EmbeddingCollection): QuantEmbeddingCollection,
}
FEATURE_PROCESSED_EBC_TYPE: str = _typename(FeatureProcessedEmbeddingBagCollection)


def _qconfig(weight_dtype: torch.dtype, output_dtype: torch.dtype,
             per_table_weight_dtype: Optional[Dict[str, torch.dtype]]) -> QuantConfig:
    return QuantConfig(
        activation=PlaceholderObserver.with_args(dtype=output_dtype),
        weight=PlaceholderObserver.with_args(dtype=weight_dtype),
        per_table_weight_dtype=per_table_weight_dtype,
    )


def quantize_feature(module: torch.nn.Module, inputs: Tuple[torch.Tensor, ...]) -> Tuple[torch.Tensor, ...]:
    """Forward pre-hook of fp16-lowered dense modules: float inputs become half."""
    def lower(x: Any) -> Any:
        is_float = isinstance(x, torch.Tensor) and x.dtype in (torch.float32, torch.float64)
        return x.half() if is_float else x

    return tuple(lower(x) for x in inputs)


def quantize_embeddings(module: nn.Module, dtype: torch.dtype, inplace: bool,
                        additional_qconfig_spec_keys: Optional[List[Type[nn.Module]]] = None,
                        additional_mapping: Optional[Dict[Type[nn.Module], Type[nn.Module]]] = None,
                        output_dtype: torch.dtype = torch.float,
                        per_table_weight_dtype: Optional[Dict[str, torch.dtype]] = None) -> nn.Module:
    """Swaps every EmbeddingBagCollection (and the additional module types) for
    its quantized counterpart.  ``dtype`` is the weight type (torch.qint8 / int8,
    quint4x2, quint2x4, half); ``per_table_weight_dtype`` overrides it per table."""
    qconfig = _qconfig(dtype, output_dtype, per_table_weight_dtype)
    swap: Dict[Type[nn.Module], Type[nn.Module]] = {EmbeddingBagCollection: QuantEmbeddingBagCollection}
    swap.update(additional_mapping or {})
    spec_types = [EmbeddingBagCollection, *(additional_qconfig_spec_keys or [])]
    return quantize_dynamic(module, qconfig_spec={t: qconfig for t in spec_types}, mapping=swap, inplace=inplace)


class PredictModule(nn.Module):
    """Serving wrapper: a subclass turns a dict of input tensors into the wrapped
    module's arguments in ``predict_forward``; ``forward`` runs it under
    ``torch.inference_mode``."""

    def __init__(self, module: nn.Module, device: Optional[str] = None) -> None:
        super().__init__()
        self._module: nn.Module = module.eval()
        self._device: Optional[torch.device] = None if not device else torch.device(device)

    @property
    def predict_module(self) -> nn.Module:
        return self._module

    @abc.abstractmethod
    def predict_forward(self, batch: Dict[str, torch.Tensor]) -> Any: ...

    def forward(self, batch: Dict[str, torch.Tensor]) -> Any:
        if self._device is None:  # resolved lazily: the serving thread picks the device
            self._device = torch.device("cuda", torch.cuda.current_device())
        with torch.inference_mode():
            return self.predict_forward(batch)

    def state_dict(self, destination=None, prefix: str = "", keep_vars: bool = False) -> Dict[str, Any]:  # type: ignore[override]
        return self._module.state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)


def quantize_dense(predict_module: PredictModule, dtype: torch.dtype,
                   additional_embedding_module_type: List[Type[nn.Module]] = []) -> nn.Module:
    """Lowers every direct child that is not an embedding collection to fp16."""
    if dtype != torch.half:
        raise NotImplementedError("only fp16 is supported for non-embedding module lowering")
    embedding_types = (float_modules.EmbeddingBagCollectionInterface, float_modules.EmbeddingCollectionInterface)
    root = predict_module.predict_module
    for name, child in list(root.named_children()):
        if isinstance(child, embedding_types) or type(child) in additional_embedding_module_type:
            continue
        lowered = child.half()
        lowered.register_forward_pre_hook(quantize_feature)
        root._modules[name] = lowered
    return predict_module


def set_pruning_data(model: torch.nn.Module, tables_to_rows_post_pruning: Dict[str, int],
                     module_types: Optional[List[Type[nn.Module]]] = None) -> torch.nn.Module:
    """Marks the collections so that quantization keeps only the first
    ``tables_to_rows_post_pruning[table]`` rows of each listed table."""
    wanted = module_types or [EmbeddingBagCollection, FeatureProcessedEmbeddingBagCollection]
    attr = quant_modules.MODULE_ATTR_EMB_CONFIG_NAME_TO_NUM_ROWS_POST_PRUNING_DICT
    for candidate in model.modules():
        if type(candidate) in wanted:
            setattr(candidate, attr, tables_to_rows_post_pruning)
    return model


def quantize_inference_model(model: torch.nn.Module,
                             quantization_mapping: Optional[Dict[str, Type[torch.nn.Module]]] = None,
                             per_table_weight_dtype: Optional[Dict[str, torch.dtype]] = None,
                             fp_weight_dtype: torch.dtype = DEFAULT_QUANTIZATION_DTYPE,
                             quantization_dtype: torch.dtype = DEFAULT_QUANTIZATION_DTYPE,
                             output_dtype: torch.dtype = torch.float) -> torch.nn.Module:
    """Module-swaps the float collections of ``model`` for the quantized ones, in
    place: EmbeddingBagCollection -> QuantEmbeddingBagCollection,
    EmbeddingCollection -> QuantEmbeddingCollection (or ``quantization_mapping``,
    keyed by type name), FeatureProcessedEmbeddingBagCollection -> its quantized
    form with ``fp_weight_dtype`` tables."""
    by_typename = DEFAULT_QUANT_MAPPING if quantization_mapping is None else quantization_mapping
    swap: Dict[Type[nn.Module], Type[nn.Module]] = {}
    feature_processed: List[str] = []
    for fqn, sub in model.named_modules():
        name = _typename(sub)
        if name in by_typename:
            swap[type(sub)] = by_typename[name]
        elif name == FEATURE_PROCESSED_EBC_TYPE:
            feature_processed.append(fqn)

    # A feature-processed collection is replaced as a whole: its tables live in
    # the collection it wraps, which must not be swapped on its own afterwards.
    fp_types = [FeatureProcessedEmbeddingBagCollection]
    for fqn in feature_processed:
        quant_modules.quant_prep_enable_register_tbes(model, fp_types)
        quant_modules.quant_prep_enable_cache_features_order(model, fp_types)
        fp_module = model.get_submodule(fqn)
        fp_module.qconfig = _qconfig(fp_weight_dtype, output_dtype, per_table_weight_dtype)  # type: ignore[assignment]
        parent_fqn, _, child = fqn.rpartition(".")
        model.get_submodule(parent_fqn).register_module(
            child, QuantFeatureProcessedEmbeddingBagCollection.from_float(fp_module)
        )

    quant_modules.quant_prep_enable_register_tbes(model, list(swap))
    quant_modules.quant_prep_enable_cache_features_order(model, [EmbeddingBagCollection, EmbeddingCollection])
    quantize_embeddings(model, quantization_dtype, True, additional_qconfig_spec_keys=list(swap),
                        additional_mapping=swap, output_dtype=output_dtype,
                        per_table_weight_dtype=per_table_weight_dtype)
    logger.info("quantized with default dtype %s, per-table overrides %s", quantization_dtype, per_table_weight_dtype)
    return model


def shard_quant_model(*args: Any, **kwargs: Any) -> Any:
    raise NotImplementedError(
        "shard_quant_model places table shards on several GPUs; this build runs the quantized path on one GPU"
    )


def _lookup_operators(model: torch.nn.Module) -> Iterator[IntNBitTableBatchedEmbeddingBagsCodegen]:
    return (m for m in model.modules() if isinstance(m, IntNBitTableBatchedEmbeddingBagsCodegen))


def get_table_to_weights_from_tbe(
    model: torch.nn.Module,
) -> Dict[str, Tuple[torch.Tensor, Optional[torch.Tensor]]]:
    """table name -> (payload bytes, scale_bias bytes or None) of every lookup operator in ``model``."""
    found: Dict[str, Tuple[torch.Tensor, Optional[torch.Tensor]]] = {}
    for op in _lookup_operators(model):
        names = [spec[0] for spec in op.embedding_specs]
        found.update(zip(names, op.split_embedding_weights()))
    return found


def assign_weights_to_tbe(
    model: torch.nn.Module, table_to_weight: Dict[str, Tuple[torch.Tensor, Optional[torch.Tensor]]]
) -> None:
    """Copies ``table_to_weight`` (as returned above) into the operators of ``model``."""
    for op in _lookup_operators(model):
        names = [spec[0] for spec in op.embedding_specs]
        missing = [n for n in names if n not in table_to_weight]
        assert not missing, f"{missing[0]} not in table_to_weight"
        op.assign_embedding_weights([table_to_weight[n] for n in names])
