"""Keys that the sharders put into ``fused_params`` to steer the per-shard
lookup modules, and their readers (same key strings and function names as
torchrec/distributed/fused_params.py:20-123).  The keys are consumed here and
never reach the lookup operator."""
from __future__ import annotations

from typing import Any, Dict, Iterable, Optional

import torch

FUSED_PARAM_REGISTER_TBE_BOOL: str = "__register_tbes_in_named_modules"
FUSED_PARAM_QUANT_STATE_DICT_SPLIT_SCALE_BIAS: str = "__register_quant_state_dict_split_scale_bias"
FUSED_PARAM_TBE_ROW_ALIGNMENT: str = "__register_tbe_row_alignment"
FUSED_PARAM_BOUNDS_CHECK_MODE: str = "__register_tbe_bounds_check_mode"
FUSED_PARAM_LENGTHS_TO_OFFSETS_LOOKUP: str = "__register_lengths_to_offsets_lookup"
FUSED_PARAM_SSD_TABLE_LIST: str = "__register_ssd_table_list"
FUSED_PARAM_IS_SSD_TABLE: str = "__register_is_ssd_table"

_NOT_FOR_THE_OPERATOR = (
    FUSED_PARAM_REGISTER_TBE_BOOL,
    FUSED_PARAM_QUANT_STATE_DICT_SPLIT_SCALE_BIAS,
    FUSED_PARAM_TBE_ROW_ALIGNMENT,
    FUSED_PARAM_BOUNDS_CHECK_MODE,
    FUSED_PARAM_LENGTHS_TO_OFFSETS_LOOKUP,
    FUSED_PARAM_SSD_TABLE_LIST,
)


class TBEToRegisterMixIn:
    """A module that owns lookup operators and can say which config each serves."""

    def get_tbes_to_register(self) -> Dict[Any, Any]:
        raise NotImplementedError


def get_tbes_to_register_from_iterable(iterable: Iterable[torch.nn.Module]) -> Dict[Any, Any]:
    found: Dict[Any, Any] = {}
    for m in iterable:
        if isinstance(m, TBEToRegisterMixIn):
            found.update(m.get_tbes_to_register())
    return found


def _get(fused_params: Optional[Dict[str, Any]], key: str, default: Any) -> Any:
    return default if not fused_params or key not in fused_params else fused_params[key]


def is_fused_param_register_tbe(fused_params: Optional[Dict[str, Any]]) -> bool:
    return bool(_get(fused_params, FUSED_PARAM_REGISTER_TBE_BOOL, False))


def is_fused_param_quant_state_dict_split_scale_bias(fused_params: Optional[Dict[str, Any]]) -> bool:
    return bool(_get(fused_params, FUSED_PARAM_QUANT_STATE_DICT_SPLIT_SCALE_BIAS, False))


def get_fused_param_tbe_row_alignment(fused_params: Optional[Dict[str, Any]]) -> Optional[int]:
    return _get(fused_params, FUSED_PARAM_TBE_ROW_ALIGNMENT, None)


def fused_param_bounds_check_mode(fused_params: Optional[Dict[str, Any]]) -> Optional[Any]:
    return _get(fused_params, FUSED_PARAM_BOUNDS_CHECK_MODE, None)


def fused_param_lengths_to_offsets_lookup(fused_params: Optional[Dict[str, Any]]) -> bool:
    return bool(_get(fused_params, FUSED_PARAM_LENGTHS_TO_OFFSETS_LOOKUP, False))


def tbe_fused_params(fused_params: Optional[Dict[str, Any]]) -> Optional[Dict[str, Any]]:
    """What is left for the lookup operator's constructor."""
    if not fused_params:
        return None
    return {k: v for k, v in fused_params.items() if k not in _NOT_FOR_THE_OPERATOR}
