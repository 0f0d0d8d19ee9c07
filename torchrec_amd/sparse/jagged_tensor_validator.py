"""Checks of the tensors a KeyedJaggedTensor was built from
(torchrec/sparse/jagged_tensor_validator.py:14-123: same function name, same
conditions, same messages).  Runs on the host view of the metadata; meant for
data-loading code, not for the lookup path."""
from __future__ import annotations

from typing import Optional

import torch

from torchrec_amd.sparse.jagged_tensor import KeyedJaggedTensor


def _fail(message: str) -> None:
    raise ValueError(message)


def _check_lengths(lengths: torch.Tensor, num_values: int) -> None:
    total = lengths.sum().item()
    if total != num_values:
        _fail(f"Sum of lengths must equal the number of values, but got {total} and {num_values}")


def _check_offsets(offsets: torch.Tensor, num_values: int) -> None:
    if offsets.numel() == 0:
        _fail("offsets cannot be empty")
    if offsets[0] != 0:
        _fail(f"Expected first offset to be 0, but got {offsets[0]} instead")
    if offsets[-1] != num_values:
        _fail(
            f"The last element of offsets must equal to the number of values, but got {offsets[-1]} and {num_values}"
        )


def validate_keyed_jagged_tensor(kjt: KeyedJaggedTensor) -> None:
    """Raises ValueError for the first inconsistency found: neither lengths nor
    offsets; lengths / offsets that disagree with each other or with the number
    of values; duplicate keys; bags that do not divide evenly among the keys;
    weights of another size than the values."""
    lengths: Optional[torch.Tensor] = kjt.lengths_or_none()
    offsets: Optional[torch.Tensor] = kjt.offsets_or_none()
    num_values = kjt.values().numel()

    if lengths is None and offsets is None:
        _fail("lengths and offsets cannot be both empty in KeyedJaggedTensor")
    if lengths is not None:
        _check_lengths(lengths, num_values)
    if offsets is not None:
        _check_offsets(offsets, num_values)
    if lengths is not None and offsets is not None:
        if lengths.numel() != offsets.numel() - 1:
            _fail(
                "Expected lengths size to be 1 more than offsets size, but got lengths size: "
                f"{lengths.numel()} and offsets size: {offsets.numel()}"
            )
        if not lengths.equal(torch.diff(offsets)):
            _fail("offsets is not equal to the cumulative sum of lengths")

    keys = kjt.keys()
    if len(set(keys)) != len(keys):
        _fail("keys must be unique")
    num_bags = lengths.numel() if lengths is not None else offsets.numel() - 1  # type: ignore[union-attr]
    if not keys:
        if num_bags > 0:
            _fail("keys is empty but lengths or offsets is not")
    elif not kjt.variable_stride_per_key() and num_bags % len(keys) != 0:
        _fail(f"lengths size must be divisible by keys size, but got {num_bags} and {len(keys)}")

    weights = kjt.weights_or_none()
    if weights is not None and weights.numel() != num_values:
        _fail(f"weights size must equal to values size, but got {weights.numel()} and {num_values}")
