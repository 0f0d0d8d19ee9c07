"""validate_keyed_jagged_tensor against the cases and messages of the
reference's own test (torchrec/sparse/tests/test_jagged_tensor_validator.py:
57-160 invalid inputs, :186-239 valid ones)."""
import pytest
import torch

from torchrec_amd import KeyedJaggedTensor
from torchrec_amd.sparse.jagged_tensor_validator import validate_keyed_jagged_tensor

V5 = torch.tensor([1, 2, 3, 4, 5])
L4 = torch.tensor([1, 2, 0, 2])
O5 = torch.tensor([0, 1, 3, 3, 5])

INVALID = [
    ("lengths and offsets cannot be both empty", ["f1", "f2"], V5, None, None, None),
    ("Expected lengths size to be 1 more than offsets size", ["f1", "f2"], V5, L4, torch.tensor([0, 1, 3, 5]), None),
    ("Sum of lengths must equal the number of values", ["f1", "f2"], V5, torch.tensor([]), None, None),
    ("Sum of lengths must equal the number of values", ["f1", "f2"], V5, torch.tensor([3, 3, 2, 1]), None, None),
    ("offsets cannot be empty", ["f1", "f2"], V5, None, torch.tensor([]), None),
    ("Expected first offset to be 0", ["f1", "f2"], V5, L4, torch.tensor([1, 2, 4, 4, 6]), None),
    ("The last element of offsets must equal to the number of values", ["f1", "f2"], V5, L4,
     torch.tensor([0, 2, 4, 4, 6]), None),
    ("offsets is not equal to the cumulative sum of lengths", ["f1", "f2"], V5, L4, torch.tensor([0, 2, 3, 3, 5]), None),
    ("keys must be unique", ["f1", "f1"], V5, L4, O5, None),
    ("keys is empty but lengths or offsets is not", [], V5, L4, O5, None),
    ("lengths size must be divisible by keys size", ["f1", "f2", "f3"], V5, L4, O5, None),
    ("weights size must equal to values size", ["f1", "f2"], V5, L4, O5, torch.tensor([0.1, 0.2, 0.3, 0.4])),
    ("weights size must equal to values size", ["f1", "f2"], V5, L4, O5,
     torch.tensor([0.1, 0.2, 0.3, 0.4, 0.5, 0.6])),
]


@pytest.mark.parametrize("message,keys,values,lengths,offsets,weights", INVALID)
def test_invalid_keyed_jagged_tensor(message, keys, values, lengths, offsets, weights):
    kjt = KeyedJaggedTensor(keys=keys, values=values, lengths=lengths, offsets=offsets, weights=weights)
    with pytest.raises(ValueError, match=message):
        validate_keyed_jagged_tensor(kjt)


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("weighted", [False, True])
def test_valid_kjt_from_lengths_and_from_offsets(seed, weighted):
    g = torch.Generator().manual_seed(seed)
    num_keys = int(torch.randint(1, 11, (1,), generator=g))
    stride = int(torch.randint(1, 11, (1,), generator=g))
    keys = [f"key{k}" for k in range(num_keys)]
    lengths = torch.randint(0, 21, (num_keys * stride,), generator=g)
    offsets = torch.cat((torch.tensor([0]), torch.cumsum(lengths, dim=0)))
    n = int(lengths.sum())
    values = torch.rand(n, generator=g) * 100
    weights = torch.rand(n, generator=g) * 100 if weighted else None
    validate_keyed_jagged_tensor(KeyedJaggedTensor.from_lengths_sync(keys=keys, values=values, weights=weights, lengths=lengths))
    validate_keyed_jagged_tensor(KeyedJaggedTensor.from_offsets_sync(keys=keys, values=values, weights=weights, offsets=offsets))
    validate_keyed_jagged_tensor(KeyedJaggedTensor(keys=keys, values=values, weights=weights, lengths=lengths, offsets=offsets))


def test_valid_empty_kjt():
    validate_keyed_jagged_tensor(KeyedJaggedTensor.empty())
    validate_keyed_jagged_tensor(KeyedJaggedTensor(keys=[], values=torch.tensor([]), lengths=torch.tensor([]),
                                                   offsets=torch.tensor([0])))
