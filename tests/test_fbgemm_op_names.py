"""torch.ops.fbgemm.* names registered by torchrec_amd.fbgemm_ops: the operators
TorchRec's quantized path calls by name resolve to this package's kernels."""
import numpy as np
import pytest
import torch

import oracle as O
import torchrec_amd.fbgemm_ops as fbgemm_ops

NAMES = ["asynchronous_complete_cumsum", "permute_2D_sparse_data", "offsets_range",
         "block_bucketize_sparse_features", "FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf"]


def test_names_resolve_on_host():
    assert set(fbgemm_ops.register()) <= set(NAMES)
    for n in NAMES:
        assert hasattr(torch.ops.fbgemm, n)
    lengths = torch.tensor([1, 2, 3, 0, 4])
    assert torch.ops.fbgemm.asynchronous_complete_cumsum(lengths).tolist() == [0, 1, 3, 6, 6, 10]
    assert torch.ops.fbgemm.offsets_range(torch.tensor([0, 2, 2, 5]), 5).tolist() == [0, 1, 0, 1, 2]
    l, v, w = torch.ops.fbgemm.permute_2D_sparse_data(
        torch.tensor([1, 0], dtype=torch.int32), torch.tensor([[1, 2], [0, 1]]), torch.tensor([10, 20, 30, 40]),
        torch.tensor([1.0, 2.0, 3.0, 4.0]), None)
    assert l.tolist() == [[0, 1], [1, 2]] and v.tolist() == [40, 10, 20, 30] and w.tolist() == [4.0, 1.0, 2.0, 3.0]


@pytest.mark.gpu
def test_names_run_the_kernels():
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(2)
    lengths = rng.integers(0, 9, 3 * 50).astype(np.int32)
    got = torch.ops.fbgemm.asynchronous_complete_cumsum(torch.from_numpy(lengths).to(dev))
    assert got.device.type == "cuda" and np.array_equal(got.cpu().numpy(), O.cumsum(lengths))
    w = rng.normal(0, 0.1, (100, 64)).astype(np.float32)
    q = torch.ops.fbgemm.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(torch.from_numpy(w).to(dev), 4)
    assert np.array_equal(q.cpu().numpy(), O.quantize_sbhalf(w, 4))
    ids = rng.integers(0, 40, int(lengths.sum())).astype(np.int32)
    block_sizes = np.asarray([10, 10, 10], dtype=np.int64)
    ol, oi, _, _ = O.bucketize(lengths, ids, block_sizes, 4, None, False, return_permute=True)
    nl, ni, nw, pos, perm = torch.ops.fbgemm.block_bucketize_sparse_features(
        torch.from_numpy(lengths).to(dev), torch.from_numpy(ids).to(dev), False, False,
        torch.from_numpy(block_sizes).to(dev), 4)
    assert nl.cpu().numpy().tolist() == ol.tolist() and ni.cpu().numpy().tolist() == oi.tolist()
    assert nw is None and pos is None and perm is None
