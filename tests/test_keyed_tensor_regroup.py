"""KeyedTensor.regroup / regroup_as_dict: the cases of the reference's test
(torchrec/sparse/tests/test_keyed_tensor.py:82-128 single and multiple
KeyedTensors, :306-332 duplicate keys), on the host and, for the one-launch
column-copy kernel, on the GPU against plain slicing."""
import numpy as np
import pytest
import torch

from torchrec_amd import KeyedTensor
from torchrec_amd.sparse.jagged_tensor import _regroup_keyed_tensors, permute_multi_embedding, regroup_kts

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("dev", DEVICES)
def test_regroup_single_kt(dev):
    tensors = [torch.randn(2, 3, device=dev) for _ in range(5)]
    kt = KeyedTensor.from_tensor_list([f"dense_{i}" for i in range(5)], tensors, 1)
    got = KeyedTensor.regroup([kt], [["dense_0", "dense_4"], ["dense_1", "dense_3"], ["dense_2"]])
    assert torch.equal(got[0], torch.cat([tensors[0], tensors[4]], 1))
    assert torch.equal(got[1], torch.cat([tensors[1], tensors[3]], 1))
    assert torch.equal(got[2], tensors[2])


@pytest.mark.parametrize("dev", DEVICES)
def test_regroup_multiple_kt_and_as_dict(dev):
    t1 = [torch.randn(2, 4, device=dev), torch.randn(2, 8, device=dev), torch.randn(2, 2, device=dev)]
    t2 = [torch.randn(2, 3, device=dev), torch.randn(2, 10, device=dev)]
    kt1 = KeyedTensor.from_tensor_list(["dense_0", "dense_1", "dense_2"], t1, 1)
    kt2 = KeyedTensor.from_tensor_list(["sparse_0", "sparse_1"], t2, 1)
    groups = [["dense_0", "sparse_1", "dense_2"], ["dense_1", "sparse_0"]]
    got = KeyedTensor.regroup([kt1, kt2], groups)
    assert torch.equal(got[0], torch.cat([t1[0], t2[1], t1[2]], 1))
    assert torch.equal(got[1], torch.cat([t1[1], t2[0]], 1))
    as_dict = KeyedTensor.regroup_as_dict([kt1, kt2], groups, ["a", "b"])
    assert list(as_dict) == ["a", "b"] and torch.equal(as_dict["b"], got[1])
    with pytest.raises(AssertionError):
        KeyedTensor.regroup_as_dict([kt1, kt2], groups, ["a"])


@pytest.mark.parametrize("dev", DEVICES)
def test_regroup_multiple_kt_duplicate_keys(dev):
    t1 = [torch.randn(2, 4, device=dev) for _ in range(2)]
    t2 = [torch.randn(2, 3, device=dev) for _ in range(3)]
    kt1 = KeyedTensor.from_tensor_list(["dense_0", "dense_1"], t1, 1)
    kt2 = KeyedTensor.from_tensor_list(["sparse_0", "sparse_1", "dense_2"], t2, 1)
    got = KeyedTensor.regroup([kt1, kt2], [["dense_0", "sparse_1"], ["dense_1", "sparse_0", "dense_0"]])
    assert torch.equal(got[0], torch.cat([t1[0], t2[1]], 1))
    assert torch.equal(got[1], torch.cat([t1[1], t2[0], t1[0]], 1))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_regroup_kernel_against_slicing(dtype):
    """Many keys (more than one launch's worth of blocks), odd widths, a key
    used twice, a key not used, an empty group."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    kts, all_keys = [], []
    for t in range(3):
        widths = rng.integers(1, 40, 70).tolist()
        keys = [f"k{t}_{i}" for i in range(len(widths))]
        values = torch.randn(257, sum(widths), device=dev).to(dtype)
        kts.append(KeyedTensor(keys=keys, length_per_key=widths, values=values))
        all_keys += keys
    order = rng.permutation(len(all_keys)).tolist()
    picked = [all_keys[i] for i in order[:-5]]  # five keys stay unused
    groups = [picked[:50], picked[50:51], [], picked[51:] + picked[:3]]
    want = _regroup_keyed_tensors(kts, groups)
    for fn in (regroup_kts, permute_multi_embedding, KeyedTensor.regroup):
        got = fn(kts, groups)
        assert len(got) == len(want)
        for g, w in zip(got, want):
            assert g.shape == w.shape and g.dtype == dtype and torch.equal(g, w)
    # a view with a row stride larger than its width (a slice of a wider output)
    wide = torch.randn(64, 100, device=dev).to(dtype)
    part = KeyedTensor(keys=["x", "y"], length_per_key=[30, 20], values=wide[:, 10:60])
    got = regroup_kts([part], [["y", "x"]])
    assert torch.equal(got[0], torch.cat([wide[:, 40:60], wide[:, 10:40]], 1))


@pytest.mark.parametrize("dev", DEVICES)
def test_kt_regroup_as_dict_module(dev):
    """torchrec/modules/tests/test_regroup.py: same result as the static method,
    on the first and on later batches; a duplicate key is refused; the cast."""
    from torchrec_amd.modules.embedding_configs import DataType
    from torchrec_amd.modules.regroup import KTRegroupAsDict

    def batch():
        t1 = [torch.randn(6, 4, device=dev), torch.randn(6, 8, device=dev), torch.randn(6, 2, device=dev)]
        t2 = [torch.randn(6, 3, device=dev), torch.randn(6, 10, device=dev)]
        return [KeyedTensor.from_tensor_list(["f1", "f2", "f3"], t1), KeyedTensor.from_tensor_list(["g1", "g2"], t2)]

    groups, keys = [["f1", "g2", "f3"], ["f2", "g1"]], ["object", "user"]
    m = KTRegroupAsDict(groups, keys)
    for _ in range(3):
        kts = batch()
        got, want = m(kts), KeyedTensor.regroup_as_dict(kts, groups, keys)
        assert list(got) == keys and all(torch.equal(got[k], want[k]) for k in keys)
    half = KTRegroupAsDict(groups, keys, emb_dtype=DataType.FP16)
    kts = batch()
    out = half(kts)
    assert out["user"].dtype == torch.float16
    assert torch.equal(out["user"], torch.cat([kts[0]["f2"], kts[1]["g1"]], 1).half())
    dup = [KeyedTensor.from_tensor_list(["f1"], [torch.randn(2, 2, device=dev)]),
           KeyedTensor.from_tensor_list(["f1"], [torch.randn(2, 2, device=dev)])]
    with pytest.raises(RuntimeError, match="Duplicate key"):
        KTRegroupAsDict([["f1"]], ["a"])(dup)
    m.clear_cache()
    assert not m._is_inited
