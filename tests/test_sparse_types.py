"""KeyedJaggedTensor / JaggedTensor / KeyedTensor against the expected values of
the reference's own unit tests (tests/golden/kjt_vectors.json), once on host
tensors and once on the GPU, where offsets, per-key totals and permutation run
in the HIP kernels.  Integer results are compared with torch.equal."""
import json
import os

import pytest
import torch

from torchrec_amd import JaggedTensor, KeyedJaggedTensor, KeyedTensor

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kjt_vectors.json")))

DEVICES = [pytest.param("cpu", id="host"), pytest.param("cuda:0", id="gpu", marks=pytest.mark.gpu)]


def T(x, device, dtype=torch.float32):
    return torch.tensor(x, dtype=dtype, device=device)


def I(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def eq(t, expected, dtype=None):
    e = torch.tensor(expected, dtype=dtype if dtype is not None else t.dtype)
    return t.shape == e.shape and torch.equal(t.cpu(), e)


@pytest.mark.parametrize("device", DEVICES)
def test_key_lookup_and_split(device):
    g = G["key_lookup"]
    kjt = KeyedJaggedTensor(values=T(G["values8"], device), keys=g["keys"], offsets=I(g["offsets"], device),
                            weights=T(G["weights8"], device))
    for via in ("getitem", "split", "to_dict"):
        if via == "getitem":
            parts = {k: kjt[k] for k in g["keys"]}
        elif via == "to_dict":
            parts = kjt.to_dict()
        else:
            s0, s1 = kjt.split([1, 1])
            assert s0.keys() == ["index_0"] and s1.keys() == ["index_1"]
            parts = {"index_0": s0, "index_1": s1}
        for k in g["keys"]:
            assert eq(parts[k].lengths(), g[k]["lengths"])
            assert eq(parts[k].weights(), g[k]["weights"])
            assert eq(parts[k].values(), g[k]["values"])
    assert kjt.stride() == 3
    assert kjt.length_per_key() == [3, 5] and kjt.offset_per_key() == [0, 3, 8]


@pytest.mark.parametrize("device", DEVICES)
def test_zero_split(device):
    g, z = G["key_lookup"], G["zero_split"]
    kjt = KeyedJaggedTensor(values=T(G["values8"], device), keys=g["keys"], offsets=I(g["offsets"], device),
                            weights=T(G["weights8"], device))
    j0, j1 = kjt.split(z["segments"])
    assert j0.keys() == [] and j0.stride() == z["j0"]["stride"]
    assert j0.lengths().numel() == 0 and j0.values().numel() == 0 and j0.weights().numel() == 0
    assert j1.keys() == z["j1"]["keys"] and j1.stride() == z["j1"]["stride"]
    assert eq(j1.lengths(), z["j1"]["lengths"])
    assert eq(j1.values(), G["values8"]) and eq(j1.weights(), G["weights8"])
    assert j1 is kjt


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weighted", [False, True])
def test_permute(device, weighted):
    g = G["permute"]
    kjt = KeyedJaggedTensor.from_lengths_sync(
        values=T(G["values8"], device), keys=g["keys"], lengths=I(g["lengths"], device),
        weights=T(G["weights8"], device) if weighted else None)
    p = kjt.permute(g["indices"])
    assert p.keys() == g["out_keys"]
    assert p.offset_per_key() == g["out_offset_per_key"]
    assert eq(p.values(), g["out_values"])
    assert eq(p.lengths(), g["out_lengths"])
    if weighted:
        assert eq(p.weights(), g["out_weights"])
    else:
        assert p.weights_or_none() is None
    assert p.stride() == 3


@pytest.mark.parametrize("device", DEVICES)
def test_permute_duplicates(device):
    g, d = G["permute"], G["permute_duplicates"]
    kjt = KeyedJaggedTensor.from_lengths_sync(values=T(G["values8"], device), keys=g["keys"],
                                              lengths=I(g["lengths"], device))
    p = kjt.permute(d["indices"])
    assert p.keys() == d["out_keys"]
    assert p.offset_per_key() == d["out_offset_per_key"]
    assert eq(p.values(), d["out_values"])
    assert eq(p.lengths(), d["out_lengths"])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("itype", [torch.int32, torch.int64])
def test_length_vs_offset(device, itype):
    g = G["length_vs_offset"]
    keys = ["index_0", "index_1"]
    j_off = KeyedJaggedTensor.from_offsets_sync(values=T(G["values8"], device), keys=keys,
                                                offsets=torch.tensor(g["offsets"], dtype=itype, device=device))
    j_len = KeyedJaggedTensor.from_lengths_sync(values=T(G["values8"], device), keys=keys,
                                                lengths=torch.tensor(g["lengths"], dtype=itype, device=device))
    assert torch.equal(j_off.lengths(), j_len.lengths()) and j_off.lengths().dtype == itype
    assert torch.equal(j_off.offsets(), j_len.offsets()) and j_len.offsets().dtype == itype
    assert eq(j_len.offsets(), g["offsets"])
    assert j_off.stride() == 4 and j_len.stride() == 4


@pytest.mark.parametrize("device", DEVICES)
def test_empty_and_float_lengths(device):
    kjt = KeyedJaggedTensor.empty(device=torch.device(device))
    assert kjt.keys() == [] and kjt.stride() == 0 and kjt.length_per_key() == []
    with pytest.raises(AssertionError):
        KeyedJaggedTensor(keys=["a"], values=T([1.0], device), lengths=T([1.0], device))
    with pytest.raises(AssertionError):
        JaggedTensor(values=T([1.0], device), offsets=T([0.0, 1.0], device))


@pytest.mark.parametrize("device", DEVICES)
def test_jagged_tensor_dense_round_trips(device):
    g = G["jt_from_dense_lengths"]
    jt = JaggedTensor.from_dense_lengths(values=T(g["values"], device), lengths=I(g["lengths"], device))
    assert eq(jt.lengths(), g["lengths"]) and eq(jt.values(), g["out_values"]) and jt.weights_or_none() is None
    assert eq(jt.offsets(), g["out_offsets"])
    rows = [T([1.0], device), T([], device), T([7.0, 8.0], device), T([10.0, 11.0, 12.0], device)]
    jd = JaggedTensor.from_dense(values=rows, weights=rows)
    assert eq(jd.offsets(), g["out_offsets"]) and eq(jd.values(), g["out_values"]) and eq(jd.weights(), g["out_values"])
    back = jd.to_dense()
    assert all(torch.equal(a, b) for a, b in zip(back, rows))
    p = G["jt_to_padded_dense"]
    jt2 = JaggedTensor(values=T(G["values8"], device), offsets=I(p["offsets"], device))
    assert eq(jt2.to_padded_dense(), p["t0"])
    assert eq(jt2.to_padded_dense(desired_length=p["t1_desired_length"], padding_value=p["t1_padding"]), p["t1"])


@pytest.mark.parametrize("device", DEVICES)
def test_keyed_tensor(device):
    tl = [T([[1.0, 1.0]], device), T([[2.0, 2.0], [3.0, 3.0]], device)]
    kt = KeyedTensor.from_tensor_list(["dense_0", "dense_1"], tl, cat_dim=0, key_dim=0)
    assert kt.key_dim() == 0
    assert torch.equal(kt["dense_0"], tl[0]) and torch.equal(kt["dense_1"], tl[1])
    d = kt.to_dict()
    assert all(torch.equal(kt[k], d[k]) for k in kt.keys())
    tl1 = [t.T for t in tl]
    kt1 = KeyedTensor.from_tensor_list(["dense_0", "dense_1"], tl1, key_dim=1)
    assert kt1.key_dim() == 1 and kt1.length_per_key() == [1, 2] and kt1.offset_per_key() == [0, 1, 3]
    assert torch.equal(kt1["dense_0"], tl1[0]) and torch.equal(kt1["dense_1"], tl1[1])


@pytest.mark.parametrize("device", DEVICES)
def test_from_jt_dict_and_concat(device):
    g = G["key_lookup"]
    kjt = KeyedJaggedTensor(values=T(G["values8"], device), keys=g["keys"], offsets=I(g["offsets"], device))
    again = KeyedJaggedTensor.from_jt_dict(kjt.to_dict())
    assert again.keys() == kjt.keys() and torch.equal(again.values(), kjt.values())
    assert torch.equal(again.lengths(), kjt.lengths())
    a, b = kjt.split([1, 1])
    cat = KeyedJaggedTensor.concat([a, b])
    assert cat.keys() == kjt.keys() and torch.equal(cat.values(), kjt.values())
    assert cat.length_per_key() == [3, 5]


def test_kjt_equality_cases():
    """kjt_is_equal on the cases of the reference's test_equality
    (torchrec/sparse/tests/test_keyed_jagged_tensor.py:892-968)."""
    from torchrec_amd.sparse.jagged_tensor import kjt_is_equal

    values = torch.Tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0])
    weights = torch.Tensor([1.0, 0.5, 1.5, 1.0, 0.5, 1.0, 1.0, 1.5])
    keys = ["index_0", "index_1"]
    offsets = torch.IntTensor([0, 0, 2, 2, 3, 4, 5, 5, 8])
    lengths = torch.IntTensor([0, 2, 0, 1, 1, 1, 0, 3])
    kt = KeyedJaggedTensor.from_offsets_sync(values=values, keys=keys, offsets=offsets)
    assert kjt_is_equal(kt, KeyedJaggedTensor.from_lengths_sync(values=values, keys=keys, lengths=lengths))
    assert not kjt_is_equal(kt, KeyedJaggedTensor(values=values, keys=["index_1", "index_0"], offsets=offsets))
    other = torch.Tensor([10.0, 4.0, 2.0, 5.0, 2.0, 6.0, 9.0, 8.0])
    assert not kjt_is_equal(kt, KeyedJaggedTensor(values=other, keys=keys, lengths=lengths))
    assert not kjt_is_equal(kt, KeyedJaggedTensor(values=values, keys=["index_0"], offsets=offsets))
    assert not kjt_is_equal(kt, KeyedJaggedTensor.from_offsets_sync(values=values, keys=keys, offsets=offsets, weights=weights))
    a = KeyedJaggedTensor.from_lengths_sync(values=values, keys=keys, lengths=torch.IntTensor([1, 2, 3, 4, 5, 6, 7, 8]))
    b = KeyedJaggedTensor.from_lengths_sync(values=values, keys=keys, lengths=torch.IntTensor([8, 7, 6, 5, 4, 3, 2, 1]))
    assert not kjt_is_equal(a, b)
    c = KeyedJaggedTensor.from_offsets_sync(values=values, keys=keys, offsets=torch.IntTensor([8, 4, 1, 5, 0, 1, 2, 1, 2]))
    assert not kjt_is_equal(kt, c)
    assert not kjt_is_equal(kt, "not a kjt")


def test_kjt_strings():
    """str() of a KJT, as the reference prints it (test_keyed_jagged_tensor.py:786-852)."""
    assert str(KeyedJaggedTensor([], torch.Tensor())) == "KeyedJaggedTensor()\n"
    one = KeyedJaggedTensor(values=torch.Tensor([1.0]), keys=["key"], offsets=torch.IntTensor([0, 1]))
    assert str(one) == 'KeyedJaggedTensor({\n    "key": [[1.0]]\n})\n'
    values = torch.Tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0])
    weights = torch.Tensor([1.0, 0.5, 1.5, 1.0, 0.5, 1.0, 1.0, 1.5])
    keys = ["index_0", "index_1"]
    offsets = torch.IntTensor([0, 2, 2, 3, 4, 5, 8])
    assert str(KeyedJaggedTensor(values=values, keys=keys, offsets=offsets)) == (
        'KeyedJaggedTensor({\n    "index_0": [[1.0, 2.0], [], [3.0]],\n'
        '    "index_1": [[4.0], [5.0], [6.0, 7.0, 8.0]]\n})\n')
    assert str(KeyedJaggedTensor(values=values, keys=keys, offsets=offsets, weights=weights)) == (
        'KeyedJaggedTensor({\n    "index_0": {\n'
        '        "values": [[1.0, 2.0], [], [3.0]],\n'
        '        "weights": [[1.0, 0.5], [], [1.5]]\n'
        '    },\n    "index_1": {\n'
        '        "values": [[4.0], [5.0], [6.0, 7.0, 8.0]],\n'
        '        "weights": [[1.0], [0.5], [1.0, 1.0, 1.5]]\n    }\n})\n')


def test_kjt_to_dict_and_empty():
    """to_dict / empty / empty_like (test_keyed_jagged_tensor.py:102-140, 225-290)."""
    values = torch.Tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0])
    weights = torch.Tensor([1.0, 0.5, 1.5, 1.0, 0.5, 1.0, 1.0, 1.5])
    keys = ["index_0", "index_1"]
    offsets = torch.IntTensor([0, 2, 2, 3, 4, 5, 8])
    d = KeyedJaggedTensor(values=values, weights=weights, keys=keys, offsets=offsets).to_dict()
    assert d["index_0"].offsets().tolist() == [0, 2, 2, 3] and d["index_0"].values().tolist() == [1.0, 2.0, 3.0]
    assert d["index_1"].offsets().tolist() == [0, 1, 2, 5] and d["index_1"].weights().tolist() == [1.0, 0.5, 1.0, 1.0, 1.5]
    e = KeyedJaggedTensor.empty()
    assert e.keys() == [] and e.values().numel() == 0 and e.to_dict() == {}
    like = KeyedJaggedTensor.empty_like(KeyedJaggedTensor(values=values, weights=weights, keys=keys, offsets=offsets))
    assert like.keys() == [] and like.values().dtype == values.dtype and like.weights().numel() == 0
