"""Managed-collision remap and the quantized collection behind it.  Expected
ids are computed with numpy's searchsorted, i.e. the reference's formula
(torchrec/modules/mc_modules.py:959-989) restated on the host."""
import numpy as np
import pytest
import torch
import torch.quantization as quant

from torchrec_amd import KeyedJaggedTensor, ops
from torchrec_amd.modules.embedding_configs import EmbeddingConfig, QuantConfig
from torchrec_amd.modules.embedding_modules import EmbeddingCollection
from torchrec_amd.modules.mc_embedding_modules import ManagedCollisionEmbeddingCollection
from torchrec_amd.modules.mc_modules import ManagedCollisionCollection, MCHManagedCollisionModule
from torchrec_amd.quant import QuantManagedCollisionEmbeddingCollection as QuantMCEC

IMAX = np.iinfo(np.int64).max


def ref_remap(values, sorted_ids, mapping, miss):
    idx = np.searchsorted(sorted_ids[:-1], values)
    hit = sorted_ids[idx] == values
    return np.where(hit, mapping[idx], miss)


def make_table(rng, size, filled):
    raw = np.sort(rng.choice(10**9, filled, replace=False)).astype(np.int64)
    sorted_ids = np.full(size, IMAX, dtype=np.int64)
    sorted_ids[:filled] = raw
    mapping = rng.permutation(size).astype(np.int64)
    return sorted_ids, mapping


@pytest.mark.parametrize("size,filled", [(1, 0), (2, 1), (64, 63), (1000, 400)])
def test_mch_remap_host(size, filled):
    rng = np.random.default_rng(size)
    sorted_ids, mapping = make_table(rng, size, filled)
    values = np.concatenate([rng.choice(sorted_ids[:max(filled, 1)], 50), rng.integers(0, 10**9, 50), [IMAX, 0]]).astype(np.int64)
    got = ops.mch_remap(torch.from_numpy(values), torch.from_numpy(sorted_ids), torch.from_numpy(mapping), size - 1)
    assert np.array_equal(got.numpy(), ref_remap(values, sorted_ids, mapping, size - 1))


@pytest.mark.gpu
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("size,filled", [(1, 0), (2, 1), (64, 63), (100_000, 60_000)])
def test_mch_remap_kernel(idt, size, filled):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(size + 1)
    sorted_ids, mapping = make_table(rng, size, filled)
    hits = rng.choice(sorted_ids[:max(filled, 1)], 5000)
    values = np.concatenate([hits, rng.integers(0, 10**9, 5000), [0, 10**9]])
    if idt == np.int64:
        values = np.concatenate([values, [IMAX, -5]])
    values = values.astype(idt)
    got = ops.mch_remap(torch.from_numpy(values).to(dev), torch.from_numpy(sorted_ids).to(dev),
                        torch.from_numpy(mapping).to(dev), size - 1)
    assert got.dtype == torch.from_numpy(values).dtype
    assert np.array_equal(got.cpu().numpy(), ref_remap(values.astype(np.int64), sorted_ids, mapping, size - 1).astype(idt))
    assert np.array_equal(got.cpu().numpy(), ops.mch_remap(torch.from_numpy(values), torch.from_numpy(sorted_ids),
                                                           torch.from_numpy(mapping), size - 1).numpy())


def build_mcec(dev):
    configs = [
        EmbeddingConfig(name="t1", embedding_dim=16, num_embeddings=40, feature_names=["f1", "f2"]),
        EmbeddingConfig(name="t2", embedding_dim=16, num_embeddings=30, feature_names=["f3"]),
    ]
    mods = {c.name: MCHManagedCollisionModule(c.num_embeddings, dev) for c in configs}
    mods["t1"].set_id_table(torch.tensor([1000, 5, 77777, 123456789]))
    mods["t2"].set_id_table(torch.tensor([9, 8, 7]), rows=torch.tensor([20, 21, 22]))
    mcc = ManagedCollisionCollection(mods, configs)
    return ManagedCollisionEmbeddingCollection(EmbeddingCollection(configs, dev), mcc, return_remapped_features=True)


def test_collection_remap_and_errors_host():
    cpu = torch.device("cpu")
    m = build_mcec(cpu).eval()
    # keys in a different order than the tables' features
    kjt = KeyedJaggedTensor(keys=["f3", "f1", "f2"], values=torch.tensor([9, 1, 7, 5, 1000, 2, 123456789, 77777]),
                            lengths=torch.tensor([2, 1, 1, 1, 2, 1]))
    out = m._managed_collision_collection(kjt)
    assert out.keys() == ["f1", "f2", "f3"]
    assert out.lengths().tolist() == [1, 1, 2, 1, 2, 1]
    # t1 sorted raw ids: 5, 1000, 77777, 123456789 -> rows 1, 0, 2, 3; miss -> 39.  t2: 7->22, 8->21, 9->20; miss -> 29
    assert out.values().tolist() == [1, 0, 39, 3, 2, 20, 29, 22]
    emb, remapped = m(kjt)
    assert set(emb.keys()) == {"f1", "f2", "f3"} and remapped.values().tolist() == out.values().tolist()
    with pytest.raises(ValueError):
        ManagedCollisionCollection({}, m._managed_collision_collection.embedding_configs())
    with pytest.raises(AssertionError):
        ManagedCollisionCollection({"t1": MCHManagedCollisionModule(7, cpu), "t2": MCHManagedCollisionModule(30, cpu)},
                                   m._managed_collision_collection.embedding_configs())
    m.train()
    with pytest.raises(NotImplementedError):
        m._managed_collision_collection(kjt)
    # the id table travels through a state_dict
    sd = m._managed_collision_collection.state_dict()
    assert "_managed_collision_modules.t1._mch_sorted_raw_ids" in sd and "_managed_collision_modules.t2._mch_remapped_ids_mapping" in sd


@pytest.mark.gpu
def test_quant_mcec_matches_float():
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    m = build_mcec(dev).eval()
    kjt = KeyedJaggedTensor(keys=["f3", "f1", "f2"],
                            values=torch.tensor([9, 1, 7, 5, 1000, 2, 123456789, 77777], device=dev),
                            lengths=torch.tensor([2, 1, 1, 1, 2, 1], device=dev))
    with torch.no_grad():
        want, want_kjt = m(kjt)
    m.qconfig = QuantConfig(activation=quant.PlaceholderObserver.with_args(dtype=torch.float),
                            weight=quant.PlaceholderObserver.with_args(dtype=torch.qint8))
    q = QuantMCEC.from_float(m)
    got, got_kjt = q(kjt)
    assert torch.equal(got_kjt.values(), want_kjt.values()) and got_kjt.keys() == want_kjt.keys()
    assert got_kjt.values().tolist() == [1, 0, 39, 3, 2, 20, 29, 22]
    for k in ("f1", "f2", "f3"):
        assert torch.equal(got[k].lengths(), want[k].lengths())
        assert torch.allclose(got[k].values(), want[k].values(), atol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_collection_remaps_all_keys_in_one_launch(idt):
    """The collection's GPU path (every key in one launch) against numpy's
    searchsorted per table: two features on one table, one key without ids, a
    key order that differs from the tables'."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(11)
    sizes = {"t1": (500, 300), "t2": (64, 63), "t3": (2000, 1500)}
    configs = [EmbeddingConfig(name="t1", embedding_dim=8, num_embeddings=500, feature_names=["a", "b"]),
               EmbeddingConfig(name="t2", embedding_dim=8, num_embeddings=64, feature_names=["c"]),
               EmbeddingConfig(name="t3", embedding_dim=8, num_embeddings=2000, feature_names=["d"])]
    modules, tables = {}, {}
    for name, (size, filled) in sizes.items():
        raw = rng.choice(2**31 - 2, filled, replace=False).astype(np.int64)
        rows = rng.permutation(size - 1)[:filled].astype(np.int64)
        mod = MCHManagedCollisionModule(size, dev)
        mod.set_id_table(torch.from_numpy(raw), torch.from_numpy(rows))
        modules[name] = mod
        tables[name] = (raw, rows, size - 1)
    mcc = ManagedCollisionCollection(modules, configs).eval()
    keys, B = ["d", "a", "c", "b"], 19
    lengths = rng.integers(0, 9, len(keys) * B)
    lengths[2 * B:3 * B] = 0  # "c" has no ids at all
    table_of = {"a": "t1", "b": "t1", "c": "t2", "d": "t3"}
    vals = []
    for k, key in enumerate(keys):
        raw = tables[table_of[key]][0]
        n = int(lengths[k * B:(k + 1) * B].sum())
        known = rng.choice(raw, n)
        unknown = rng.integers(0, 2**31 - 2, n)
        vals.append(np.where(rng.random(n) < 0.6, known, unknown))
    values = np.concatenate(vals).astype(np.int64)
    kjt = KeyedJaggedTensor(keys=keys, values=torch.from_numpy(values).to(idt).to(dev),
                            lengths=torch.from_numpy(lengths).to(dev))
    out = mcc(kjt)
    assert out.keys() == ["a", "b", "c", "d"] and out.values().dtype == idt
    per_key = dict(zip(keys, vals))
    want = []
    for key in out.keys():
        raw, rows, miss = tables[table_of[key]]
        lut = dict(zip(raw.tolist(), rows.tolist()))
        want += [lut.get(int(v), miss) for v in per_key[key]]
    assert out.values().cpu().tolist() == want
    assert out.lengths().cpu().tolist() == np.concatenate(
        [lengths[keys.index(k) * B:(keys.index(k) + 1) * B] for k in out.keys()]).tolist()
