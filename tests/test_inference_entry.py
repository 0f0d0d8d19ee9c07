"""Module-swap entry points (quantize_inference_model, set_pruning_data,
get/assign_weights_to_tbe) and the feature-processed collection.  The cases
follow torchrec/inference/tests/test_inference.py:151-227, 368-398 and
torchrec/modules/tests/test_fp_embedding_modules.py; host cases build the
float model on the meta device (no arithmetic), GPU cases compare the
quantized model with the float one."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle as O
from torchrec_amd import JaggedTensor, KeyedJaggedTensor, ops
from torchrec_amd.inference.modules import (
    assign_weights_to_tbe,
    get_table_to_weights_from_tbe,
    quantize_embeddings,
    quantize_inference_model,
    set_pruning_data,
    shard_quant_model,
)
from torchrec_amd.modules.embedding_configs import DataType, EmbeddingBagConfig, EmbeddingConfig, PoolingType
from torchrec_amd.modules.embedding_modules import EmbeddingBagCollection, EmbeddingCollection
from torchrec_amd.modules.feature_processor_ import PositionWeightedModule, PositionWeightedModuleCollection
from torchrec_amd.modules.fp_embedding_modules import FeatureProcessedEmbeddingBagCollection
from torchrec_amd.quant import (
    EmbeddingBagCollection as QuantEBC,
    EmbeddingCollection as QuantEC,
    FeatureProcessedEmbeddingBagCollection as QuantFPEBC,
)
from torchrec_amd.tbe import SparseType

DIM = 16


def tables(prefix, n, weighted_names=False):
    return [
        EmbeddingBagConfig(name=f"{prefix}table_{i}", embedding_dim=DIM, num_embeddings=50 + 10 * i,
                           feature_names=[f"{prefix}feature_{i}"])
        for i in range(n)
    ]


class SparseArch(nn.Module):
    """Unweighted + weighted collections, optionally one behind position weights."""

    def __init__(self, device, max_feature_lengths=None, with_ec=False):
        super().__init__()
        self.t, self.wt = tables("", 4), tables("weighted_", 2)
        fp_tables = []
        if max_feature_lengths:
            fp_tables = [t for t in self.t if t.feature_names[0] in max_feature_lengths]
            self.t = [t for t in self.t if t.feature_names[0] not in max_feature_lengths]
        self.ebc = EmbeddingBagCollection(self.t, False, device)
        self.weighted_ebc = EmbeddingBagCollection(self.wt, True, device)
        self.fp_ebc = None
        if fp_tables:
            self.fp_ebc = FeatureProcessedEmbeddingBagCollection(
                EmbeddingBagCollection(fp_tables, True, device),
                PositionWeightedModuleCollection(max_feature_lengths, device if device.type != "meta" else None),
            )
        self.ec = None
        if with_ec:
            self.ec = EmbeddingCollection(
                [EmbeddingConfig(name="seq_table", embedding_dim=DIM, num_embeddings=40, feature_names=["seq_feature"])],
                device,
            )

    def forward(self, kjt, wkjt, fpkjt=None):
        outs = [self.ebc(kjt).values(), self.weighted_ebc(wkjt).values()]
        if self.fp_ebc is not None:
            outs.append(self.fp_ebc(fpkjt).values())
        return torch.cat(outs, dim=1)


class Model(nn.Module):
    def __init__(self, device, **kw):
        super().__init__()
        self.sparse = SparseArch(device, **kw)
        self.dense = nn.Linear(4, 4)

    def forward(self, *a):
        return self.sparse(*a)


META = torch.device("meta")


def tbes(model):
    return [m for m in model.modules() if m.__class__.__name__ == "IntNBitTableBatchedEmbeddingBagsCodegen"]


# --------------------------------------------------------------------------- host
def test_swap_types_and_default_dtype():
    model = quantize_inference_model(Model(META, with_ec=True))
    assert type(model.sparse.ebc) is QuantEBC and type(model.sparse.weighted_ebc) is QuantEBC
    assert type(model.sparse.ec) is QuantEC
    assert isinstance(model.dense, nn.Linear)
    assert model.sparse.weighted_ebc.is_weighted() and not model.sparse.ebc.is_weighted()
    for t in tbes(model):
        assert all(spec[3] == SparseType.INT8 for spec in t.embedding_specs)
    # register_tbes is switched on by the entry point: the operators are visible as submodules
    assert len(model.sparse.ebc.tbes) == 1 and len(model.sparse.weighted_ebc.tbes) == 1
    assert model.sparse.ebc.output_dtype() == torch.float


def test_set_pruning_data():
    model = Model(META)
    pruning = {t.name: t.num_embeddings - 1 for t in model.sparse.t}
    set_pruning_data(model, pruning)
    q = quantize_inference_model(model)
    seen = 0
    for m in q.modules():
        if isinstance(m, QuantEBC):
            for c in m.embedding_bag_configs():
                if c.name in pruning:
                    assert c.num_embeddings_post_pruning == pruning[c.name]
        elif m.__class__.__name__ == "IntNBitTableBatchedEmbeddingBagsCodegen":
            for i, spec in enumerate(m.embedding_specs):
                if spec[0] in pruning:
                    assert spec[1] == pruning[spec[0]]
                    assert m.split_embedding_weights()[i][0].size(0) == pruning[spec[0]]
                    seen += 1
    assert seen == len(pruning)


def test_quantize_per_table_dtype_with_fp_ebc():
    mfl = {"feature_0": 100, "feature_1": 100}
    model = Model(META, max_feature_lengths=mfl)
    per_table = {t.name: torch.quint4x2 for t in tables("", 4) + tables("weighted_", 2)}
    q = quantize_inference_model(model, per_table_weight_dtype=per_table)
    assert type(q.sparse.fp_ebc) is QuantFPEBC
    assert isinstance(q.sparse.fp_ebc.feature_processor, PositionWeightedModuleCollection)
    ops_ = tbes(q)
    assert len(ops_) == 3  # one per collection: fp_ebc, ebc, weighted_ebc
    for t in ops_:
        assert all(spec[3] == SparseType.INT4 for spec in t.embedding_specs)


def test_tbe_count_different_pooling():
    model = Model(META)
    model.sparse.ebc.embedding_bag_configs()[0].pooling = PoolingType.MEAN
    q = quantize_inference_model(model)
    assert len(q.sparse.ebc.tbes) == 2 and len(q.sparse.weighted_ebc.tbes) == 1


def test_quantize_embeddings_not_inplace_and_shard_refused():
    model = Model(META)
    q = quantize_embeddings(model, dtype=torch.quint2x4, inplace=False, output_dtype=torch.half)
    assert type(model.sparse.ebc) is EmbeddingBagCollection and type(q.sparse.ebc) is QuantEBC
    assert q.sparse.ebc.output_dtype() == torch.half
    assert all(spec[3] == SparseType.INT2 for t in tbes(q) for spec in t.embedding_specs)
    with pytest.raises(NotImplementedError):
        shard_quant_model(q)


def test_fp_ebc_requires_weighted_and_matching_processors():
    ebc = EmbeddingBagCollection(tables("", 2), False, META)
    with pytest.raises(AssertionError):
        FeatureProcessedEmbeddingBagCollection(ebc, PositionWeightedModuleCollection({"feature_0": 3}))
    webc = EmbeddingBagCollection(tables("", 2), True, META)
    with pytest.raises(AssertionError):
        FeatureProcessedEmbeddingBagCollection(webc, {"feature_0": PositionWeightedModule(3)})


def test_position_weights_host():
    """Host path of the position-weight processors against a loop."""
    rng = np.random.default_rng(0)
    keys, B = ["a", "b", "c"], 5
    lengths = rng.integers(0, 4, len(keys) * B)
    values = torch.arange(int(lengths.sum()))
    kjt = KeyedJaggedTensor(keys=keys, values=values, lengths=torch.from_numpy(lengths))
    pw = PositionWeightedModuleCollection({"a": 4, "c": 4})
    with torch.no_grad():
        pw.position_weights["a"].copy_(torch.tensor([1.0, 2.0, 3.0, 4.0]))
        pw.position_weights["c"].copy_(torch.tensor([10.0, 20.0, 30.0, 40.0]))
    got = pw(kjt).weights().detach().numpy()
    want = []
    for k, key in enumerate(keys):
        for b in range(B):
            for p in range(lengths[k * B + b]):
                want.append({"a": p + 1.0, "b": 1.0, "c": 10.0 * (p + 1)}[key])
    assert np.array_equal(got, np.asarray(want, dtype=np.float32))
    assert np.array_equal(ops.offsets_range(kjt.offsets(), values.numel()).numpy(),
                          np.concatenate([np.arange(l) for l in lengths]))
    jt = PositionWeightedModule(4)(JaggedTensor(values=torch.arange(5), lengths=torch.tensor([2, 3])))
    assert jt.weights().tolist() == [1.0] * 5


# --------------------------------------------------------------------------- GPU
def _kjt(rng, keys, rows, B, dev, weighted=False, max_len=6):
    lengths = rng.integers(0, max_len, len(keys) * B).astype(np.int64)
    per = lengths.reshape(len(keys), B).sum(1)
    vals = np.concatenate([rng.integers(0, rows[k], per[k]) for k in range(len(keys))]) if len(keys) else np.zeros(0)
    w = torch.from_numpy(rng.random(int(lengths.sum())).astype(np.float32)).to(dev) if weighted else None
    return KeyedJaggedTensor(keys=keys, values=torch.from_numpy(vals.astype(np.int64)).to(dev),
                             lengths=torch.from_numpy(lengths).to(dev), weights=w)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,atol", [(torch.qint8, 2e-2), (torch.quint4x2, 0.3), (torch.half, 2e-3)])
def test_quantized_model_matches_float(dtype, atol):
    dev = torch.device("cuda:0")
    torch.manual_seed(1)
    rng = np.random.default_rng(1)
    mfl = {"feature_0": 8, "feature_1": 8}
    model = Model(dev, max_feature_lengths=mfl).eval()
    with torch.no_grad():
        for p in model.sparse.fp_ebc._feature_processors.position_weights.values():
            p.copy_(torch.rand_like(p) + 0.5)
    B = 9
    s = model.sparse
    kjt = _kjt(rng, [t.feature_names[0] for t in s.t], [t.num_embeddings for t in s.t], B, dev)
    wkjt = _kjt(rng, [t.feature_names[0] for t in s.wt], [t.num_embeddings for t in s.wt], B, dev, weighted=True)
    fp_cfg = s.fp_ebc._embedding_bag_collection.embedding_bag_configs()
    fpkjt = _kjt(rng, [t.feature_names[0] for t in fp_cfg], [t.num_embeddings for t in fp_cfg], B, dev)
    with torch.no_grad():
        want = model(kjt, wkjt, fpkjt)
    q = quantize_inference_model(model, quantization_dtype=dtype, fp_weight_dtype=dtype)
    assert type(q.sparse.fp_ebc) is QuantFPEBC and len(tbes(q)) == 3
    with torch.inference_mode():
        got = q(kjt, wkjt, fpkjt)
    assert got.shape == want.shape
    assert torch.allclose(got, want, atol=atol), float((got - want).abs().max())

    # weights out of the operators and back in: same outputs
    table_to_weight = get_table_to_weights_from_tbe(q)
    assert set(table_to_weight) == {t.name for t in tables("", 4) + tables("weighted_", 2)}
    saved = {k: (w.clone(), None if sb is None else sb.clone()) for k, (w, sb) in table_to_weight.items()}
    for t in tbes(q):
        t.weights_dev.zero_()
    with torch.inference_mode():
        assert not torch.equal(q(kjt, wkjt, fpkjt), got)
    assign_weights_to_tbe(q, saved)
    with torch.inference_mode():
        assert torch.equal(q(kjt, wkjt, fpkjt), got)


@pytest.mark.gpu
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_position_weights_kernel(idt):
    """One-launch position weights == host computation; offsets_range likewise;
    positions beyond the table length take the last entry."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(4)
    keys, B = ["k0", "k1", "k2", "k3"], 37
    lengths = rng.integers(0, 12, len(keys) * B)
    lengths[5] = 40  # longer than any table below
    n = int(lengths.sum())
    host = KeyedJaggedTensor(keys=keys, values=torch.arange(n, dtype=idt), lengths=torch.from_numpy(lengths).to(idt))
    pw = PositionWeightedModuleCollection({"k0": 12, "k2": 16, "k3": 12})
    with torch.no_grad():
        for p in pw.position_weights.values():
            p.copy_(torch.rand_like(p))
    # host reference, with the clamp applied by hand
    want = []
    for k, key in enumerate(keys):
        for b in range(B):
            for p in range(lengths[k * B + b]):
                if key in pw.position_weights_dict:
                    t = pw.position_weights_dict[key].detach()
                    want.append(float(t[min(p, t.numel() - 1)]))
                else:
                    want.append(1.0)
    got = pw.to(dev)(host.to(dev)).weights()
    assert got.device.type == "cuda"
    assert np.array_equal(got.cpu().numpy(), np.asarray(want, dtype=np.float32))
    r = ops.offsets_range(host.offsets().to(dev), n)
    assert r.dtype == idt and np.array_equal(r.cpu().numpy(), np.concatenate([np.arange(l) for l in lengths]))


@pytest.mark.gpu
def test_quant_fp_ebc_bit_exact_against_oracle():
    """QuantFeatureProcessedEmbeddingBagCollection == oracle lookup with the position weights as per-sample weights."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(9)
    T, rows, D, B = 3, 300, 64, 21
    cfgs, quantized, otables = [], {}, []
    for t in range(T):
        q = O.quantize_sbhalf(rng.normal(0, 0.1, (rows, D)).astype(np.float32), 4)
        cfgs.append(EmbeddingBagConfig(name=f"t{t}", embedding_dim=D, num_embeddings=rows, feature_names=[f"f{t}"],
                                       data_type=DataType.INT4, pooling=PoolingType.SUM))
        qt = torch.from_numpy(q)
        quantized[f"t{t}"] = (qt[:, :-4].to(dev), qt[:, -4:].to(dev))
        otables.append((O.INT4, D, q))
    pw = PositionWeightedModuleCollection({"f0": 10, "f2": 10}, dev)
    with torch.no_grad():
        for p in pw.position_weights.values():
            p.copy_(torch.rand_like(p) * 2 - 1)
    m = QuantFPEBC(cfgs, True, dev, output_dtype=torch.float, table_name_to_quantized_weights=quantized,
                   feature_processor=pw)
    lengths = rng.integers(0, 10, T * B).astype(np.int32)
    offsets = np.zeros(T * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lengths)
    ids = rng.integers(0, rows, int(offsets[-1])).astype(np.int32)
    kjt = KeyedJaggedTensor(keys=["f0", "f1", "f2"], values=torch.from_numpy(ids).to(dev),
                            lengths=torch.from_numpy(lengths).to(dev))
    got = m(kjt).values().cpu().numpy()
    psw = np.ones(len(ids), dtype=np.float32)
    for k, key in enumerate(["f0", "f1", "f2"]):
        if key in pw.position_weights_dict:
            t = pw.position_weights_dict[key].detach().cpu().numpy()
            for b in range(B):
                s, e = offsets[k * B + b], offsets[k * B + b + 1]
                psw[s:e] = t[: e - s]
    want = O.tbe_forward(O.pack_store(otables), [0, 1, 2], B, ids, offsets, psw, O.SUM, O.FP32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("B,max_len,idt,from_offsets", [
    (21, 10, torch.int32, False),      # small: static kernel
    (33, 30, torch.int64, True),       # bags longer than the weight vectors (clamped), int64 ids, KJT with offsets
    (4096, 40, torch.int32, False),    # window kernel, offsets derived inside the lookup kernel
    (4096, 40, torch.int32, True),     # window kernel from offsets
])
def test_position_weights_inside_the_lookup_kernel(B, max_len, idt, from_offsets):
    """The feature-processed collection looks the position weights up inside
    the lookup kernel.  Same bits as materializing them first (the weights are
    the same fp32 values either way), for a key order that differs from the
    module's, a key without weights, an unused key, MEAN and SUM tables."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(B + max_len)
    rows, D = 500, 64
    names = ["a", "b", "c", "d"]
    cfgs, quantized = [], {}
    for t, name in enumerate(names):
        q = torch.from_numpy(O.quantize_sbhalf(rng.normal(0, 0.1, (rows, D)).astype(np.float32), 4 if t % 2 else 8))
        cfgs.append(EmbeddingBagConfig(name=f"t_{name}", embedding_dim=D, num_embeddings=rows, feature_names=[name],
                                       data_type=DataType.INT4 if t % 2 else DataType.INT8,
                                       pooling=PoolingType.MEAN if t == 3 and B < 1000 else PoolingType.SUM))
        quantized[f"t_{name}"] = (q[:, :-4].to(dev), q[:, -4:].to(dev))
    pw = PositionWeightedModuleCollection({"a": 20, "c": 7, "d": 20}, dev)  # "b" has none: weight 1
    with torch.no_grad():
        for p in pw.position_weights.values():
            p.copy_(torch.rand_like(p) * 2 - 1)
    m = QuantFPEBC(cfgs, True, dev, output_dtype=torch.half, table_name_to_quantized_weights=quantized,
                   feature_processor=pw)
    keys = ["c", "unused", "a", "d", "b"]
    lengths = rng.integers(0, max_len + 1, len(keys) * B).astype(np.int64)
    ids = rng.integers(0, rows, int(lengths.sum()))
    kw = dict(keys=keys, values=torch.from_numpy(ids).to(idt).to(dev))
    if from_offsets:
        offsets = np.zeros(len(lengths) + 1, dtype=np.int64)
        offsets[1:] = np.cumsum(lengths)
        kjt = KeyedJaggedTensor(offsets=torch.from_numpy(offsets).to(idt).to(dev), **kw)
    else:
        kjt = KeyedJaggedTensor(lengths=torch.from_numpy(lengths).to(idt).to(dev), **kw)
    fused = m(kjt)
    materialized = QuantEBC.forward(m, pw(kjt))
    assert fused.keys() == materialized.keys()
    assert torch.equal(fused.values().view(torch.int16), materialized.values().view(torch.int16))
    # a replaced weight vector is picked up
    with torch.no_grad():
        pw.position_weights["a"].mul_(0.5)
    assert torch.equal(m(kjt).values().view(torch.int16), QuantEBC.forward(m, pw(kjt)).values().view(torch.int16))
    assert not torch.equal(m(kjt).values(), fused.values())


@pytest.mark.gpu
def test_scratch_address_follows_a_replaced_buffer():
    """The operator remembers the scratch address per call shape.  A larger call
    replaces the stream's buffer: the addresses remembered for smaller shapes go
    with it, on the plain route and on the position-weighted one alike."""
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    rows, D = 300, 32
    q = torch.from_numpy(O.quantize_sbhalf(rng.normal(0, 0.1, (rows, D)).astype(np.float32), 8))
    cfg = EmbeddingBagConfig(name="t", embedding_dim=D, num_embeddings=rows, feature_names=["a", "b"],
                             data_type=DataType.INT8)
    pw = PositionWeightedModuleCollection({"a": 9, "b": 9}, dev)
    with torch.no_grad():
        for p in pw.position_weights.values():
            p.copy_(torch.rand_like(p) + 0.5)
    m = QuantFPEBC([cfg], True, dev, table_name_to_quantized_weights={"t": (q[:, :-4].to(dev), q[:, -4:].to(dev))},
                   feature_processor=pw)
    op = m._emb_modules[0]

    def kjt_of(B):
        lengths = rng.integers(0, 9, 2 * B).astype(np.int32)
        ids = rng.integers(0, rows, int(lengths.sum())).astype(np.int32)
        return KeyedJaggedTensor(keys=["a", "b"], values=torch.from_numpy(ids).to(dev),
                                 lengths=torch.from_numpy(lengths).to(dev))

    def remembered_addresses_are_live():
        for (_, _, _, stream), address in op._ws_ptr.items():
            assert address == op._workspace[stream].data_ptr()

    def weighted_from_lengths(kjt):
        # the weights materialized, the KJT still without offsets: the plain lengths route
        return KeyedJaggedTensor(keys=kjt.keys(), values=kjt.values(), weights=pw(kjt).weights(),
                                 lengths=kjt.lengths())

    small, large = kjt_of(48), kjt_of(20000)
    plain_small = QuantEBC.forward(m, weighted_from_lengths(small)).values().clone()
    fused_small = m(small).values().clone()                         # position-weighted route, same shape
    assert torch.equal(plain_small, fused_small)
    assert op._ws_ptr, "neither route took scratch: the test covers nothing"
    remembered_addresses_are_live()
    fused_large = m(large).values().clone()                         # replaces the buffer
    remembered_addresses_are_live()
    assert torch.equal(QuantEBC.forward(m, weighted_from_lengths(small)).values(), plain_small)
    assert torch.equal(m(small).values(), fused_small)
    remembered_addresses_are_live()
    assert torch.equal(fused_large, QuantEBC.forward(m, weighted_from_lengths(large)).values())
    assert torch.equal(fused_large, QuantEBC.forward(m, pw(large)).values())


@pytest.mark.gpu
def test_position_weighted_entry_checks_its_layout():
    """The C entry point validates the host-side layout against the table."""
    dev = torch.device("cuda:0")
    rows, D, B = 50, 32, 4
    q = torch.from_numpy(O.quantize_sbhalf(np.zeros((rows, D), dtype=np.float32), 8))
    cfg = EmbeddingBagConfig(name="t", embedding_dim=D, num_embeddings=rows, feature_names=["f"], data_type=DataType.INT8)
    m = QuantEBC([cfg], True, dev, table_name_to_quantized_weights={"t": (q[:, :-4].to(dev), q[:, -4:].to(dev))})
    op = m._emb_modules[0]
    ids = torch.zeros(8, dtype=torch.int32, device=dev)
    offsets = torch.arange(0, 10, 2, dtype=torch.int32, device=dev)
    table = torch.ones(6, device=dev)
    op(ids, offsets, position_weights=(table, [0], [6]))
    with pytest.raises(RuntimeError, match="outside the table"):
        op(ids, offsets, position_weights=(table, [2], [6]))
    with pytest.raises(RuntimeError, match="outside the table"):
        op(ids, offsets, position_weights=(table, [-1], [3]))
    with pytest.raises(AssertionError):
        op(ids, offsets, position_weights=(table, [], []))


@pytest.mark.gpu
def test_forward_rejects_misaligned_buffers():
    """Ids, bag boundaries, weights and the output must sit at multiples of
    their element size: the C entry point says so instead of launching."""
    from torchrec_amd import _lib

    dev = torch.device("cuda:0")
    rows, D, B = 50, 32, 4
    q = torch.from_numpy(O.quantize_sbhalf(np.zeros((rows, D), dtype=np.float32), 8))
    cfg = EmbeddingBagConfig(name="t", embedding_dim=D, num_embeddings=rows, feature_names=["f"], data_type=DataType.INT8)
    m = QuantEBC([cfg], True, dev, table_name_to_quantized_weights={"t": (q[:, :-4].to(dev), q[:, -4:].to(dev))})
    op = m._emb_modules[0]
    ids = torch.zeros(10, dtype=torch.int64, device=dev)
    offsets = torch.arange(0, 10, 2, dtype=torch.int64, device=dev)
    out = torch.empty(B, D, dtype=torch.float32, device=dev)
    l, plan, stream = _lib.lib(), op._get_plan(None), _lib.current_stream(dev)

    def call(w, i, o, dst):
        return l.tra_tbe_forward(plan, w, i, o, 1, None, B, 8, 0, _lib.FP32, dst, D, stream)

    w = op.weights_dev.data_ptr()
    assert call(w, ids.data_ptr(), offsets.data_ptr(), out.data_ptr()) == 0
    for args in (
        (w + 2, ids.data_ptr(), offsets.data_ptr(), out.data_ptr()),
        (w, ids.data_ptr() + 4, offsets.data_ptr(), out.data_ptr()),
        (w, ids.data_ptr(), offsets.data_ptr() + 4, out.data_ptr()),
        (w, ids.data_ptr(), offsets.data_ptr(), out.data_ptr() + 2),
    ):
        assert call(*args) == -1 and b"aligned" in l.tra_last_error()
    torch.cuda.synchronize()


@pytest.mark.gpu
def test_operator_built_on_cpu_then_moved():
    """An operator filled on the CPU and moved with ``.to()`` looks up like one
    built on the GPU."""
    from torchrec_amd.tbe import PoolingMode
    from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import IntNBitTableBatchedEmbeddingBagsCodegen

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    rows, D, B = 200, 64, 16
    q = torch.from_numpy(O.quantize_sbhalf(rng.standard_normal((rows, D)).astype(np.float32), 4))
    pair = [(q[:, :-4].contiguous(), q[:, -4:].contiguous())]
    spec = [("t", rows, D, SparseType.INT4, None)]
    on_gpu = IntNBitTableBatchedEmbeddingBagsCodegen(
        spec, device=dev, pooling_mode=PoolingMode.SUM, weight_lists=[(w.to(dev), s.to(dev)) for w, s in pair]
    )
    moved = IntNBitTableBatchedEmbeddingBagsCodegen(
        spec, device=torch.device("cpu"), pooling_mode=PoolingMode.SUM, weight_lists=pair
    ).to(dev)
    assert moved.current_device == dev and moved.weights_dev.is_cuda
    lengths = torch.from_numpy(rng.integers(0, 9, size=B).astype(np.int32))
    ids = torch.from_numpy(rng.integers(0, rows, size=int(lengths.sum())).astype(np.int32)).to(dev)
    offsets = torch.cat([torch.zeros(1, dtype=torch.int32), lengths.cumsum(0).int()]).to(dev)
    assert torch.equal(on_gpu(ids, offsets), moved(ids, offsets))
