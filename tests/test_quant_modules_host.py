"""Host-side behaviour of the quantized modules that needs no GPU: grouping,
naming, key order, dtype mapping, state_dict layout and aliasing, error
behaviour.  Expectations follow the reference's tests
(torchrec/quant/tests/test_embedding_modules.py:238-275, 311, 342-402, 849,
999-1025; torchrec/quant/tests/test_tensor_types.py:24-50)."""
import pytest
import torch

from torchrec_amd import _lib, KeyedJaggedTensor
from torchrec_amd.modules.embedding_configs import (
    data_type_to_sparse_type,
    DataType,
    dtype_to_data_type,
    EmbeddingBagConfig,
    EmbeddingConfig,
    pooling_type_to_pooling_mode,
    PoolingType,
)
from torchrec_amd.modules.embedding_modules import get_embedding_names_by_table
from torchrec_amd.quant.embedding_modules import (
    _fx_trec_unwrap_kjt,
    EmbeddingBagCollection as QuantEBC,
    EmbeddingCollection as QuantEC,
)
from torchrec_amd.tbe import PoolingMode, SparseType
from torchrec_amd.tensor_types import UInt2Tensor, UInt4Tensor

CPU = torch.device("cpu")


def test_dtype_maps():
    assert dtype_to_data_type(torch.quint4x2) == DataType.INT4
    assert dtype_to_data_type(torch.quint2x4) == DataType.INT2
    assert dtype_to_data_type(torch.qint8) == DataType.INT8 == dtype_to_data_type(torch.quint8)
    assert dtype_to_data_type(torch.uint8) == DataType.UINT8
    assert dtype_to_data_type(torch.half) == DataType.FP16 and dtype_to_data_type(torch.float) == DataType.FP32
    assert data_type_to_sparse_type(DataType.UINT8) == SparseType.INT8
    assert [SparseType.FP32.as_int(), SparseType.FP16.as_int(), SparseType.INT8.as_int(),
            SparseType.INT4.as_int(), SparseType.INT2.as_int()] == [0, 1, 2, 3, 4]
    assert pooling_type_to_pooling_mode(PoolingType.MEAN) == PoolingMode.MEAN
    with pytest.raises(Exception):
        dtype_to_data_type(torch.complex64)


def test_grouping_names_and_order():
    tables = [
        EmbeddingBagConfig(name="t1", embedding_dim=16, num_embeddings=10, feature_names=["f1", "f3"], data_type=DataType.INT4),
        EmbeddingBagConfig(name="t2", embedding_dim=32, num_embeddings=10, feature_names=["f2"], data_type=DataType.INT8, pooling=PoolingType.MEAN),
        EmbeddingBagConfig(name="t3", embedding_dim=8, num_embeddings=10, feature_names=["f1"], data_type=DataType.FP16),
    ]
    q = QuantEBC(tables, False, CPU, output_dtype=torch.half)
    # grouped by pooling: SUM tables (t1, t3) first, then MEAN (t2); shared feature f1 gets @table
    assert [len(m.embedding_specs) for m in q._emb_modules] == [2, 1]
    assert q._feature_names == ["f1", "f3", "f1", "f2"]
    assert q._feature_splits == [3, 1]
    assert q._embedding_names == ["f1@t1", "f3", "f1@t3", "f2"]
    assert q._length_per_key == [16, 16, 8, 32]
    assert q._emb_modules[0].pooling_mode == PoolingMode.SUM and q._emb_modules[1].pooling_mode == PoolingMode.MEAN
    assert get_embedding_names_by_table(tables) == [["f1@t1", "f3"], ["f2"], ["f1@t3"]]
    assert q.output_dtype() == torch.half and not q.is_weighted() and q.device == CPU
    with pytest.raises(ValueError, match="Duplicate table name"):
        QuantEBC([tables[0], tables[0]], False, CPU)


def test_ec_dim_mismatch_and_grouping():
    t = [EmbeddingConfig(name="a", embedding_dim=16, num_embeddings=10, feature_names=["fa"], data_type=DataType.INT8),
         EmbeddingConfig(name="b", embedding_dim=16, num_embeddings=10, feature_names=["fb"], data_type=DataType.INT4),
         EmbeddingConfig(name="c", embedding_dim=16, num_embeddings=10, feature_names=["fc"], data_type=DataType.INT8)]
    q = QuantEC(t, CPU)
    assert q._feature_names == ["fa", "fc", "fb"] and q._feature_splits == [2, 1]
    assert q.embedding_names_by_table() == [["fa"], ["fb"], ["fc"]] and q.embedding_dim() == 16
    with pytest.raises(ValueError, match="same embedding dimension"):
        QuantEC(t + [EmbeddingConfig(name="d", embedding_dim=8, num_embeddings=10, feature_names=["fd"])], CPU)


@pytest.mark.parametrize("split", [False, True])
def test_state_dict_layout_and_aliasing(split):
    tables = [
        EmbeddingBagConfig(name="t8", embedding_dim=16, num_embeddings=10, feature_names=["a"], data_type=DataType.INT8),
        EmbeddingBagConfig(name="t4", embedding_dim=16, num_embeddings=10, feature_names=["b"], data_type=DataType.INT4),
        EmbeddingBagConfig(name="t2", embedding_dim=16, num_embeddings=10, feature_names=["c"], data_type=DataType.INT2),
        EmbeddingBagConfig(name="th", embedding_dim=16, num_embeddings=10, feature_names=["d"], data_type=DataType.FP16),
    ]
    q = QuantEBC(tables, False, CPU, quant_state_dict_split_scale_bias=split)
    sd = q.state_dict()
    keys = set(sd.keys())
    assert {f"embedding_bags.{t.name}.weight" for t in tables} <= keys
    if split:
        assert {"embedding_bags.t8.weight_qscale", "embedding_bags.t4.weight_qbias"} <= keys
        assert sd["embedding_bags.t8.weight"].shape == (10, 16)
        assert sd["embedding_bags.t4.weight"].shape == (10, 16) and isinstance(sd["embedding_bags.t4.weight"], UInt4Tensor)
        assert sd["embedding_bags.t2.weight"].shape == (10, 16) and isinstance(sd["embedding_bags.t2.weight"], UInt2Tensor)
        assert sd["embedding_bags.t4.weight"].view(torch.uint8).shape == (10, 8)
        assert sd["embedding_bags.t8.weight_qscale"].dtype == torch.float16
        assert sd["embedding_bags.th.weight"].shape == (10, 32)  # fp16 bytes
    else:
        assert sd["embedding_bags.t8.weight"].shape == (10, 32)  # 16 + 4 -> padded to 32
    # buffers alias the packed store: loading a state dict rewrites the store in place
    tbe = q._emb_modules[0]
    before = tbe.weights_dev.clone()
    new_sd = {k: (v.view(torch.uint8).clone() if isinstance(v, (UInt4Tensor, UInt2Tensor)) else v.clone()) for k, v in sd.items()}
    for k in new_sd:
        if new_sd[k].dtype == torch.uint8:
            new_sd[k].fill_(0x5A)
    wrapped = {}
    for k, v in new_sd.items():
        orig = sd[k]
        wrapped[k] = type(orig)(v) if isinstance(orig, (UInt4Tensor, UInt2Tensor)) else v
    q.load_state_dict(wrapped)
    assert not torch.equal(before, tbe.weights_dev)
    assert (tbe.weights_dev == 0x5A).any()


def test_uintx_tensors():
    e = torch.arange(64, dtype=torch.uint8).view(4, 16)
    t4 = UInt4Tensor(e)
    assert t4.shape == (4, 32) and t4.dtype == torch.uint8
    assert torch.equal(t4.view(torch.uint8), e)
    assert torch.equal(t4[:, :8].view(torch.uint8), e[:, :4]) and t4[:, :8].shape == (4, 8)
    assert torch.equal(t4[1:3].view(torch.uint8), e[1:3])
    t2 = UInt2Tensor(e)
    assert t2.shape == (4, 64) and torch.equal(t2[:, 8:16].view(torch.uint8), e[:, 2:4])
    c = t4.clone()
    assert isinstance(c, UInt4Tensor) and torch.equal(c.view(torch.uint8), e)
    c.copy_(UInt4Tensor(torch.zeros_like(e)))
    assert not c.view(torch.uint8).any() and e.any()
    assert t4.view(8, 16).shape == (8, 16)


def test_unwrap_kjt_dtype_rule_host():
    for dt in (torch.int32, torch.int64):
        kjt = KeyedJaggedTensor(keys=["a"], values=torch.tensor([1, 2], dtype=dt), lengths=torch.tensor([2], dtype=torch.int32))
        i, o = _fx_trec_unwrap_kjt(kjt)
        assert i.dtype == dt and o.dtype == dt


def test_forward_without_gpu_fails_loudly():
    tables = [EmbeddingBagConfig(name="t", embedding_dim=16, num_embeddings=10, feature_names=["f"], data_type=DataType.INT8)]
    q = QuantEBC(tables, False, CPU)
    kjt = KeyedJaggedTensor(keys=["f"], values=torch.tensor([1, 2]), lengths=torch.tensor([2]))
    with pytest.raises(_lib.TorchrecAmdError, match="MI355X"):
        q(kjt)
    with pytest.raises(ValueError):  # missing feature
        q(KeyedJaggedTensor(keys=["g"], values=torch.tensor([1]), lengths=torch.tensor([1])))


def test_feature_order_is_resolved_per_key_order():
    """The module remembers the order it resolved for a key order, and resolves a
    different key order afresh (the reference's cache_features_order flag, which
    pins the first order seen, is honoured separately)."""
    tables = [
        EmbeddingBagConfig(name="t1", embedding_dim=16, num_embeddings=10, feature_names=["f1", "f3"], data_type=DataType.INT4),
        EmbeddingBagConfig(name="t2", embedding_dim=32, num_embeddings=10, feature_names=["f2"], data_type=DataType.INT8, pooling=PoolingType.MEAN),
    ]
    q = QuantEBC(tables, False, CPU)
    assert q._feature_names == ["f1", "f3", "f2"]
    a = q._resolve_order(["f1", "f2", "f3"])
    assert a == [0, 2, 1] and q._resolve_order(["f1", "f2", "f3"]) is a
    assert q._group_positions(a) == [(0, 2), (1,)] and q._group_positions(a) is q._group_positions(a)
    b = q._resolve_order(["x", "f3", "f2", "f1"])
    assert b == [3, 1, 2] and q._group_positions(b) == [(3, 1), (2,)]
    with pytest.raises(ValueError):
        q._resolve_order(["f1", "f2"])  # a missing feature is a list.index error, as in the reference
    pinned = QuantEBC(tables, False, CPU, cache_features_order=True)
    first = pinned._resolve_order(["f3", "f2", "f1"])
    assert first == [2, 0, 1] and pinned._resolve_order(["f1", "f2", "f3"]) is first


def test_create_on_meta_device_without_providing_weights():
    """torchrec/quant/tests/test_embedding_modules.py:220-236."""
    from torchrec_amd.modules.embedding_configs import EmbeddingBagConfig, EmbeddingConfig
    from torchrec_amd.quant import EmbeddingBagCollection as QEBC, EmbeddingCollection as QEC

    qebc = QEBC([EmbeddingBagConfig(name="t1", embedding_dim=16, num_embeddings=10, feature_names=["f1"])],
                is_weighted=False, device=torch.device("meta"))
    assert qebc.state_dict()["embedding_bags.t1.weight"].device.type == "meta"
    qec = QEC([EmbeddingConfig(name="t1", embedding_dim=16, num_embeddings=10, feature_names=["f1"])],
              device=torch.device("meta"))
    assert qec.state_dict()["embeddings.t1.weight"].device.type == "meta"


def test_operator_follows_its_buffer_between_devices():
    """``.to()`` moves the packed buffer; the operator's launch device follows
    and a lookup away from the GPU still fails with a message, not a fault."""
    from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import IntNBitTableBatchedEmbeddingBagsCodegen

    op = IntNBitTableBatchedEmbeddingBagsCodegen(
        [("t", 10, 8, SparseType.INT8, None)], device=CPU, pooling_mode=PoolingMode.SUM
    )
    op.initialize_weights()
    assert op.current_device == CPU and op.weights_dev.device == CPU
    op.to("meta")
    assert op.current_device.type == "meta" and op.weights_dev.device.type == "meta"
    with pytest.raises(_lib.TorchrecAmdError, match="MI355X"):
        op(torch.zeros(2, dtype=torch.int32), torch.tensor([0, 2], dtype=torch.int32))


def test_operator_copies_and_pickles_without_its_plans():
    """Launch plans are C handles owned by one object: a deep copy or a pickle
    carries the packed bytes and configuration and starts with no plans."""
    import copy
    import ctypes
    import io

    from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import IntNBitTableBatchedEmbeddingBagsCodegen

    op = IntNBitTableBatchedEmbeddingBagsCodegen(
        [("t", 10, 8, SparseType.INT8, None)], device=CPU, pooling_mode=PoolingMode.SUM
    )
    op.initialize_weights()
    op.weights_dev.fill_(7)
    op._plans[None] = ctypes.c_void_p(0)  # stands in for a plan handle (NULL: destroy is a no-op)
    twin = copy.deepcopy(op)
    assert twin._plans == {} and len(op._plans) == 1
    assert torch.equal(twin.weights_dev, op.weights_dev) and twin.weights_dev.data_ptr() != op.weights_dev.data_ptr()
    buf = io.BytesIO()
    torch.save(op, buf)
    buf.seek(0)
    back = torch.load(buf, weights_only=False)
    assert back._plans == {} and torch.equal(back.weights_dev, op.weights_dev)
    assert back.embedding_specs == op.embedding_specs and back.row_bytes == op.row_bytes


def test_row_padding_layout_and_views():
    """Rows of at most 128 bytes lie at the next power-of-two stride (no row straddles a
    128-byte line) while the padded store fits the budget; every view keeps the row's width."""
    from torchrec_amd import tbe as tbe_pkg
    from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
        IntNBitTableBatchedEmbeddingBagsCodegen as TBE,
        line_padded_row_stride,
    )

    assert [line_padded_row_stride(w) for w in (4, 12, 16, 20, 48, 64, 68, 80, 128, 132, 144, 272)] == [
        4, 16, 16, 32, 64, 64, 128, 128, 128, 132, 144, 272]
    specs = [("a", 10, 128, SparseType.INT4, None), ("b", 7, 256, SparseType.INT8, None), ("c", 5, 32, SparseType.FP16, None)]
    op = TBE(specs, device=CPU, pooling_mode=PoolingMode.SUM)  # the default: "line"
    assert tbe_pkg.get_default_row_padding() == "line" and op.row_padding == "line"
    assert op.row_bytes == [80, 272, 64] and op.row_stride == [128, 272, 64]
    assert op.weights_physical_offsets == [0, 1280, 1280 + 2048] and op.weights_size == 1280 + 2048 + 512
    op.initialize_weights()
    for mode, widths in ((0, [80, 272, 64]), (1, [64, 256, 64]), (2, [64, 256, 64])):
        for t, (w, s, b) in enumerate(op.split_embedding_weights_with_scale_bias(mode)):
            assert w.shape == (specs[t][1], widths[t]) and w.stride() == (op.row_stride[t], 1)
            assert w.untyped_storage().data_ptr() == op.weights_dev.untyped_storage().data_ptr()
    w, scale, bias = op.split_embedding_weights_with_scale_bias(2)[0]
    assert scale.dtype == torch.float16 and scale.shape == (10, 1) and scale.stride(0) == 64
    # writing through the views lands in the rows of the packed buffer, 128 bytes apart
    w.fill_(0x21)
    scale.fill_(1.0)
    bias.fill_(-2.0)
    raw = op.weights_dev[:1280].view(10, 128)
    assert (raw[:, 4:68] == 0x21).all() and (raw[:, 80:] == 0).all() and (raw[:, 68:80] == 0).all()
    assert raw[:, :4].reshape(-1).tolist() == [0x00, 0x3C, 0x00, 0xC0] * 10
    # the same operator with its rows at their width
    tight = TBE(specs, device=CPU, pooling_mode=PoolingMode.SUM, row_padding="none")
    assert tight.row_stride == tight.row_bytes == [80, 272, 64] and tight.weights_size == 1024 + 2048 + 512
    # assigning weights gives the same table contents in either layout
    tight.initialize_weights()
    tight.assign_embedding_weights([(a, b) for a, b in op.split_embedding_weights(True)])
    for (x, xs), (y, ys) in zip(op.split_embedding_weights(True), tight.split_embedding_weights(True)):
        assert torch.equal(x, y) and (xs is None or torch.equal(xs, ys))
    with pytest.raises(ValueError, match="row_padding"):
        TBE(specs, device=CPU, row_padding="page")


def test_row_padding_budget_and_default_switch(monkeypatch):
    """An operator whose padded store would exceed the budget keeps its rows at their width
    (the 68-byte rows of a 136 GB store stay 68 bytes apart); the default can be switched."""
    from torchrec_amd import tbe as tbe_pkg
    from torchrec_amd.tbe import split_table_batched_embeddings_ops_inference as mod

    big = [("t", 250_000_000, 128, SparseType.INT4, None)] * 8
    op = mod.IntNBitTableBatchedEmbeddingBagsCodegen(
        [(f"t{i}",) + s[1:] for i, s in enumerate(big)], device=torch.device("meta"), row_alignment=4)
    assert op.row_bytes == [68] * 8 and op.row_stride == [68] * 8 and op.weights_size == 136_000_000_000
    monkeypatch.setattr(mod, "ROW_PADDING_BUDGET_BYTES", 1000)
    small = mod.IntNBitTableBatchedEmbeddingBagsCodegen([("t", 10, 128, SparseType.INT4, None)], device=CPU)
    assert small.row_stride == [80]  # 10 x 128 bytes would not fit a budget of 1000
    monkeypatch.undo()
    previous = tbe_pkg.set_default_row_padding("none")
    try:
        assert previous == "line"
        assert mod.IntNBitTableBatchedEmbeddingBagsCodegen([("t", 10, 128, SparseType.INT4, None)], device=CPU).row_stride == [80]
    finally:
        tbe_pkg.set_default_row_padding(previous)
    assert mod.IntNBitTableBatchedEmbeddingBagsCodegen([("t", 10, 128, SparseType.INT4, None)], device=CPU).row_stride == [128]
    with pytest.raises(ValueError):
        tbe_pkg.set_default_row_padding("page")


def _stub_lookups(module, calls):
    """Stand-ins for the operators' GPU lookup: zeros into the caller's buffer, and a record of
    whether the operator was reached through ``__call__`` (hooks fire) or through ``forward``."""
    for i, op in enumerate(module._emb_modules):
        def fake_forward(*args, _i=i, **kw):
            calls.append(("forward", _i))
            kw["out"].zero_()
            return kw["out"]
        op.forward = fake_forward  # type: ignore[method-assign]
        op.register_forward_pre_hook(lambda m, a, kw=None, _i=i: calls.append(("hook", _i)))


def test_ec_batching_hint_follows_the_prepared_lengths_form(monkeypatch):
    """The order of the reference's graph (torchrec/quant/embedding_modules.py:943-950, pinned by
    torchrec/quant/tests/test_embedding_modules.py:1027-1117): by default the batching hint sees
    the flattened lengths and the lengths are unflattened afterwards; prepared with
    ``__use_unflattened_lengths_for_batching`` the hint is a user of the unflattened lengths;
    with ``__use_batching_hinted_output`` off (and flattened lengths) there is no hint."""
    from torchrec_amd.quant import embedding_modules as qm

    t = [EmbeddingConfig(name="t1", embedding_dim=16, num_embeddings=10, feature_names=["f1", "f2"], data_type=DataType.FP16),
         EmbeddingConfig(name="t2", embedding_dim=16, num_embeddings=10, feature_names=["f3", "f4"], data_type=DataType.FP16)]
    q = QuantEC(t, CPU, output_dtype=torch.half)
    calls = []
    _stub_lookups(q, calls)
    seen = []
    real_unflatten, real_hint = qm._get_unflattened_lengths, qm._get_batching_hinted_output
    monkeypatch.setattr(qm, "_get_unflattened_lengths",
                        lambda lengths, n: (seen.append(("unflatten", tuple(lengths.shape))), real_unflatten(lengths, n))[1])
    monkeypatch.setattr(qm, "_get_batching_hinted_output",
                        lambda lengths, output: (seen.append(("hint", tuple(lengths.shape))), real_hint(lengths=lengths, output=output))[1])
    kjt = KeyedJaggedTensor(keys=["f1", "f2", "f3", "f4"], values=torch.arange(6) % 10,
                            lengths=torch.tensor([1, 0, 2, 0, 1, 1, 0, 1]))
    out = q(kjt)
    assert seen == [("hint", (8,)), ("unflatten", (8,))]
    assert [tuple(out[k].values().shape) for k in ("f1", "f2", "f3", "f4")] == [(1, 16), (2, 16), (2, 16), (1, 16)]
    assert out["f3"].lengths().tolist() == [1, 1]
    seen.clear()
    setattr(q, qm.MODULE_ATTR_USE_UNFLATTENED_LENGTHS_FOR_BATCHING, True)
    q(kjt)
    assert seen == [("unflatten", (8,)), ("hint", (4, 2))]
    seen.clear()
    setattr(q, qm.MODULE_ATTR_USE_UNFLATTENED_LENGTHS_FOR_BATCHING, False)
    setattr(q, qm.MODULE_ATTR_USE_BATCHING_HINTED_OUTPUT, False)
    q(kjt)
    assert seen == [("unflatten", (8,))]
    # every lookup above went through the operators' forward (they are not registered)
    assert calls and all(kind == "forward" for kind, _ in calls)


def test_ec_remove_padding_drops_rows_behind_the_last_bag():
    """``__remove_stbe_padding``: a values tensor longer than the lengths add up to (padding at
    its end) yields per-feature rows of the bags only, and the buffer is cut at the last bag's end
    (construct_jagged_tensors_inference(remove_padding=True), torchrec/modules/utils.py:315-316)."""
    from torchrec_amd.quant import embedding_modules as qm

    t = [EmbeddingConfig(name="t1", embedding_dim=8, num_embeddings=10, feature_names=["f1", "f2"], data_type=DataType.INT8)]
    q = QuantEC(t, CPU, output_dtype=torch.float, need_indices=True)
    _stub_lookups(q, [])
    values = torch.tensor([3, 4, 5, 6, 7, 9, 9, 9])  # three entries of padding
    kjt = KeyedJaggedTensor(keys=["f1", "f2"], values=values, lengths=torch.tensor([2, 1, 0, 2]))
    for flag in (False, True):
        setattr(q, qm.MODULE_ATTR_REMOVE_STBE_PADDING_BOOL, flag)
        out = q(kjt)
        assert out["f1"].values().shape == (3, 8) and out["f2"].values().shape == (2, 8)
        assert out["f1"].weights().tolist() == [3, 4, 5] and out["f2"].weights().tolist() == [6, 7]
        base = out["f1"].values()
        rows_in_buffer = base.untyped_storage().nbytes() // (8 * 4)
        assert rows_in_buffer == 8  # one buffer for the whole KJT either way; the views stop at row 5


@pytest.mark.parametrize("cls", ["ebc", "ec"])
def test_registered_operators_are_called_as_modules(cls):
    """``register_tbes``: the operators are submodules (``tbes``) and the collection calls them
    through ``__call__``, so hooks see every lookup; unregistered operators are reached through
    ``forward`` (torchrec/quant/embedding_modules.py:546-557, 938-942)."""
    for register in (False, True):
        if cls == "ebc":
            t = [EmbeddingBagConfig(name="t1", embedding_dim=8, num_embeddings=10, feature_names=["f1"], data_type=DataType.INT8),
                 EmbeddingBagConfig(name="t2", embedding_dim=8, num_embeddings=10, feature_names=["f2"], data_type=DataType.INT8,
                                    pooling=PoolingType.MEAN)]
            q = QuantEBC(t, False, CPU, output_dtype=torch.float, register_tbes=register)
        else:
            t = [EmbeddingConfig(name="t1", embedding_dim=8, num_embeddings=10, feature_names=["f1"], data_type=DataType.INT8),
                 EmbeddingConfig(name="t2", embedding_dim=8, num_embeddings=10, feature_names=["f2"], data_type=DataType.INT4)]
            q = QuantEC(t, CPU, output_dtype=torch.float, register_tbes=register)
        assert hasattr(q, "tbes") == register
        calls = []
        _stub_lookups(q, calls)
        q(KeyedJaggedTensor(keys=["f1", "f2"], values=torch.tensor([1, 2, 3]), offsets=torch.tensor([0, 1, 2, 2, 3])))
        kinds = [kind for kind, _ in calls]
        assert kinds.count("forward") == 2
        assert kinds.count("hook") == (2 if register else 0)


@pytest.mark.parametrize("split", [False, True])
def test_state_dict_moves_between_row_paddings(split):
    """A state dict saved from a collection whose rows lie at their width loads into one whose rows
    are line-padded (and back): the buffers have the same names and shapes in either layout, and
    the table contents (payload, scale, bias of every row) arrive unchanged."""
    from torchrec_amd import tbe as tbe_pkg

    tables = [
        EmbeddingBagConfig(name="t4", embedding_dim=128, num_embeddings=12, feature_names=["a"], data_type=DataType.INT4),
        EmbeddingBagConfig(name="t8", embedding_dim=32, num_embeddings=9, feature_names=["b"], data_type=DataType.INT8),
        EmbeddingBagConfig(name="th", embedding_dim=16, num_embeddings=7, feature_names=["c"], data_type=DataType.FP16),
    ]

    def build(padding):
        previous = tbe_pkg.set_default_row_padding(padding)
        try:
            return QuantEBC(tables, False, CPU, quant_state_dict_split_scale_bias=split)
        finally:
            tbe_pkg.set_default_row_padding(previous)

    tight, padded = build("none"), build("line")
    assert tight._emb_modules[0].row_stride == [80, 48, 32] and padded._emb_modules[0].row_stride == [128, 64, 32]
    gen = torch.Generator().manual_seed(3)
    src = tight._emb_modules[0]
    src.weights_dev.copy_(torch.randint(0, 256, src.weights_dev.shape, dtype=torch.uint8, generator=gen))
    sd = tight.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {k: tuple(v.shape) for k, v in padded.state_dict().items()}
    padded.load_state_dict(sd)
    contents = lambda m: [(w.clone(), None if s is None else s.clone())
                          for w, s in m._emb_modules[0].split_embedding_weights(True)]
    for (w0, s0), (w1, s1) in zip(contents(tight), contents(padded)):
        assert torch.equal(w0, w1) and (s0 is None or torch.equal(s0, s1))
    # and back into a fresh tight collection
    again = build("none")
    again.load_state_dict(padded.state_dict())
    for (w0, s0), (w1, s1) in zip(contents(tight), contents(again)):
        assert torch.equal(w0, w1) and (s0 is None or torch.equal(s0, s1))
