"""Every benchmark configuration under `pytest -m gpu`, built by bench.py's own
workload generator (same seeds, row counts and id distributions as the
benchmark: log-uniform table sizes, Zipf ids through a permutation, Poisson
lengths, the 68-byte-row store), at full size where the device holds it.

Full-size outputs cannot all go through the scalar CPU oracle in test time,
so each configuration is checked two ways: (1) a sample of samples (all their
features) against the oracle, run on the rows those bags touch, gathered from
the module's own packed store; (2) size-independent properties over the whole
output: every route (window kernel from lengths, from offsets, static kernel)
gives the same bits; MEAN == SUM * (1/len).  The bar is 0 differing bit
patterns."""
import argparse
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402
import oracle as O  # noqa: E402
from helpers import bits_equal  # noqa: E402
from torchrec_amd import KeyedJaggedTensor, _lib  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
CODE = {"fp32": O.FP32, "fp16": O.FP16, "int8": O.INT8, "int4": O.INT4, "int2": O.INT2}


@pytest.fixture(autouse=True)
def _release_device_memory():
    """The stores here are large (up to 136 GB): hand them back after each test."""
    yield
    import gc
    gc.collect()
    torch.cuda.empty_cache()


def _workload(config, scale=1.0, batches=1, row_alignment=None):
    if row_alignment is None:
        row_alignment = 4 if config == "c5" else 16
    args = argparse.Namespace(config=config, batches=batches, row_alignment=row_alignment, scale=scale, batch_size=None)
    return bench.build_workload(args, DEV)


def _free_bytes():
    free, _ = torch.cuda.mem_get_info()
    return free


def _oracle_on_samples(wl, values, lengths, weights, samples, pooling, out_dtype):
    """Oracle output for samples `samples` (all features): the rows their bags
    touch are gathered from the module's packed store into a compact store."""
    tbe = wl["module"]._emb_modules[0]
    T, B = wl["T"], wl["B"]
    assert list(tbe.feature_table_map) == list(range(T))
    lens = lengths.cpu().numpy().astype(np.int64)
    offs = np.zeros(T * B + 1, dtype=np.int64)
    offs[1:] = np.cumsum(lens)
    Bs = len(samples)
    pick = np.concatenate([np.arange(offs[t * B + b], offs[t * B + b + 1]) for t in range(T) for b in samples]) \
        if Bs else np.zeros(0, np.int64)
    pick_t = torch.from_numpy(pick).to(DEV)
    ids = values[pick_t].cpu().numpy().astype(np.int64)
    w = None if weights is None else weights[pick_t].cpu().numpy()
    sub_len = lens.reshape(T, B)[:, samples].reshape(-1)
    sub_off = np.zeros(T * Bs + 1, dtype=np.int32)
    sub_off[1:] = np.cumsum(sub_len)
    pieces, t_off, t_rows, base = [], [], [], 0
    for t in range(T):
        seg = ids[sub_off[t * Bs]:sub_off[(t + 1) * Bs]]
        uniq = np.unique(seg)
        ids[sub_off[t * Bs]:sub_off[(t + 1) * Bs]] = np.searchsorted(uniq, seg)
        rb = tbe.row_bytes[t]
        view = tbe._rows_view(t)
        rows = view[torch.from_numpy(uniq).to(DEV)].cpu().numpy() if len(uniq) else np.zeros((0, rb), np.uint8)
        if len(uniq) == 0:  # the oracle wants a row to exist
            rows = np.zeros((1, rb), np.uint8)
        pieces.append(rows.reshape(-1))
        t_off.append(base)
        t_rows.append(rows.shape[0])
        pad = O.round_up(rows.size, 128) - rows.size
        pieces.append(np.zeros(pad, np.uint8))
        base += rows.size + pad
    store = O.Store(np.concatenate(pieces), np.asarray(t_off, np.int64), np.asarray(t_rows, np.int64),
                    np.asarray(tbe.dims, np.int32), np.asarray([CODE[str(x)] for x in tbe.weight_tys], np.int32),
                    np.asarray(tbe.row_bytes, np.int32))  # (rows were gathered at their width)
    return O.tbe_forward(store, list(range(T)), Bs, ids.astype(np.int32), sub_off, w, pooling, out_dtype)


def _forward(wl, i=0, with_offsets=False):
    v, l, w = wl["batches"][i]
    if with_offsets:
        off = torch.zeros(l.numel() + 1, dtype=torch.int32, device=DEV)
        off[1:] = torch.cumsum(l, 0)
        kjt = KeyedJaggedTensor(keys=wl["keys"], values=v, offsets=off, weights=w, stride=wl["B"])
    else:
        kjt = KeyedJaggedTensor(keys=wl["keys"], values=v, lengths=l, weights=w)
    return wl["module"](kjt)


def _check_routes_agree(wl, out):
    """from-lengths == from-offsets == static kernel, bit for bit, over the whole output."""
    view = torch.int16 if out.dtype == torch.float16 else torch.int32
    b = _forward(wl, with_offsets=True).values()
    assert torch.equal(out.view(view), b.view(view))
    _lib.set_tuning(balanced=0)
    try:
        c = _forward(wl, with_offsets=True).values()
    finally:
        _lib.set_tuning(balanced=None)
    assert torch.equal(out.view(view), c.view(view))


def test_config1_full():
    """C1 at full size, the whole output against the oracle."""
    wl = _workload("c1")
    out = _forward(wl).values()
    v, l, w = wl["batches"][0]
    want = _oracle_on_samples(wl, v, l, w, np.arange(wl["B"]), O.SUM, O.FP16)
    assert out.shape == (512, 512) and bits_equal(out.cpu().numpy(), want) == 0


def test_config2_full_size_zipf_log_uniform_rows():
    """C2 as the benchmark builds it: 26 tables of log-uniform[1e3, 4e7] rows (6 GB),
    B 2048, lengths U[1,40] with 5 % empty, Zipf(1.05) ids through a permutation."""
    if _free_bytes() < 12e9:
        pytest.skip("needs 12 GB of free device memory")
    wl = _workload("c2", batches=2)
    assert min(wl["rows"]) < 5_000 and max(wl["rows"]) > 10_000_000  # the log-uniform spread is there
    out = _forward(wl).values()
    v, l, w = wl["batches"][0]
    # Zipf: a handful of rows take a large share of the lookups
    seg = v[: int(l[:wl["B"]].sum())]
    assert torch.bincount(seg.long()).max().item() > 20
    # one permutation per table, shared by the batches: the hottest row of every table is the
    # same row in both batches (and is the rank-1 row of the generator), the ids are not
    B = wl["B"]
    big = max(range(wl["T"]), key=lambda t: wl["rows"][t])
    for t in (0, big, wl["T"] - 1):
        top = []
        for vb, lb, _ in wl["batches"]:
            ends = torch.cumsum(lb.view(wl["T"], B).sum(dim=1), 0)
            seg_t = vb[int(ends[t - 1]) if t else 0: int(ends[t])].long()
            top.append(int(torch.bincount(seg_t).argmax()))
        assert top[0] == top[1] == int(wl["hot_ids"][t][0]), (t, top)
    assert not torch.equal(wl["batches"][0][0][:1000], wl["batches"][1][0][:1000])
    samples = np.arange(0, wl["B"], 16)  # 128 samples x 26 features
    want = _oracle_on_samples(wl, v, l, w, samples, O.SUM, O.FP16)
    assert bits_equal(np.ascontiguousarray(out[torch.from_numpy(samples).to(DEV)].cpu().numpy()), want) == 0
    _check_routes_agree(wl, out)
    assert wl["module"]._emb_modules[0].out_of_range_count() == 0


def test_config3_all_64_tables():
    """C3 as the benchmark builds it: 64 tables, dims {32,64,128,256} x {int8,int4,int2,fp16},
    rows log-uniform[1e5, 1e7] (14 GB), B 4096, Poisson(30) lengths, weighted SUM, fp32 out."""
    if _free_bytes() < 24e9:
        pytest.skip("needs 24 GB of free device memory")
    wl = _workload("c3")
    assert wl["T"] == 64 and len(set(zip(wl["dims"], wl["dts"]))) == 16
    out = _forward(wl).values()
    v, l, w = wl["batches"][0]
    samples = np.arange(0, wl["B"], 128)  # 32 samples x 64 features
    want = _oracle_on_samples(wl, v, l, w, samples, O.SUM, O.FP32)
    got = np.ascontiguousarray(out[torch.from_numpy(samples).to(DEV)].cpu().numpy())
    assert bits_equal(got, want) == 0
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)  # the stated tolerance, for the record
    _check_routes_agree(wl, out)


def test_config4_sequence_full_size():
    """C4 as the benchmark builds it: 16 tables x 1e6 x 128 int8 (2.3 GB), B 1024, lengths
    U[0,256], uniform ids, jagged fp16 output; the rows of 8 samples per feature against the oracle."""
    if _free_bytes() < 8e9:
        pytest.skip("needs 8 GB of free device memory")
    wl = _workload("c4")
    v, l, w = wl["batches"][0]
    out = wl["module"](KeyedJaggedTensor(keys=wl["keys"], values=v, lengths=l))
    T, B = wl["T"], wl["B"]
    lens = l.cpu().numpy().astype(np.int64)
    offs = np.zeros(T * B + 1, dtype=np.int64)
    offs[1:] = np.cumsum(lens)
    tbe = wl["module"]._emb_modules[0]
    for t in (0, 7, 15):
        jt = out[f"f{t}"]
        assert jt.values().shape == (int(lens[t * B:(t + 1) * B].sum()), 128) and jt.values().dtype == torch.float16
        assert torch.equal(jt.lengths().cpu(), l[t * B:(t + 1) * B].cpu())
        lo, hi = offs[t * B + 100], offs[t * B + 108]  # samples 100..107 of the feature
        ids = v[lo:hi].cpu().numpy().astype(np.int64)
        uniq = np.unique(ids)
        rows = tbe._rows_view(t)[torch.from_numpy(uniq).to(DEV)].cpu().numpy()
        store = O.Store(rows.reshape(-1), np.asarray([0], np.int64), np.asarray([len(uniq)], np.int64),
                        np.asarray([128], np.int32), np.asarray([O.INT8], np.int32), np.asarray([tbe.row_bytes[t]], np.int32))
        n = len(ids)
        want = O.tbe_forward(store, [0], 1, np.searchsorted(uniq, ids).astype(np.int32), np.asarray([0, n], np.int32),
                             None, O.NONE, O.FP16)
        first = offs[t * B]
        got = jt.values()[lo - first:hi - first].cpu().numpy()
        assert bits_equal(np.ascontiguousarray(got), want) == 0, t


def test_config5_shape_shortened_tables_whole_output():
    """C5's shape with tables of 1 M rows: 8 tables x 128 int4 at row_alignment 4 (68-byte
    rows), B 16384, L = 80, Zipf(0.8) ids through the affine bijection, MEAN, fp16 out;
    the whole [16384, 1024] output against the oracle."""
    wl = _workload("c5", scale=1e6 / 250e6)
    tbe = wl["module"]._emb_modules[0]
    assert tbe.row_bytes == [68] * 8 and wl["rows"] == [1_000_000] * 8 and wl["B"] == 16384
    out = _forward(wl).values()
    v, l, w = wl["batches"][0]
    assert int(l.min()) == 80 == int(l.max())
    want = _oracle_on_samples(wl, v, l, w, np.arange(wl["B"]), O.MEAN, O.FP16)
    assert out.shape == (16384, 1024) and bits_equal(out.cpu().numpy(), want) == 0
    _check_routes_agree(wl, out)


def test_config5_full_136_GB_store():
    """C5 at full size: 8 x 250 M rows of 68 bytes = 136 GB resident, 10.5 M lookups per call.
    512 samples (all 8 features) against the oracle on the rows they touch; every route gives
    the same bits; MEAN equals SUM * (1/80) computed from a SUM lookup over the same store."""
    if _free_bytes() < 150e9:
        pytest.skip("needs 150 GB of free device memory for the 136 GB store")
    wl = _workload("c5")
    tbe = wl["module"]._emb_modules[0]
    assert tbe.weights_size >= 136e9 and tbe.row_bytes == [68] * 8
    out = _forward(wl).values()
    v, l, w = wl["batches"][0]
    samples = np.arange(0, wl["B"], 32)
    want = _oracle_on_samples(wl, v, l, w, samples, O.MEAN, O.FP16)
    assert bits_equal(np.ascontiguousarray(out[torch.from_numpy(samples).to(DEV)].cpu().numpy()), want) == 0
    _check_routes_agree(wl, out)
    # MEAN == SUM * (1/80): a SUM operator over the same packed bytes (no second store), fp32 out
    from torchrec_amd.tbe import EmbeddingLocation, PoolingMode, SparseType
    from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import IntNBitTableBatchedEmbeddingBagsCodegen as TBE
    mk = lambda mode: TBE(embedding_specs=[(f"t{i}", 250_000_000, 128, SparseType.INT4, EmbeddingLocation.DEVICE) for i in range(8)],
                          pooling_mode=mode, device=DEV, output_dtype=SparseType.FP32, row_alignment=4)
    outs = {}
    for mode in (PoolingMode.SUM, PoolingMode.MEAN):
        op = mk(mode)
        assert op.weights_size == tbe.weights_size
        op.weights_dev = tbe.weights_dev  # alias the resident store
        op._weights_initialized = True
        outs[mode] = op(v, None, lengths=l, batch_size=wl["B"])
    inv = torch.ones(1, device=DEV) / torch.full((1,), 80.0, device=DEV)  # 1.0f / 80.0f, as the kernel forms it
    assert torch.equal(outs[PoolingMode.MEAN], outs[PoolingMode.SUM] * inv)
