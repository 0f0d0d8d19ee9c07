"""Parity of the HIP lookup (through IntNBitTableBatchedEmbeddingBagsCodegen and
the C ABI) against the CPU oracle.  The oracle's formula is reproducible
bit-for-bit and the kernels evaluate it in the same order, so the bar here is
0 differing bit patterns; that is stricter than the stated tolerance
(1e-5 relative for fp32 outputs, 2 ulp for fp16 outputs)."""
import itertools

import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_equal, make_bags, make_table, weight_pair
from torchrec_amd.tbe import EmbeddingLocation, PoolingMode, SparseType
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen as TBE,
)

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
ST = {O.FP32: SparseType.FP32, O.FP16: SparseType.FP16, O.INT8: SparseType.INT8,
      O.INT4: SparseType.INT4, O.INT2: SparseType.INT2}
POOL = {O.SUM: PoolingMode.SUM, O.MEAN: PoolingMode.MEAN, O.NONE: PoolingMode.NONE}


def build(rng, specs, ftm, pooling, out_dtype, row_alignment, row_padding=None, bounds_check_mode=None):
    """specs: [(dtype, rows, dim)].  Returns (TBE on GPU, oracle Store).  The packed store's row
    padding (rows of up to 128 bytes at a power-of-two stride, or every row at its width) is drawn
    from the test's generator unless given: the oracle has its own copy of the tables, so the
    lookups must not depend on it."""
    if row_padding is None:
        row_padding = ("line", "none")[int(rng.integers(2))]
    datas = [make_table(rng, dt, rows, dim) for dt, rows, dim in specs]
    store = O.pack_store([(dt, dim, d) for (dt, _, dim), d in zip(specs, datas)], row_alignment=row_alignment)
    weight_lists = []
    for (dt, _, _), d in zip(specs, datas):
        w, sb = weight_pair(dt, d)
        weight_lists.append((torch.from_numpy(np.ascontiguousarray(w)).to(DEV),
                             None if sb is None else torch.from_numpy(np.ascontiguousarray(sb)).to(DEV)))
    tbe = TBE(
        embedding_specs=[(f"t{i}", rows, dim, ST[dt], EmbeddingLocation.DEVICE) for i, (dt, rows, dim) in enumerate(specs)],
        feature_table_map=ftm, pooling_mode=POOL[pooling], device=DEV, weight_lists=weight_lists,
        output_dtype=ST[out_dtype], row_alignment=row_alignment, row_padding=row_padding,
        bounds_check_mode=bounds_check_mode,
    )
    return tbe, store


def run_both(tbe, store, ftm, B, ids, offsets, psw, pooling, out_dtype):
    got = tbe(
        torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV),
        None if psw is None else torch.from_numpy(psw).to(DEV),
    ).cpu().numpy()
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, pooling, out_dtype)
    return got, want


@pytest.mark.parametrize("dtype", [O.INT8, O.INT4, O.INT2, O.FP16, O.FP32])
@pytest.mark.parametrize("pooling,weighted", [(O.SUM, False), (O.SUM, True), (O.MEAN, False), (O.MEAN, True), (O.NONE, False)])
def test_lookup_bit_exact_all_dims(dtype, pooling, weighted):
    """Every weight type x pooling x {fp32, fp16} out x {int32, int64} ids x dims 32..256,
    bags 0..80 long with empties, row_alignment 16 and the tight packing."""
    rng = np.random.default_rng(100 + dtype * 10 + pooling)
    for dim, out_dtype, idt, align in itertools.product(
        (32, 64, 128, 256), (O.FP32, O.FP16), (np.int32, np.int64), (16, 4)
    ):
        rows, B = 2000, 37
        specs = [(dtype, rows, dim), (dtype, rows + 13, dim)]
        ftm = [0, 1, 0]
        tbe, store = build(rng, specs, ftm, pooling, out_dtype, align)
        lengths, offsets, ids = make_bags(rng, [rows, rows + 13, rows], B, 80, idt)
        psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
        got, want = run_both(tbe, store, ftm, B, ids, offsets, psw, pooling, out_dtype)
        assert bits_equal(got, want) == 0, (dim, out_dtype, idt, align)
        assert tbe.out_of_range_count() == 0


def test_mixed_group_one_call():
    """One TBE group mixing all weight types and dims 32/64/128/256 (weighted SUM, fp32 out)."""
    rng = np.random.default_rng(3)
    specs = []
    for t in range(16):
        specs.append(([O.INT8, O.INT4, O.INT2, O.FP16][(t // 4) % 4], 500 + 7 * t, [32, 64, 128, 256][t % 4]))
    ftm = list(range(16))
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP32, 16)
    B = 64
    lengths, offsets, ids = make_bags(rng, [s[1] for s in specs], B, 40)
    psw = rng.uniform(0, 1, len(ids)).astype(np.float32)
    got, want = run_both(tbe, store, ftm, B, ids, offsets, psw, O.SUM, O.FP32)
    assert bits_equal(got, want) == 0
    # stated tolerance, for the record
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)


@pytest.mark.parametrize("dtype,dim", [(O.INT8, 8), (O.INT8, 12), (O.INT8, 24), (O.INT4, 8), (O.INT4, 24),
                                       (O.INT4, 40), (O.INT2, 16), (O.INT2, 48), (O.FP16, 2), (O.FP16, 6),
                                       (O.FP16, 20), (O.FP32, 1), (O.FP32, 3), (O.FP32, 10), (O.INT8, 1040), (O.INT8, 520), (O.INT4, 1048),
                                       (O.INT2, 2064),
                                       (O.FP16, 1000), (O.FP32, 520)])
def test_odd_dims(dtype, dim):
    """Payloads that are not multiples of 16 bytes (8- and 4-byte lane chunks) and
    rows wider than one wave of 16-byte chunks (column slices)."""
    rng = np.random.default_rng(dim)
    for pooling in (O.SUM, O.NONE):
        rows, B = 300, 19
        tbe, store = build(rng, [(dtype, rows, dim)], [0], pooling, O.FP32, 4)
        lengths, offsets, ids = make_bags(rng, [rows], B, 9)
        got, want = run_both(tbe, store, [0], B, ids, offsets, None, pooling, O.FP32)
        assert bits_equal(got, want) == 0


@pytest.mark.parametrize("route", ["static", "window", "lengths", "static-lengths"])
def test_wide_rows_next_to_ordinary_ones(tuning, route):
    """int-N rows too wide for one wave of 8- or 4-byte lane chunks are cut into column slices and get
    a launch class of their own (the header is loaded separately there); ordinary rows of the same
    weight type keep the class whose first lane receives the header with its chunk.  Both in one
    operator, weighted MEAN, every pooled kernel and both entries, against the oracle."""
    tuning(balanced=1 if route in ("window", "lengths") else 0)
    rng = np.random.default_rng(len(route))
    rows, B = 400, 160
    specs = [(O.INT8, rows, 520), (O.INT4, rows, 128), (O.INT8, rows, 64), (O.INT4, rows, 1048), (O.INT2, rows, 2064),
             (O.INT2, rows, 64)]
    ftm = [0, 1, 2, 3, 4, 5, 1]
    tbe, store = build(rng, specs, ftm, O.MEAN, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * len(ftm), B, 30)
    psw = rng.uniform(-1, 1, len(ids)).astype(np.float32)
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, O.MEAN, O.FP16)
    if route.endswith("lengths"):
        got = _from_lengths(tbe, ids, lengths, psw, B)
    else:
        got = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV), torch.from_numpy(psw).to(DEV)).cpu().numpy()
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0


def test_edge_bags():
    """All-empty input, a single very long bag, pruned ids (-1), and out-of-range ids."""
    rng = np.random.default_rng(11)
    rows, dim, B = 1000, 128, 8
    tbe, store = build(rng, [(O.INT4, rows, dim)], [0], O.SUM, O.FP16, 16)
    # all bags empty -> exact zeros
    offsets = np.zeros(B + 1, dtype=np.int32)
    ids = np.zeros(0, dtype=np.int32)
    got, want = run_both(tbe, store, [0], B, ids, offsets, None, O.SUM, O.FP16)
    assert bits_equal(got, want) == 0 and not got.any()
    # the same with an (empty) per-sample weight tensor
    got = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV),
              torch.zeros(0, device=DEV)).cpu().numpy()
    assert not got.any()
    # one bag of 5000 ids, the rest empty
    offsets = np.zeros(B + 1, dtype=np.int32)
    offsets[4:] = 5000
    ids = rng.integers(0, rows, 5000).astype(np.int32)
    got, want = run_both(tbe, store, [0], B, ids, offsets, None, O.SUM, O.FP16)
    assert bits_equal(got, want) == 0
    # -1 ids are skipped, exactly as the CPU kernels do
    ids2 = ids.copy()
    ids2[::7] = -1
    got, want = run_both(tbe, store, [0], B, ids2, offsets, None, O.SUM, O.FP16)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0
    # ids >= rows are skipped and counted
    ids3 = ids.copy()
    ids3[:5] = rows + 3
    got = tbe(torch.from_numpy(ids3).to(DEV), torch.from_numpy(offsets).to(DEV)).cpu().numpy()
    ids3[:5] = -1
    want = O.tbe_forward(store, [0], B, ids3, offsets, None, O.SUM, O.FP16)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 5
    assert tbe.out_of_range_count() == 0


def test_feature_positions_and_out_columns():
    """Lookup straight from a key order that differs from the operator's features,
    with an unused key in between, writing into a slice of a wider output."""
    rng = np.random.default_rng(5)
    rows, dim, B = 800, 64, 33
    specs = [(O.INT8, rows, dim), (O.INT4, rows, dim)]
    tbe, store = build(rng, specs, [0, 1], O.SUM, O.FP32, 16)
    # KJT keys: [f1, unused, f0]
    lengths, offsets, ids = make_bags(rng, [rows, rows, rows], B, 20)
    out = torch.full((B, 3 * dim + 5), 7.0, device=DEV)
    tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV), feature_positions=[2, 0],
        batch_size=B, out=out, out_col=dim)
    # oracle: reorder by hand
    seg = [ids[offsets[k * B]:offsets[(k + 1) * B]] for k in range(3)]
    L = lengths.reshape(3, B)
    o_len = np.concatenate([L[2], L[0]])
    o_off = np.zeros(2 * B + 1, dtype=np.int32)
    o_off[1:] = np.cumsum(o_len)
    want = O.tbe_forward(store, [0, 1], B, np.concatenate([seg[2], seg[0]]), o_off, None, O.SUM, O.FP32)
    got = out.cpu().numpy()
    assert bits_equal(np.ascontiguousarray(got[:, dim:3 * dim]), want) == 0
    assert (got[:, :dim] == 7.0).all() and (got[:, 3 * dim:] == 7.0).all()


def test_config1_shape_full():
    """The smallest benchmark workload at full size: 8 tables x 100k x 64 int8, B=512, L=20, SUM, fp16 out."""
    rng = np.random.default_rng(1001)
    T, rows, dim, B = 8, 100_000, 64, 512
    specs = [(O.INT8, rows, dim)] * T
    tbe, store = build(rng, specs, list(range(T)), O.SUM, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 20, fixed_len=20)
    got, want = run_both(tbe, store, list(range(T)), B, ids, offsets, None, O.SUM, O.FP16)
    assert got.shape == (512, 512)
    assert bits_equal(got, want) == 0


def test_properties_large():
    """Size-independent properties on a larger problem (no oracle run):
    weighted with w == 1 equals unweighted; MEAN == SUM * (1/len) in fp32;
    permuting features permutes output columns only."""
    rng = np.random.default_rng(77)
    T, rows, dim, B = 12, 200_000, 128, 2048
    specs = [(O.INT4, rows, dim)] * T
    datas = [make_table(rng, O.INT4, rows, dim) for _ in range(T)]
    wl = [(torch.from_numpy(np.ascontiguousarray(d[:, :-4])).to(DEV), torch.from_numpy(np.ascontiguousarray(d[:, -4:])).to(DEV)) for d in datas]
    mk = lambda pooling, order: TBE(
        embedding_specs=[(f"t{i}", rows, dim, SparseType.INT4, EmbeddingLocation.DEVICE) for i in order],
        pooling_mode=pooling, device=DEV, weight_lists=[wl[i] for i in order], output_dtype=SparseType.FP32)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 40)
    ti, to = torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV)
    s = mk(PoolingMode.SUM, range(T))
    a = s(ti, to)
    b = s(ti, to, torch.ones(len(ids), device=DEV))
    assert torch.equal(a, b)
    m = mk(PoolingMode.MEAN, range(T))(ti, to)
    ln = torch.from_numpy(lengths.astype(np.int64)).to(DEV).view(T, B).t().float()  # [B, T]
    inv = torch.where(ln > 0, 1.0 / ln, torch.ones_like(ln)).repeat_interleave(dim, dim=1)
    assert torch.equal(m, a * inv)
    order = list(rng.permutation(T))
    p = mk(PoolingMode.SUM, order)(ti, to, feature_positions=order, batch_size=B)
    assert torch.equal(p.view(B, T, dim), a.view(B, T, dim)[:, order, :])


def test_sequence_properties_at_scale():
    """Sequence lookup at the shape of the unpooled workload (16 features, int8
    x 128, 1024 samples of 0..256 ids, ~2.1 M ids; tables shortened to 100 K
    rows), without an oracle run: a row of the output is the SUM-pooled bag that
    holds just that id (same arithmetic, other kernel); equal ids give equal
    rows; permuting a feature's ids permutes its rows; id -1 gives a zero row."""
    rng = np.random.default_rng(404)
    T, rows, dim, B = 16, 100_000, 128, 1024
    datas = [make_table(rng, O.INT8, rows, dim) for _ in range(T)]
    wl = [(torch.from_numpy(np.ascontiguousarray(d[:, :-4])).to(DEV), torch.from_numpy(np.ascontiguousarray(d[:, -4:])).to(DEV)) for d in datas]
    seq = TBE(embedding_specs=[(f"t{i}", rows, dim, SparseType.INT8, EmbeddingLocation.DEVICE) for i in range(T)],
              pooling_mode=PoolingMode.NONE, device=DEV, weight_lists=wl, output_dtype=SparseType.FP16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 256)
    ids[rng.integers(0, len(ids), 1000)] = -1
    ti, to = torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV)
    out = seq(ti, to)
    assert out.shape == (len(ids), dim) and out.dtype == torch.float16
    # feature 3 alone through the pooled kernels, one id per bag
    f = 3
    lo, hi = int(offsets[f * B]), int(offsets[(f + 1) * B])
    pooled = TBE(embedding_specs=[("t", rows, dim, SparseType.INT8, EmbeddingLocation.DEVICE)],
                 pooling_mode=PoolingMode.SUM, device=DEV, weight_lists=[wl[f]], output_dtype=SparseType.FP16)
    one_each = torch.arange(hi - lo + 1, dtype=ti.dtype, device=DEV)
    want = pooled(ti[lo:hi].contiguous(), one_each)
    assert torch.equal(out[lo:hi].view(torch.int16), want.view(torch.int16))
    # equal ids, equal rows; -1 is a zero row
    seg = ti[lo:hi]
    order = torch.argsort(seg, stable=True)
    same = seg[order][1:] == seg[order][:-1]
    rows_sorted = out[lo:hi][order]
    assert torch.equal(rows_sorted[1:][same], rows_sorted[:-1][same])
    assert not out[ti == -1].any()
    # a permutation of one feature's ids permutes its rows and leaves the others alone
    perm = torch.randperm(hi - lo, device=DEV)
    ti2 = ti.clone()
    ti2[lo:hi] = seg[perm]
    out2 = seq(ti2, to)
    assert torch.equal(out2[lo:hi], out[lo:hi][perm])
    assert torch.equal(out2[:lo], out[:lo]) and torch.equal(out2[hi:], out[hi:])


# The pooled lookup has two kernels: a static bag->wave mapping for small calls
# and a per-CU window kernel that ranks bags by length (taken when a call has
# at least 10240 bags and 163840 ids).  The library's tuning overrides
# (tra_set_tuning: "balanced", "window") put oracle-sized inputs through the
# window kernel in the tests below; the `tuning` fixture restores the defaults.

@pytest.mark.parametrize("dtype", [O.INT8, O.INT4, O.INT2, O.FP16, O.FP32])
@pytest.mark.parametrize("pooling,weighted", [(O.SUM, False), (O.SUM, True), (O.MEAN, False), (O.MEAN, True)])
def test_window_kernel_bit_exact(tuning, dtype, pooling, weighted):
    """Window kernel vs oracle: every weight type x pooling, both id widths and
    output types, several windows per feature and a ragged last window."""
    tuning(balanced=1)
    rng = np.random.default_rng(900 + dtype * 10 + pooling + weighted)
    for dim, out_dtype, idt, window in ((128, O.FP32, np.int32, 64), (64, O.FP16, np.int64, 100),
                                        (256, O.FP16, np.int32, 0), (32, O.FP32, np.int64, 2048)):
        tuning(window=window)
        rows, B = 3000, 211
        specs = [(dtype, rows, dim), (dtype, rows + 13, dim)]
        ftm = [0, 1, 0]
        tbe, store = build(rng, specs, ftm, pooling, out_dtype, 16)
        lengths, offsets, ids = make_bags(rng, [rows, rows + 13, rows], B, 60, idt)
        psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
        got, want = run_both(tbe, store, ftm, B, ids, offsets, psw, pooling, out_dtype)
        assert bits_equal(got, want) == 0, (dim, out_dtype, idt, window)
        assert tbe.out_of_range_count() == 0


def test_window_kernel_mixed_and_edges(tuning):
    """Window kernel: one group mixing weight types and dims (several launch
    classes and sub-classes), bags longer than the exact length bins, empty
    bags, -1 and out-of-range ids, and a key order that differs from the
    operator's feature order."""
    tuning(balanced=1)
    tuning(window=96)
    rng = np.random.default_rng(41)
    specs = [([O.INT8, O.INT4, O.INT2, O.FP16][(t // 4) % 4], 500 + 7 * t, [32, 64, 128, 256][t % 4]) for t in range(16)]
    ftm = list(range(16))
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP32, 16)
    B = 77
    lengths, offsets, ids = make_bags(rng, [s[1] for s in specs], B, 40)
    psw = rng.uniform(0, 1, len(ids)).astype(np.float32)
    got, want = run_both(tbe, store, ftm, B, ids, offsets, psw, O.SUM, O.FP32)
    assert bits_equal(got, want) == 0

    rows, dim, B = 1000, 128, 40
    tbe, store = build(rng, [(O.INT4, rows, dim)], [0, 0], O.MEAN, O.FP16, 16)
    lens = rng.integers(0, 30, 2 * B)
    lens[3], lens[50], lens[51] = 700, 5000, 193   # coarse bins, last bin, first coarse bin
    lens[10:20] = 0
    offsets = np.zeros(2 * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lens)
    ids = rng.integers(0, rows, offsets[-1]).astype(np.int32)
    ids[::7] = -1
    got, want = run_both(tbe, store, [0, 0], B, ids, offsets, None, O.MEAN, O.FP16)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0
    bad = ids.copy()
    pos = np.flatnonzero(bad >= 0)[:9]
    bad[pos] = rows + 5
    got = tbe(torch.from_numpy(bad).to(DEV), torch.from_numpy(offsets).to(DEV)).cpu().numpy()
    bad[pos] = -1
    want = O.tbe_forward(store, [0, 0], B, bad, offsets, None, O.MEAN, O.FP16)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 9

    # all bags empty
    z = np.zeros(2 * B + 1, dtype=np.int32)
    got, want = run_both(tbe, store, [0, 0], B, np.zeros(0, dtype=np.int32), z, None, O.MEAN, O.FP16)
    assert bits_equal(got, want) == 0 and not got.any()

    # keys [f1, unused, f0] read in place, written into a slice of a wider output
    rows, dim, B = 800, 64, 133
    tbe, store = build(rng, [(O.INT8, rows, dim), (O.INT4, rows, dim)], [0, 1], O.SUM, O.FP32, 16)
    lengths, offsets, ids = make_bags(rng, [rows, rows, rows], B, 20)
    out = torch.full((B, 3 * dim + 5), 7.0, device=DEV)
    tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV), feature_positions=[2, 0],
        batch_size=B, out=out, out_col=dim)
    seg = [ids[offsets[k * B]:offsets[(k + 1) * B]] for k in range(3)]
    L = lengths.reshape(3, B)
    o_off = np.zeros(2 * B + 1, dtype=np.int32)
    o_off[1:] = np.cumsum(np.concatenate([L[2], L[0]]))
    want = O.tbe_forward(store, [0, 1], B, np.concatenate([seg[2], seg[0]]), o_off, None, O.SUM, O.FP32)
    got = out.cpu().numpy()
    assert bits_equal(np.ascontiguousarray(got[:, dim:3 * dim]), want) == 0
    assert (got[:, :dim] == 7.0).all() and (got[:, 3 * dim:] == 7.0).all()


def _position_psw(lens, table, key_start, key_len, B):
    """Per-id weights the position-weighted entry applies: the id at place k of a
    bag of key p gets table[key_start[p] + min(k, key_len[p] - 1)]."""
    out = []
    for bag, n in enumerate(lens):
        p = bag // B
        k = np.minimum(np.arange(n), key_len[p] - 1)
        out.append(table[key_start[p] + k])
    return np.concatenate(out).astype(np.float32) if out else np.zeros(0, np.float32)


def _run_entry(tbe, entry, ids, lens, offsets, B, table=None, key_start=None, key_len=None):
    ti = torch.from_numpy(ids).to(DEV)
    kw = {}
    if entry.startswith("position"):
        kw["position_weights"] = (torch.from_numpy(table).to(DEV), list(key_start), list(key_len))
    if entry in ("lengths", "position_lengths"):
        return tbe(ti, None, lengths=torch.from_numpy(lens.astype(ids.dtype)).to(DEV), batch_size=B, **kw).cpu().numpy()
    return tbe(ti, torch.from_numpy(offsets).to(DEV), batch_size=B, **kw).cpu().numpy()


LONG_BAG_CASES = {
    # two bags that share the sort bin 192..255 and meet in one round, the shorter first
    "200_250": lambda rng, n: _with(rng, n, {0: 200, 1: 250, 9: 255, 10: 192, 17: 254, 30: 193}),
    # the open last bin (>= 4224)
    "last_bin": lambda rng, n: _with(rng, n, {2: 4300, 3: 6000, 40: 4224, 41: 9000}),
    # every bag long, lengths spread over several 64-wide bins
    "random_150_600": lambda rng, n: rng.integers(150, 601, n),
    # 64-wide bins 256..319 and 320..383 with many members each
    "bins_256_383": lambda rng, n: rng.integers(256, 384, n),
}


def _with(rng, n, fixed):
    lens = rng.integers(0, 12, n)
    for i, v in fixed.items():
        lens[i] = v
    return lens


@pytest.mark.parametrize("entry", ["offsets", "lengths", "position_offsets", "position_lengths"])
@pytest.mark.parametrize("pooling", [O.SUM, O.MEAN])
@pytest.mark.parametrize("case", sorted(LONG_BAG_CASES))
def test_window_kernel_long_bags(tuning, entry, pooling, case):
    """Bags of 192 ids and more, whose sort bins hold a range of lengths, several
    of them in one window and one round of the window kernel: every id of every
    bag is pooled (the reference pools a bag whatever its length,
    torchrec/quant/embedding_modules.py:547-557).  Offsets, lengths and
    position-weighted entries, SUM and MEAN, against the oracle bit for bit."""
    tuning(balanced=1, window=128)
    rng = np.random.default_rng(sum(map(ord, case)) + pooling)
    rows, dim, B, F = 2000, 128, 48, 2
    tbe, store = build(rng, [(O.INT4, rows, dim), (O.INT8, rows + 7, dim)], [0, 1], pooling, O.FP32, 16)
    lens = LONG_BAG_CASES[case](rng, F * B).astype(np.int64)
    offsets = np.zeros(F * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lens)
    ids = np.concatenate([rng.integers(0, rows, int(lens[f * B:(f + 1) * B].sum())) for f in range(F)]).astype(np.int32)
    ids[::11] = -1
    table = rng.uniform(0.5, 1.5, 40).astype(np.float32)
    key_start, key_len = [0, 25], [25, 15]
    psw = _position_psw(lens, table, key_start, key_len, B) if entry.startswith("position") else None
    want = O.tbe_forward(store, [0, 1], B, ids, offsets, psw, pooling, O.FP32)
    got = _run_entry(tbe, entry, ids, lens, offsets, B, table, key_start, key_len)
    assert bits_equal(got, want) == 0, (case, entry, pooling)
    assert tbe.out_of_range_count() == 0


@pytest.mark.parametrize("entry", ["offsets", "lengths"])
@pytest.mark.parametrize("pooling,weighted", [(O.SUM, False), (O.MEAN, True)])
def test_long_bags_default_route_at_scale(entry, pooling, weighted):
    """The same long bags where the window kernel is the default route (12 x
    1024 bags, lengths 150..600 mixed with short ones, ~1.2 M ids): equal to the
    static kernel's bits everywhere, and a sample of bags equal to the oracle."""
    from torchrec_amd import _lib
    rng = np.random.default_rng(515 + pooling)
    T, rows, dim, B = 12, 20_000, 128, 1024
    tbe, store = build(rng, [(O.INT4, rows, dim)] * T, list(range(T)), pooling, O.FP16, 16)
    lens = rng.integers(0, 30, T * B)
    long_ = rng.random(T * B) < 0.25
    lens[long_] = rng.integers(150, 601, int(long_.sum()))
    offsets = np.zeros(T * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lens)
    ids = rng.integers(0, rows, int(offsets[-1])).astype(np.int32)
    psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
    ti = torch.from_numpy(ids).to(DEV)
    tw = None if psw is None else torch.from_numpy(psw).to(DEV)
    import ctypes
    buf = ctypes.create_string_buffer(512)
    _lib.check(_lib.lib().tra_tbe_launch_info(tbe._get_plan(None), B, len(ids), int(tbe.pooling_mode),
                                              T if entry == "lengths" else 0, buf, 512))
    assert b"tbe_pooled_cu_kernel" in buf.value
    if entry == "lengths":
        a = tbe(ti, None, tw, lengths=torch.from_numpy(lens.astype(np.int32)).to(DEV), batch_size=B)
    else:
        a = tbe(ti, torch.from_numpy(offsets).to(DEV), tw)
    _lib.set_tuning(balanced=0)
    try:
        b = tbe(ti, torch.from_numpy(offsets).to(DEV), tw)
    finally:
        _lib.set_tuning(balanced=None)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    Bs = 24
    sub_len = lens.reshape(T, B)[:, :Bs]
    sub_off = np.zeros(T * Bs + 1, dtype=np.int32)
    sub_off[1:] = np.cumsum(sub_len.reshape(-1))
    pick = np.concatenate([np.arange(offsets[f * B], offsets[f * B + Bs]) for f in range(T)])
    want = O.tbe_forward(store, list(range(T)), Bs, ids[pick], sub_off, None if psw is None else psw[pick], pooling, O.FP16)
    assert bits_equal(np.ascontiguousarray(a[:Bs].cpu().numpy()), want) == 0


def test_window_kernel_equals_static_at_scale(tuning):
    """At a size where the window kernel is the default (26 features x 2048
    samples, ~1M ids) both kernels give the same bits, and a sample of bags
    matches the oracle."""
    rng = np.random.default_rng(2024)
    T, rows, dim, B = 26, 50_000, 128, 2048
    specs = [(O.INT4, rows, dim)] * T
    ftm = list(range(T))
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 40, empty_frac=0.02)
    ti, to = torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV)
    tuning(balanced=None)
    tuning(window=None)
    a = tbe(ti, to)
    tuning(balanced=0)
    b = tbe(ti, to)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # oracle on the first 64 samples of every feature
    Bs = 64
    sub_len = lengths.reshape(T, B)[:, :Bs]
    sub_off = np.zeros(T * Bs + 1, dtype=np.int32)
    sub_off[1:] = np.cumsum(sub_len.reshape(-1))
    sub_ids = np.concatenate([ids[offsets[f * B]:offsets[f * B + Bs]] for f in range(T)])
    want = O.tbe_forward(store, ftm, Bs, sub_ids, sub_off, None, O.SUM, O.FP16)
    assert bits_equal(np.ascontiguousarray(a[:Bs].cpu().numpy()), want) == 0


def test_mixed_types_weighted_at_scale(tuning):
    """The mixed workload's shape (weight types and dims mixed, weighted SUM,
    fp32 out, 4096 samples, Poisson(30) bag lengths; 16 tables of 50 K rows):
    several launch classes and sub-classes of the window kernel.  Same bits as
    the static kernel; doubling every weight doubles every output exactly; a
    sample of bags matches the oracle."""
    rng = np.random.default_rng(303)
    dts = [O.INT8, O.INT4, O.INT2, O.FP16]
    dims = [32, 64, 128, 256]
    T, rows, B = 16, 50_000, 4096
    specs = [(dts[t % 4], rows, dims[(t // 4) % 4]) for t in range(T)]
    ftm = list(range(T))
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP32, 16)
    lengths = rng.poisson(30, T * B).astype(np.int32)
    offsets = np.zeros(T * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lengths)
    ids = rng.integers(0, rows, int(offsets[-1])).astype(np.int32)
    psw = rng.uniform(0, 1, len(ids)).astype(np.float32)
    ti, to, tw = (torch.from_numpy(x).to(DEV) for x in (ids, offsets, psw))
    tuning(balanced=None)
    a = tbe(ti, to, tw)
    tuning(balanced=0)
    b = tbe(ti, to, tw)
    tuning(balanced=None)
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert torch.equal(tbe(ti, to, tw * 2), a * 2)
    Bs = 8
    sub_len = lengths.reshape(T, B)[:, :Bs]
    sub_off = np.zeros(T * Bs + 1, dtype=np.int32)
    sub_off[1:] = np.cumsum(sub_len.reshape(-1))
    pick = np.concatenate([np.arange(offsets[f * B], offsets[f * B + Bs]) for f in range(T)])
    want = O.tbe_forward(store, ftm, Bs, ids[pick], sub_off, psw[pick], O.SUM, O.FP32)
    assert bits_equal(np.ascontiguousarray(a[:Bs].cpu().numpy()), want) == 0


@pytest.mark.parametrize("from_lengths", [False, True])
def test_window_kernel_many_features(tuning, from_lengths):
    """More features than the window kernel keeps close at hand: 300 features
    on three tables (over 128 per launch class: key positions then come from
    the descriptors, not the launch arguments), 3 samples each, 128 bags per
    window (over 32 features per window: their descriptors are read from global
    memory, not from LDS), keys in reverse order."""
    tuning(balanced=1)
    tuning(window=128)
    rng = np.random.default_rng(300)
    F, B = 300, 3
    specs = [(O.INT4, 400, 64), (O.INT8, 300, 64), (O.INT4, 500, 32)]
    ftm = [f % 3 for f in range(F)]
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP32, 16)
    rows_f = [specs[t][1] for t in ftm]
    lengths, offsets, ids = make_bags(rng, rows_f, B, 12)
    want = O.tbe_forward(store, ftm, B, ids, offsets, None, O.SUM, O.FP32)
    ti = torch.from_numpy(ids).to(DEV)
    if from_lengths:
        got = tbe(ti, None, lengths=torch.from_numpy(lengths.astype(np.int32)).to(DEV), batch_size=B)
    else:
        got = tbe(ti, torch.from_numpy(offsets).to(DEV))
    assert bits_equal(got.cpu().numpy(), want) == 0
    # the same bags addressed through a reversed key order
    rev = list(range(F - 1, -1, -1))
    L = lengths.reshape(F, B)
    seg = [ids[offsets[f * B]:offsets[(f + 1) * B]] for f in range(F)]
    r_len = np.concatenate([L[f] for f in rev]).astype(np.int32)
    r_off = np.zeros(F * B + 1, dtype=np.int32)
    r_off[1:] = np.cumsum(r_len)
    r_ids = torch.from_numpy(np.concatenate([seg[f] for f in rev])).to(DEV)
    if from_lengths:
        got = tbe(r_ids, None, lengths=torch.from_numpy(r_len).to(DEV), batch_size=B, feature_positions=rev)
    else:
        got = tbe(r_ids, torch.from_numpy(r_off).to(DEV), batch_size=B, feature_positions=rev)
    assert bits_equal(got.cpu().numpy(), want) == 0


def test_lookup_under_hip_graph():
    """The lookup captured in a HIP graph: several replays, with eager work and
    synchronisation in between, each equal to the eager result."""
    rng = np.random.default_rng(8)
    T, rows, dim, B = 6, 5000, 128, 256
    specs = [(O.INT4, rows, dim)] * T
    tbe, store = build(rng, specs, list(range(T)), O.SUM, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 30)
    cap = int(len(ids) * 1.5)
    ti = torch.zeros(cap, dtype=torch.int32, device=DEV)
    to = torch.zeros(T * B + 1, dtype=torch.int32, device=DEV)
    out = torch.zeros(B, T * dim, dtype=torch.float16, device=DEV)

    def load(seed):
        r = np.random.default_rng(seed)
        l, o, i = make_bags(r, [rows] * T, B, 30)
        assert len(i) <= cap
        ti.zero_()
        ti[: len(i)].copy_(torch.from_numpy(i))
        to.copy_(torch.from_numpy(o))
        return i, o

    load(0)
    tbe(ti, to, batch_size=B, out=out)  # plan creation outside capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            tbe(ti, to, batch_size=B, out=out)
    torch.cuda.synchronize()
    for seed in (1, 2, 3, 4):
        i, o = load(seed)
        g.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy().copy()
        eager = tbe(ti, to, batch_size=B).cpu().numpy()
        want = O.tbe_forward(store, list(range(T)), B, i, o, None, O.SUM, O.FP16)
        assert bits_equal(got, want) == 0, seed
        assert bits_equal(eager, want) == 0, seed


def _from_lengths(tbe, ids, lengths, psw, B, **kw):
    return tbe(torch.from_numpy(ids).to(DEV), None, None if psw is None else torch.from_numpy(psw).to(DEV),
               lengths=torch.from_numpy(lengths).to(DEV), batch_size=B, **kw).cpu().numpy()


@pytest.mark.parametrize("window", [None, 64, 100, 0, 2048])
@pytest.mark.parametrize("dtype,pooling,weighted,idt", [
    (O.INT4, O.SUM, False, np.int32), (O.INT8, O.MEAN, True, np.int64), (O.FP16, O.SUM, True, np.int32),
    (O.INT2, O.MEAN, False, np.int64), (O.FP32, O.SUM, False, np.int32)])
def test_forward_from_lengths(tuning, window, dtype, pooling, weighted, idt):
    """forward(offsets=None, lengths=...) against the oracle: the small-call route
    (scan + lookup, window None) and the window kernel deriving the bag starts
    itself, with windows that span feature boundaries."""
    if window is not None:
        tuning(balanced=1)
        tuning(window=window)
    rng = np.random.default_rng(300 + dtype + pooling + (window or 7))
    rows, B, dim = 3000, 211, 64
    specs = [(dtype, rows, dim), (dtype, rows + 13, dim), (dtype, rows + 5, dim)]
    ftm = [0, 1, 2, 0, 1]
    tbe, store = build(rng, specs, ftm, pooling, O.FP32, 16)
    rows_f = [specs[t][1] for t in ftm]
    lengths, offsets, ids = make_bags(rng, rows_f, B, 50, idt)
    psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, pooling, O.FP32)
    got = _from_lengths(tbe, ids, lengths, psw, B)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0


def test_forward_from_lengths_scattered_keys(tuning):
    """Window kernel from lengths when the operator's features sit at scattered,
    descending and repeated-gap key positions of a wider KJT (every feature
    boundary inside a window starts a new run), plus an int64 total beyond the
    first features and empty leading keys."""
    tuning(balanced=1)
    tuning(window=150)
    rng = np.random.default_rng(17)
    rows, B, dim = 900, 97, 128
    specs = [(O.INT4, rows, dim)] * 4
    tbe, store = build(rng, specs, [0, 1, 2, 3], O.SUM, O.FP16, 16)
    K = 7
    positions = [5, 2, 3, 0]           # keys 1, 4, 6 unused; 2 -> 3 is the only adjacent pair
    lengths, offsets, ids = make_bags(rng, [rows] * K, B, 30)
    got = _from_lengths(tbe, ids, lengths, None, B, feature_positions=positions)
    seg = [ids[offsets[k * B]:offsets[(k + 1) * B]] for k in range(K)]
    Lm = lengths.reshape(K, B)
    o_off = np.zeros(4 * B + 1, dtype=np.int32)
    o_off[1:] = np.cumsum(np.concatenate([Lm[p] for p in positions]))
    want = O.tbe_forward(store, [0, 1, 2, 3], B, np.concatenate([seg[p] for p in positions]), o_off, None, O.SUM, O.FP16)
    assert bits_equal(got, want) == 0
    # same through the offsets entry point
    got2 = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV), feature_positions=positions,
               batch_size=B).cpu().numpy()
    assert bits_equal(got2, want) == 0
    # an unaligned lengths view takes the scan + lookup route and gives the same bits
    padded = torch.zeros(len(lengths) + 1, dtype=torch.int32, device=DEV)
    padded[1:] = torch.from_numpy(lengths)
    assert padded[1:].data_ptr() % 16 != 0
    got3 = tbe(torch.from_numpy(ids).to(DEV), None, lengths=padded[1:], feature_positions=positions,
               batch_size=B).cpu().numpy()
    assert bits_equal(got3, want) == 0


def test_forward_from_lengths_at_scale():
    """Default routing at 26 x 2048 bags (~1M ids): lengths entry == offsets entry, bit for bit."""
    rng = np.random.default_rng(2025)
    T, rows, dim, B = 26, 50_000, 128, 2048
    tbe, store = build(rng, [(O.INT4, rows, dim)] * T, list(range(T)), O.SUM, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 40, empty_frac=0.05)
    ti = torch.from_numpy(ids).to(DEV)
    a = tbe(ti, torch.from_numpy(offsets).to(DEV))
    b = tbe(ti, None, lengths=torch.from_numpy(lengths).to(DEV), batch_size=B)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def _launch_text(tbe, B, n_ids, n_keys):
    import ctypes
    from torchrec_amd import _lib
    buf = ctypes.create_string_buffer(1024)
    _lib.check(_lib.lib().tra_tbe_launch_info(tbe._get_plan(None), B, n_ids, int(tbe.pooling_mode), n_keys, buf, 1024))
    return buf.value.decode()


@pytest.mark.parametrize("B,idt,pooling,weighted", [
    (1, np.int32, O.SUM, False), (37, np.int64, O.MEAN, True), (512, np.int32, O.SUM, True),
    (1170, np.int32, O.MEAN, False), (1171, np.int64, O.SUM, False)])
def test_small_call_from_lengths_one_launch(tuning, B, idt, pooling, weighted):
    """A call too small for the window kernel, given lengths: up to 16384 lengths the static kernel sums
    the lengths in front of each block itself (one launch, no scan kernel); beyond, or with
    fused_scan=0, a scan runs first.  Both against the oracle, mixed row widths (1 to 32 lanes per
    row), 12 features at shuffled positions of a 14-key KJT, batch sizes that leave tiles partly empty."""
    rng = np.random.default_rng(4000 + B)
    dims = [32, 64, 128, 256, 8, 16]
    dts = [O.INT8, O.INT4, O.FP16, O.INT2, O.FP32, O.INT8]
    specs = [(dts[t], 700 + 13 * t, dims[t]) for t in range(6)]
    ftm = [0, 1, 2, 3, 4, 5, 0, 1, 2, 3, 4, 5]
    K = 14
    positions = list(rng.permutation(K)[:12])
    tbe, store = build(rng, specs, ftm, pooling, O.FP32, 16)
    # (few enough ids that the call stays with the static kernel at the larger batch sizes)
    lengths, offsets, ids = make_bags(rng, [700] * K, B, 33 if B < 1000 else 10, idt, empty_frac=0.2)
    psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
    seg = [ids[offsets[k * B]:offsets[(k + 1) * B]] for k in range(K)]
    wseg = None if psw is None else [psw[offsets[k * B]:offsets[(k + 1) * B]] for k in range(K)]
    Lm = lengths.reshape(K, B)
    o_off = np.zeros(12 * B + 1, dtype=idt)
    o_off[1:] = np.cumsum(np.concatenate([Lm[p] for p in positions]))
    want = O.tbe_forward(store, ftm, B, np.concatenate([seg[p] for p in positions]), o_off,
                         None if psw is None else np.concatenate([wseg[p] for p in positions]), pooling, O.FP32)
    fused_expected = K * B <= 16384
    text = _launch_text(tbe, B, len(ids), K)
    assert ("tbe_pooled_kernel" in text) and (("from_lengths" in text) == fused_expected) and (("scan" in text) != fused_expected), text
    got = _from_lengths(tbe, ids, lengths, psw, B, feature_positions=positions)
    assert bits_equal(got, want) == 0
    tuning(fused_scan=0)
    assert "scan" in _launch_text(tbe, B, len(ids), K)
    got = _from_lengths(tbe, ids, lengths, psw, B, feature_positions=positions)
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0


@pytest.mark.parametrize("pooling", [O.SUM, O.MEAN])
def test_negative_lengths_same_on_every_route(tuning, pooling):
    """A malformed KJT with a few negative lengths: bag starts are the running
    sum of the lengths as they stand and a negative length makes its own bag
    empty.  The same on every route a lengths call can take (scan + lookup, the
    static kernel summing its own prefix, the window kernel staged by one wave
    and by the whole block) and through the offsets entry fed with the running
    sum: all outputs bit for bit equal."""
    rng = np.random.default_rng(606 + pooling)
    T, B, rows, dim = 3, 400, 500, 64
    tbe, store = build(rng, [(O.INT4, rows, dim)] * T, list(range(T)), pooling, O.FP32, 16)
    lengths = rng.integers(0, 12, T * B).astype(np.int32)
    bad = rng.choice(np.arange(5, T * B - 5), 9, replace=False)
    lengths[bad] = -rng.integers(1, 4, len(bad)).astype(np.int32)   # never below the running sum's start
    offsets = np.zeros(T * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lengths)
    assert offsets.min() >= 0
    ids = rng.integers(0, rows, int(offsets.max()) + 8).astype(np.int32)
    ti = torch.from_numpy(ids).to(DEV)
    tl = torch.from_numpy(lengths).to(DEV)
    ref = tbe(ti, torch.from_numpy(offsets).to(DEV), batch_size=B).cpu().numpy()
    empty_rows = ref.reshape(B, T, dim)[(bad % B), (bad // B)]
    assert not empty_rows.any()                      # the negative bags pooled nothing
    outs = {}
    outs["static, own prefix"] = tbe(ti, None, lengths=tl, batch_size=B).cpu().numpy()
    tuning(fused_scan=0)
    outs["scan + lookup"] = tbe(ti, None, lengths=tl, batch_size=B).cpu().numpy()
    tuning(fused_scan=None)
    tuning(balanced=1, window=100)
    outs["window, one wave stages"] = tbe(ti, None, lengths=tl, batch_size=B).cpu().numpy()
    outs["window, offsets"] = tbe(ti, torch.from_numpy(offsets).to(DEV), batch_size=B).cpu().numpy()
    tuning(window=300)
    outs["window, block stages"] = tbe(ti, None, lengths=tl, batch_size=B).cpu().numpy()
    for name, got in outs.items():
        assert bits_equal(got, ref) == 0, name


@pytest.mark.parametrize("T,B,route", [(1, 70_000, "offsets"), (1, 70_000, "lengths"), (2, 40_000, "lengths"),
                                       (1, 1_100_000, "offsets"), (1, 1_100_000, "lengths"),
                                       (300, 3, "offsets"), (300, 3, "lengths"), (300, 40, "lengths"),
                                       (300, 100, "lengths")])
def test_extreme_shapes(tuning, T, B, route):
    """Very tall and very wide calls: a batch beyond what a window entry can
    index (the static kernel takes over), and hundreds of features with a
    handful of bags each, through both entries, window kernel requested."""
    tuning(balanced=1)
    rng = np.random.default_rng(T * 1000 + B)
    rows, dim = 500, 32
    dts = [O.INT4, O.INT8, O.FP16]
    specs = [(dts[t % 3], rows + t, dim) for t in range(T)]
    ftm = list(range(T))
    tbe, store = build(rng, specs, ftm, O.MEAN, O.FP16, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 6)
    want = O.tbe_forward(store, ftm, B, ids, offsets, None, O.MEAN, O.FP16)
    if route == "lengths":
        got = _from_lengths(tbe, ids, lengths, None, B)
    else:
        got = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV)).cpu().numpy()
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0


@pytest.mark.parametrize("route", ["static", "window", "lengths"])
def test_padded_id_buffer(tuning, route):
    """An id buffer longer than the bags describe (a fixed-size serving buffer
    with a padded tail): the excess is never looked up, as with the
    reference's offsets, whichever entry and kernel runs."""
    tuning(balanced=0 if route == "static" else 1)
    rng = np.random.default_rng(31)
    rows, B, dim = 2000, 300, 64
    specs = [(O.INT4, rows, dim), (O.INT8, rows, dim)]
    tbe, store = build(rng, specs, [0, 1], O.SUM, O.FP32, 16)
    lengths, offsets, ids = make_bags(rng, [rows, rows], B, 25)
    psw = rng.uniform(-1, 1, len(ids)).astype(np.float32)
    want = O.tbe_forward(store, [0, 1], B, ids, offsets, psw, O.SUM, O.FP32)
    pad = 777
    ids_p = np.concatenate([ids, np.full(pad, rows + 5, dtype=ids.dtype)])  # the tail would count as out of range
    psw_p = np.concatenate([psw, np.full(pad, np.float32(np.nan))])
    if route == "lengths":
        got = _from_lengths(tbe, ids_p, lengths, psw_p, B)
    else:
        got = tbe(torch.from_numpy(ids_p).to(DEV), torch.from_numpy(offsets).to(DEV),
                  torch.from_numpy(psw_p).to(DEV)).cpu().numpy()
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == 0


@pytest.mark.parametrize("window", [None, 256, 100])
@pytest.mark.parametrize("B,idt", [(8192, np.int32), (4096, np.int64)])
def test_forward_from_lengths_long_prefix(tuning, B, idt, window):
    """Enough bags that the blocks of the last windows sum the lengths in front
    of them in many batches of loads (26 x 8192 int32 lengths, 26 x 4096 int64
    ones): lengths entry == offsets entry, bit for bit, and the launch really
    is the from-lengths one.  Default windows (several hundred bags: staged by
    the whole block) and forced small ones (staged by the block's first wave
    while the other waves sum the prefix, here up to 850 KB of it)."""
    if window is not None:
        tuning(balanced=1, window=window)
    rng = np.random.default_rng(77 + B)
    T, rows, dim = 26, 20_000, 64
    tbe, store = build(rng, [(O.INT8, rows, dim)] * T, list(range(T)), O.MEAN, O.FP32, 16)
    lengths, offsets, ids = make_bags(rng, [rows] * T, B, 12, idt, empty_frac=0.1)
    psw = torch.from_numpy(rng.uniform(-1, 1, len(ids)).astype(np.float32)).to(DEV)
    ti = torch.from_numpy(ids).to(DEV)
    a = tbe(ti, torch.from_numpy(offsets).to(DEV), psw)
    b = tbe(ti, None, psw, lengths=torch.from_numpy(lengths).to(DEV), batch_size=B)
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    import ctypes
    from torchrec_amd import _lib
    buf = ctypes.create_string_buffer(512)
    _lib.check(_lib.lib().tra_tbe_launch_info(tbe._get_plan(None), B, len(ids), int(tbe.pooling_mode), T, buf, 512))
    assert b"from_lengths" in buf.value


@pytest.mark.parametrize("seed", range(64))
def test_random_plans(tuning, seed):
    """Seeded random operators (table count, weight types, dims, rows, shared and
    shuffled features, pooling, weights, id and output types, row alignment,
    pruned ids) through a random route (static kernel, window kernel with a
    random window, lengths entry) against the oracle, bit for bit."""
    rng = np.random.default_rng(9000 + seed)
    T = int(rng.integers(1, 11))
    pooling = [O.SUM, O.MEAN, O.NONE][int(rng.choice(3, p=[0.45, 0.35, 0.2]))]
    dims_pool = [16, 32, 48, 64, 96, 128, 160, 256, 320, 512]
    one_dim = dims_pool[int(rng.integers(0, len(dims_pool)))]
    specs = []
    for _ in range(T):
        dt = [O.INT8, O.INT4, O.INT2, O.FP16, O.FP32][int(rng.integers(0, 5))]
        dim = one_dim if pooling == O.NONE else dims_pool[int(rng.integers(0, len(dims_pool)))]
        rows = int(rng.choice([1, 2, 37, 500, 3000]))
        specs.append((dt, rows, dim))
    ftm = list(range(T)) + [int(x) for x in rng.integers(0, T, int(rng.integers(0, 4)))]
    rng.shuffle(ftm)
    out_dtype = [O.FP32, O.FP16][int(rng.integers(0, 2))]
    ra = int(rng.choice([4, 8, 16, 64]))
    idt = [np.int32, np.int64][int(rng.integers(0, 2))]
    B = int(rng.choice([1, 7, 64, 257, 1500]))
    max_len = int(rng.choice([1, 3, 20, 70, 300, 5000]))
    if max_len >= 300:  # long bags: fewer of them, so the oracle stays quick
        B = min(B, 64 if max_len == 300 else 7)
    weighted = pooling != O.NONE and bool(rng.integers(0, 2))
    route = ["static", "window", "lengths"][int(rng.integers(0, 3))]
    window = int(rng.choice([0, 64, 100, 300, 2048]))
    if route != "static":
        tuning(balanced=1)
        tuning(window=window)
    else:
        tuning(balanced=0)
    tbe, store = build(rng, specs, ftm, pooling, out_dtype, ra)
    rows_f = [specs[t][1] for t in ftm]
    lengths, offsets, ids = make_bags(rng, rows_f, B, max_len, idt, empty_frac=float(rng.choice([0.0, 0.1, 0.6])))
    if len(ids) and pooling != O.NONE:
        ids[rng.random(len(ids)) < 0.05] = -1  # pruned ids are skipped
    psw = rng.uniform(-2, 2, len(ids)).astype(np.float32) if weighted else None
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, pooling, out_dtype)
    tag = (seed, T, pooling, specs, ftm, out_dtype, ra, idt.__name__, B, max_len, weighted, route, window)
    if route == "lengths":
        got = _from_lengths(tbe, ids, lengths, psw, B)
    else:
        got = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV),
                  None if psw is None else torch.from_numpy(psw).to(DEV)).cpu().numpy()
    assert got.shape == want.shape, tag
    assert bits_equal(got, want) == 0, tag
    assert tbe.out_of_range_count() == 0, tag


@pytest.mark.parametrize("seed", range(48))
def test_random_natural_key_order(tuning, seed):
    """Seeded random operators whose features sit at consecutive key positions
    (what a collection with one feature per table launches), window kernel
    forced with windows of 64 - 300 bags: the lengths entry (up to 256 bags the
    window is staged by one wave while the others sum the prefix) and the
    offsets entry against the oracle, bit for bit."""
    rng = np.random.default_rng(50000 + seed)
    nt = int(rng.integers(1, 9))
    pooling = [O.SUM, O.MEAN][int(rng.integers(0, 2))]
    dims_pool = [16, 32, 64, 128, 256]
    same = bool(rng.integers(0, 2))
    dt0 = [O.INT8, O.INT4, O.INT2, O.FP16][int(rng.integers(0, 4))]
    d0 = dims_pool[int(rng.integers(0, 5))]
    specs = []
    for _ in range(nt):
        dt = dt0 if same else [O.INT8, O.INT4, O.INT2, O.FP16, O.FP32][int(rng.integers(0, 5))]
        dim = d0 if same else dims_pool[int(rng.integers(0, 5))]
        specs.append((dt, int(rng.choice([3, 500, 3000])), dim))
    ftm = list(range(nt))
    out_dtype = [O.FP32, O.FP16][int(rng.integers(0, 2))]
    ra = int(rng.choice([4, 16, 64]))
    idt = [np.int32, np.int64][int(rng.integers(0, 2))]
    B = int(rng.choice([3, 64, 100, 257, 700]))
    max_len = int(rng.choice([1, 5, 40, 200, 400]))
    if max_len >= 200:
        B = min(B, 64)
    weighted = bool(rng.integers(0, 2))
    window = int(rng.choice([64, 100, 208, 256, 300]))
    tuning(balanced=1)
    tuning(window=window)
    tbe, store = build(rng, specs, ftm, pooling, out_dtype, ra)
    lengths, offsets, ids = make_bags(rng, [s[1] for s in specs], B, max_len, idt,
                                      empty_frac=float(rng.choice([0.0, 0.1, 0.5])))
    if len(ids):
        ids[rng.random(len(ids)) < 0.03] = -1
    psw = rng.uniform(-2, 2, len(ids)).astype(np.float32) if weighted else None
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, pooling, out_dtype)
    tag = (seed, specs, pooling, out_dtype, ra, idt.__name__, B, max_len, weighted, window)
    assert bits_equal(_from_lengths(tbe, ids, lengths, psw, B), want) == 0, tag
    got = tbe(torch.from_numpy(ids).to(DEV), torch.from_numpy(offsets).to(DEV),
              None if psw is None else torch.from_numpy(psw).to(DEV)).cpu().numpy()
    assert bits_equal(got, want) == 0, tag


@pytest.mark.parametrize("seed", range(48))
def test_random_position_weights(tuning, seed):
    """Seeded random operators with the position weights looked up inside the
    lookup kernel (static and window kernel, offsets and lengths entry, keys with
    0, 1 or many weights, bags longer than their weight vector): same bits as
    the oracle fed with the weights materialized per id."""
    rng = np.random.default_rng(70000 + seed)
    nt = int(rng.integers(1, 7))
    pooling = [O.SUM, O.MEAN][int(rng.integers(0, 2))]
    dims_pool = [16, 32, 64, 128, 256]
    specs = [([O.INT8, O.INT4, O.INT2, O.FP16, O.FP32][int(rng.integers(0, 5))], int(rng.choice([3, 500, 3000])),
              dims_pool[int(rng.integers(0, 5))]) for _ in range(nt)]
    ftm = list(range(nt)) + [int(x) for x in rng.integers(0, nt, int(rng.integers(0, 3)))]
    if rng.integers(0, 2):
        rng.shuffle(ftm)
    nk = len(ftm)
    out_dtype = [O.FP32, O.FP16][int(rng.integers(0, 2))]
    ra = int(rng.choice([4, 16, 64]))
    idt = [np.int32, np.int64][int(rng.integers(0, 2))]
    B = int(rng.choice([3, 64, 257, 700]))
    max_len = int(rng.choice([1, 5, 40, 200]))
    if max_len >= 200:
        B = min(B, 64)
    route = ["static", "window"][int(rng.integers(0, 2))]
    window = int(rng.choice([64, 100, 208, 256, 300]))
    from_lengths = bool(rng.integers(0, 2))
    key_len = [int(rng.choice([0, 1, 7, 30, 250])) for _ in range(nk)]
    key_start, tot = [], 0
    for n_ in key_len:
        key_start.append(tot)
        tot += n_
    table = rng.uniform(-1.5, 1.5, max(tot, 1)).astype(np.float32)
    tuning(balanced=1 if route == "window" else 0)
    if route == "window":
        tuning(window=window)
    tbe, store = build(rng, specs, ftm, pooling, out_dtype, ra)
    lengths, offsets, ids = make_bags(rng, [specs[t][1] for t in ftm], B, max_len, idt,
                                      empty_frac=float(rng.choice([0.0, 0.1, 0.5])))
    psw = np.ones(len(ids), dtype=np.float32)
    for k in range(nk):
        if key_len[k] == 0:
            continue  # a key without weights: every id weighs 1
        for b in range(B):
            s, e = int(offsets[k * B + b]), int(offsets[k * B + b + 1])
            psw[s:e] = table[key_start[k] + np.minimum(np.arange(e - s), key_len[k] - 1)]
    want = O.tbe_forward(store, ftm, B, ids, offsets, psw, pooling, out_dtype)
    pw = (torch.from_numpy(table).to(DEV), key_start, key_len)
    ti = torch.from_numpy(ids).to(DEV)
    if from_lengths:
        got = tbe(ti, None, None, lengths=torch.from_numpy(lengths).to(DEV), batch_size=B, position_weights=pw)
    else:
        got = tbe(ti, torch.from_numpy(offsets).to(DEV), None, position_weights=pw)
    tag = (seed, specs, ftm, pooling, out_dtype, ra, idt.__name__, B, max_len, route, window, from_lengths, key_len)
    assert bits_equal(got.cpu().numpy(), want) == 0, tag


def test_table_beyond_2_31_rows(tuning):
    """A table with more than 2^31 rows (fp32, dim 1: 8.6 GB): int64 ids beyond 2^31 address the
    right rows; int32 ids see every non-negative id as in range; ids >= rows are skipped and counted."""
    rows, B = 2**31 + 1000, 4
    free, _ = torch.cuda.mem_get_info()
    if free < rows * 4 + (1 << 30):
        pytest.skip("not enough free device memory for an 8.6 GB table")
    tbe = TBE(embedding_specs=[("big", rows, 1, SparseType.FP32, EmbeddingLocation.DEVICE)],
              pooling_mode=PoolingMode.SUM, device=DEV, output_dtype=SparseType.FP32, row_alignment=4)
    tbe.initialize_weights()
    assert tbe.row_stride == [4]
    w = tbe.weights_dev.view(torch.float32)
    assert w.numel() >= rows
    w.zero_()
    picks = [0, 5, 2**31 - 1, 2**31, 2**31 + 7, rows - 1]
    for k, r in enumerate(picks):
        w[r] = float(k + 1)
    ids = torch.tensor([picks[3], picks[4], picks[5], picks[0], rows, picks[2], picks[1], -1], dtype=torch.int64, device=DEV)
    offsets = torch.tensor([0, 2, 5, 6, 8], dtype=torch.int64, device=DEV)
    got = tbe(ids, offsets).cpu().view(-1).tolist()
    assert got == [4.0 + 5.0, 6.0 + 1.0, 3.0, 2.0]
    assert tbe.out_of_range_count() == 1
    # window kernel, same ids (forced)
    tuning(balanced=1)
    got = tbe(ids, offsets).cpu().view(-1).tolist()
    assert got == [4.0 + 5.0, 6.0 + 1.0, 3.0, 2.0]
    assert tbe.out_of_range_count() == 1
    # int32 ids: every non-negative id is a row of this table
    ids32 = torch.tensor([2**31 - 1, 5, 0, -1], dtype=torch.int32, device=DEV)
    off32 = torch.tensor([0, 1, 2, 3, 4], dtype=torch.int32, device=DEV)
    assert tbe(ids32, off32).cpu().view(-1).tolist() == [3.0, 2.0, 1.0, 0.0]
    assert tbe.out_of_range_count() == 0
    del tbe, w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("mode", ["WARNING", "IGNORE"])
def test_bounds_check_warning_and_ignore_pool_row_zero(mode, tuning):
    """BoundsCheckMode.WARNING / IGNORE: an id outside its table (too large, or negative other than
    -1) pools row 0 of that table, which is what the lookup sees in fbgemm_gpu after
    bounds_check_indices has rewritten the id to 0 (the reference's sharded call site asks for
    WARNING by default, torchrec/distributed/quant_embedding_kernel.py:337-339); -1 is still
    skipped; every bad id is counted.  Parity unpinned: fbgemm_gpu is not in this image, the
    expectation is its documented behaviour restated on the oracle (bad ids replaced by 0).
    Covered: both pooled kernels, ids a block at a time (8 lanes per row) and one by one, per-sample
    weights, MEAN, both id widths, the lookup from lengths, and the sequence lookup."""
    from torchrec_amd.tbe.enums import BoundsCheckMode
    bcm = getattr(BoundsCheckMode, mode)
    rng = np.random.default_rng(77 + len(mode))
    for (dt, dim), pooling, weighted, idt, balanced in itertools.product(
        ((O.INT4, 128), (O.INT8, 32), (O.FP16, 64), (O.INT2, 256)), (O.SUM, O.MEAN), (False, True),
        (np.int32, np.int64), (0, 1),
    ):
        rows, B = 500, 70
        specs = [(dt, rows, dim), (dt, rows + 40, dim)]
        ftm = [0, 1, 1]
        rows_f = [rows, rows + 40, rows + 40]
        tbe, store = build(rng, specs, ftm, pooling, O.FP32, 16, bounds_check_mode=bcm)
        tuning(balanced=balanced)
        lengths, offsets, ids = make_bags(rng, rows_f, B, 45, idt)
        feat_of = np.repeat(np.arange(3), B)
        owner = np.repeat(feat_of, lengths)  # feature of every id
        bad = ids.copy()
        pick = rng.choice(len(ids), 60, replace=False)
        bad[pick[:20]] = -1                                              # pruned: skipped, not counted
        bad[pick[20:40]] = np.asarray(rows_f)[owner[pick[20:40]]] + rng.integers(0, 5, 20)  # too large
        bad[pick[40:]] = -2 - rng.integers(0, 1000, 20)                   # negative, not -1
        expect, n_bad = O.bounds_check_indices(rows_f, B, bad, offsets, mode)
        assert n_bad == 40 and (expect[pick[20:]] == 0).all() and (expect[pick[:20]] == -1).all()
        psw = rng.uniform(-1, 1, len(ids)).astype(np.float32) if weighted else None
        tag = (dt, dim, pooling, weighted, idt, balanced)
        want = O.tbe_forward(store, ftm, B, expect, offsets, psw, pooling, O.FP32)
        got = tbe(torch.from_numpy(bad).to(DEV), torch.from_numpy(offsets).to(DEV),
                  None if psw is None else torch.from_numpy(psw).to(DEV)).cpu().numpy()
        assert bits_equal(got, want) == 0, tag
        assert tbe.out_of_range_count() == 40, tag
        if not weighted:
            # the same from the lengths (the collection's route)
            got = tbe(torch.from_numpy(bad).to(DEV), None, None, lengths=torch.from_numpy(lengths.astype(idt)).to(DEV),
                      batch_size=B).cpu().numpy()
            assert bits_equal(got, want) == 0, tag
            assert tbe.out_of_range_count() == 40, tag
    # sequence lookup: the row of a bad id is row 0 of its table, that of -1 is zeros
    rows, dim, B = 300, 64, 9
    tbe, store = build(rng, [(O.INT8, rows, dim), (O.INT8, rows, dim)], [0, 1], O.NONE, O.FP16, 16, bounds_check_mode=bcm)
    lengths, offsets, ids = make_bags(rng, [rows, rows], B, 12, np.int32)
    bad = ids.copy()
    bad[::5] = rows + 1
    bad[1::7] = -1
    expect, n_bad = O.bounds_check_indices([rows, rows], B, bad, offsets, mode)
    assert n_bad == int((bad == rows + 1).sum())
    want = O.tbe_forward(store, [0, 1], B, expect, offsets, None, O.NONE, O.FP16)
    got = tbe(torch.from_numpy(bad).to(DEV), torch.from_numpy(offsets).to(DEV)).cpu().numpy()
    assert bits_equal(got, want) == 0
    assert tbe.out_of_range_count() == int((bad == rows + 1).sum())


def test_multi_class_call_on_two_streams(tuning):
    """A plan of five or more launch classes runs every other launch on its own second stream,
    forked from and joined to the caller's stream inside the call.  Checked: the same bits as with
    everything on the caller's stream (tuning fork=0) and as the oracle on a sample of bags; the call
    is ordered behind work queued on the caller's stream before it (inputs written by a kernel just
    before the call) and ahead of work queued after it (the output read right after, no wait in
    between); calls on the same plan from several caller streams and host threads at once; and a
    captured call (which stays on the captured stream) replayed against the eager result."""
    import threading
    rng = np.random.default_rng(909)
    dts = [O.INT8, O.INT4, O.INT2, O.FP16]
    dims = [32, 64, 128, 256]
    T, rows, B = 16, 20_000, 2048
    specs = [(dts[t % 4], rows, dims[(t // 4) % 4]) for t in range(T)]
    ftm = list(range(T))
    tbe, store = build(rng, specs, ftm, O.SUM, O.FP32, 16)
    lengths = rng.poisson(30, T * B).astype(np.int32)
    offsets = np.zeros(T * B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lengths)
    n = int(offsets[-1])
    batches = [rng.integers(0, rows, n).astype(np.int32) for _ in range(4)]
    to = torch.from_numpy(offsets).to(DEV)
    import ctypes
    from torchrec_amd import _lib

    def launches():
        buf = ctypes.create_string_buffer(4096)
        _lib.check(_lib.lib().tra_tbe_launch_info(tbe._get_plan(None), B, n, int(tbe.pooling_mode), 0, buf, 4096))
        return buf.value.decode().split("; ")

    tuning(fork=0)
    assert len(launches()) == 7 and not any("stream" in x for x in launches())
    want = [tbe(torch.from_numpy(b).to(DEV), to).clone() for b in batches]
    torch.cuda.synchronize()
    tuning(fork=None)
    # seven launch classes: every other launch, largest class first, goes to the second stream
    assert [("second stream" in x) for x in launches()] == [False, True, False, True, False, True, False], launches()
    # ordering on the caller's stream: ids copied in just before the call, output summed right after
    ti = torch.empty(n, dtype=torch.int32, device=DEV)
    for k in (0, 1, 2, 3, 0):
        src = torch.from_numpy(batches[k]).to(DEV)
        ti.copy_(src)                      # queued before the call
        got = tbe(ti, to)
        chk = got.view(torch.int32).eq(want[k].view(torch.int32)).all()  # queued after the call
        ti.zero_()                         # also after the call: must not reach the lookups
        assert bool(chk), k
    Bs = 4
    sub_off = np.zeros(T * Bs + 1, dtype=np.int32)
    sub_off[1:] = np.cumsum(lengths.reshape(T, B)[:, :Bs].reshape(-1))
    pick = np.concatenate([np.arange(offsets[f * B], offsets[f * B + Bs]) for f in range(T)])
    ref = O.tbe_forward(store, ftm, Bs, batches[0][pick], sub_off, None, O.SUM, O.FP32)
    assert bits_equal(np.ascontiguousarray(want[0][:Bs].cpu().numpy()), ref) == 0
    # several caller streams from several host threads, the same plan
    errors = []

    def worker(k):
        try:
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                t_ids = torch.from_numpy(batches[k]).to(DEV)
                for _ in range(6):
                    out = tbe(t_ids, to)
                    if not torch.equal(out.view(torch.int32), want[k].view(torch.int32)):
                        errors.append(k)
            st.synchronize()
        except Exception as e:  # surfaced below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    # captured: the call stays on the captured stream; replays equal the eager result
    out = torch.zeros(B, sum(s[2] for s in specs), dtype=torch.float32, device=DEV)
    ti.copy_(torch.from_numpy(batches[1]).to(DEV))
    tbe(ti, to, batch_size=B, out=out)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            tbe(ti, to, batch_size=B, out=out)
    torch.cuda.synchronize()
    for k in (2, 3, 0):
        ti.copy_(torch.from_numpy(batches[k]).to(DEV))
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), want[k].view(torch.int32)), k
