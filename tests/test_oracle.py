"""Pins the CPU oracle (oracle/tbe_oracle.c) before anything is compared with it:
against the fbgemm library itself (the kernels TorchRec's CPU path runs),
against torch's own prepack / embedding_bag ops, and against what the
mathematics fixes.  No GPU."""
import itertools

import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_equal, bucketize_python


def _rows(rng, dim, n=400, bits=4):
    w = rng.normal(0, 0.1, (n, dim)).astype(np.float32)
    w[0] = 0.25
    w[1] = np.linspace(0, 2**bits - 1, dim)
    w[2] *= 1e-9
    w[3] *= 1e4
    w[4] = 0.0
    return w


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_quantizer_matches_fbgemm_bytes(bits):
    rng = np.random.default_rng(bits)
    for dim in (8, 16, 32, 64, 128, 256):
        w = _rows(rng, dim, bits=bits)
        a = O.quantize_sbhalf(w, bits, "c")
        assert np.array_equal(a, O.quantize_sbhalf(w, bits, "fbgemm"))
        assert np.array_equal(a, O.quantize_sbhalf(w, bits, "fbgemm_ref"))


def test_quantizer_closed_forms():
    # constant row: range 0 -> scale 1, bias = the constant (fp16), every q = 0
    w = np.full((1, 16), 0.25, dtype=np.float32)
    q = O.quantize_sbhalf(w, 4)
    assert not q[0, :8].any()
    assert q[0, 8:10].view(np.float16)[0] == 1.0 and q[0, 10:12].view(np.float16)[0] == 0.25
    # exact ramp 0..15: scale 1, bias 0, q = the value; low nibble is the even element
    w = np.arange(16, dtype=np.float32)[None, :]
    q = O.quantize_sbhalf(w, 4)
    assert q[0, :8].tolist() == [(2 * i) | ((2 * i + 1) << 4) for i in range(8)]
    # int2 unpacks LSB first
    w = np.array([[0, 1, 2, 3, 3, 2, 1, 0]], dtype=np.float32)
    q = O.quantize_sbhalf(w, 2)
    assert q[0, :2].tolist() == [0 | 1 << 2 | 2 << 4 | 3 << 6, 3 | 2 << 2 | 1 << 4 | 0 << 6]


def test_quantizer_matches_torch_prepack():
    """torch.ops.quantized.embedding_bag_{4,2}bit_prepack produce the same SBHalf rows."""
    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.1, (200, 64)).astype(np.float32)
    for bits, op in ((4, torch.ops.quantized.embedding_bag_4bit_prepack), (2, torch.ops.quantized.embedding_bag_2bit_prepack)):
        want = op(torch.from_numpy(w)).numpy()
        assert np.array_equal(O.quantize_sbhalf(w, bits), want)


def test_half_conversions_exhaustive():
    """fp16 -> fp32 for all 65536 patterns and fp32 -> fp16 (RNE) on a dense sample, against numpy."""
    lib = O.c_lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_half_to_float(int(h)) for h in allh], dtype=np.float32)
    ok = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert ok.all()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.normal(0, 1, 20000), rng.normal(0, 1e-5, 20000), rng.normal(0, 1e4, 5000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001, 2.0**-14, 1e-8]),
        (allh.view(np.float16).astype(np.float32)[:31744] + allh.view(np.float16).astype(np.float32)[1:31745]) / 2,  # exact ties
    ]).astype(np.float32)
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([lib.oracle_float_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


CASES = list(itertools.product(
    (O.INT8, O.INT4, O.INT2, O.FP16, O.FP32), (32, 128), (O.SUM, O.MEAN, O.NONE), (False, True),
    (O.FP32, O.FP16), (np.int32, np.int64)))


def _table(rng, dtype, dim, rows):
    w = rng.normal(0, 0.1, (rows, dim)).astype(np.float32)
    if dtype in (O.INT8, O.INT4, O.INT2):
        return (dtype, dim, O.quantize_sbhalf(w, O.BITS[dtype]))
    return (dtype, dim, w.astype(np.float16) if dtype == O.FP16 else w)


@pytest.mark.parametrize("dtype,dim,pooling,weighted,out_dtype,idt", CASES)
def test_lookup_matches_fbgemm_bits(dtype, dim, pooling, weighted, out_dtype, idt):
    """The restated formula equals fbgemm's JIT kernels bit-for-bit (header-first rows,
    padded stride, 1 and 4 threads)."""
    if pooling == O.NONE and weighted:
        pytest.skip("sequence lookups take no per-sample weights")
    rng = np.random.default_rng(dtype * 1000 + dim + pooling)
    rows, B = 1500, 40
    for align in (16, 4):
        store = O.pack_store([_table(rng, dtype, dim, rows), _table(rng, dtype, dim, rows + 17)], row_alignment=align)
        lengths = rng.integers(0, 81, 2 * B)
        lengths[3] = 0
        offsets = np.zeros(2 * B + 1, dtype=idt)
        offsets[1:] = np.cumsum(lengths)
        idx = rng.integers(0, rows, int(offsets[-1])).astype(idt)
        psw = rng.uniform(-1, 1, len(idx)).astype(np.float32) if weighted else None
        a = O.tbe_forward(store, [0, 1], B, idx, offsets, psw, pooling, out_dtype, "c")
        b = O.tbe_forward(store, [0, 1], B, idx, offsets, psw, pooling, out_dtype, "fbgemm")
        c = O.tbe_forward(store, [0, 1], B, idx, offsets, psw, pooling, out_dtype, "fbgemm", nthreads=4)
        assert bits_equal(a, b) == 0 and bits_equal(b, c) == 0


def test_lookup_brute_force_float64():
    """Dequantize-then-sum in float64 on a tiny input: a dropped term, a wrong nibble
    order or a transposed header would be off by far more than fp32 rounding."""
    rng = np.random.default_rng(9)
    rows, dim, B = 50, 16, 6
    for dtype in (O.INT8, O.INT4, O.INT2):
        bits = O.BITS[dtype]
        w = rng.normal(0, 0.1, (rows, dim)).astype(np.float32)
        q = O.quantize_sbhalf(w, bits)
        payload = dim * bits // 8
        scale = q[:, payload:payload + 2].copy().view(np.float16).astype(np.float64)[:, 0]
        bias = q[:, payload + 2:payload + 4].copy().view(np.float16).astype(np.float64)[:, 0]
        epb = 8 // bits
        deq = np.zeros((rows, dim))
        for c in range(dim):
            deq[:, c] = ((q[:, c // epb] >> ((c % epb) * bits)) & (2**bits - 1)) * scale + bias
        assert np.abs(deq - w).max() <= (w.max(axis=1) - w.min(axis=1)).max() / (2**bits - 1) * 0.51 + 1e-3
        store = O.pack_store([(dtype, dim, q)])
        lengths = rng.integers(0, 7, B)
        offsets = np.zeros(B + 1, dtype=np.int64)
        offsets[1:] = np.cumsum(lengths)
        idx = rng.integers(0, rows, int(offsets[-1]))
        psw = rng.uniform(0, 1, len(idx)).astype(np.float32)
        for pooling, weighted in ((O.SUM, False), (O.SUM, True), (O.MEAN, False)):
            got = O.tbe_forward(store, [0], B, idx, offsets, psw if weighted else None, pooling, O.FP32)
            want = np.zeros((B, dim))
            for b in range(B):
                for j in range(offsets[b], offsets[b + 1]):
                    want[b] += (psw[j] if weighted else 1.0) * deq[idx[j]]
                if pooling == O.MEAN and lengths[b]:
                    want[b] /= lengths[b]
            np.testing.assert_allclose(got, want, rtol=0, atol=2e-6)


def test_lookup_invariants():
    rng = np.random.default_rng(4)
    rows, dim, B = 300, 64, 20
    t = _table(rng, O.INT4, dim, rows)
    store = O.pack_store([t])
    lengths = rng.integers(0, 10, B)
    lengths[0] = 0
    offsets = np.zeros(B + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(lengths)
    idx = rng.integers(0, rows, int(offsets[-1])).astype(np.int32)
    s = O.tbe_forward(store, [0], B, idx, offsets, None, O.SUM, O.FP32)
    assert not s[0].any()                                              # empty bag -> exact zeros
    ones = np.ones(len(idx), dtype=np.float32)
    assert bits_equal(s, O.tbe_forward(store, [0], B, idx, offsets, ones, O.SUM, O.FP32)) == 0
    m = O.tbe_forward(store, [0], B, idx, offsets, None, O.MEAN, O.FP32)
    inv = np.where(lengths > 0, np.float32(1.0) / np.maximum(lengths, 1).astype(np.float32), np.float32(1.0))
    assert bits_equal(m, (s * inv[:, None].astype(np.float32)).astype(np.float32)) == 0
    # sequence row == a bag holding just that id
    n = O.tbe_forward(store, [0], B, idx, offsets, None, O.NONE, O.FP32)
    single_off = np.arange(len(idx) + 1, dtype=np.int32)
    assert bits_equal(n, O.tbe_forward(store, [0], len(idx), idx, single_off, None, O.SUM, O.FP32)) == 0
    # out-of-range ids are rejected, -1 is skipped
    bad = idx.copy()
    bad[2] = rows
    with pytest.raises(IndexError):
        O.tbe_forward(store, [0], B, bad, offsets, None, O.SUM, O.FP32)
    skip = idx.copy()
    skip[2] = -1
    assert bits_equal(O.tbe_forward(store, [0], B, skip, offsets, None, O.SUM, O.FP32),
                      O.tbe_forward(store, [0], B, skip, offsets, None, O.SUM, O.FP32, "fbgemm")) == 0


def test_lookup_matches_torch_embedding_bag_4bit():
    """torch.ops.quantized.embedding_bag_4bit_rowwise_offsets (trailer layout, fp32 out)
    agrees with the oracle to fp32 rounding on the same quantized rows."""
    rng = np.random.default_rng(12)
    rows, dim, B = 400, 64, 30
    w = rng.normal(0, 0.1, (rows, dim)).astype(np.float32)
    q = O.quantize_sbhalf(w, 4)
    lengths = rng.integers(0, 12, B)
    offsets = np.zeros(B + 1, dtype=np.int64)
    offsets[1:] = np.cumsum(lengths)
    idx = rng.integers(0, rows, int(offsets[-1]))
    want = torch.ops.quantized.embedding_bag_4bit_rowwise_offsets(
        torch.from_numpy(q), torch.from_numpy(idx), torch.from_numpy(offsets), include_last_offset=True).numpy()
    got = O.tbe_forward(O.pack_store([(O.INT4, dim, q)]), [0], B, idx, offsets, None, O.SUM, O.FP32)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)


def test_index_math_oracles():
    rng = np.random.default_rng(1)
    for dt in (np.int32, np.int64):
        l = rng.integers(0, 100, 1000).astype(dt)
        o = O.cumsum(l)
        assert o[0] == 0 and np.array_equal(o[1:], np.cumsum(l, dtype=dt))
    # permute: golden vector of the reference (test_keyed_jagged_tensor.py:415-452)
    lengths = np.array([[0, 2, 0], [1, 1, 1], [0, 3, 0]], dtype=np.int32)
    values = np.arange(1, 9, dtype=np.float32)
    weights = np.array([1.0, 0.5, 1.5, 1.0, 0.5, 1.0, 1.0, 1.5], dtype=np.float32)
    pl, pv, pw = O.permute_2d([1, 0, 2], lengths, values, weights)
    assert pl.reshape(-1).tolist() == [1, 1, 1, 0, 2, 0, 0, 3, 0]
    assert pv.tolist() == [3.0, 4.0, 5.0, 1.0, 2.0, 6.0, 7.0, 8.0]
    assert pw.tolist() == [1.5, 1.0, 0.5, 1.0, 0.5, 1.0, 1.0, 1.5]
    pl, pv, _ = O.permute_2d([1, 0, 2, 1, 1], lengths, values)
    assert pv.tolist() == [3.0, 4.0, 5.0, 1.0, 2.0, 6.0, 7.0, 8.0, 3.0, 4.0, 5.0, 3.0, 4.0, 5.0]


def test_bucketize_oracle_hand_case():
    """oracle_bucketize on a case small enough to do by hand: 2 features x 2
    samples, 2 buckets, block sizes 3 and 5; the id 9 of feature 0 lies beyond
    the last bucket (9 // 3 = 3 >= 2) and is dropped."""
    lengths = np.array([2, 1, 1, 2], dtype=np.int64)         # bags (f0,b0) (f0,b1) (f1,b0) (f1,b1)
    ids = np.array([4, 1, 9, 7, 2, 5], dtype=np.int64)       # f0: [4 1] [9]   f1: [7] [2 5]
    w = np.array([.1, .2, .3, .4, .5, .6], dtype=np.float32)
    # bucket of each id: 4//3=1, 1//3=0, 9//3=3 (dropped), 7//5=1, 2//5=0, 5//5=1
    nl, ni, nw, perm = O.bucketize(lengths, ids, [3, 5], 2, w, False, return_permute=True)
    assert nl.tolist() == [1, 0, 0, 1,   1, 0, 1, 1]         # bucket-major: [W, F, B]
    assert ni.tolist() == [1, 2,   1, 2, 0]                  # id % block size, input order inside a bag
    assert nw.tolist() == [np.float32(x) for x in (.2, .5, .1, .4, .6)]
    assert perm.tolist() == [2, 0, -1, 3, 1, 4]              # where each input id went; -1 = dropped
    nl2, ni2, _, _ = O.bucketize(lengths, ids, [3, 5], 2, w, True, return_permute=True)
    assert nl2.tolist() == nl.tolist() and ni2.tolist() == [1, 2, 4, 7, 5]  # keep_orig_idx: ids as given


@pytest.mark.parametrize("F,B,W", [(1, 1, 1), (2, 3, 2), (4, 15, 5), (15, 15, 129), (3, 200, 8)])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("keep", [False, True])
def test_bucketize_oracle_matches_python_rule(F, B, W, idt, keep):
    """oracle_bucketize against an independent pure-Python statement of the rule
    (the rule of block_bucketize_ref, torchrec/distributed/tests/test_utils.py:379-466):
    new lengths, new ids, weights and the unbucketize permute, with ids beyond the
    last bucket dropped, with and without keep_orig_idx."""
    rng = np.random.default_rng(F * 100 + B * 10 + W)
    lengths = rng.integers(0, 6, F * B).astype(idt)
    block_sizes = rng.integers(1, 50, F).astype(np.int64)
    hi = np.repeat(block_sizes * (W + 1), B)  # some ids fall beyond the last bucket
    ids = (np.concatenate([rng.integers(0, hi[i], lengths[i]) for i in range(F * B)]).astype(idt)
           if lengths.sum() else np.zeros(0, idt))
    weights = rng.random(len(ids)).astype(np.float32)
    pl, pi, pw, pu = bucketize_python(lengths.tolist(), ids.tolist(), weights.tolist(), block_sizes.tolist(), W, keep)
    ol, oi, ow, ou = O.bucketize(lengths, ids, block_sizes, W, weights, keep, return_permute=True)
    assert ol.tolist() == pl and oi.tolist() == pi and ou.tolist() == pu
    assert np.array_equal(ow, np.asarray(pw, dtype=np.float32))
    assert (np.asarray(pu) == -1).sum() == len(ids) - len(pi)  # exactly the dropped ids have no place
    # without weights / without the permute the other outputs do not change
    ol2, oi2, ow2, ou2 = O.bucketize(lengths, ids, block_sizes, W, None, keep)
    assert ol2.tolist() == pl and oi2.tolist() == pi and ow2 is None and ou2 is None


def test_bounds_check_oracle_hand_case():
    """The restated id rewrite of fbgemm_gpu's bounds_check_indices on a case worked by hand: three
    features x two bags; -1 stays, every other id outside its own feature's table becomes 0 in
    WARNING / IGNORE and stays in NONE; an id that is fine for a larger table is bad for a smaller
    one.  (Unpinned against fbgemm_gpu itself, which this image does not have.)"""
    rows = [4, 10, 6]
    offsets = np.array([0, 2, 3, 6, 6, 8, 9])
    ids = np.array([3, 4, -1, 9, 10, -7, 5, 6, 0])
    #               f0    | f0 | f1        | f1 (empty) | f2   | f2
    for mode in ("WARNING", "IGNORE"):
        out, bad = O.bounds_check_indices(rows, 2, ids, offsets, mode)
        assert out.tolist() == [3, 0, -1, 9, 0, 0, 5, 0, 0] and bad == 4
    out, bad = O.bounds_check_indices(rows, 2, ids, offsets, "NONE")
    assert out.tolist() == ids.tolist() and bad == 4
    assert ids.tolist() == [3, 4, -1, 9, 10, -7, 5, 6, 0]  # the input is not modified
