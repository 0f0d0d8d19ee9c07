"""HIP index-math and quantization kernels against the CPU oracle / numpy.
Integer outputs: torch.equal.  Quantized bytes: identical."""
import itertools

import numpy as np
import pytest
import torch

import oracle as O
from helpers import bucketize_python
from torchrec_amd import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 2047, 2048, 2049, 4095, 4096, 4097, 53_248, 100_003,
                               131_071, 131_072, 131_073, 200_001, 262_143, 262_144, 262_145, 1_048_577])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_cumsum(n, dtype):
    rng = np.random.default_rng(n)
    lengths = rng.integers(0, 50, n).astype(dtype)
    got = ops.asynchronous_complete_cumsum(torch.from_numpy(lengths).to(DEV)).cpu().numpy()
    want = O.cumsum(lengths)
    assert got.dtype == want.dtype and np.array_equal(got, want)
    assert np.array_equal(want[1:], np.cumsum(lengths, dtype=dtype))  # closed form


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_cumsum_unaligned_view(dtype):
    """Input that starts 4 (or 8) bytes into an allocation: no 16-byte loads."""
    rng = np.random.default_rng(5)
    lengths = rng.integers(0, 50, 20_001).astype(dtype)
    view = torch.from_numpy(lengths).to(DEV)[1:]
    assert view.data_ptr() % 16 != 0
    got = ops.asynchronous_complete_cumsum(view).cpu().numpy()
    assert np.array_equal(got, O.cumsum(lengths[1:]))


def test_cumsum_int64_beyond_32_bits():
    lengths = np.full(5000, 2**31 - 7, dtype=np.int64)
    got = ops.asynchronous_complete_cumsum(torch.from_numpy(lengths).to(DEV)).cpu().numpy()
    assert np.array_equal(got[1:], np.cumsum(lengths))


@pytest.mark.parametrize("F,B", [(1, 1), (3, 7), (26, 2048), (64, 4096), (5, 300)])
def test_length_per_key(F, B):
    rng = np.random.default_rng(F * B)
    lengths = rng.integers(0, 41, F * B).astype(np.int32)
    got = ops.length_per_key(torch.from_numpy(lengths).to(DEV), F, B)
    assert got == lengths.reshape(F, B).sum(axis=1).tolist()
    # the two-step form: queued now, collected after other work has been queued behind it
    later = ops.length_per_key_async(torch.from_numpy(lengths).to(DEV), F, B)
    busy = torch.empty(1 << 22, device=DEV).normal_()
    assert later() == got
    del busy


@pytest.mark.parametrize("T,B,Tp", [(3, 3, 3), (5, 17, 9), (26, 512, 26), (4, 1000, 2), (2, 1, 6)])
@pytest.mark.parametrize("idt,vdt,weighted", [(np.int32, np.int64, True), (np.int64, np.int32, False), (np.int32, np.float32, True)])
def test_permute_2d(T, B, Tp, idt, vdt, weighted):
    rng = np.random.default_rng(T * 1000 + B + Tp)
    lengths = rng.integers(0, 9, (T, B)).astype(idt)
    total = int(lengths.sum())
    values = rng.integers(0, 10**6, total).astype(vdt)
    weights = rng.random(total).astype(np.float32) if weighted else None
    perm = rng.integers(0, T, Tp).astype(np.int32)  # repeats allowed
    wl, wv, ww = O.permute_2d(perm, lengths, values, weights)
    gl, gv, gw = ops.permute_2D_sparse_data(
        torch.from_numpy(perm).to(DEV), torch.from_numpy(lengths).to(DEV), torch.from_numpy(values).to(DEV),
        None if weights is None else torch.from_numpy(weights).to(DEV))
    assert np.array_equal(gl.cpu().numpy(), wl)
    assert np.array_equal(gv.cpu().numpy(), wv)
    if weighted:
        assert np.array_equal(gw.cpu().numpy(), ww)
    else:
        assert gw is None


@pytest.mark.gpu
@pytest.mark.parametrize("weighted", [False, True])
def test_permute_2d_selecting_only_empty_features(weighted):
    """A permutation that picks nothing but features without ids, out of an input
    that has ids (and weights) elsewhere: empty outputs, no call with null outputs."""
    lengths = np.array([[2, 1, 3], [0, 0, 0], [1, 1, 1], [0, 0, 0]], dtype=np.int64)
    total = int(lengths.sum())
    values = np.arange(total, dtype=np.int64)
    weights = np.linspace(0, 1, total).astype(np.float32) if weighted else None
    perm = np.array([3, 1, 1], dtype=np.int32)
    gl, gv, gw = ops.permute_2D_sparse_data(
        torch.from_numpy(perm).to(DEV), torch.from_numpy(lengths).to(DEV), torch.from_numpy(values).to(DEV),
        None if weights is None else torch.from_numpy(weights).to(DEV))
    assert gl.shape == (3, 3) and int(gl.sum()) == 0
    assert gv.numel() == 0 and gv.dtype == torch.int64
    assert (gw is None) if not weighted else (gw.numel() == 0 and gw.dtype == torch.float32)
    # through the KJT: the permuted tensor is usable
    from torchrec_amd import KeyedJaggedTensor
    kjt = KeyedJaggedTensor(keys=["a", "b", "c", "d"], values=torch.from_numpy(values).to(DEV),
                            lengths=torch.from_numpy(lengths.reshape(-1)).to(DEV),
                            weights=None if weights is None else torch.from_numpy(weights).to(DEV))
    p = kjt.permute([3, 1])
    assert p.keys() == ["d", "b"] and p.values().numel() == 0 and p.lengths().tolist() == [0] * 6


@pytest.mark.gpu
def test_ops_with_bags_but_no_ids_to_write():
    """Operators whose output is empty while their input is not (or whose bags
    hold no ids at all) return empty tensors; they pass no null output on."""
    F, B, W = 3, 4, 2
    zero = torch.zeros(F * B, dtype=torch.int64, device=DEV)
    offsets0 = torch.zeros(F * B + 1, dtype=torch.int64, device=DEV)
    # position weights of bags without ids
    out = ops.position_weights(offsets0, F, B, torch.zeros(F, dtype=torch.int32, device=DEV),
                               torch.full((F,), 5, dtype=torch.int32, device=DEV), torch.ones(15, device=DEV), 0)
    assert out.numel() == 0 and out.dtype == torch.float32
    assert ops.offsets_range(offsets0[:-1], 0).numel() == 0
    # bucketize: no ids at all
    empty = torch.zeros(0, dtype=torch.int64, device=DEV)
    bs = torch.full((F,), 10, dtype=torch.int64, device=DEV)
    nl, ni, nw, _, nu = ops.block_bucketize_sparse_features(zero, empty, False, True, bs, W, torch.zeros(0, device=DEV))
    assert int(nl.sum()) == 0 and ni.numel() == 0 and nw.numel() == 0 and nu.numel() == 0
    # bucketize: ids and weights present, every id beyond the last bucket (dropped)
    lengths = torch.ones(F * B, dtype=torch.int64, device=DEV)
    ids = torch.full((F * B,), 10 * W + 3, dtype=torch.int64, device=DEV)
    nl, ni, nw, _, _ = ops.block_bucketize_sparse_features(lengths, ids, False, False, bs, W, torch.rand(F * B, device=DEV))
    want = O.bucketize(lengths.cpu().numpy(), ids.cpu().numpy(), bs.cpu().numpy(), W,
                       np.ones(F * B, dtype=np.float32), False)
    assert nl.cpu().numpy().tolist() == want[0].tolist() and int(nl.sum()) == 0
    assert ni.numel() == len(want[1]) == 0 and nw.numel() == 0


@pytest.mark.parametrize("F,B,W", [(1, 1, 1), (2, 3, 2), (4, 15, 5), (15, 15, 129), (3, 200, 8)])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("keep", [False, True])
def test_bucketize(F, B, W, idt, keep):
    rng = np.random.default_rng(F * 100 + B * 10 + W)
    lengths = rng.integers(0, 6, F * B).astype(idt)
    block_sizes = rng.integers(1, 50, F).astype(np.int64)
    # some ids fall beyond the last bucket and are dropped
    hi = np.repeat(block_sizes * (W + 1), B)
    ids = np.concatenate([rng.integers(0, hi[i], lengths[i]) for i in range(F * B)]).astype(idt) if lengths.sum() else np.zeros(0, idt)
    weights = rng.random(len(ids)).astype(np.float32)
    pl, pi, pw, pu = bucketize_python(lengths.tolist(), ids.tolist(), weights.tolist(), block_sizes.tolist(), W, keep)
    ol, oi, ow, ou = O.bucketize(lengths, ids, block_sizes, W, weights, keep, return_permute=True)
    assert ol.tolist() == pl and oi.tolist() == pi and ou.tolist() == pu  # oracle pinned by the python rule
    gl, gi, gw, _, gu = ops.block_bucketize_sparse_features(
        torch.from_numpy(lengths).to(DEV), torch.from_numpy(ids).to(DEV), False, True,
        torch.from_numpy(block_sizes).to(DEV), W, torch.from_numpy(weights).to(DEV), keep)
    assert gl.cpu().numpy().tolist() == pl
    assert gi.cpu().numpy().tolist() == pi
    assert gu.cpu().numpy().tolist() == pu
    assert np.array_equal(gw.cpu().numpy(), np.asarray(pw, dtype=np.float32))


@pytest.mark.parametrize("is_sequence", [False, True])
def test_bucketize_kjt(is_sequence):
    """KJT-level wrappers: keys repeated per bucket, lengths/values of the op, and for
    sequence features the unbucketize permute and the bucket of every input id."""
    from torchrec_amd import KeyedJaggedTensor
    from torchrec_amd.sparse.bucketize import bucketize_kjt_before_all2all, bucketize_kjt_inference

    rng = np.random.default_rng(12)
    keys, B, W = ["a", "b", "c"], 11, 4
    lengths = rng.integers(0, 6, len(keys) * B).astype(np.int64)
    block_sizes = np.asarray([7, 13, 29], dtype=np.int64)
    hi = np.repeat(block_sizes * W, B)  # every id lands in a bucket
    ids = np.concatenate([rng.integers(0, hi[i], lengths[i]) for i in range(len(lengths))]).astype(np.int64)
    weights = rng.random(len(ids)).astype(np.float32)
    kjt = KeyedJaggedTensor(keys=keys, values=torch.from_numpy(ids).to(DEV), lengths=torch.from_numpy(lengths).to(DEV),
                            weights=torch.from_numpy(weights).to(DEV))
    ol, oi, ow, ou = O.bucketize(lengths, ids, block_sizes, W, weights, False, return_permute=True)
    out, perm, mapping = bucketize_kjt_inference(kjt, W, torch.from_numpy(block_sizes), is_sequence=is_sequence)
    assert out.keys() == keys * W and out.stride() == B
    assert out.lengths().cpu().numpy().tolist() == ol.tolist()
    assert out.values().cpu().numpy().tolist() == oi.tolist()
    assert np.array_equal(out.weights().cpu().numpy(), ow)
    if is_sequence:
        assert perm.cpu().numpy().tolist() == ou.tolist()
        per_id_block = np.repeat(np.repeat(block_sizes, B), lengths)
        assert mapping.cpu().numpy().tolist() == (ids // per_id_block).tolist()
        # ids come back in input order through the permute
        restored = out.values()[perm] + mapping * torch.from_numpy(per_id_block).to(DEV)
        assert restored.cpu().numpy().tolist() == ids.tolist()
    else:
        assert perm is None and mapping is None
    out2, perm2 = bucketize_kjt_before_all2all(kjt, W, torch.from_numpy(block_sizes), output_permute=is_sequence)
    assert out2.keys() == keys * W and out2.values().cpu().numpy().tolist() == oi.tolist()
    assert (perm2 is not None) == is_sequence
    with pytest.raises(NotImplementedError):
        bucketize_kjt_inference(kjt, W, torch.from_numpy(block_sizes), bucketize_pos=True)


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_quantize_rows_bytes_identical(bits):
    rng = np.random.default_rng(bits)
    for dim in (8, 16, 32, 64, 128, 256, 1024):
        w = rng.normal(0, 0.1, (3000, dim)).astype(np.float32)
        w[0] = 0.25                                   # constant row: scale 1, all q = 0
        w[1] = np.linspace(0, 2**bits - 1, dim)       # exact ramp
        w[2] *= 1e-9                                  # tiny range: fp16 scale underflows
        w[3] *= 1e4
        w[4] = 0.0
        want = O.quantize_sbhalf(w, bits)
        got = ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(torch.from_numpy(w).to(DEV), bits).cpu().numpy()
        assert got.shape == want.shape and np.array_equal(got, want), (bits, dim, int((got != want).sum()))
        # a host tensor is staged through the GPU and comes back on the host
        got_h = ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(torch.from_numpy(w[:100]), bits)
        assert got_h.device.type == "cpu" and np.array_equal(got_h.numpy(), want[:100])


def _lengths_like(kind, n, rng):
    if kind == "short":
        ln = rng.integers(0, 41, n)
        ln[rng.random(n) < 0.05] = 0
    elif kind == "poisson":
        ln = rng.poisson(30.0, n)
    else:  # a few very long bags among empty and short ones: chunks of 64 ids inside one bag
        ln = rng.integers(0, 4, n)
        ln[rng.integers(0, n, max(1, n // 500))] = rng.integers(65, 700, max(1, n // 500))
    return ln


@pytest.mark.parametrize("F,B,W,kind", [
    (26, 2048, 8, "short"),      # 8 bags per wave
    (64, 4096, 4, "poisson"),    # 64 bags per wave
    (8, 16384, 16, "long"),
    (3, 5000, 1, "long"),
    (5, 1000, 700, "short"),     # one bag per wave (wide bucketization)
    (2, 300, 1500, "short"),     # beyond the wave kernels' bucket limit: thread-per-bag kernels
])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_bucketize_at_scale(F, B, W, kind, idt):
    rng = np.random.default_rng(F * B + W)
    n = F * B
    lengths = _lengths_like(kind, n, rng).astype(idt)
    block_sizes = rng.integers(1000, 200_000, F).astype(np.int64)
    if idt == np.int64:
        block_sizes[0] = (1 << 33) + 12345  # 64-bit division
    L = int(lengths.sum())
    per_id_bs = np.repeat(np.repeat(block_sizes, B), lengths)
    top = np.minimum(per_id_bs * (W + 1), np.iinfo(idt).max)  # some ids fall beyond the last bucket
    ids = (rng.random(L) * top).astype(idt)
    weights = rng.random(L).astype(np.float32)
    for keep in (False, True):
        ol, oi, ow, ou = O.bucketize(lengths, ids, block_sizes, W, weights, keep, return_permute=True)
        gl, gi, gw, _, gu = ops.block_bucketize_sparse_features(
            torch.from_numpy(lengths).to(DEV), torch.from_numpy(ids).to(DEV), False, True,
            torch.from_numpy(block_sizes).to(DEV), W, torch.from_numpy(weights).to(DEV), keep)
        assert np.array_equal(gl.cpu().numpy(), ol)
        assert np.array_equal(gi.cpu().numpy(), oi)
        assert np.array_equal(gu.cpu().numpy(), ou)
        assert np.array_equal(gw.cpu().numpy(), ow)
    # what the layout itself fixes: every kept id sits in the bucket its value names, in input order
    kept = ou >= 0
    assert int(ol.sum()) == int(kept.sum())
    assert np.array_equal(oi[ou[kept]], ids[kept])  # (keep=True run is the last one)


@pytest.mark.parametrize("F,B,kind", [(26, 2048, "short"), (64, 4096, "poisson"), (8, 16384, "long"), (1, 1, "long"),
                                      (3, 77, "short")])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_offsets_range_and_position_weights_at_scale(F, B, kind, idt):
    rng = np.random.default_rng(F + B)
    n = F * B
    lengths = _lengths_like(kind, n, rng).astype(idt)
    L = int(lengths.sum())
    offsets = np.zeros(n + 1, dtype=idt)
    offsets[1:] = np.cumsum(lengths)
    want_range = (np.arange(L) - np.repeat(offsets[:-1], lengths)).astype(idt)
    got = ops.offsets_range(torch.from_numpy(offsets[:-1].copy()).to(DEV), L)
    assert got.dtype == torch.from_numpy(offsets).dtype and np.array_equal(got.cpu().numpy(), want_range)
    # a range cut short: ids at or beyond range_size are not produced
    if L > 10:
        cut = L - 7
        assert np.array_equal(ops.offsets_range(torch.from_numpy(offsets[:-1].copy()).to(DEV), cut).cpu().numpy(),
                              want_range[:cut])
    # position weights: key k has a table of key_len[k] entries (0: no table -> 1.0); positions
    # beyond the table take its last entry
    key_len = rng.integers(0, 50, F).astype(np.int32)
    key_len[rng.integers(0, F)] = 0
    key_start = np.zeros(F, dtype=np.int32)
    key_start[1:] = np.cumsum(key_len)[:-1]
    table = rng.random(max(int(key_len.sum()), 1)).astype(np.float32)
    key_of_id = np.repeat(np.repeat(np.arange(F), B), lengths)
    klen = key_len[key_of_id]
    pos = np.minimum(want_range, np.maximum(klen - 1, 0))
    want_w = np.where(klen > 0, table[np.minimum(key_start[key_of_id] + pos, len(table) - 1)], np.float32(1.0)).astype(np.float32)
    got_w = ops.position_weights(torch.from_numpy(offsets).to(DEV), F, B, torch.from_numpy(key_start).to(DEV),
                                 torch.from_numpy(key_len).to(DEV), torch.from_numpy(table).to(DEV), L)
    assert np.array_equal(got_w.cpu().numpy(), want_w)


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_quantize_rows_odd_dims(bits):
    """Dims on either side of the dword-per-lane kernel's alignment rule, rows wider than one wave's
    worth of dwords, and a row count that leaves the last wave partly idle."""
    rng = np.random.default_rng(100 + bits)
    for dim in (4, 12, 20, 40, 96, 200, 520, 2048):
        if dim % (8 // bits):
            continue
        w = rng.normal(0, 1.0, (1237, dim)).astype(np.float32)
        want = O.quantize_sbhalf(w, bits)
        got = ops.FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(torch.from_numpy(w).to(DEV), bits).cpu().numpy()
        assert np.array_equal(got, want), (bits, dim, int((got != want).sum()))
