"""tra_tbe_forward_lengths_static: the lengths entry whose scratch (the offsets
array and the scan's partial sums) is a static device array of the library, so
the call allocates nothing.  Called through the C ABI and compared, bit for
bit, with tra_tbe_forward_lengths on a caller-allocated workspace: two calls in
a row, the second on a smaller input (the array keeps the first call's
contents), on the routes that use the scratch (scan + lookup).  The call must
leave the device's free memory and torch's pools as they were, and it is the
entry for callers under HIP graph capture: a captured call is replayed several
times, with eager work in between, against the eager result."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_equal, make_bags, make_table, weight_pair
from torchrec_amd import _lib
from torchrec_amd.tbe import EmbeddingLocation, PoolingMode, SparseType
from torchrec_amd.tbe.split_table_batched_embeddings_ops_inference import (
    IntNBitTableBatchedEmbeddingBagsCodegen as TBE,
)

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _operator(rng, specs):
    datas = [make_table(rng, dt, rows, dim) for dt, rows, dim in specs]
    wl = []
    for (dt, _, _), d in zip(specs, datas):
        w, sb = weight_pair(dt, d)
        wl.append((torch.from_numpy(np.ascontiguousarray(w)).to(DEV),
                   None if sb is None else torch.from_numpy(np.ascontiguousarray(sb)).to(DEV)))
    st = {O.INT8: SparseType.INT8, O.INT4: SparseType.INT4}
    tbe = TBE(embedding_specs=[(f"t{i}", rows, dim, st[dt], EmbeddingLocation.DEVICE) for i, (dt, rows, dim) in enumerate(specs)],
              pooling_mode=PoolingMode.SUM, device=DEV, weight_lists=wl, output_dtype=SparseType.FP16)
    store = O.pack_store([(dt, dim, d) for (dt, _, dim), d in zip(specs, datas)], row_alignment=16)
    return tbe, store


def _both_entries(tbe, ids, lengths, B, K, total_D):
    """(static-scratch entry, workspace entry) outputs of one lookup."""
    lib = _lib.lib()
    ti = torch.from_numpy(ids).to(DEV)
    tl = torch.from_numpy(lengths).to(DEV)
    plan = tbe._get_plan(None)
    stream = _lib.current_stream(DEV)
    out_static = torch.full((B, total_D), 7.0, dtype=torch.float16, device=DEV)
    out_ws = torch.full((B, total_D), 9.0, dtype=torch.float16, device=DEV)
    ws_bytes = lib.tra_tbe_forward_lengths_workspace_bytes(K, B, 0)
    assert 0 < ws_bytes <= lib.tra_tbe_forward_lengths_static_max_bytes()
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    args = (plan, _lib.ptr(tbe.weights_dev), _lib.ptr(ti), _lib.ptr(tl), 0, None, B, K, len(ids),
            _lib.POOL_SUM, _lib.FP16)
    # the static entry allocates nothing: neither from the device (hipMemGetInfo) nor from torch's pools
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(DEV)
    reserved_before, allocated_before = torch.cuda.memory_reserved(DEV), torch.cuda.memory_allocated(DEV)
    _lib.check(lib.tra_tbe_forward_lengths_static(*args, out_static.data_ptr(), total_D, stream))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(DEV)
    assert free_after == free_before
    assert (torch.cuda.memory_reserved(DEV), torch.cuda.memory_allocated(DEV)) == (reserved_before, allocated_before)
    _lib.check(lib.tra_tbe_forward_lengths(*args, out_ws.data_ptr(), total_D, ws.data_ptr(), stream))
    torch.cuda.synchronize()
    return out_static.cpu().numpy(), out_ws.cpu().numpy()


def test_static_scratch_entry_two_calls_in_a_row():
    rng = np.random.default_rng(2718)
    # two weight types = two launches: the lengths are scanned into the scratch
    # once and both launches read the offsets from it
    specs = [(O.INT4, 3000, 64), (O.INT8, 2500, 64), (O.INT4, 2000, 64), (O.INT8, 1500, 64)]
    tbe, store = _operator(rng, specs)
    K, total_D = len(specs), 64 * len(specs)
    rows_f = [s[1] for s in specs]
    buf = ctypes.create_string_buffer(512)
    # call 1: 4 x 40000 bags: scan in tiles (partial sums in the scratch), window kernel from offsets
    # call 2: 4 x 5000 bags of few ids: one-launch scan into the scratch, static kernel
    # (a call of at most 16384 lengths would not touch the scratch at all: its one kernel
    # derives the bag starts itself)
    for B, max_len in ((40_000, 6), (5000, 5)):
        lengths, offsets, ids = make_bags(rng, rows_f, B, max_len)
        _lib.check(_lib.lib().tra_tbe_launch_info(tbe._get_plan(None), B, len(ids), _lib.POOL_SUM, K, buf, 512))
        assert b"from_lengths" not in buf.value and b"scan" in buf.value, buf.value
        got_static, got_ws = _both_entries(tbe, ids, lengths, B, K, total_D)
        assert bits_equal(got_static, got_ws) == 0, B
        if B <= 5000:
            want = O.tbe_forward(store, list(range(K)), B, ids, offsets, None, O.SUM, O.FP16)
            assert bits_equal(got_static, want) == 0


def test_static_scratch_entry_refuses_what_does_not_fit():
    rng = np.random.default_rng(3)
    tbe, _ = _operator(rng, [(O.INT4, 100, 64)])
    lib = _lib.lib()
    K, B = 1, 3_000_000  # 12 MB of offsets: beyond the 8 MiB array
    assert lib.tra_tbe_forward_lengths_workspace_bytes(K, B, 0) > lib.tra_tbe_forward_lengths_static_max_bytes()
    out = torch.empty(8, dtype=torch.float16, device=DEV)
    rc = lib.tra_tbe_forward_lengths_static(tbe._get_plan(None), _lib.ptr(tbe.weights_dev), _lib.ptr(out), _lib.ptr(out),
                                            0, None, B, K, 1, _lib.POOL_SUM, _lib.FP16, out.data_ptr(), 64,
                                            _lib.current_stream(DEV))
    assert rc == -5  # TRA_ERR_TOO_LARGE, nothing launched
    assert b"static" in lib.tra_last_error()


def test_static_scratch_entry_under_graph_capture():
    """The context the entry is for: captured in a HIP graph (a scan + lookup call, more than
    16384 bags, so the scratch is used), replayed four times with new inputs and eager work
    between the replays; every replay equals the workspace entry run eagerly on the same inputs."""
    rng = np.random.default_rng(99)
    specs = [(O.INT4, 3000, 64), (O.INT8, 2500, 64), (O.INT4, 2000, 64), (O.INT8, 1500, 64)]
    tbe, _ = _operator(rng, specs)
    K, total_D, B = len(specs), 64 * len(specs), 6000
    assert K * B > 16384
    rows_f = [s[1] for s in specs]
    lib = _lib.lib()
    plan = tbe._get_plan(None)
    cap = K * B * 5
    ti = torch.zeros(cap, dtype=torch.int32, device=DEV)
    tl = torch.zeros(K * B, dtype=torch.int32, device=DEV)
    out = torch.zeros(B, total_D, dtype=torch.float16, device=DEV)
    ws = torch.empty(lib.tra_tbe_forward_lengths_workspace_bytes(K, B, 0), dtype=torch.uint8, device=DEV)

    def load(seed):
        lengths, _, ids = make_bags(np.random.default_rng(seed), rows_f, B, 5)
        ti.zero_()
        ti[: len(ids)].copy_(torch.from_numpy(ids))
        tl.copy_(torch.from_numpy(lengths))
        return len(ids)

    # the captured call reads its id count from the launch arguments: every replay uses inputs
    # padded to the same count (ids past the bags are never read)
    n0 = load(0)
    n_ids = cap

    def call_static(stream):
        _lib.check(lib.tra_tbe_forward_lengths_static(plan, _lib.ptr(tbe.weights_dev), _lib.ptr(ti), _lib.ptr(tl), 0, None,
                                                      B, K, n_ids, _lib.POOL_SUM, _lib.FP16, out.data_ptr(), total_D, stream))

    call_static(_lib.current_stream(DEV))  # geometry of this call shape, outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            call_static(_lib.current_stream(DEV))
    torch.cuda.synchronize()
    assert n0 <= cap
    for seed in (1, 2, 3, 4):
        load(seed)
        out.fill_(3.0)
        g.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy().copy()
        eager = torch.full((B, total_D), 5.0, dtype=torch.float16, device=DEV)
        _lib.check(lib.tra_tbe_forward_lengths(plan, _lib.ptr(tbe.weights_dev), _lib.ptr(ti), _lib.ptr(tl), 0, None, B, K,
                                               n_ids, _lib.POOL_SUM, _lib.FP16, eager.data_ptr(), total_D, ws.data_ptr(),
                                               _lib.current_stream(DEV)))
        torch.cuda.synchronize()
        assert bits_equal(got, eager.cpu().numpy()) == 0, seed
