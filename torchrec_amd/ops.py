"""Tensor-level front ends of the index-math and quantization kernels.

Function names follow the ``torch.ops.fbgemm.*`` operators the reference calls
at torchrec/sparse/jagged_tensor.py:79-80 (complete cumsum), :2573-2583
(permute_2D_sparse_data), torchrec/distributed/embedding_sharding.py:153-198
(block_bucketize_sparse_features) and torchrec/quant/embedding_modules.py:
261-265 (FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf).

Tensors on the GPU always go through the HIP kernels of libtorchrec_amd.so.
Index tensors that still live on the host (a KeyedJaggedTensor that has not
been moved to the device yet) are handled with plain torch integer arithmetic;
quantization and bucketization have no host form.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import _lib

_INT_TYPES = (torch.int32, torch.int64)


def _check_int(t: torch.Tensor, what: str) -> None:
    if t.dtype not in _INT_TYPES:
        raise TypeError(f"{what} must be int32 or int64, got {t.dtype}")


def asynchronous_complete_cumsum(lengths: torch.Tensor) -> torch.Tensor:
    """[n] -> [n + 1]: out[0] = 0, out[i + 1] = lengths[0] + ... + lengths[i]."""
    _check_int(lengths, "lengths")
    lengths = lengths.reshape(-1)
    n = lengths.numel()
    if lengths.device.type != "cuda":
        out = lengths.new_zeros(n + 1)
        if n:
            torch.cumsum(lengths, 0, out=out[1:])
        return out
    lengths = lengths.contiguous()
    out = torch.empty(n + 1, dtype=lengths.dtype, device=lengths.device)
    l = _lib.lib()
    ws_bytes = l.tra_cumsum_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=lengths.device) if ws_bytes else None
    _lib.check(
        l.tra_cumsum(
            _lib.ptr(lengths), n, int(lengths.dtype == torch.int64), _lib.ptr(out), _lib.ptr(ws),
            _lib.current_stream(lengths.device),
        )
    )
    return out


def length_per_key(lengths: torch.Tensor, num_features: int, stride: int) -> List[int]:
    """Per-feature totals of a feature-major [F * B] lengths tensor as a Python list.

    One reduction kernel and one F-element device-to-host copy (the reference
    does torch.sum(lengths.view(F, B), 1).tolist(), jagged_tensor.py:1201-1212).
    """
    if num_features == 0:
        return []
    if lengths.numel() == 0:
        return [0] * num_features
    _check_int(lengths, "lengths")
    if lengths.device.type != "cuda":
        return torch.sum(lengths.reshape(num_features, stride), dim=1).tolist()
    lengths = lengths.contiguous()
    out = torch.empty(num_features, dtype=torch.int64, device=lengths.device)
    _lib.check(
        _lib.lib().tra_length_per_key(
            _lib.ptr(lengths), num_features, stride, int(lengths.dtype == torch.int64),
            _lib.ptr(out), _lib.current_stream(lengths.device),
        )
    )
    return out.tolist()


_side_streams: dict = {}  # device index -> a second stream (default priority) for small reads that need not order with the main one


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    idx = device.index if device.index is not None else torch.cuda.current_device()
    s = _side_streams.get(idx)
    if s is None:
        s = _side_streams[idx] = torch.cuda.Stream(device=idx)
    return s


def length_per_key_async(lengths: torch.Tensor, num_features: int, stride: int):
    """``length_per_key`` split in two: the reduction and its copy to pinned host memory are queued now, on a
    second stream that waits for what the current stream holds at this moment (whatever produced ``lengths``),
    and the returned function waits for that copy alone and yields the Python list.  Work queued on the
    current stream afterwards (a lookup, say) neither waits for the reduction nor holds the host up.
    ``lengths`` must stay alive until the returned function has been called."""
    _check_int(lengths, "lengths")
    lengths = lengths.contiguous()
    dev = lengths.device
    side = _side_stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        out = torch.empty(num_features, dtype=torch.int64, device=dev)
        _lib.check(
            _lib.lib().tra_length_per_key(
                _lib.ptr(lengths), num_features, stride, int(lengths.dtype == torch.int64),
                _lib.ptr(out), _lib.current_stream(dev),
            )
        )
        host = torch.empty(num_features, dtype=torch.int64, pin_memory=True)
        host.copy_(out, non_blocking=True)
        arrived = torch.cuda.Event()
        arrived.record(side)

    # The side stream reads ``lengths`` (possibly a contiguous copy made above, which nobody else
    # holds): the allocator is told so, and the returned function keeps the tensor until the copy
    # has arrived, so that its memory is not handed to a later allocation of the current stream.
    lengths.record_stream(side)

    def finish(_held=lengths) -> List[int]:
        arrived.synchronize()
        return host.tolist()

    return finish


def permute_2D_sparse_data(
    permute: torch.Tensor,
    lengths: torch.Tensor,
    values: torch.Tensor,
    weights: Optional[torch.Tensor] = None,
    permuted_lengths_sum: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """lengths [T, B]; returns (lengths[permute], values / weights regrouped)."""
    _check_int(lengths, "lengths")
    assert lengths.dim() == 2
    T, B = lengths.shape
    Tp = permute.numel()
    if lengths.device.type != "cuda":
        perm = permute.to(torch.int64)
        out_lengths = lengths[perm]
        per_feature = lengths.sum(dim=1).tolist()
        starts = [0]
        for x in per_feature:
            starts.append(starts[-1] + x)
        pieces = [values[starts[p] : starts[p + 1]] for p in perm.tolist()]
        out_values = torch.cat(pieces) if pieces else values[:0]
        out_weights = None
        if weights is not None:
            wp = [weights[starts[p] : starts[p + 1]] for p in perm.tolist()]
            out_weights = torch.cat(wp) if wp else weights[:0]
        return out_lengths, out_values, out_weights

    dev = lengths.device
    l = _lib.lib()
    stream = _lib.current_stream(dev)
    is64 = int(lengths.dtype == torch.int64)
    lengths = lengths.contiguous()
    values = values.contiguous()
    if values.element_size() not in (4, 8):
        raise TypeError(f"values must have 4- or 8-byte elements, got {values.dtype}")
    permute = permute.to(device=dev, dtype=torch.int32).contiguous()
    out_lengths = torch.empty((Tp, B), dtype=lengths.dtype, device=dev)
    _lib.check(
        l.tra_permute_2d_lengths(
            _lib.ptr(permute), Tp, T, B, _lib.ptr(lengths), is64, _lib.ptr(out_lengths), stream
        )
    )
    in_offsets = asynchronous_complete_cumsum(lengths.view(-1))
    out_offsets = asynchronous_complete_cumsum(out_lengths.view(-1))
    if permuted_lengths_sum is None:
        permuted_lengths_sum = int(out_offsets[-1].item())
    out_values = torch.empty(permuted_lengths_sum, dtype=values.dtype, device=dev)
    out_weights = None
    if weights is not None:
        weights = weights.contiguous()
        if weights.dtype != torch.float32:
            raise TypeError(f"weights must be float32, got {weights.dtype}")
        out_weights = torch.empty(permuted_lengths_sum, dtype=torch.float32, device=dev)
    if permuted_lengths_sum > 0:  # (nothing to move otherwise, and empty outputs have no address to pass)
        _lib.check(
            l.tra_permute_2d_data(
                _lib.ptr(permute), Tp, B, _lib.ptr(in_offsets), _lib.ptr(out_offsets), is64,
                _lib.ptr(values), values.element_size(), _lib.ptr(weights), _lib.ptr(out_values),
                _lib.ptr(out_weights), stream,
            )
        )
    return out_lengths, out_values, out_weights


def block_bucketize_sparse_features(
    lengths: torch.Tensor,
    indices: torch.Tensor,
    bucketize_pos: bool,
    sequence: bool,
    block_sizes: torch.Tensor,
    my_size: int,
    weights: Optional[torch.Tensor] = None,
    keep_orig_idx: bool = False,
) -> Tuple[
    torch.Tensor, torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]
]:
    """Returns (new_lengths [W*F*B], new_indices, new_weights, new_pos, unbucketize_permute).

    new_pos (positions inside the original bag) is not produced: bucketize_pos
    must be False.  ``sequence`` asks for unbucketize_permute.
    """
    if bucketize_pos:
        raise NotImplementedError("bucketize_pos is not supported")
    _lib.require_gpu(lengths, "block_bucketize_sparse_features")
    _check_int(lengths, "lengths")
    _check_int(indices, "indices")
    # The kernels take ids and lengths in one width; lengths of another width
    # (a KJT usually carries int32 lengths beside int64 ids) are widened or
    # narrowed on the way in and the new lengths given back in the caller's.
    lengths_dtype = lengths.dtype
    if indices.dtype != lengths_dtype:
        lengths = lengths.to(indices.dtype)
    dev = lengths.device
    l = _lib.lib()
    stream = _lib.current_stream(dev)
    is64 = int(lengths.dtype == torch.int64)
    lengths = lengths.contiguous().view(-1)
    indices = indices.contiguous()
    F = block_sizes.numel()
    n = lengths.numel()
    B = n // F if F else 0
    W = int(my_size)
    bs = block_sizes.to(device=dev, dtype=torch.int64).contiguous()
    offsets = asynchronous_complete_cumsum(lengths)
    new_lengths = torch.empty(W * n, dtype=lengths.dtype, device=dev)
    _lib.check(
        l.tra_bucketize_lengths(
            _lib.ptr(offsets), _lib.ptr(indices), is64, _lib.ptr(bs), F, B, W, _lib.ptr(new_lengths), stream
        )
    )
    new_offsets = asynchronous_complete_cumsum(new_lengths)
    total = int(new_offsets[-1].item())
    new_indices = torch.empty(total, dtype=indices.dtype, device=dev)
    new_weights = None
    if weights is not None:
        weights = weights.contiguous().to(torch.float32)
        new_weights = torch.empty(total, dtype=torch.float32, device=dev)
    unbucketize = (
        torch.empty(indices.numel(), dtype=torch.int64, device=dev) if sequence else None
    )
    ws_bytes = l.tra_bucketize_workspace_bytes(F, B, W)
    cursor = torch.empty(ws_bytes // 8, dtype=torch.int64, device=dev) if ws_bytes else None
    _lib.check(
        l.tra_bucketize_scatter(
            # (no id kept, e.g. all beyond the last bucket: no weight is moved, and the empty
            # output has no address to pass)
            _lib.ptr(offsets), _lib.ptr(indices), is64, _lib.ptr(weights if total > 0 else None), _lib.ptr(bs), F, B, W,
            int(keep_orig_idx), _lib.ptr(new_offsets), _lib.ptr(cursor), _lib.ptr(new_indices),
            _lib.ptr(new_weights), _lib.ptr(unbucketize), stream,
        )
    )
    if new_lengths.dtype != lengths_dtype:
        new_lengths = new_lengths.to(lengths_dtype)
    return new_lengths, new_indices, new_weights, None, unbucketize


def FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(weight: torch.Tensor, bit_rate: int) -> torch.Tensor:
    """[rows, D] fp32/fp16 -> uint8 [rows, D*bits/8 + 4]: payload, fp16 scale, fp16 bias.

    Runs on the GPU.  A host tensor is staged through the current GPU and the
    result returned on the host, so callers that quantize a CPU-resident float
    module (the usual from_float flow) keep their device placement.
    """
    if weight.dim() != 2:
        raise ValueError("expected a [rows, dim] tensor")
    if not torch.cuda.is_available():
        raise _lib.TorchrecAmdError("row-wise quantization runs on an MI355X GPU; none is visible")
    src_device = weight.device
    dev = src_device if src_device.type == "cuda" else torch.device("cuda", torch.cuda.current_device())
    rows, dim = weight.shape
    out_cols = dim * bit_rate // 8 + 4
    out_host = torch.empty((rows, out_cols), dtype=torch.uint8, device=src_device)
    # Chunked so a large host table never needs a full fp32 copy on the device.
    step = max(1, (1 << 28) // max(dim * 4, 1))
    for r0 in range(0, max(rows, 1), step):
        chunk = weight[r0 : r0 + step].to(device=dev, dtype=torch.float32).contiguous()
        n = chunk.shape[0]
        out = torch.empty((n, out_cols), dtype=torch.uint8, device=dev)
        _lib.check(
            _lib.lib().tra_quantize_rows_sbhalf(
                _lib.ptr(chunk), n, dim, bit_rate, _lib.ptr(out), _lib.current_stream(dev)
            )
        )
        out_host[r0 : r0 + n].copy_(out)
    return out_host


def offsets_range(offsets: torch.Tensor, range_size: int) -> torch.Tensor:
    """[num_bags] bag starts -> [range_size] position of every element inside its bag
    (torch.ops.fbgemm.offsets_range; torchrec/modules/feature_processor_.py:82-84)."""
    _check_int(offsets, "offsets")
    offsets = offsets.reshape(-1).contiguous()
    n = offsets.numel()
    if offsets.device.type != "cuda":
        if n == 0 or range_size == 0:
            return offsets.new_zeros(range_size)
        ends = torch.cat([offsets[1:], offsets.new_tensor([range_size])])
        lengths = (ends - offsets).clamp(min=0)
        starts = torch.repeat_interleave(offsets, lengths)
        return torch.arange(range_size, dtype=offsets.dtype)[: starts.numel()] - starts
    out = torch.zeros(range_size, dtype=offsets.dtype, device=offsets.device)
    _lib.check(
        _lib.lib().tra_offsets_range(
            _lib.ptr(offsets), n, int(offsets.dtype == torch.int64), range_size, _lib.ptr(out),
            _lib.current_stream(offsets.device),
        )
    )
    return out


def position_weights(
    offsets: torch.Tensor,
    num_keys: int,
    batch_size: int,
    key_start: torch.Tensor,
    key_len: torch.Tensor,
    table: torch.Tensor,
    num_values: int,
) -> torch.Tensor:
    """Per-id weights ``table[key_start[k] + position in bag]`` (1.0 where ``key_len[k] <= 0``)
    for a feature-major KJT with ``offsets`` of ``num_keys * batch_size + 1`` entries."""
    _check_int(offsets, "offsets")
    _lib.require_gpu(offsets, "offsets")
    offsets = offsets.contiguous()
    assert offsets.numel() >= num_keys * batch_size + 1
    assert key_start.dtype == torch.int32 and key_len.dtype == torch.int32 and table.dtype == torch.float32
    out = torch.empty(num_values, dtype=torch.float32, device=offsets.device)
    if num_values == 0:  # (bags without ids: nothing to weigh, and an empty output has no address to pass)
        return out
    _lib.check(
        _lib.lib().tra_position_weights(
            _lib.ptr(offsets), int(offsets.dtype == torch.int64), num_keys, batch_size, _lib.ptr(key_start),
            _lib.ptr(key_len), _lib.ptr(table.contiguous()), _lib.ptr(out), _lib.current_stream(offsets.device),
        )
    )
    return out


def mch_remap(
    values: torch.Tensor, sorted_ids: torch.Tensor, mapping: torch.Tensor, miss_id: int
) -> torch.Tensor:
    """Ids found in ``sorted_ids[:-1]`` (or equal to the last entry when nothing smaller is found)
    become ``mapping[position]``, all others ``miss_id`` (torchrec/modules/mc_modules.py:959-989)."""
    _check_int(values, "values")
    assert sorted_ids.dtype == torch.int64 and mapping.dtype == torch.int64
    assert sorted_ids.numel() == mapping.numel() and sorted_ids.numel() > 0
    if values.device.type != "cuda":
        idx = torch.searchsorted(sorted_ids[:-1], values.long())
        hit = sorted_ids[idx] == values
        return torch.where(hit, mapping[idx], torch.full_like(idx, miss_id)).to(values.dtype)
    values = values.contiguous()
    out = torch.empty_like(values)
    _lib.check(
        _lib.lib().tra_mch_remap(
            _lib.ptr(values), values.numel(), int(values.dtype == torch.int64), _lib.ptr(sorted_ids.contiguous()),
            _lib.ptr(mapping.contiguous()), sorted_ids.numel(), int(miss_id), _lib.ptr(out),
            _lib.current_stream(values.device),
        )
    )
    return out


def mch_remap_keys(
    values: torch.Tensor,
    offsets: torch.Tensor,
    batch_size: int,
    sorted_ids: List[torch.Tensor],
    mappings: List[torch.Tensor],
    miss_ids: List[int],
) -> torch.Tensor:
    """``mch_remap`` for every key of a KeyedJaggedTensor in one launch: key ``k`` (ids
    ``values[offsets[k*B] : offsets[(k+1)*B]]``) is looked up in ``sorted_ids[k]`` / ``mappings[k]``."""
    import ctypes

    _lib.require_gpu(values, "mch_remap_keys")
    _check_int(values, "values")
    K = len(sorted_ids)
    assert len(mappings) == K and len(miss_ids) == K
    assert offsets.numel() == K * batch_size + 1, "offsets must have num_keys * B + 1 entries"
    for s_, m_ in zip(sorted_ids, mappings):
        assert s_.dtype == torch.int64 and m_.dtype == torch.int64 and s_.numel() == m_.numel() > 0
        assert s_.is_contiguous() and m_.is_contiguous() and s_.device == values.device and m_.device == values.device
    values = values.contiguous()
    if offsets.dtype != values.dtype:
        offsets = offsets.to(values.dtype)
    offsets = offsets.contiguous()
    out = torch.empty_like(values)
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    _lib.check(
        _lib.lib().tra_mch_remap_keys(
            _lib.ptr(values), values.numel(), _lib.ptr(offsets), int(values.dtype == torch.int64), K, int(batch_size),
            (vp * max(K, 1))(*[t.data_ptr() for t in sorted_ids]), (vp * max(K, 1))(*[t.data_ptr() for t in mappings]),
            (i64 * max(K, 1))(*[t.numel() for t in sorted_ids]), (i64 * max(K, 1))(*[int(m) for m in miss_ids]),
            _lib.ptr(out), _lib.current_stream(values.device),
        )
    )
    return out
