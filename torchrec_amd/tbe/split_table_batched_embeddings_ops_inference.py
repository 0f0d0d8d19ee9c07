"""Table-batched quantized embedding operator for MI355X.

``IntNBitTableBatchedEmbeddingBagsCodegen`` keeps the constructor keywords,
methods and attributes the reference uses from fbgemm_gpu's class of the same
name (call sites: torchrec/quant/embedding_modules.py:427-438, 461-467,
547-557, 828-842, 938-942; torchrec/inference/modules.py:628-655; the contract
as stated by MockTBE, torchrec/distributed/test_utils/infer_utils.py:1037-1096).
Storage and lookup are this package's own:

* one ``uint8`` buffer per group holds every table; table ``t`` starts at a
  256-byte aligned offset; a row is ``[fp16 scale][fp16 bias][payload][pad]``
  for INT8/INT4/INT2 and ``[payload][pad]`` for FP16/FP32, padded to
  ``row_alignment`` bytes (its *width*, what every view of the table shows);
* rows lie ``row_stride`` bytes apart.  HBM is fetched in 128-byte lines, so a
  random row costs the lines it touches: an 80-byte row at an 80-byte stride
  straddles two lines half of the time.  With row padding "line" (the default)
  a row of at most 128 bytes is stored at the next power-of-two stride, where
  it never straddles a line, as long as the padded store of the operator stays
  within ``ROW_PADDING_BUDGET_BYTES``; otherwise, and with row padding "none",
  the stride is the width.  Views of a table are ``[rows, width]`` slices of
  the strided buffer either way;
* ``forward`` launches the HIP gather/dequantize/pool kernels of
  ``libtorchrec_amd.so`` on the current stream.  There is no host lookup: on a
  CPU device the module can be built, inspected and (de)serialized, but
  ``forward`` raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import nn, Tensor

from torchrec_amd import _lib
from torchrec_amd.tbe.enums import BoundsCheckMode, EmbeddingLocation, PoolingMode, SparseType

# TORCHREC_AMD_BOUNDS_CHECK=1 (read when this module is imported): every forward
# fetches the count of out-of-range ids and raises if there were any (synchronizes).
_ENV_BOUNDS_CHECK = os.environ.get("TORCHREC_AMD_BOUNDS_CHECK", "0") == "1"
_INT_DTYPES = (torch.int32, torch.int64)
_BOUNDS_FATAL = int(BoundsCheckMode.FATAL)
_FORWARD_LENGTHS = None  # the library's tra_tbe_forward_lengths, bound on first use

_SUPPORTED_WEIGHTS = (SparseType.FP32, SparseType.FP16, SparseType.INT8, SparseType.INT4, SparseType.INT2)
_TABLE_ALIGNMENT = 256
_LINE_BYTES = 128
# Row padding trades spare HBM for bandwidth; an operator whose padded store would exceed this
# keeps its rows at their width (a fixed figure, not a share of the device's memory: the layout
# of an operator must not depend on where it was built).
ROW_PADDING_BUDGET_BYTES = 64 << 30
_ROW_PADDING_MODES = ("line", "none")
_default_row_padding = os.environ.get("TORCHREC_AMD_ROW_PADDING", "line")
if _default_row_padding not in _ROW_PADDING_MODES:
    raise ValueError(f"TORCHREC_AMD_ROW_PADDING={_default_row_padding!r}: expected one of {_ROW_PADDING_MODES}")


def set_default_row_padding(mode: str) -> str:
    """Row padding of operators built from now on ("line" or "none"); returns the previous default."""
    global _default_row_padding
    if mode not in _ROW_PADDING_MODES:
        raise ValueError(f"row padding {mode!r}: expected one of {_ROW_PADDING_MODES}")
    previous, _default_row_padding = _default_row_padding, mode
    return previous


def get_default_row_padding() -> str:
    return _default_row_padding


def line_padded_row_stride(row_bytes: int) -> int:
    """Distance between rows of ``row_bytes`` bytes under row padding "line": the next power
    of two for rows of at most one 128-byte line, the width for wider rows."""
    if row_bytes > _LINE_BYTES:
        return row_bytes
    stride = 4
    while stride < row_bytes:
        stride *= 2
    return stride


def round_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


def unpadded_row_size_in_bytes(dim: int, weight_ty: SparseType, scale_bias_size_in_bytes: int = 4) -> int:
    payload = dim * weight_ty.bit_rate() // 8
    if weight_ty in (SparseType.INT8, SparseType.INT4, SparseType.INT2):
        return payload + scale_bias_size_in_bytes
    return payload


def rounded_row_size_in_bytes(
    dim: int, weight_ty: SparseType, row_alignment: int, scale_bias_size_in_bytes: int = 4
) -> int:
    return round_up(unpadded_row_size_in_bytes(dim, weight_ty, scale_bias_size_in_bytes), row_alignment)


class IntNBitTableBatchedEmbeddingBagsCodegen(nn.Module):
    """Inference-only table-batched embedding lookup over packed int-N / fp16 rows."""

    def __init__(
        self,
        embedding_specs: List[Tuple[str, int, int, SparseType, EmbeddingLocation]],
        feature_table_map: Optional[List[int]] = None,
        index_remapping: Optional[List[Tensor]] = None,
        pooling_mode: PoolingMode = PoolingMode.SUM,
        device: Optional[torch.device] = None,
        bounds_check_mode: Optional[int] = None,
        weight_lists: Optional[List[Tuple[Tensor, Optional[Tensor]]]] = None,
        output_dtype: SparseType = SparseType.FP16,
        row_alignment: Optional[int] = None,
        uvm_host_mapped: bool = False,
        feature_names_per_table: Optional[List[List[str]]] = None,
        row_padding: Optional[str] = None,
        **unsupported,
    ) -> None:
        super().__init__()
        # uvm_host_mapped chooses how host-mapped tables are allocated; every
        # table here lives in HBM, so it has nothing to act on.
        self.feature_names_per_table = feature_names_per_table
        if index_remapping:
            raise NotImplementedError("index_remapping (pruning hash maps) is not supported")
        for k, v in unsupported.items():
            if v not in (None, False, 0):
                raise NotImplementedError(f"IntNBitTableBatchedEmbeddingBagsCodegen: option {k}={v!r}")
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")
        elif not isinstance(device, torch.device):
            device = torch.device(device)
        if device.type == "cuda" and device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.current_device: torch.device = device
        self.embedding_specs = embedding_specs
        self.pooling_mode = pooling_mode
        self.output_dtype: int = output_dtype.as_int()
        # An id outside [0, rows) is counted in every mode.  WARNING / IGNORE: it
        # pools row 0, as in fbgemm_gpu, whose bounds_check_indices rewrites such
        # an id to 0 in these modes before the lookup.  Not given, NONE (unchecked
        # in fbgemm_gpu) and FATAL: it is skipped (adds nothing); FATAL also raises
        # after the call, which waits for the kernel.
        self.bounds_check_mode_int: int = -1 if bounds_check_mode is None else int(bounds_check_mode)
        if output_dtype not in (SparseType.FP32, SparseType.FP16):
            raise NotImplementedError(f"output dtype {output_dtype} (fp32 and fp16 are supported)")
        self.scale_bias_size_in_bytes = 4
        self.row_alignment: int = 16 if row_alignment is None else int(row_alignment)
        if self.row_alignment < 1:
            raise ValueError("row_alignment must be positive")

        T_ = len(embedding_specs)
        self.feature_table_map: List[int] = (
            list(feature_table_map) if feature_table_map is not None else list(range(T_))
        )
        assert T_ <= len(self.feature_table_map), "every table needs at least one feature"
        for t in self.feature_table_map:
            assert 0 <= t < T_, f"feature_table_map entry {t} out of range"
        self.embedding_names: List[str] = [e[0] for e in embedding_specs]
        rows: List[int] = [int(e[1]) for e in embedding_specs]
        dims: List[int] = [int(e[2]) for e in embedding_specs]
        self.weight_tys: List[SparseType] = [e[3] for e in embedding_specs]
        for ty in self.weight_tys:
            if ty not in _SUPPORTED_WEIGHTS:
                raise NotImplementedError(f"weight type {ty} (INT8/INT4/INT2/FP16/FP32 are supported)")
        for name, d, ty in zip(self.embedding_names, dims, self.weight_tys):
            if (d * ty.bit_rate()) % 32 != 0:
                raise ValueError(
                    f"table {name}: embedding_dim {d} at {ty.bit_rate()} bits is not a whole number of 4-byte words"
                )
        self.rows = rows
        self.dims = dims
        self.max_D: int = max(dims) if dims else 0
        D_offsets = [0]
        for t in self.feature_table_map:
            D_offsets.append(D_offsets[-1] + dims[t])
        self.D_offsets: List[int] = D_offsets
        self.total_D: int = D_offsets[-1]

        # row_bytes: width of a row (header, payload, padding to row_alignment); row_stride: distance
        # between rows in the packed buffer (>= width, see the module docstring).
        self.row_bytes: List[int] = []
        for d, ty in zip(dims, self.weight_tys):
            rb = rounded_row_size_in_bytes(d, ty, self.row_alignment, self.scale_bias_size_in_bytes)
            if device.type == "cuda" and rb % 4 != 0:
                raise ValueError(
                    f"row_alignment {self.row_alignment} gives {rb}-byte rows; the GPU kernels need a multiple of 4"
                )
            self.row_bytes.append(rb)
        self.row_padding: str = _default_row_padding if row_padding is None else row_padding
        if self.row_padding not in _ROW_PADDING_MODES:
            raise ValueError(f"row_padding {self.row_padding!r}: expected one of {_ROW_PADDING_MODES}")

        def layout(strides: List[int]) -> Tuple[List[int], int]:
            offsets, total = [], 0
            for r, st in zip(rows, strides):
                offsets.append(total)
                total = round_up(total + r * st, _TABLE_ALIGNMENT)
            return offsets, total

        self.row_stride: List[int] = list(self.row_bytes)
        self.weights_physical_offsets, self.weights_size = layout(self.row_stride)
        if self.row_padding == "line":
            padded = [line_padded_row_stride(rb) for rb in self.row_bytes]
            offsets, total = layout(padded)
            if total <= ROW_PADDING_BUDGET_BYTES:
                self.row_stride, self.weights_physical_offsets, self.weights_size = padded, offsets, total
        self._plans: Dict[Optional[Tuple[int, ...]], ctypes.c_void_p] = {}
        self._plan_address: Dict[Optional[Tuple[int, ...]], int] = {}  # the same handles as integers
        self._identity_positions: Tuple[int, ...] = tuple(range(len(self.feature_table_map)))
        self._num_keys: Dict[Tuple[int, ...], int] = {}
        self._workspace: Dict[int, Tensor] = {}  # per stream: scratch of forward(offsets=None, lengths=...)
        self._ws_bytes: Dict[Tuple[int, int, int], int] = {}  # size of that scratch per (keys, batch size, id width)
        self._ws_ptr: Dict[Tuple[int, int, int, int], int] = {}  # its address per (keys, batch size, id width, stream)
        self._weights_initialized = False
        self.weight_initialized = False
        self.register_buffer("weights_dev", torch.empty(0, dtype=torch.uint8, device=device), persistent=False)
        if weight_lists is not None:
            self.initialize_weights()
            self.assign_embedding_weights(weight_lists)

    # -- storage ------------------------------------------------------------
    def initialize_weights(self) -> None:
        if not self._weights_initialized:
            self.weights_dev = torch.zeros(self.weights_size, dtype=torch.uint8, device=self.current_device)
            self._weights_initialized = True
            self.weight_initialized = True
            self._drop_plan()

    def _apply(self, fn, recurse: bool = True):  # type: ignore[no-untyped-def]
        """``.to()`` / ``.cuda()`` / ``.cpu()`` move the packed buffer; the device the
        operator launches on follows it, and plans made for the old device go."""
        super()._apply(fn, recurse)
        dev = self.weights_dev.device
        if dev.type == "cuda" and dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        if dev != self.current_device:
            self.current_device = dev
            self._drop_plan()
            self._workspace.clear()
            self._ws_ptr.clear()
        return self

    def _num_keys_of(self, positions: Tuple[int, ...]) -> int:
        """Smallest number of KJT keys that covers ``positions`` (remembered per placement)."""
        n = self._num_keys.get(positions)
        if n is None:
            n = self._num_keys[positions] = max(positions) + 1
        return n

    def _rows_view(self, t: int) -> Tensor:
        """Table ``t`` as ``[rows, row_bytes]`` bytes of the packed buffer (rows ``row_stride`` apart)."""
        off, r, rb, st = self.weights_physical_offsets[t], self.rows[t], self.row_bytes[t], self.row_stride[t]
        view = self.weights_dev.detach()[off : off + r * st].view(r, st)
        return view if st == rb else view[:, :rb]

    def split_embedding_weights_with_scale_bias(
        self, split_scale_bias_mode: int = 1
    ) -> List[Tuple[Tensor, Optional[Tensor], Optional[Tensor]]]:
        """Per-table views that alias the packed buffer.

        mode 0: ``(rows incl. header and padding, None, None)``;
        mode 1: ``(payload, scale_bias uint8 [rows, 4], None)``;
        mode 2: ``(payload, scale fp16 [rows, 1], bias fp16 [rows, 1])``.
        FP16 / FP32 tables have no header: ``(payload, None, None)``.
        """
        assert split_scale_bias_mode in (0, 1, 2)
        if not self._weights_initialized:
            self.initialize_weights()
        sb = self.scale_bias_size_in_bytes
        splits: List[Tuple[Tensor, Optional[Tensor], Optional[Tensor]]] = []
        for t, ty in enumerate(self.weight_tys):
            view = self._rows_view(t)
            if split_scale_bias_mode == 0:
                splits.append((view, None, None))
                continue
            view = view[:, : unpadded_row_size_in_bytes(self.dims[t], ty, sb)]
            if ty in (SparseType.INT8, SparseType.INT4, SparseType.INT2):
                if split_scale_bias_mode == 1:
                    splits.append((view[:, sb:], view[:, :sb], None))
                else:
                    splits.append(
                        (
                            view[:, sb:],
                            view[:, : sb // 2].view(torch.float16),
                            view[:, sb // 2 : sb].view(torch.float16),
                        )
                    )
            else:
                splits.append((view, None, None))
        return splits

    def split_embedding_weights(self, split_scale_shifts: bool = True) -> List[Tuple[Tensor, Optional[Tensor]]]:
        mode = 1 if split_scale_shifts else 0
        return [(w, s) for (w, s, _) in self.split_embedding_weights_with_scale_bias(mode)]

    def assign_embedding_weights(self, q_weight_list: List[Tuple[Tensor, Optional[Tensor]]]) -> None:
        """Copy ``(payload, scale_bias)`` per table into the packed buffer."""
        if not self._weights_initialized:
            self.initialize_weights()
        dest = self.split_embedding_weights(split_scale_shifts=True)
        assert len(q_weight_list) == len(dest), "one (weight, scale_shift) pair per table"
        if self.current_device.type == "meta":
            return
        for (dw, ds), (sw, ss) in zip(dest, q_weight_list):
            sw = sw.view(torch.uint8) if sw.dtype != torch.uint8 else sw
            assert dw.shape == sw.shape, f"weight shape {tuple(sw.shape)} != table shape {tuple(dw.shape)}"
            dw.copy_(sw)
            if ds is not None:
                assert ss is not None, "quantized tables need a scale_shift tensor"
                ss = ss.view(torch.uint8) if ss.dtype != torch.uint8 else ss
                ds.copy_(ss.reshape(ds.shape))

    # -- lookup -----------------------------------------------------------------
    def _drop_plan(self) -> None:
        plans = getattr(self, "_plans", None)
        if plans:
            for plan in plans.values():
                try:
                    _lib.lib().tra_tbe_destroy(plan)
                except Exception:  # interpreter shutdown
                    pass
            plans.clear()
        addresses = getattr(self, "_plan_address", None)
        if addresses:
            addresses.clear()

    def __del__(self) -> None:
        self._drop_plan()

    def __getstate__(self):  # type: ignore[no-untyped-def]
        """Copies (``copy.deepcopy``) and pickles carry the packed buffer and the
        configuration; launch plans and scratch buffers belong to this object
        and are made again on the copy's first lookup."""
        state = self.__dict__.copy()
        state["_plans"] = {}
        state["_plan_address"] = {}
        state["_workspace"] = {}
        state["_ws_ptr"] = {}
        return state

    def _get_plan(self, feature_positions: Optional[Tuple[int, ...]] = None) -> ctypes.c_void_p:
        """Launch plan for one placement of the features among the input keys
        (None: feature f is the f-th key).  Plans are cached per placement."""
        plan = self._plans.get(feature_positions)
        if plan is None:
            T_ = len(self.embedding_specs)
            specs = (_lib.TableSpec * max(T_, 1))()
            for t in range(T_):
                specs[t].offset = self.weights_physical_offsets[t]
                specs[t].rows = self.rows[t]
                specs[t].dim = self.dims[t]
                specs[t].dtype = self.weight_tys[t].as_int()
                specs[t].row_bytes = self.row_stride[t]
            F = len(self.feature_table_map)
            ftm = (ctypes.c_int32 * max(F, 1))(*self.feature_table_map)
            pos = None
            if feature_positions is not None:
                assert len(feature_positions) == F, "one position per feature"
                pos = (ctypes.c_int32 * max(F, 1))(*feature_positions)
            plan = ctypes.c_void_p()
            with torch.cuda.device(self.current_device):
                _lib.check(_lib.lib().tra_tbe_create(specs, T_, ftm, pos, F, ctypes.byref(plan)))
            if self.bounds_check_mode_int >= 0:
                _lib.check(_lib.lib().tra_tbe_set_bounds_check_mode(plan, self.bounds_check_mode_int))
            self._plans[feature_positions] = plan
        return plan

    def forward(
        self,
        indices: Tensor,
        offsets: Tensor,
        per_sample_weights: Optional[Tensor] = None,
        feature_positions: Optional[Sequence[int]] = None,
        batch_size: Optional[int] = None,
        out: Optional[Tensor] = None,
        out_col: int = 0,
        lengths: Optional[Tensor] = None,
        position_weights: Optional[Tuple[Tensor, Sequence[int], Sequence[int]]] = None,
    ) -> Tensor:
        """Pooled: ``[B, total_D]``; ``PoolingMode.NONE``: ``[indices.numel(), D]``.

        The first three arguments are the reference operator's.  The others let
        a caller look up straight from a KeyedJaggedTensor whose keys are in a
        different order (or a superset): ``feature_positions[f]`` is the index
        of feature ``f`` among the KJT keys, so its bags are
        ``offsets[feature_positions[f] * B + b]`` with ``B = batch_size``;
        ``out`` / ``out_col`` make the operator write into columns
        ``out_col ..`` of a caller-owned ``[B, >= out_col + total_D]`` tensor
        (``[L, D]`` for PoolingMode.NONE).  With ``offsets=None`` and
        ``lengths`` (the KJT's ``[K * B]`` lengths, ``batch_size`` required) the
        operator derives the offsets itself, inside the lookup kernel when the
        call is large enough for that to pay.  ``position_weights`` =
        ``(table, key_start, key_len)`` replaces ``per_sample_weights`` by
        weights looked up inside the kernel: the id at position ``k`` of a bag
        of input key ``p`` gets ``table[key_start[p] + min(k, key_len[p] - 1)]``
        (1 when ``key_len[p]`` is 0); ``table`` is one fp32 device tensor.
        """
        dev = self.current_device
        if dev.type != "cuda":
            raise _lib.TorchrecAmdError(
                f"IntNBitTableBatchedEmbeddingBagsCodegen.forward on device {dev}: "
                "the lookup runs on an MI355X GPU only"
            )
        if not self._weights_initialized:
            raise _lib.TorchrecAmdError("weights are not initialized (call initialize_weights())")
        if self.weights_dev.device != dev:  # e.g. the buffer was replaced by hand
            raise _lib.TorchrecAmdError(f"packed weights are on {self.weights_dev.device}, the operator on {dev}")
        idt = indices.dtype
        if not indices.is_cuda:
            _lib.require_gpu(indices, "indices")
        if idt not in _INT_DTYPES:
            raise TypeError(f"indices must be int32 or int64, got {idt}")
        if not indices.is_contiguous():
            indices = indices.contiguous()
        if offsets is None:
            assert lengths is not None and batch_size is not None, "offsets=None needs lengths and batch_size"
            if not lengths.is_cuda:
                _lib.require_gpu(lengths, "lengths")
            if lengths.dtype != idt:
                lengths = lengths.to(idt)
            if lengths.dim() != 1 or not lengths.is_contiguous():
                lengths = lengths.contiguous().view(-1)
        else:
            if not offsets.is_cuda:
                _lib.require_gpu(offsets, "offsets")
            if offsets.dtype != idt:
                offsets = offsets.to(idt)
            if not offsets.is_contiguous():
                offsets = offsets.contiguous()
        F = len(self.feature_table_map)
        positions: Optional[Tuple[int, ...]] = None
        if feature_positions is not None:
            positions = (
                feature_positions if type(feature_positions) is tuple else tuple(int(p) for p in feature_positions)
            )
            if positions == self._identity_positions:
                positions = None
        if batch_size is None:
            assert positions is None, "batch_size is required with feature_positions"
            assert F > 0 and (offsets.numel() - 1) % F == 0, "offsets must have F * B + 1 entries"
            batch_size = (offsets.numel() - 1) // F
        B = int(batch_size)
        n_keys = F if positions is None else self._num_keys_of(positions)
        if offsets is None:
            assert B == 0 or lengths.numel() % B == 0, "lengths must have K * B entries"
            k_total = lengths.numel() // B if B else n_keys
            assert k_total >= n_keys, "lengths shorter than the features it must cover"
        else:
            assert offsets.numel() >= n_keys * B + 1, "offsets shorter than the features it must cover"
        L = indices.numel()
        out_dtype = torch.float16 if self.output_dtype == _lib.FP16 else torch.float32
        nobag = self.pooling_mode == PoolingMode.NONE
        psw = None
        pos_args = None
        if position_weights is not None:
            assert not nobag, "position weights apply to pooled lookups"
            assert per_sample_weights is None, "position weights take the place of per_sample_weights"
            table, key_start, key_len = position_weights
            _lib.require_gpu(table, "position weight table")
            assert table.dtype == torch.float32 and table.is_contiguous() and table.numel() >= 1
            n_k = len(key_start)
            assert len(key_len) == n_k >= n_keys, "one (start, length) pair per input key"
            pos_args = (
                table, (ctypes.c_int32 * max(n_k, 1))(*key_start), (ctypes.c_int32 * max(n_k, 1))(*key_len), n_k
            )
        if per_sample_weights is not None and not nobag:
            psw = per_sample_weights.contiguous()
            if psw.dtype != torch.float32:
                psw = psw.float()
            assert psw.numel() == L, "per_sample_weights must have one entry per index"
        if out is None:
            shape = (L, self.max_D) if nobag else (B, self.total_D)
            out = torch.empty(shape, dtype=out_dtype, device=dev)
            out_col = 0
        else:
            assert out.dtype == out_dtype and out.device == dev and out.dim() == 2 and out.stride(1) == 1
            if nobag:
                assert out_col == 0 and out.shape[0] >= L and out.shape[1] == self.max_D
            else:
                assert out.shape[0] >= B and out.shape[1] >= out_col + self.total_D
        out_stride = out.stride(0)
        out_ptr = out.data_ptr() + out_col * out.element_size()
        i64 = int(idt == torch.int64)
        if pos_args is not None:
            table, c_start, c_len, n_k = pos_args
            stream = _lib.current_stream(dev)
            ws_ptr = None
            if offsets is None:
                assert k_total == n_k, "one (start, length) pair per key of the lengths"
                ws_ptr = self._scratch_address(k_total, B, i64, stream)
            _lib.check(
                _lib.lib().tra_tbe_forward_position_weighted(
                    self._get_plan(positions), _lib.ptr(self.weights_dev), _lib.ptr(indices),
                    _lib.ptr(lengths if offsets is None else offsets), int(offsets is None), i64,
                    _lib.ptr(table), table.numel(), c_start, c_len, n_k, B, L, int(self.pooling_mode),
                    self.output_dtype, out_ptr, out_stride, ws_ptr, stream,
                )
            )
        elif offsets is None:
            self._launch_from_lengths(positions, indices, lengths, i64, psw, B, k_total, L, out_ptr, out_stride)
            return out
        else:
            _lib.check(
                _lib.lib().tra_tbe_forward(
                    self._get_plan(positions), _lib.ptr(self.weights_dev), _lib.ptr(indices), _lib.ptr(offsets),
                    i64, _lib.ptr(psw), B, L, int(self.pooling_mode),
                    self.output_dtype, out_ptr, out_stride, _lib.current_stream(dev),
                )
            )
        if _ENV_BOUNDS_CHECK or self.bounds_check_mode_int == _BOUNDS_FATAL:
            bad = self.out_of_range_count()
            if bad:
                raise IndexError(f"{bad} embedding indices were out of range")
        return out

    def _scratch_address(self, k_total: int, B: int, i64: int, stream: int) -> int:
        """Device address of the lengths entry points' scratch for this call shape on this stream
        (one buffer per stream: calls queued on different streams must not share it).  A shape seen
        before costs one dictionary lookup."""
        ws_key = (k_total, B, i64, stream)
        ws_ptr = self._ws_ptr.get(ws_key)
        if ws_ptr is None:
            dev = self.current_device
            ws_bytes = _lib.lib().tra_tbe_forward_lengths_workspace_bytes(k_total, B, i64)
            ws = self._workspace.get(stream)
            if ws is None or ws.numel() < ws_bytes or ws.device != dev:
                ws = self._workspace[stream] = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
                # a larger buffer replaced the stream's old one: forget the addresses handed out from it
                for k in [k for k in self._ws_ptr if k[3] == stream]:
                    del self._ws_ptr[k]
            ws_ptr = self._ws_ptr[ws_key] = ws.data_ptr()
        return ws_ptr

    def _launch_from_lengths(
        self,
        positions: Optional[Tuple[int, ...]],
        indices: Tensor,
        lengths: Tensor,
        i64: int,
        psw: Optional[Tensor],
        B: int,
        k_total: int,
        L: int,
        out_ptr: int,
        out_stride: int,
    ) -> None:
        """The launch of ``forward(offsets=None, lengths=...)``.  The caller has checked the arguments:
        contiguous device tensors on this operator's GPU, ``lengths`` of the ids' type with ``k_total * B``
        entries, ``psw`` fp32 or None."""
        stream = _lib.current_stream(self.current_device)
        ws_ptr = self._scratch_address(k_total, B, i64, stream)
        global _FORWARD_LENGTHS
        fn = _FORWARD_LENGTHS
        if fn is None:
            fn = _FORWARD_LENGTHS = _lib.forward_lengths_entry()
        # (fn takes the plan's address as an integer: the extension module reads plain ints)
        plan = self._plan_address.get(positions)
        if plan is None:
            plan = self._plan_address[positions] = self._get_plan(positions).value
        rc = fn(
            plan, self._buffers["weights_dev"].data_ptr(), indices.data_ptr(),
            lengths.data_ptr(), i64, None if psw is None else psw.data_ptr(), B, k_total, L,
            int(self.pooling_mode), self.output_dtype, out_ptr, out_stride, ws_ptr, stream,
        )
        if rc != 0:
            _lib.check(rc)
        if _ENV_BOUNDS_CHECK or self.bounds_check_mode_int == _BOUNDS_FATAL:
            bad = self.out_of_range_count()
            if bad:
                raise IndexError(f"{bad} embedding indices were out of range")

    def out_of_range_count(self) -> int:
        """Ids outside [0, rows) (other than -1) seen since the last call.  Synchronizes."""
        total = 0
        for plan in self._plans.values():
            n = ctypes.c_int64(0)
            _lib.check(
                _lib.lib().tra_tbe_error_count(plan, _lib.current_stream(self.current_device), ctypes.byref(n))
            )
            total += int(n.value)
        return total

    def extra_repr(self) -> str:
        return (
            f"tables={len(self.embedding_specs)}, features={len(self.feature_table_map)}, "
            f"pooling={self.pooling_mode.name}, bytes={self.weights_size}, row_alignment={self.row_alignment}, "
            f"row_padding={self.row_padding}"
        )
