"""uint8-backed tensors whose logical elements are 4 or 2 bits wide.

The quantized modules register int4 / int2 table payloads in their
``state_dict`` through these wrappers so the reported shape is
``[rows, embedding_dim]`` rather than the packed byte shape.  Behaviour follows
torchrec/tensor_types.py:61-176: ``.view(torch.uint8)`` returns the packed
bytes, slicing / ``view`` / ``select`` work in logical elements (the last
dimension must stay byte aligned), ``detach`` / ``clone`` / ``copy_`` /
``to(device)`` act on the bytes.
"""
from __future__ import annotations

import itertools
from typing import Any, Callable, Dict, List, Tuple

import torch

aten = torch.ops.aten


def down_size(n: int, size: torch.Size) -> Tuple[int, ...]:
    assert size[-1] % n == 0, f"{size} last dim not divisible by {n}"
    return (*size[:-1], size[-1] // n)


def up_size(n: int, size: torch.Size) -> Tuple[int, ...]:
    return (*size[:-1], size[-1] * n)


def _first_of_type(values, ty):
    for v in values:
        if isinstance(v, ty):
            return v
    return None


class UIntXTensor(torch.Tensor):
    """N logical elements per byte; dtype reported as uint8."""

    __torch_function__ = torch._C._disabled_torch_function_impl

    @staticmethod
    def __new__(cls, N: int, elem: torch.Tensor):
        assert elem.dtype is torch.uint8
        return torch.Tensor._make_wrapper_subclass(
            cls, up_size(N, elem.shape), dtype=torch.uint8, device=elem.device
        )

    def __init__(self, N: int, elem: torch.Tensor) -> None:
        self.N: int = N
        self.elem: torch.Tensor = elem

    def tolist(self) -> List:
        return self.elem.tolist()

    def __repr__(self) -> str:
        return f"UInt{8 // self.N}Tensor(shape={self.shape}, elem={self.elem})"

    # -- dispatch handlers ---------------------------------------------------
    @classmethod
    def _detach(cls, args, kwargs):
        (self,) = args
        with torch.inference_mode(False):
            return cls(aten.detach.default(self.elem))

    @classmethod
    def _clone(cls, args, kwargs):
        return cls(aten.clone.default(args[0].elem))

    @classmethod
    def _copy_(cls, args, kwargs):
        dst, src = args[0], args[1]
        dst.elem.copy_(src.elem if isinstance(src, UIntXTensor) else src)
        return dst

    @classmethod
    def _view_dtype(cls, args, kwargs):
        self, dtype = args
        if dtype != torch.uint8:
            raise NotImplementedError(f"view(dtype={dtype})")
        return self.elem

    @classmethod
    def _to_copy(cls, args, kwargs):
        self = args[0]
        everything = itertools.chain(args, (kwargs or {}).values())
        everything = list(everything)
        dtype = _first_of_type(everything, torch.dtype)
        device = _first_of_type(everything, torch.device)
        if device is None:
            raise NotImplementedError("_to_copy without a device")
        assert dtype is None or dtype == torch.uint8
        return cls(self.elem.to(device))

    @classmethod
    def _slice(cls, args, kwargs):
        self = args[0]
        dim = args[1] if len(args) > 1 else 0
        start = args[2] if len(args) > 2 else None
        end = args[3] if len(args) > 3 else None
        step = args[4] if len(args) > 4 else 1
        if dim < 0:
            dim += self.dim()
        if dim != self.dim() - 1:
            return cls(aten.slice.Tensor(self.elem, dim, start, end, step))
        if step != 1:
            raise NotImplementedError(f"slice step={step}")
        start = 0 if start is None else start
        end = self.shape[dim] if end is None else end
        assert start % self.N == 0, start
        assert end >= self.shape[dim] or end % self.N == 0, end
        return cls(aten.slice.Tensor(self.elem, dim, start // self.N, end // self.N, 1))

    @classmethod
    def _view(cls, args, kwargs):
        self, size = args
        size = torch._prims_common.infer_size(size, self.numel())
        return cls(self.elem.reshape(down_size(self.N, size)))

    @classmethod
    def _select(cls, args, kwargs):
        self, dim, index = args
        if dim < 0:
            dim += self.dim()
        if dim == self.dim() - 1:
            raise NotImplementedError(f"select dim={dim}")
        return cls(aten.select.int(self.elem, dim, index))

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs=None):
        handlers: Dict[Any, Callable] = {
            aten.detach.default: cls._detach,
            aten.clone.default: cls._clone,
            aten.copy_.default: cls._copy_,
            aten.view.dtype: cls._view_dtype,
            aten._to_copy.default: cls._to_copy,
            aten.slice.Tensor: cls._slice,
            aten.view.default: cls._view,
            aten.select.int: cls._select,
        }
        h = handlers.get(func)
        if h is None:
            raise NotImplementedError(f"{func} args:{args} kwargs:{kwargs}")
        return h(args, kwargs)


class UInt4Tensor(UIntXTensor):
    N: int = 2

    @staticmethod
    def __new__(cls, elem: torch.Tensor):
        return UIntXTensor.__new__(cls, cls.N, elem)

    def __init__(self, elem: torch.Tensor) -> None:
        super().__init__(UInt4Tensor.N, elem)


class UInt2Tensor(UIntXTensor):
    N: int = 4

    @staticmethod
    def __new__(cls, elem: torch.Tensor):
        return UIntXTensor.__new__(cls, cls.N, elem)

    def __init__(self, elem: torch.Tensor) -> None:
        super().__init__(UInt2Tensor.N, elem)
