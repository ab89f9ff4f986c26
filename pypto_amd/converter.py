"""``from_torch``: the tensor hand-over of the reference's legacy jit front end.

Reference: python/pypto/converter.py:35-112.  There the call returns a ``pypto.Tensor`` carrying
shape (with dynamic axes marked), dtype, name, data pointer, format and device.  Here the kernels
are pre-compiled and every shape is a launch argument, so ``dynamic_axis`` and ``tensor_format``
carry no information; the wrapper keeps the torch tensor and exposes the same attributes.
The error behaviour is the reference's: ``TypeError`` for anything that is not a torch tensor,
``RuntimeError`` for a non-contiguous one (converter.py:76-80).
"""
from __future__ import annotations

from typing import List, Optional

import torch


class Tensor:
    """Thin handle on a contiguous torch tensor (device memory stays owned by the caller)."""

    __slots__ = ("_t", "name", "dynamic_axis", "format")

    def __init__(self, t: torch.Tensor, name: str = "", dynamic_axis: Optional[List[int]] = None, fmt=None):
        self._t = t
        self.name = name
        self.dynamic_axis = list(dynamic_axis) if dynamic_axis is not None else None
        self.format = fmt

    @property
    def shape(self):
        return list(self._t.shape) if self._t.dim() else [1]

    @property
    def ori_shape(self):
        return list(self._t.shape)

    @property
    def dtype(self):
        return self._t.dtype

    @property
    def device(self):
        return self._t.device

    @property
    def data_ptr(self):
        return self._t.data_ptr()

    def torch(self) -> torch.Tensor:
        return self._t

    def __repr__(self):
        return f"pypto_amd.Tensor(name={self.name!r}, shape={self.shape}, dtype={self.dtype}, device={self.device})"


def from_torch(tensor, name: str = "", dynamic_axis: Optional[List[int]] = None, tensor_format=None) -> Tensor:
    if not isinstance(tensor, torch.Tensor):
        raise TypeError("input type is not currently supported.")
    if not tensor.is_contiguous():
        raise RuntimeError("not all tensors are contiguous")
    return Tensor(tensor, name, dynamic_axis, tensor_format)


def as_torch(x, what: str) -> torch.Tensor:
    """Operator-side unwrapping: accepts the wrapper or a bare torch tensor."""
    if isinstance(x, Tensor):
        return x.torch()
    if isinstance(x, torch.Tensor):
        if not x.is_contiguous():
            raise RuntimeError(f"{what}: not all tensors are contiguous")
        return x
    raise TypeError(f"{what}: input type is not currently supported.")


def copy_unless_same(dst: torch.Tensor, src: torch.Tensor, what: str) -> None:
    """The cache-out arguments of the prolog operators: normally the very tensor passed as cache-in (the
    kernels then update the rows named by the cache index in place and nothing is copied).  A different
    tensor receives a copy of the whole cache first -- the reference's semantics, and gigabytes per call at
    real cache sizes, so in-place use is the intended path.  Two views that share memory without being the
    same range would be copied onto themselves: refused."""
    if dst.data_ptr() == src.data_ptr():
        return
    lo_d, lo_s = dst.data_ptr(), src.data_ptr()
    hi_d, hi_s = lo_d + dst.numel() * dst.element_size(), lo_s + src.numel() * src.element_size()
    if lo_d < hi_s and lo_s < hi_d:
        raise ValueError(f"{what} and {what}_out overlap in memory without being the same tensor")
    dst.copy_(src.reshape(dst.shape))
