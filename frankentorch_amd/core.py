"""Boundary types mirrored from `ft-core`: DType, Device (with the HIP id the backend adds),
TensorMeta, and the error carriers `KernelError` / `HipError`.

TensorMeta follows crates/ft-core/src/lib.rs:340-420 (shape, strides in elements, storage_offset,
dtype, device; `from_shape` builds contiguous strides). KernelError follows
crates/ft-kernel-cpu/src/lib.rs:1697-1733; HipError follows ft_kernel_metal::Error
(crates/ft-kernel-metal/src/lib.rs:60-77).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from enum import IntEnum
from typing import Sequence

from . import _lib


class DType(IntEnum):
    F64 = 0
    F32 = 1


class Device(IntEnum):
    Cpu = 0
    Cuda = 1
    Hip = 2


def contiguous_strides(shape: Sequence[int]) -> list[int]:
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * int(shape[i + 1])
    return strides


@dataclass
class TensorMeta:
    shape: list[int]
    strides: list[int] = field(default_factory=list)
    storage_offset: int = 0
    dtype: DType = DType.F32
    device: Device = Device.Cpu

    @classmethod
    def from_shape(cls, shape, dtype: DType = DType.F32, device: Device = Device.Cpu) -> "TensorMeta":
        shape = [int(s) for s in shape]
        return cls(shape, contiguous_strides(shape), 0, dtype, device)

    @classmethod
    def from_shape_and_strides(cls, shape, strides, storage_offset, dtype: DType = DType.F32,
                               device: Device = Device.Cpu) -> "TensorMeta":
        return cls([int(s) for s in shape], [int(s) for s in strides], int(storage_offset), dtype, device)

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def to_c(self) -> _lib.Meta:
        if len(self.shape) > _lib.MAX_DIMS or len(self.shape) != len(self.strides):
            raise ValueError("TensorMeta rank %d not representable (max %d)" % (len(self.shape), _lib.MAX_DIMS))
        m = _lib.Meta()
        m.ndim = len(self.shape)
        m.dtype = int(self.dtype)
        m.device = int(self.device)
        for i, (s, st) in enumerate(zip(self.shape, self.strides)):
            m.shape[i] = s
            m.strides[i] = st
        m.storage_offset = self.storage_offset
        return m


class KernelError(Exception):
    """`KernelError` of the reference; `.kind` is the variant name, payload fields as attributes."""

    KINDS = {
        1: "Incompatible(DTypeMismatch)",
        2: "Incompatible(DeviceMismatch)",
        3: "ShapeMismatch",
        4: "UnsupportedLayout",
        5: "StorageSpanOverflow",
        6: "InsufficientStorage",
        7: "InvalidDimension",
        8: "ShapeOverflow",
        9: "EmptyReductionDim",
    }

    def __init__(self, code: int, info: _lib.ErrorInfo):
        self.code = code
        self.kind = self.KINDS.get(code, "Unknown")
        self.side = info.side.decode()
        self.lhs = list(info.lhs_shape[: info.lhs_ndim])
        self.rhs = list(info.rhs_shape[: info.rhs_ndim])
        self.a = int(info.a)
        self.b = int(info.b)
        self.message = info.message.decode(errors="replace")
        super().__init__("%s: %s" % (self.kind, self.message))

    # Named views of the payload, as the reference's variants spell them.
    @property
    def dim(self):
        return self.a

    @property
    def ndim(self):
        return self.b

    @property
    def needed(self):
        return self.a

    @property
    def available(self):
        return self.b


class HipError(Exception):
    """Backend failure: Unavailable | Kernel | SizeOverflow | BufferTooLarge | CommandBuffer | ..."""

    def __init__(self, code: int, info: _lib.ErrorInfo):
        self.code = code
        self.kind = _lib.load().fth_status_name(code).decode()
        self.message = info.message.decode(errors="replace")
        super().__init__("%s: %s" % (self.kind, self.message))


def check(rc: int) -> None:
    """Raises the exception that corresponds to a non-zero status."""
    if rc == 0:
        return
    info = _lib.last_error()
    if 1 <= rc <= 9:
        raise KernelError(rc, info)
    raise HipError(rc, info)
