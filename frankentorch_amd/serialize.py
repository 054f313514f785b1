"""Host-side mirror of the loading surface of `ft-serialize`: the safetensors functions
(crates/ft-serialize/src/lib.rs:2170-2286: `load_safetensors`, `load_safetensors_from_bytes`,
`load_safetensors_metadata`) and the native state-dict ones (:996-1160: `load_state_dict`,
`load_state_dict_from_bytes`), over the C ABI's memory-mapped reader. The device-side path
(`SafeTensorsFile.read_dev`, `fused.Gpt2Hip.from_safetensors`) moves tensors straight into resident
buffers instead of building host tensors first.

Errors: `core.HipError` with kind "Corrupt" where the reference returns TensorIOError::Corrupt,
"Io" for TensorIOError::Io, "InvalidMagic" and "UnsupportedVersion" for the native container's
two header variants.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional

import numpy as np

from . import _lib
from .core import check

DTYPE_F64, DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2, 3
DTYPE_NAMES = {DTYPE_F64: "F64", DTYPE_F32: "F32", DTYPE_F16: "F16", DTYPE_BF16: "BF16"}
# BF16 has no numpy type: its tensors come back as uint16 bit patterns (`bf16_to_f32` widens them).
_NUMPY = {DTYPE_F64: np.float64, DTYPE_F32: np.float32, DTYPE_F16: np.float16, DTYPE_BF16: np.uint16}


class TensorInfo(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("ndim", C.c_int32), ("shape", C.c_uint64 * _lib.MAX_DIMS), ("numel", C.c_uint64),
                ("byte_len", C.c_uint64)]


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


class SafeTensorsFile:
    """An open, validated safetensors container (a path, or bytes that stay referenced)."""

    _OPEN, _OPEN_BYTES = "fth_safetensors_open", "fth_safetensors_open_bytes"

    def __init__(self, source):
        h = C.c_void_p()
        lib = _lib.load()
        if isinstance(source, (bytes, bytearray, memoryview)):
            self._keep = bytes(source)
            check(getattr(lib, self._OPEN_BYTES)(self._keep, len(self._keep), C.byref(h)))
        else:
            self._keep = None
            check(getattr(lib, self._OPEN)(str(source).encode(), C.byref(h)))
        self._h = h.value

    def close(self) -> None:
        if self._h:
            _lib.load().fth_safetensors_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def names(self):
        lib = _lib.load()
        return [lib.fth_safetensors_name(self._h, i).decode() for i in range(lib.fth_safetensors_count(self._h))]

    def info(self, name: str):
        """(dtype code, shape tuple)."""
        t = TensorInfo()
        check(_lib.load().fth_safetensors_info(self._h, name.encode(), C.byref(t)))
        return t.dtype, tuple(int(t.shape[i]) for i in range(t.ndim))

    def read(self, name: str) -> np.ndarray:
        """The tensor as stored (F64 / F32 / F16 arrays; BF16 as uint16 bit patterns)."""
        dtype, shape = self.info(name)
        out = np.empty(shape, dtype=_NUMPY[dtype])
        check(_lib.load().fth_safetensors_read(self._h, name.encode(), out.ctypes.data, out.nbytes))
        return out

    def read_dev(self, name: str, dst, transpose: bool = False, stream=None) -> None:
        """Into a device buffer of f32 or f64 elements, converted (and transposed, for a matrix) on the GPU."""
        fn = _lib.load().fth_safetensors_read_f32_dev if dst.dtype == np.float32 else _lib.load().fth_safetensors_read_f64_dev
        check(fn(self._h, name.encode(), 1 if transpose else 0, dst.ptr, dst.size, stream))

    def metadata(self) -> Optional[Dict[str, str]]:
        """The "__metadata__" map, or None if the file has none. Keys are looked up one by one."""
        n = _lib.load().fth_safetensors_metadata_count(self._h)
        return None if n < 0 else _MetadataView(self, n)

    def metadata_value(self, key: str) -> Optional[str]:
        v = _lib.load().fth_safetensors_metadata(self._h, key.encode())
        return None if v is None else v.decode()


class _MetadataView:
    def __init__(self, f: SafeTensorsFile, n: int):
        self._f, self._n = f, n

    def __len__(self):
        return self._n

    def get(self, key, default=None):
        v = self._f.metadata_value(key)
        return default if v is None else v

    def __getitem__(self, key):
        v = self._f.metadata_value(key)
        if v is None:
            raise KeyError(key)
        return v

    def __contains__(self, key):
        return self._f.metadata_value(key) is not None


def load_safetensors_from_bytes(data) -> Dict[str, np.ndarray]:
    """crates/ft-serialize/src/lib.rs:2179: name -> tensor, in name order."""
    with SafeTensorsFile(data) as f:
        return {n: f.read(n) for n in f.names()}


def load_safetensors(path) -> Dict[str, np.ndarray]:
    """crates/ft-serialize/src/lib.rs:2170."""
    with SafeTensorsFile(path) as f:
        return {n: f.read(n) for n in f.names()}


def load_safetensors_metadata(path) -> Optional[Dict[str, str]]:
    """crates/ft-serialize/src/lib.rs:2274. Returns a plain dict only for the keys asked through `.get`; the container
    does not enumerate keys through the C ABI, so the view object is returned."""
    f = SafeTensorsFile(path)
    return f.metadata()


class StateDictFile(SafeTensorsFile):
    """An open, validated native state-dict container ("FTSV"). Same listing and read calls; no metadata map."""

    _OPEN, _OPEN_BYTES = "fth_statedict_open", "fth_statedict_open_bytes"


def load_state_dict_from_bytes(data) -> Dict[str, np.ndarray]:
    """crates/ft-serialize/src/lib.rs:1005: name -> tensor, in name order (BF16 tensors as uint16 bit patterns)."""
    with StateDictFile(data) as f:
        return {n: f.read(n) for n in f.names()}


def load_state_dict(path) -> Dict[str, np.ndarray]:
    """crates/ft-serialize/src/lib.rs:996."""
    with StateDictFile(path) as f:
        return {n: f.read(n) for n in f.names()}
