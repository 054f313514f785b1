"""ctypes binding of libft_kernel_hip.so.

Prototypes are read from include/ft_kernel_hip.h at import time, so the Python side can never
drift from the C ABI: every declared function gets its argtypes/restype from its declaration.
There is no fallback: if the shared library is missing, loading raises with the build command.
"""
from __future__ import annotations

import ctypes as C
import os
import re

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
HEADER = os.path.join(REPO_ROOT, "include", "ft_kernel_hip.h")
LIB_PATH = os.path.join(PKG_DIR, "libft_kernel_hip.so")

MAX_DIMS = 8


class Meta(C.Structure):
    """fth_meta: the flattened TensorMeta."""

    _fields_ = [
        ("ndim", C.c_int32),
        ("dtype", C.c_int32),
        ("device", C.c_int32),
        ("reserved", C.c_int32),
        ("shape", C.c_uint64 * MAX_DIMS),
        ("strides", C.c_uint64 * MAX_DIMS),
        ("storage_offset", C.c_uint64),
    ]


class ErrorInfo(C.Structure):
    _fields_ = [
        ("code", C.c_int32),
        ("lhs_ndim", C.c_int32),
        ("rhs_ndim", C.c_int32),
        ("reserved", C.c_int32),
        ("lhs_shape", C.c_uint64 * MAX_DIMS),
        ("rhs_shape", C.c_uint64 * MAX_DIMS),
        ("a", C.c_uint64),
        ("b", C.c_uint64),
        ("side", C.c_char * 16),
        ("message", C.c_char * 200),
    ]


class GemmDesc(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("m", "n", "k", "lda", "ldb", "ldc", "batch", "stride_a", "stride_b", "stride_c")] + [
        ("trans_b", C.c_int32),
        ("epilogue", C.c_int32),
        ("trans_a", C.c_int32),
        ("reserved", C.c_int32),
    ]


class SdpaDesc(C.Structure):
    _fields_ = [
        (n, C.c_int64)
        for n in (
            "num_bh", "heads", "seq_q", "seq_k", "d_k", "d_v",
            "q_batch_stride", "q_head_stride", "q_row_stride",
            "k_batch_stride", "k_head_stride", "k_row_stride",
            "v_batch_stride", "v_head_stride", "v_row_stride",
            "o_batch_stride", "o_head_stride", "o_row_stride",
        )
    ] + [("causal", C.c_int32), ("kv_group", C.c_int32)]


class LayerWeights(C.Structure):
    _fields_ = [
        (n, C.c_void_p)
        for n in ("ln1_w", "ln1_b", "wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "ln2_w", "ln2_b", "w1", "b1", "w2", "b2")
    ]


_SCALARS = {
    "int8_t": C.c_int8,
    "int32_t": C.c_int32,
    "int64_t": C.c_int64,
    "uint64_t": C.c_uint64,
    "size_t": C.c_size_t,
    "float": C.c_float,
    "double": C.c_double,
    "fth_stream": C.c_void_p,
    "fth_event": C.c_void_p,
}


def _ctype_of(decl: str):
    decl = decl.replace("const", " ").strip()
    if "*" in decl:
        if re.match(r"^\s*char\s*\*", decl):
            return C.c_char_p
        return C.c_void_p
    base = decl.split()[0]
    if base not in _SCALARS:
        raise ValueError("unknown C type in header: %r" % decl)
    return _SCALARS[base]


def parse_header(path: str = HEADER):
    """Returns {name: (restype, [argtypes])} for every function the header declares."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(fth_\w+)\s*\(([^;{}()]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        if ret.startswith("typedef") or not ret:
            continue
        if ret == "void":
            restype = None
        elif "*" in ret:
            restype = C.c_char_p if "char" in ret else C.c_void_p
        else:
            restype = _SCALARS[ret.replace("const", "").split()[0]]
        argtypes = []
        if args and args != "void":
            for a in args.split(","):
                argtypes.append(_ctype_of(a))
        protos[name] = (restype, argtypes)
    return protos


_lib = None
_protos = None


def protos():
    global _protos
    if _protos is None:
        _protos = parse_header()
    return _protos


def load() -> C.CDLL:
    """Loads the HIP library. Raises if it has not been built: there is no other code path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing. Build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950). This package has no CPU fallback." % LIB_PATH
        )
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in protos().items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error() -> ErrorInfo:
    info = ErrorInfo()
    load().fth_last_error(C.byref(info))
    return info
