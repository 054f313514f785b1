"""numpy front end of the CPU checker (oracle/ft_oracle.cpp). TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py import this module.
Every function takes and returns C-contiguous numpy arrays and mirrors one `ft_kernel_cpu`
entry point (names and argument meaning follow the reference; see ft_oracle.cpp for file:line).
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libft_oracle.so")
_lib = None

_i64 = C.c_int64
_vp = C.c_void_p


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            import importlib.util

            spec = importlib.util.spec_from_file_location("build_oracle", os.path.join(_HERE, "build_oracle.py"))
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            mod.build_oracle()
        _lib = C.CDLL(_LIB_PATH)
        _lib.fto_threads.restype = C.c_int
        _lib.fto_index_select_f32.restype = _i64
        _lib.fto_index_select_f64.restype = _i64
        _lib.fto_gpt2_forward_f32.restype = _i64
        _lib.fto_sgemm_blocked.restype = C.c_int
    return _lib


def threads() -> int:
    return lib().fto_threads()


def set_threads(n: int) -> None:
    lib().fto_set_threads(C.c_int(n))


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _c(a, dtype=None):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype if dtype is not None else a.dtype)


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError("oracle computes f32 and f64 only, got %s" % dtype)


def softmax(x, dim: int = -1):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    dim = dim % x.ndim
    outer = int(np.prod(x.shape[:dim], dtype=np.int64))
    reduce = x.shape[dim]
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    y = np.empty_like(x)
    getattr(lib(), "fto_softmax_" + sfx)(_p(x), _p(y), _i64(outer), _i64(reduce), _i64(inner))
    return y


def layer_norm(x, weight, bias, eps):
    x = _c(x)
    sfx, ct = _sfx(x.dtype)
    batch, n = x.reshape(-1, x.shape[-1]).shape
    y = np.empty_like(x)
    getattr(lib(), "fto_layer_norm_" + sfx)(_p(x), _p(_c(weight)), _p(_c(bias)), _p(y), _i64(batch), _i64(n), ct(eps))
    return y


def add_layer_norm(a, b, weight, bias, eps):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    batch, n = a.reshape(-1, a.shape[-1]).shape
    y = np.empty_like(a)
    lib().fto_add_layer_norm_f32(_p(a), _p(b), _p(_c(weight)), _p(_c(bias)), _p(y), _i64(batch), _i64(n), C.c_float(eps))
    return y


def rms_norm(x, weight, eps):
    x = _c(x)
    sfx, ct = _sfx(x.dtype)
    batch, n = x.reshape(-1, x.shape[-1]).shape
    y = np.empty_like(x)
    getattr(lib(), "fto_rms_norm_" + sfx)(_p(x), _p(_c(weight)), _p(y), _i64(batch), _i64(n), ct(eps))
    return y


def gelu(x):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    y = np.empty_like(x)
    getattr(lib(), "fto_gelu_" + sfx)(_p(x), _p(y), _i64(x.size))
    return y


def gelu_tanh(x):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    y = np.empty_like(x)
    getattr(lib(), "fto_gelu_tanh_" + sfx)(_p(x), _p(y), _i64(x.size))
    return y


def add(a, b):
    a = _c(a)
    b = _c(b)
    sfx, _ = _sfx(a.dtype)
    y = np.empty_like(a)
    getattr(lib(), "fto_add_" + sfx)(_p(a), _p(b), _p(y), _i64(a.size))
    return y


def bias_add(x, bias, residual=None):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    rows, cols = x.reshape(-1, x.shape[-1]).shape
    y = np.empty_like(x)
    getattr(lib(), "fto_bias_add_" + sfx)(_p(x), _p(_c(bias)), _p(_c(residual)), _p(y), _i64(rows), _i64(cols))
    return y


def gemm(a, b, trans_b: bool = False):
    """a [m,k] . b ([k,n], or [n,k] when trans_b) -> [m,n]; wide accumulation, one rounding."""
    a = _c(a)
    b = _c(b)
    sfx, _ = _sfx(a.dtype)
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == k
    c = np.empty((m, n), dtype=a.dtype)
    getattr(lib(), "fto_gemm_" + sfx)(C.c_int(1 if trans_b else 0), _i64(m), _i64(n), _i64(k), _p(a), _i64(k), _p(b),
                                      _i64(b.shape[1]), _p(c), _i64(n))
    return c


def sgemm_blocked(a, b):
    """Timed stand-in for matrixmultiply's f32 kernel; returns None without AVX2/FMA."""
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), dtype=np.float32)
    ok = lib().fto_sgemm_blocked(_i64(m), _i64(n), _i64(k), _p(a), _i64(k), _p(b), _i64(n), _p(c), _i64(n))
    return c if ok else None


def bmm(a, b):
    a = _c(a)
    b = _c(b)
    sfx, _ = _sfx(a.dtype)
    batch, m, k = a.shape
    n = b.shape[2]
    c = np.empty((batch, m, n), dtype=a.dtype)
    getattr(lib(), "fto_bmm_" + sfx)(_i64(batch), _i64(m), _i64(n), _i64(k), _p(a), _p(b), _p(c))
    return c


def addmm(inp, mat1, mat2, beta, alpha):
    mat1 = _c(mat1)
    mat2 = _c(mat2)
    inp = _c(inp)
    sfx, ct = _sfx(mat1.dtype)
    m, k = mat1.shape
    n = mat2.shape[1]
    out = np.empty((m, n), dtype=mat1.dtype)
    getattr(lib(), "fto_addmm_" + sfx)(_p(inp), C.c_int(1 if inp.ndim == 1 else 0), _p(mat1), _p(mat2), _i64(m),
                                       _i64(n), _i64(k), ct(beta), ct(alpha), _p(out))
    return out


def linear(x, weight, bias=None):
    x = _c(x)
    weight = _c(weight)
    sfx, _ = _sfx(x.dtype)
    batch, in_f = x.shape
    out_f = weight.shape[0]
    y = np.empty((batch, out_f), dtype=x.dtype)
    getattr(lib(), "fto_linear_" + sfx)(_p(x), _p(weight), _p(_c(bias)), _i64(batch), _i64(in_f), _i64(out_f), _p(y))
    return y


def sdpa_forward(q, k, v, scale, causal):
    q = _c(q)
    k = _c(k)
    v = _c(v)
    sfx, ct = _sfx(q.dtype)
    num_bh, seq_q, d_k = q.shape
    seq_k = k.shape[1]
    d_v = v.shape[2]
    out = np.zeros((num_bh, seq_q, d_v), dtype=q.dtype)
    getattr(lib(), "fto_sdpa_forward_" + sfx)(_p(q), _p(k), _p(v), _i64(num_bh), _i64(seq_q), _i64(seq_k), _i64(d_k),
                                              _i64(d_v), ct(scale), C.c_int(1 if causal else 0), _p(out))
    return out


def sdpa_forward_masked_gqa(q, k, v, scale, mask):
    """q [batch, h_q, seq_q, d_k]; k, v [batch, h_kv, seq_k, d]; additive mask [seq_q, seq_k] (shared) or
    [batch * h_q, seq_q, seq_k] (crates/ft-kernel-cpu/src/lib.rs:4777-4850)."""
    q, k, v, mask = _c(q), _c(k), _c(v), _c(np.asarray(mask, dtype=q.dtype))
    sfx, ct = _sfx(q.dtype)
    batch, h_q, seq_q, d_k = q.shape
    h_kv, seq_k = k.shape[1], k.shape[2]
    d_v = v.shape[3]
    assert h_q % h_kv == 0 and mask.shape[-2:] == (seq_q, seq_k)
    stride = 0 if mask.ndim == 2 else seq_q * seq_k
    assert mask.ndim == 2 or mask.shape[0] == batch * h_q
    out = np.zeros((batch, h_q, seq_q, d_v), dtype=q.dtype)
    getattr(lib(), "fto_sdpa_forward_masked_gqa_" + sfx)(_p(q), _p(k), _p(v), _i64(batch), _i64(h_q), _i64(h_kv), _i64(seq_q),
                                                         _i64(seq_k), _i64(d_k), _i64(d_v), ct(scale), _p(mask), _i64(stride), _p(out))
    return out


def sdpa_forward_masked(q, k, v, scale, mask):
    """q, k, v [num_bh, seq, d]: the h_q == h_kv case (crates/ft-kernel-cpu/src/lib.rs:4661-4741)."""
    q, k, v = _c(q), _c(k), _c(v)
    return sdpa_forward_masked_gqa(q[None], k[None], v[None], scale, mask)[0]


def quantize_rows_i8(x):
    """Per-row symmetric int8 of a [rows, cols] f32 matrix -> (q int8, scales f32); also quantize_per_output_channel_i8."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    q, scales = np.empty((rows, cols), np.int8), np.empty(rows, np.float32)
    lib().fto_quantize_rows_i8(_p(x), _i64(rows), _i64(cols), _p(q), _p(scales))
    return q, scales


def linear_int8_dynamic(x, w_i8, w_scales, bias=None):
    x, w_i8, w_scales = _c(x, np.float32), _c(w_i8, np.int8), _c(w_scales, np.float32)
    m, k = x.shape
    n = w_i8.shape[0]
    out = np.empty((m, n), np.float32)
    lib().fto_linear_int8_dynamic_f32(_p(x), _i64(m), _i64(k), _p(w_i8), _p(w_scales), _i64(n), _p(_c(bias, np.float32)), _p(out))
    return out


def log_softmax(x, dim: int = -1):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    dim = dim % x.ndim
    outer = int(np.prod(x.shape[:dim], dtype=np.int64))
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    y = np.empty_like(x)
    getattr(lib(), "fto_log_softmax_" + sfx)(_p(x), _p(y), _i64(outer), _i64(x.shape[dim]), _i64(inner))
    return y


def cross_entropy_forward(logits, target):
    """Per-row loss lse(logits) - logits[target]; raises IndexError on a target outside [0, classes)."""
    logits = _c(logits)
    sfx, _ = _sfx(logits.dtype)
    batch, classes = logits.shape
    t = _c(np.asarray(target, dtype=np.int64))
    loss = np.empty(batch, logits.dtype)
    fn = getattr(lib(), "fto_cross_entropy_forward_" + sfx)
    fn.restype = C.c_int64
    bad = fn(_p(logits), _p(t), _i64(batch), _i64(classes), _p(loss))
    if bad >= 0:
        raise IndexError("target of row %d is out of range" % bad)
    return loss


def cross_entropy_backward(logits, target, dloss):
    logits, dloss = _c(logits), _c(dloss)
    sfx, _ = _sfx(logits.dtype)
    batch, classes = logits.shape
    t = _c(np.asarray(target, dtype=np.int64))
    out = np.empty_like(logits)
    fn = getattr(lib(), "fto_cross_entropy_backward_" + sfx)
    fn.restype = C.c_int64
    bad = fn(_p(logits), _p(t), _p(dloss), _i64(batch), _i64(classes), _p(out))
    if bad >= 0:
        raise IndexError("target of row %d is out of range" % bad)
    return out


def layer_norm_backward(dy, x, weight, eps):
    """Returns (dx, dweight, dbias) for y = layer_norm(x) * weight + bias over the last dim."""
    dy, x, weight = _c(dy), _c(x), _c(weight)
    sfx, ct = _sfx(x.dtype)
    batch, n = x.reshape(-1, x.shape[-1]).shape
    dx, dw, db = np.empty_like(x), np.empty(n, x.dtype), np.empty(n, x.dtype)
    getattr(lib(), "fto_layer_norm_backward_" + sfx)(_p(dy), _p(x), _p(weight), _i64(batch), _i64(n), ct(eps), _p(dx), _p(dw), _p(db))
    return dx, dw, db


def rms_norm_backward(dy, x, weight, eps):
    """Returns (dx, dweight or None)."""
    dy, x, weight = _c(dy), _c(x), _c(weight)
    sfx, ct = _sfx(x.dtype)
    batch, n = x.reshape(-1, x.shape[-1]).shape
    dx = np.empty_like(x)
    dw = None if weight is None else np.empty(n, x.dtype)
    getattr(lib(), "fto_rms_norm_backward_" + sfx)(_p(dy), _p(x), _p(weight), _i64(batch), _i64(n), ct(eps), _p(dx), _p(dw))
    return dx, dw


def linear_backward(dy, x, weight, need_bias=True):
    """Returns (dx, dweight, dbias or None) for y = x . weight^T + bias."""
    dy, x, weight = _c(dy), _c(x), _c(weight)
    sfx, _ = _sfx(x.dtype)
    batch, in_f = x.shape
    out_f = weight.shape[0]
    dx, dw = np.zeros((batch, in_f), x.dtype), np.zeros((out_f, in_f), x.dtype)
    db = np.zeros(out_f, x.dtype) if need_bias else None
    getattr(lib(), "fto_linear_backward_" + sfx)(_p(dy), _p(x), _p(weight), _i64(batch), _i64(in_f), _i64(out_f), _p(dx), _p(dw), _p(db))
    return dx, dw, db


def sdpa_backward(q, k, v, dout, scale, causal):
    """Returns (dq, dk, dv) for out = sdpa_forward(q, k, v, scale, causal)."""
    q, k, v, dout = _c(q), _c(k), _c(v), _c(dout)
    sfx, ct = _sfx(q.dtype)
    num_bh, seq_q, d_k = q.shape
    seq_k, d_v = k.shape[1], v.shape[2]
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    getattr(lib(), "fto_sdpa_backward_" + sfx)(_p(q), _p(k), _p(v), _p(dout), _i64(num_bh), _i64(seq_q), _i64(seq_k), _i64(d_k),
                                               _i64(d_v), ct(scale), C.c_int(1 if causal else 0), _p(dq), _p(dk), _p(dv))
    return dq, dk, dv


def sdpa_backward_unit_dout(q, k, v, scale, causal):
    """(dq, dk, dv) for dout = ones, without that tensor (crates/ft-kernel-cpu/src/lib.rs:5662-5770)."""
    q, k, v = _c(q), _c(k), _c(v)
    sfx, ct = _sfx(q.dtype)
    num_bh, seq_q, d_k = q.shape
    seq_k, d_v = k.shape[1], v.shape[2]
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    getattr(lib(), "fto_sdpa_backward_unit_dout_" + sfx)(_p(q), _p(k), _p(v), _i64(num_bh), _i64(seq_q), _i64(seq_k), _i64(d_k), _i64(d_v),
                                                         ct(scale), C.c_int(1 if causal else 0), _p(dq), _p(dk), _p(dv))
    return dq, dk, dv


def sdpa_backward_masked(q, k, v, dout, scale, mask, mask_bh_stride=None):
    """(dq, dk, dv) for out = sdpa_forward_masked(q, k, v, scale, mask); mask [seq_q, seq_k] shared (stride 0) or [num_bh, seq_q, seq_k]."""
    q, k, v, dout = _c(q), _c(k), _c(v), _c(dout)
    mask = _c(np.asarray(mask, dtype=q.dtype))
    sfx, ct = _sfx(q.dtype)
    num_bh, seq_q, d_k = q.shape
    seq_k, d_v = k.shape[1], v.shape[2]
    if mask_bh_stride is None:
        mask_bh_stride = 0 if mask.ndim == 2 else seq_q * seq_k
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    getattr(lib(), "fto_sdpa_backward_masked_" + sfx)(_p(q), _p(k), _p(v), _p(dout), _i64(num_bh), _i64(seq_q), _i64(seq_k), _i64(d_k),
                                                      _i64(d_v), ct(scale), _p(mask), _i64(mask_bh_stride), _p(dq), _p(dk), _p(dv))
    return dq, dk, dv


def index_select(x, dim, indices):
    """Returns (out, bad): bad is the position of the first invalid index, or -1."""
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    idx = _c(np.asarray(indices, dtype=np.float64))
    outer = int(np.prod(x.shape[:dim], dtype=np.int64))
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    out = np.zeros(x.shape[:dim] + (idx.size,) + x.shape[dim + 1:], dtype=x.dtype)
    bad = getattr(lib(), "fto_index_select_" + sfx)(_p(x), _i64(outer), _i64(x.shape[dim]), _i64(inner), _p(idx),
                                                    _i64(idx.size), _p(out))
    return out, int(bad)


def argmax(x, dim):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    dim = dim % x.ndim
    outer = int(np.prod(x.shape[:dim], dtype=np.int64))
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    out = np.empty(x.shape[:dim] + x.shape[dim + 1:], dtype=x.dtype)
    getattr(lib(), "fto_argmax_" + sfx)(_p(x), _i64(outer), _i64(x.shape[dim]), _i64(inner), _p(out))
    return out


def permute_0213(x):
    x = _c(x)
    sfx, _ = _sfx(x.dtype)
    d0, d1, d2, d3 = x.shape
    out = np.empty((d0, d2, d1, d3), dtype=x.dtype)
    getattr(lib(), "fto_permute_0213_" + sfx)(_p(x), _p(out), _i64(d0), _i64(d1), _i64(d2), _i64(d3))
    return out


LAYER_KEYS = ("ln1_w", "ln1_b", "wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "ln2_w", "ln2_b", "w1", "b1", "w2", "b2")


def _layer_ptrs(layers):
    keep = []
    arr = (_vp * (16 * len(layers)))()
    for li, lw in enumerate(layers):
        for ki, key in enumerate(LAYER_KEYS):
            a = _c(lw[key], np.float32)
            keep.append(a)
            arr[li * 16 + ki] = a.ctypes.data
    return arr, keep


def encoder_layer(layer, x, batch, seq, heads, eps, causal, gelu_tanh=False):
    """One pre-LN block on x [batch*seq, d_model]; returns a new array."""
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    d_model = x.shape[-1]
    d_ff = layer["w1"].shape[0]
    arr, keep = _layer_ptrs([layer])
    fn = lib().fto_encoder_layer_gelu_tanh_f32 if gelu_tanh else lib().fto_encoder_layer_f32
    fn(arr, _p(x), _i64(batch), _i64(seq), _i64(d_model), _i64(heads), _i64(d_ff), C.c_float(eps), C.c_int(1 if causal else 0))
    del keep
    return x


def gpt2_forward(wte, wpe, layers, lnf_w, lnf_b, ids, batch, seq, heads, eps, want_logits=True):
    """Returns dict(hidden, logits (or None), argmax, bad)."""
    wte = _c(wte, np.float32)
    wpe = _c(wpe, np.float32)
    vocab, d_model = wte.shape
    d_ff = layers[0]["w1"].shape[0]
    arr, keep = _layer_ptrs(layers)
    ids = _c(np.asarray(ids, dtype=np.float64).reshape(-1))
    tokens = batch * seq
    hidden = np.empty((tokens, d_model), dtype=np.float32)
    logits = np.empty((tokens, vocab), dtype=np.float32) if want_logits else None
    am = np.empty((tokens,), dtype=np.float32)
    bad = lib().fto_gpt2_forward_f32(_i64(vocab), _i64(wpe.shape[0]), _i64(d_model), _i64(heads), _i64(d_ff),
                                     C.c_float(eps), _p(wte), _p(wpe), arr, _i64(len(layers)), _p(_c(lnf_w, np.float32)),
                                     _p(_c(lnf_b, np.float32)), _p(ids), _i64(batch), _i64(seq), _p(hidden), _p(logits),
                                     _p(am))
    del keep
    return {"hidden": hidden, "logits": logits, "argmax": am, "bad": int(bad)}


def transpose_2d(x):
    """transpose_2d_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:42406-42439, 42286-42318): [rows, cols] -> [cols, rows], a
    copy of the bits."""
    x = np.asarray(x)
    return np.ascontiguousarray(x.T)


def transpose_batched(x):
    """transpose_batched_materialize_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:42526-42556, 42490-42519):
    [batch, rows, cols] -> [batch, cols, rows]."""
    x = np.asarray(x)
    return np.ascontiguousarray(x.transpose(0, 2, 1))


# ---- native state-dict container ---------------------------------------------------------------
class StateDictError(Exception):
    """kind: "InvalidMagic" | "UnsupportedVersion" | "Corrupt" (TensorIOError, crates/ft-serialize/src/lib.rs:607-619)."""

    def __init__(self, kind, reason=""):
        self.kind, self.reason = kind, reason
        super().__init__("%s: %s" % (kind, reason))


def load_state_dict_from_bytes(data):
    """load_state_dict_from_bytes (crates/ft-serialize/src/lib.rs:1005-1160) restated step for step in plain Python:
    returns {key: (dtype_tag, shape tuple, payload bytes)} in key order, or raises StateDictError with the reference's
    variant and reason text. (The rank-1 width-4 F64 fast path :1165-1260 returns the same map and is not restated.)"""
    data = bytes(data)
    n = len(data)
    pos = 0

    def corrupt(reason):
        return StateDictError("Corrupt", reason)

    def u64(what="truncated u64"):
        nonlocal pos
        if pos + 8 > n:  # read_fixed_bytes :1472-1486
            raise corrupt(what)
        v = int.from_bytes(data[pos:pos + 8], "little")
        pos += 8
        return v

    if n < 4 or data[:4] != b"FTSV":  # :1011
        raise StateDictError("InvalidMagic")
    pos = 4
    if pos + 4 > n:
        raise corrupt("truncated u32")
    version = int.from_bytes(data[4:8], "little")
    pos = 8
    if version > 1:  # :1018
        raise StateDictError("UnsupportedVersion", "found %d max 1" % version)
    count = u64()
    remaining = n - pos
    if count > remaining // 17:  # :1029-1040
        raise corrupt("claimed %d tensors but only %d bytes remain (min 17 per tensor)" % (count, remaining))
    width = {0: 8, 1: 4, 2: 2, 3: 2}
    names = {0: "f64", 1: "f32", 2: "f16", 3: "bf16"}
    out = {}
    for _ in range(count):
        key_len = u64()
        key_end = pos + key_len
        if key_end >= 1 << 64:
            raise corrupt("key length overflow")
        if key_end > n:
            raise corrupt("truncated key data")
        try:
            key = data[pos:key_end].decode("utf-8")
        except UnicodeDecodeError:
            raise corrupt("invalid UTF-8 in key")
        pos = key_end
        if key in out:
            raise corrupt("duplicate tensor key in native state dict: '%s'" % key)
        ndim = u64()
        if ndim > (n - pos) // 8:
            raise corrupt("truncated shape data for tensor '%s'" % key)
        shape, numel, overflow = [], 1, False
        for _ in range(ndim):
            dim = u64()
            if not overflow:
                if numel * dim >= 1 << 64:
                    overflow = True
                else:
                    numel *= dim
            shape.append(dim)
        if pos >= n:
            raise corrupt("truncated dtype")
        tag = data[pos]
        if tag > 3:
            raise corrupt("unknown dtype tag: %d" % tag)
        pos += 1
        if overflow:
            raise corrupt("shape overflow in native state dict tensor '%s'" % key)
        needed = numel * width[tag]
        if needed >= 1 << 64 or pos + needed >= 1 << 64:
            raise corrupt("byte count overflow for %s tensor '%s'" % (names[tag], key))
        if pos + needed > n:
            raise corrupt("truncated %s data" % names[tag])
        out[key] = (tag, tuple(shape), data[pos:pos + needed])
        pos += needed
    if pos != n:
        raise corrupt("trailing bytes after state dict payload: remaining=%d" % (n - pos))
    # BTreeMap<String, _> iterates in byte order of the UTF-8 keys
    return {k: out[k] for k in sorted(out, key=lambda s: s.encode("utf-8"))}


def encode_state_dict(tensors):
    """The layout write_state_dict_to_writer produces (crates/ft-serialize/src/lib.rs:786-860), for building test inputs:
    `tensors` is {key: numpy array of float64 / float32 / float16, or (uint16 array, "bf16")}; keys are written in
    byte order."""
    tag_of = {np.dtype(np.float64): 0, np.dtype(np.float32): 1, np.dtype(np.float16): 2}
    out = [b"FTSV", (1).to_bytes(4, "little"), len(tensors).to_bytes(8, "little")]
    for key in sorted(tensors, key=lambda s: s.encode("utf-8")):
        v = tensors[key]
        if isinstance(v, tuple):
            arr, tag = np.ascontiguousarray(v[0], dtype=np.uint16), 3
        else:
            arr = np.ascontiguousarray(v)
            tag = tag_of[arr.dtype]
        kb = key.encode("utf-8")
        out += [len(kb).to_bytes(8, "little"), kb, arr.ndim.to_bytes(8, "little")]
        out += [int(d).to_bytes(8, "little") for d in arr.shape]
        out += [bytes([tag]), arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes()]
    return b"".join(out)
