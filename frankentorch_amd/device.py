"""Device-pointer tier (fth_dev_*): hipMalloc-backed buffers with explicit copies, streams,
events, and one thin Python function per kernel. Inputs are already resident in HBM; nothing here
copies implicitly, and nothing computes on the host.
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np

from . import _lib
from .core import check

EPI_NONE, EPI_BIAS, EPI_GELU, EPI_RESIDUAL, EPI_GELU_TANH = 0, 1, 2, 4, 8
ACT_GELU_ERF, ACT_GELU_TANH = 0, 1


def is_available() -> bool:
    """ft_kernel_metal::fused::is_available: True when a gfx950 device can run the kernels."""
    return bool(_lib.load().fth_is_available())


def device_info() -> dict:
    arch = C.create_string_buffer(64)
    cus, eclk, mclk, hbm = C.c_int32(), C.c_int32(), C.c_int32(), C.c_uint64()
    check(_lib.load().fth_device_info(arch, 64, C.byref(cus), C.byref(hbm), C.byref(eclk), C.byref(mclk)))
    return {"arch": arch.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value,
            "engine_clock_khz": eclk.value, "memory_clock_khz": mclk.value}


class DeviceBuffer:
    """A typed, hipMalloc-backed array. Copies are explicit: `from_host`, `to_host`."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__len__") else (shape,)))
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape, dtype=np.int64))
        self.nbytes = self.size * self.dtype.itemsize
        p = C.c_void_p()
        check(_lib.load().fth_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value or 0
        self._owned = True

    @classmethod
    def from_host(cls, array) -> "DeviceBuffer":
        array = np.ascontiguousarray(array)
        buf = cls(array.shape, array.dtype)
        if buf.nbytes:
            check(_lib.load().fth_memcpy_h2d(buf.ptr, array.ctypes.data, buf.nbytes))
        return buf

    def to_host(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            check(_lib.load().fth_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def view(self, offset_elems: int) -> "DeviceView":
        """A non-owning typed pointer to element `offset_elems` (keeps this buffer alive)."""
        return DeviceView(self, offset_elems)

    def free(self) -> None:
        if self._owned and self.ptr:
            _lib.load().fth_free(self.ptr)
        self.ptr = 0
        self._owned = False

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DeviceView:
    """Typed device address inside a DeviceBuffer; accepted wherever a DeviceBuffer operand is."""

    def __init__(self, base: DeviceBuffer, offset_elems: int):
        self.base = base
        self.dtype = base.dtype
        self.ptr = base.ptr + offset_elems * base.dtype.itemsize


def synchronize() -> None:
    check(_lib.load().fth_device_synchronize())


class Event:
    def __init__(self):
        e = C.c_void_p()
        check(_lib.load().fth_event_create(C.byref(e)))
        self.handle = e.value

    def record(self, stream=None) -> None:
        check(_lib.load().fth_event_record(self.handle, stream))

    def synchronize(self) -> None:
        check(_lib.load().fth_event_synchronize(self.handle))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(_lib.load().fth_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            _lib.load().fth_event_destroy(self.handle)
        except Exception:
            pass


class PinnedArray:
    """A page-locked host array (fth_host_malloc) exposed as numpy; the DMA engines read and write it in place."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__len__") else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(_lib.load().fth_host_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value or 0
        raw = (C.c_char * self.nbytes).from_address(self.ptr) if self.nbytes else b""
        self.array = np.frombuffer(raw, dtype=self.dtype).reshape(self.shape)

    def free(self) -> None:
        if self.ptr:
            self.array = None
            _lib.load().fth_host_free(self.ptr)
        self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        s = C.c_void_p()
        check(_lib.load().fth_stream_create(C.byref(s)))
        self.handle = s.value

    def synchronize(self) -> None:
        check(_lib.load().fth_stream_synchronize(self.handle))

    def __del__(self):
        try:
            _lib.load().fth_stream_destroy(self.handle)
        except Exception:
            pass


def link_rates(nbytes: int, reps: int = 5) -> dict:
    """GB/s of the host link for one pinned buffer of `nbytes`: each direction alone, then both at once on two streams."""
    import time

    L = _lib.load()
    hin, hout = PinnedArray((nbytes,), np.uint8), PinnedArray((nbytes,), np.uint8)
    hin.array[:] = 1
    hout.array[:] = 0
    din, dout = DeviceBuffer((nbytes,), np.uint8), DeviceBuffer((nbytes,), np.uint8)
    s1, s2 = Stream(), Stream()

    def timed(up, down):
        best = float("inf")
        for _ in range(reps + 1):
            t0 = time.perf_counter()
            if up:
                check(L.fth_memcpy_async(din.ptr, hin.ptr, nbytes, 1, s1.handle))
            if down:
                check(L.fth_memcpy_async(hout.ptr, dout.ptr, nbytes, 2, s2.handle))
            s1.synchronize()
            s2.synchronize()
            best = min(best, time.perf_counter() - t0)
        return nbytes / best / 1e9

    h2d, d2h, both = timed(True, False), timed(False, True), timed(True, True)
    res = {"h2d": round(h2d, 2), "d2h": round(d2h, 2), "h2d_duplex": round(both, 2), "d2h_duplex": round(both, 2)}
    hin.free()
    hout.free()
    return res


def _sfx(buf: DeviceBuffer) -> str:
    if buf.dtype == np.float32:
        return "f32"
    if buf.dtype == np.float64:
        return "f64"
    raise TypeError("kernels compute f32 and f64 only, got %s" % buf.dtype)


def _ptr(buf):
    return None if buf is None else (buf.ptr if hasattr(buf, "ptr") else int(buf))


def _real(buf, v):
    return C.c_float(v) if buf.dtype == np.float32 else C.c_double(v)


def softmax_lastdim(x, y, rows, cols, stream=None):
    check(getattr(_lib.load(), "fth_dev_softmax_lastdim_" + _sfx(x))(_ptr(x), _ptr(y), rows, cols, stream))


def softmax_strided(x, y, outer, reduce, inner, stream=None):
    check(getattr(_lib.load(), "fth_dev_softmax_strided_" + _sfx(x))(_ptr(x), _ptr(y), outer, reduce, inner, stream))


def log_softmax_strided(x, y, outer, reduce, inner, stream=None):
    check(getattr(_lib.load(), "fth_dev_log_softmax_strided_" + _sfx(x))(_ptr(x), _ptr(y), outer, reduce, inner, stream))


def cross_entropy_forward(logits, target, batch, classes, loss, bad_index=None, stream=None):
    """loss[i] = lse(logits[i]) - logits[i][target[i]]; target is an int64 tensor of class indices."""
    check(getattr(_lib.load(), "fth_dev_cross_entropy_forward_" + _sfx(logits))(_ptr(logits), _ptr(target), batch, classes,
                                                                                _ptr(loss), _ptr(bad_index), stream))


def cross_entropy_backward(logits, target, dloss, batch, classes, dlogits, bad_index=None, stream=None):
    check(getattr(_lib.load(), "fth_dev_cross_entropy_backward_" + _sfx(logits))(_ptr(logits), _ptr(target), _ptr(dloss), batch,
                                                                                 classes, _ptr(dlogits), _ptr(bad_index), stream))


def layer_norm(x, weight, bias, y, batch, norm_size, eps, stream=None):
    check(getattr(_lib.load(), "fth_dev_layer_norm_" + _sfx(x))(_ptr(x), _ptr(weight), _ptr(bias), _ptr(y), batch,
                                                                norm_size, _real(x, eps), stream))


def add_layer_norm(a, b, weight, bias, y, batch, norm_size, eps, stream=None):
    if a.dtype != np.float32:
        raise TypeError("add_layer_norm exists for float32 only (add_layer_norm_forward_f32 has no f64 twin)")
    check(_lib.load().fth_dev_add_layer_norm_f32(_ptr(a), _ptr(b), _ptr(weight), _ptr(bias), _ptr(y), batch, norm_size,
                                                 C.c_float(eps), stream))


def rms_norm(x, weight, y, batch, norm_size, eps, stream=None):
    check(getattr(_lib.load(), "fth_dev_rms_norm_" + _sfx(x))(_ptr(x), _ptr(weight), _ptr(y), batch, norm_size,
                                                              _real(x, eps), stream))


def gelu(x, y, n, stream=None):
    check(getattr(_lib.load(), "fth_dev_gelu_" + _sfx(x))(_ptr(x), _ptr(y), n, stream))


def gelu_tanh(x, y, n, stream=None):
    check(getattr(_lib.load(), "fth_dev_gelu_tanh_" + _sfx(x))(_ptr(x), _ptr(y), n, stream))


def add(a, b, y, n, stream=None):
    check(getattr(_lib.load(), "fth_dev_add_" + _sfx(a))(_ptr(a), _ptr(b), _ptr(y), n, stream))


def bias_add(x, bias, y, rows, cols, stream=None):
    check(getattr(_lib.load(), "fth_dev_bias_add_" + _sfx(x))(_ptr(x), _ptr(bias), _ptr(y), rows, cols, stream))


def bias_residual_add(x, bias, residual, y, rows, cols, stream=None):
    check(getattr(_lib.load(), "fth_dev_bias_residual_add_" + _sfx(x))(_ptr(x), _ptr(bias), _ptr(residual), _ptr(y), rows, cols, stream))


def index_select(inp, outer, dim_size, inner, indices, num_indices, out, bad_index=None, stream=None):
    check(getattr(_lib.load(), "fth_dev_index_select_" + _sfx(inp))(_ptr(inp), outer, dim_size, inner, _ptr(indices),
                                                                    num_indices, _ptr(out), _ptr(bad_index), stream))


def embedding_add(wte, vocab, wpe, max_pos, ids, tokens, seq, width, out, bad_index=None, stream=None):
    check(_lib.load().fth_dev_embedding_add_f32(_ptr(wte), vocab, _ptr(wpe), max_pos, _ptr(ids), tokens, seq, width,
                                                _ptr(out), _ptr(bad_index), stream))


def argmax(x, outer, reduce, inner, out, stream=None):
    check(getattr(_lib.load(), "fth_dev_argmax_" + _sfx(x))(_ptr(x), outer, reduce, inner, _ptr(out), stream))


def linear_argmax_workspace_floats(rows, out_features) -> int:
    return int(_lib.load().fth_dev_linear_argmax_workspace_floats(rows, out_features))


def linear_argmax(x, w, rows, out_features, in_features, logits, out, workspace=None, stream=None):
    """logits = x . w^T and out = argmax over the last dim of the logits (fp32); workspace: a float32 DeviceBuffer of
    linear_argmax_workspace_floats(rows, out_features) elements, or None for the two separate kernels."""
    n = 0 if workspace is None else workspace.size
    check(_lib.load().fth_dev_linear_argmax_f32(_ptr(x), _ptr(w), rows, out_features, in_features, _ptr(logits), _ptr(out),
                                                _ptr(workspace), n, stream))


def copy(x, y, n, stream=None):
    check(getattr(_lib.load(), "fth_dev_copy_" + _sfx(x))(_ptr(x), _ptr(y), n, stream))


def transpose_2d(src, dst, rows, cols, stream=None):
    check(getattr(_lib.load(), "fth_dev_transpose_2d_" + _sfx(src))(_ptr(src), _ptr(dst), rows, cols, stream))


def transpose_batched(src, dst, batch, rows, cols, stream=None):
    check(getattr(_lib.load(), "fth_dev_transpose_batched_" + _sfx(src))(_ptr(src), _ptr(dst), batch, rows, cols, stream))


def memory_info():
    """(free, total) device memory in bytes."""
    f, tot = C.c_uint64(), C.c_uint64()
    check(_lib.load().fth_device_memory_info(C.byref(f), C.byref(tot)))
    return f.value, tot.value


def gemm_workspace_info():
    """(live, retired) bytes of the GEMM unit's split-tile / transposed-operand workspaces."""
    live, ret = C.c_uint64(), C.c_uint64()
    check(_lib.load().fth_device_workspace_info(C.byref(live), C.byref(ret)))
    return live.value, ret.value


def permute_0213(src, dst, d0, d1, d2, d3, stream=None):
    check(getattr(_lib.load(), "fth_dev_permute_0213_" + _sfx(src))(_ptr(src), _ptr(dst), d0, d1, d2, d3, stream))


def gemm_desc(m, n, k, trans_b=False, batch=1, epilogue=EPI_NONE, lda=None, ldb=None, ldc=None, stride_a=None,
              stride_b=None, stride_c=None, trans_a=False) -> _lib.GemmDesc:
    d = _lib.GemmDesc()
    d.m, d.n, d.k = m, n, k
    d.trans_a = 1 if trans_a else 0
    d.lda = (m if trans_a else k) if lda is None else lda
    d.ldb = (k if trans_b else n) if ldb is None else ldb
    d.ldc = n if ldc is None else ldc
    d.batch = batch
    d.stride_a = m * k if stride_a is None else stride_a
    d.stride_b = k * n if stride_b is None else stride_b
    d.stride_c = m * n if stride_c is None else stride_c
    d.trans_b = 1 if trans_b else 0
    d.epilogue = epilogue
    return d


def gemm(desc, a, b, c, bias=None, residual=None, alpha=1.0, stream=None):
    """C = alpha * A . op(B) (+ bias, GELU, residual per desc.epilogue)."""
    check(getattr(_lib.load(), "fth_dev_gemm_" + _sfx(a))(C.byref(desc), _real(a, alpha), _ptr(a), _ptr(b), _ptr(c),
                                                          _ptr(bias), _ptr(residual), stream))


def _dtype_code(buf) -> int:
    return 0 if buf.dtype == np.float64 else 1  # FTH_DTYPE_F64 / FTH_DTYPE_F32


def _workspace(nbytes, workspace):
    """The caller's workspace buffer, or a fresh one of the size the library asks for."""
    if workspace is not None:
        return workspace
    return DeviceBuffer((max(int(nbytes), 16) + 3) // 4, np.float32)


def norm_backward_workspace_bytes(rows, cols, dtype=np.float32) -> int:
    return _lib.load().fth_dev_norm_backward_workspace_bytes(rows, cols, 0 if np.dtype(dtype) == np.float64 else 1)


def layer_norm_backward(dy, x, weight, dx, dweight, dbias, rows, cols, eps, workspace=None, stream=None):
    """layer_norm_backward_f32 / _f64: dx [rows, cols], dweight / dbias [cols]; mean / rstd recomputed from x."""
    ws = _workspace(_lib.load().fth_dev_norm_backward_workspace_bytes(rows, cols, _dtype_code(x)), workspace)
    check(getattr(_lib.load(), "fth_dev_layer_norm_backward_" + _sfx(x))(_ptr(dy), _ptr(x), _ptr(weight), rows, cols, _real(x, eps),
                                                                         _ptr(dx), _ptr(dweight), _ptr(dbias), ws.ptr, ws.nbytes, stream))
    return ws


def layer_norm_backward_noalloc(dy, x, weight, dx, dweight, dbias, rows, cols, eps, stream=None):
    """fth_dev_layer_norm_backward_f32_noalloc: the fp32 LayerNorm backward with its partial sums in the library's built-in
    device array; raises (BufferTooLarge) for shapes beyond layer_norm_backward_noalloc_max_bytes()."""
    check(_lib.load().fth_dev_layer_norm_backward_f32_noalloc(_ptr(dy), _ptr(x), _ptr(weight), rows, cols, float(eps), _ptr(dx),
                                                              _ptr(dweight), _ptr(dbias), stream))


def layer_norm_backward_noalloc_max_bytes() -> int:
    return int(_lib.load().fth_dev_layer_norm_backward_noalloc_max_bytes())


def rms_norm_backward(dy, x, weight, dx, dweight, rows, cols, eps, workspace=None, stream=None):
    """rms_norm_backward_f32 / _f64: weight and dweight may both be None."""
    ws = _workspace(_lib.load().fth_dev_norm_backward_workspace_bytes(rows, cols, _dtype_code(x)), workspace)
    check(getattr(_lib.load(), "fth_dev_rms_norm_backward_" + _sfx(x))(_ptr(dy), _ptr(x), _ptr(weight), rows, cols, _real(x, eps),
                                                                       _ptr(dx), _ptr(dweight), ws.ptr, ws.nbytes, stream))
    return ws


def linear_backward(dy, x, weight, dx, dweight, dbias, batch, in_features, out_features, workspace=None, stream=None):
    """linear_backward: dx = dy . W, dweight = dy^T . x, dbias = column sums of dy (None: not wanted)."""
    ws = _workspace(_lib.load().fth_dev_linear_backward_workspace_bytes(batch, out_features, _dtype_code(x)), workspace)
    check(getattr(_lib.load(), "fth_dev_linear_backward_" + _sfx(x))(_ptr(dy), _ptr(x), _ptr(weight), batch, in_features, out_features,
                                                                     _ptr(dx), _ptr(dweight), _ptr(dbias), ws.ptr, ws.nbytes, stream))
    return ws


def sdpa_backward(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace=None, stream=None):
    """sdpa_backward_f32 / _f64 on contiguous [num_bh, seq, d] operands."""
    ws = _workspace(_lib.load().fth_dev_sdpa_backward_workspace_bytes(num_bh, seq_q, seq_k, _dtype_code(q)), workspace)
    check(getattr(_lib.load(), "fth_dev_sdpa_backward_" + _sfx(q))(_ptr(q), _ptr(k), _ptr(v), _ptr(dout), num_bh, seq_q, seq_k, d_k, d_v,
                                                                   _real(q, scale), 1 if causal else 0, _ptr(dq), _ptr(dk), _ptr(dv),
                                                                   ws.ptr, ws.nbytes, stream))
    return ws


def sdpa_backward_unit_dout(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace=None, stream=None):
    """sdpa_backward_f32_unit_dout (and an f64 twin): the backward for dout = ones, which is not passed."""
    ws = _workspace(_lib.load().fth_dev_sdpa_backward_unit_dout_workspace_bytes(num_bh, seq_q, seq_k, d_v, _dtype_code(q)), workspace)
    check(getattr(_lib.load(), "fth_dev_sdpa_backward_unit_dout_" + _sfx(q))(_ptr(q), _ptr(k), _ptr(v), num_bh, seq_q, seq_k, d_k, d_v,
                                                                             _real(q, scale), 1 if causal else 0, _ptr(dq), _ptr(dk),
                                                                             _ptr(dv), ws.ptr, ws.nbytes, stream))
    return ws


def sdpa_backward_masked(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride, dq, dk, dv, workspace=None,
                         stream=None):
    """sdpa_backward_masked_f64 and its f32 twin: P = softmax(scale * Q.K^T + mask); mask_bh_stride 0 shares one [seq_q, seq_k] mask."""
    ws = _workspace(_lib.load().fth_dev_sdpa_backward_workspace_bytes(num_bh, seq_q, seq_k, _dtype_code(q)), workspace)
    check(getattr(_lib.load(), "fth_dev_sdpa_backward_masked_" + _sfx(q))(_ptr(q), _ptr(k), _ptr(v), _ptr(dout), num_bh, seq_q, seq_k, d_k,
                                                                          d_v, _real(q, scale), _ptr(mask), mask_bh_stride, _ptr(dq),
                                                                          _ptr(dk), _ptr(dv), ws.ptr, ws.nbytes, stream))
    return ws


def sdpa_desc_contiguous(num_bh, seq_q, seq_k, d_k, d_v, causal) -> _lib.SdpaDesc:
    d = _lib.SdpaDesc()
    _lib.load().fth_sdpa_desc_contiguous(C.byref(d), num_bh, seq_q, seq_k, d_k, d_v, 1 if causal else 0)
    return d


def sdpa_forward(desc, scale, q, k, v, out, stream=None):
    check(getattr(_lib.load(), "fth_dev_sdpa_forward_" + _sfx(q))(C.byref(desc), _real(q, scale), _ptr(q), _ptr(k),
                                                                  _ptr(v), _ptr(out), stream))


def sdpa_desc_gqa(batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, causal=False) -> _lib.SdpaDesc:
    """Contiguous q [batch, h_q, seq_q, d_k] and k / v [batch, h_kv, seq_k, d]: query head h reads K/V head h // (h_q // h_kv)."""
    if h_kv <= 0 or h_q % h_kv:
        raise ValueError("h_kv must divide h_q")
    d = sdpa_desc_contiguous(batch * h_q, seq_q, seq_k, d_k, d_v, causal)
    d.heads, d.kv_group = h_q, h_q // h_kv
    d.q_batch_stride, d.q_head_stride = h_q * seq_q * d_k, seq_q * d_k
    d.k_batch_stride, d.k_head_stride = h_kv * seq_k * d_k, seq_k * d_k
    d.v_batch_stride, d.v_head_stride = h_kv * seq_k * d_v, seq_k * d_v
    d.o_batch_stride, d.o_head_stride = h_q * seq_q * d_v, seq_q * d_v
    return d


def sdpa_forward_masked(desc, scale, q, k, v, mask, mask_bh_stride, out, stream=None):
    """softmax(scale * q k^T + mask) v; mask_bh_stride 0 shares one [seq_q, seq_k] mask, seq_q * seq_k reads one per head."""
    check(getattr(_lib.load(), "fth_dev_sdpa_forward_masked_" + _sfx(q))(C.byref(desc), _real(q, scale), _ptr(q), _ptr(k), _ptr(v),
                                                                         _ptr(mask), mask_bh_stride, _ptr(out), stream))


def quantize_rows_i8(x, rows, cols, q, scales, stream=None):
    """Per-row symmetric int8 (activations, or weights per output channel): q int8 [rows, cols], scales f32 [rows]."""
    check(_lib.load().fth_dev_quantize_rows_i8(_ptr(x), rows, cols, _ptr(q), _ptr(scales), stream))


def linear_int8_workspace_bytes(m, k) -> int:
    return int(_lib.load().fth_dev_linear_int8_workspace_bytes(m, k))


def linear_int8_dynamic(x, m, k, w_i8, w_scales, n, bias, out, workspace=None, stream=None):
    """out [m, n] = dequant(quant_rows(x) . w_i8^T) + bias; returns the workspace buffer so callers can reuse it."""
    workspace = _workspace(linear_int8_workspace_bytes(m, k), workspace)
    check(_lib.load().fth_dev_linear_int8_dynamic_f32(_ptr(x), m, k, _ptr(w_i8), _ptr(w_scales), n, _ptr(bias), _ptr(out),
                                                      _ptr(workspace), workspace.nbytes, stream))
    return workspace


def default_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
