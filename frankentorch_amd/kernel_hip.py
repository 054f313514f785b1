"""`ft_kernel_hip`: the operator entry points of `ft_kernel_cpu`, same names, same argument
meaning, same errors -- host arrays in, a freshly allocated host array out -- computed on the
MI355X through the host-slice tier of the C ABI.

The reference's signatures take `&[T]` slices plus `&TensorMeta`; here a slice is a 1-D
C-contiguous numpy array (f32 or f64) and the meta is `core.TensorMeta`. Fallible entry points
raise `core.KernelError` with the reference's variant; the fused entry points that the reference
leaves infallible (and that panic on short slices) raise `core.HipError(InvalidArgument)`.

Reference lines (crates/ft-kernel-cpu/src/lib.rs): matmul :37752 / :17355, bmm :38496 / :17785,
addmm :41562 / :17514, linear :17306 / :17162, matmul_rhs_transposed :17408 / :17381,
softmax_dim :39193 / :18350, layer_norm_forward :5877 / :5824, add_layer_norm_forward :5932,
rms_norm_forward :6459 / :6418, gelu :37123, add :36870, sdpa_forward :5200 / :4572,
index_select :40216, argmax_dim :39443 / :18653, transpose_2d :42406 / :42286,
transpose_batched_materialize :42526 / :42490.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .core import TensorMeta, check


def _slice(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a.reshape(-1)


def _opt(a, dtype):
    return None if a is None else _slice(a, dtype)


def _p(a):
    return None if a is None else a.ctypes.data


def _call_sized(fn, dtype, *args_before_out):
    """Two-step call: validate and size (out == NULL), then run into an exact-size array."""
    out_len = C.c_size_t(0)
    check(fn(*args_before_out, None, 0, C.byref(out_len)))
    out = np.empty(out_len.value, dtype=dtype)
    if out_len.value:
        check(fn(*args_before_out, out.ctypes.data, out.size, C.byref(out_len)))
    return out


def _binary(name, dtype, lhs, rhs, lhs_meta: TensorMeta, rhs_meta: TensorMeta):
    lhs, rhs = _slice(lhs, dtype), _slice(rhs, dtype)
    lm, rm = lhs_meta.to_c(), rhs_meta.to_c()
    return _call_sized(getattr(_lib.load(), name), dtype, _p(lhs), lhs.size, _p(rhs), rhs.size, C.byref(lm), C.byref(rm))


def matmul_tensor_contiguous_f32(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_matmul_tensor_contiguous_f32", np.float32, lhs, rhs, lhs_meta, rhs_meta)


def matmul_tensor_contiguous_f64(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_matmul_tensor_contiguous_f64", np.float64, lhs, rhs, lhs_meta, rhs_meta)


def bmm_tensor_contiguous_f32(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_bmm_tensor_contiguous_f32", np.float32, lhs, rhs, lhs_meta, rhs_meta)


def bmm_tensor_contiguous_f64(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_bmm_tensor_contiguous_f64", np.float64, lhs, rhs, lhs_meta, rhs_meta)


def add_tensor_contiguous_f32(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_add_tensor_contiguous_f32", np.float32, lhs, rhs, lhs_meta, rhs_meta)


def add_tensor_contiguous_f64(lhs, rhs, lhs_meta, rhs_meta):
    return _binary("fth_add_tensor_contiguous_f64", np.float64, lhs, rhs, lhs_meta, rhs_meta)


def _addmm(name, dtype, ctype, inp, mat1, mat2, input_meta, mat1_meta, mat2_meta, beta, alpha):
    inp, mat1, mat2 = _slice(inp, dtype), _slice(mat1, dtype), _slice(mat2, dtype)
    im, m1, m2 = input_meta.to_c(), mat1_meta.to_c(), mat2_meta.to_c()
    return _call_sized(getattr(_lib.load(), name), dtype, _p(inp), inp.size, _p(mat1), mat1.size, _p(mat2), mat2.size,
                       C.byref(im), C.byref(m1), C.byref(m2), ctype(beta), ctype(alpha))


def addmm_tensor_contiguous_f32(inp, mat1, mat2, input_meta, mat1_meta, mat2_meta, beta, alpha):
    return _addmm("fth_addmm_tensor_contiguous_f32", np.float32, C.c_float, inp, mat1, mat2, input_meta, mat1_meta,
                  mat2_meta, beta, alpha)


def addmm_tensor_contiguous_f64(inp, mat1, mat2, input_meta, mat1_meta, mat2_meta, beta, alpha):
    return _addmm("fth_addmm_tensor_contiguous_f64", np.float64, C.c_double, inp, mat1, mat2, input_meta, mat1_meta,
                  mat2_meta, beta, alpha)


def _linear(name, dtype, x, weight, bias, batch, in_features, out_features):
    x, weight, bias = _slice(x, dtype), _slice(weight, dtype), _opt(bias, dtype)
    return _call_sized(getattr(_lib.load(), name), dtype, _p(x), x.size, _p(weight), weight.size, _p(bias),
                       0 if bias is None else bias.size, batch, in_features, out_features)


def linear_tensor_f32(x, weight, bias, batch, in_features, out_features):
    return _linear("fth_linear_tensor_f32", np.float32, x, weight, bias, batch, in_features, out_features)


def linear_tensor_f64(x, weight, bias, batch, in_features, out_features):
    return _linear("fth_linear_tensor_f64", np.float64, x, weight, bias, batch, in_features, out_features)


def _matmul_bt(name, dtype, m, k, n, lhs, rhs_nk):
    lhs, rhs_nk = _slice(lhs, dtype), _slice(rhs_nk, dtype)
    return _call_sized(getattr(_lib.load(), name), dtype, m, k, n, _p(lhs), lhs.size, _p(rhs_nk), rhs_nk.size)


def matmul_rhs_transposed_contiguous_f32(m, k, n, lhs, rhs_nk):
    return _matmul_bt("fth_matmul_rhs_transposed_contiguous_f32", np.float32, m, k, n, lhs, rhs_nk)


def matmul_rhs_transposed_contiguous_f64(m, k, n, lhs, rhs_nk):
    return _matmul_bt("fth_matmul_rhs_transposed_contiguous_f64", np.float64, m, k, n, lhs, rhs_nk)


def _unary_dim(name, dtype, inp, meta: TensorMeta, dim):
    inp = _slice(inp, dtype)
    m = meta.to_c()
    return _call_sized(getattr(_lib.load(), name), dtype, _p(inp), inp.size, C.byref(m), dim)


def softmax_dim_tensor_contiguous_f32(inp, meta, dim):
    return _unary_dim("fth_softmax_dim_tensor_contiguous_f32", np.float32, inp, meta, dim)


def softmax_dim_tensor_contiguous_f64(inp, meta, dim):
    return _unary_dim("fth_softmax_dim_tensor_contiguous_f64", np.float64, inp, meta, dim)


def log_softmax_dim_tensor_contiguous_f32(inp, meta, dim):
    """crates/ft-kernel-cpu/src/lib.rs:39298."""
    return _unary_dim("fth_log_softmax_dim_tensor_contiguous_f32", np.float32, inp, meta, dim)


def log_softmax_dim_tensor_contiguous_f64(inp, meta, dim):
    """crates/ft-kernel-cpu/src/lib.rs:18504."""
    return _unary_dim("fth_log_softmax_dim_tensor_contiguous_f64", np.float64, inp, meta, dim)


def _cross_entropy(sfx, dtype, logits, target, dloss, batch, classes):
    logits = _slice(logits, dtype)
    target = np.ascontiguousarray(target, dtype=np.uint64).reshape(-1)
    fn = getattr(_lib.load(), "fth_cross_entropy_%s_%s" % ("forward" if dloss is None else "backward", sfx))
    if dloss is None:
        out = np.empty(batch, dtype=dtype)
        check(fn(_p(logits), logits.size, _p(target), target.size, batch, classes, _p(out), out.size))
    else:
        dloss = _slice(dloss, dtype)
        out = np.empty(batch * classes, dtype=dtype)
        check(fn(_p(logits), logits.size, _p(target), target.size, _p(dloss), dloss.size, batch, classes, _p(out), out.size))
    return out


def cross_entropy_forward_f32(logits, target, batch, classes):
    """Per-row loss, crates/ft-kernel-cpu/src/lib.rs:6717."""
    return _cross_entropy("f32", np.float32, logits, target, None, batch, classes)


def cross_entropy_forward_f64(logits, target, batch, classes):
    """crates/ft-kernel-cpu/src/lib.rs:6649."""
    return _cross_entropy("f64", np.float64, logits, target, None, batch, classes)


def cross_entropy_backward_f32(logits, target, dloss, batch, classes):
    """dlogits, crates/ft-kernel-cpu/src/lib.rs:6745."""
    return _cross_entropy("f32", np.float32, logits, target, dloss, batch, classes)


def cross_entropy_backward_f64(logits, target, dloss, batch, classes):
    """crates/ft-kernel-cpu/src/lib.rs:6679."""
    return _cross_entropy("f64", np.float64, logits, target, dloss, batch, classes)


def argmax_dim_tensor_contiguous_f32(inp, meta, dim):
    return _unary_dim("fth_argmax_dim_tensor_contiguous_f32", np.float32, inp, meta, dim)


def argmax_dim_tensor_contiguous_f64(inp, meta, dim):
    return _unary_dim("fth_argmax_dim_tensor_contiguous_f64", np.float64, inp, meta, dim)


def _gelu(name, dtype, inp, meta: TensorMeta):
    inp = _slice(inp, dtype)
    m = meta.to_c()
    return _call_sized(getattr(_lib.load(), name), dtype, _p(inp), inp.size, C.byref(m))


def gelu_tensor_contiguous_f32(inp, meta):
    return _gelu("fth_gelu_tensor_contiguous_f32", np.float32, inp, meta)


def gelu_tensor_contiguous_f64(inp, meta):
    return _gelu("fth_gelu_tensor_contiguous_f64", np.float64, inp, meta)


def gelu_tanh_tensor_contiguous_f32(inp, meta):
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), GELU::tanh() (crates/ft-nn/src/lib.rs:1949-1957)."""
    return _gelu("fth_gelu_tanh_tensor_contiguous_f32", np.float32, inp, meta)


def gelu_tanh_tensor_contiguous_f64(inp, meta):
    return _gelu("fth_gelu_tanh_tensor_contiguous_f64", np.float64, inp, meta)


def _index_select(name, dtype, inp, meta: TensorMeta, dim, indices):
    inp = _slice(inp, dtype)
    idx = _slice(indices, np.float64)
    m = meta.to_c()
    return _call_sized(getattr(_lib.load(), name), dtype, _p(inp), inp.size, C.byref(m), dim, _p(idx), idx.size)


def index_select_tensor_contiguous_f32(inp, meta, dim, indices):
    return _index_select("fth_index_select_tensor_contiguous_f32", np.float32, inp, meta, dim, indices)


def index_select_tensor_contiguous_f64(inp, meta, dim, indices):
    return _index_select("fth_index_select_tensor_contiguous_f64", np.float64, inp, meta, dim, indices)


def layer_norm_forward_f32(x, weight, bias, batch, norm_size, eps):
    x, weight, bias = _slice(x, np.float32), _opt(weight, np.float32), _opt(bias, np.float32)
    out = np.empty(batch * norm_size, dtype=np.float32)
    check(_lib.load().fth_layer_norm_forward_f32(_p(x), x.size, _p(weight), _p(bias), batch, norm_size, eps, _p(out), out.size))
    return out


def layer_norm_forward_f64(x, weight, bias, batch, norm_size, eps):
    x, weight, bias = _slice(x, np.float64), _opt(weight, np.float64), _opt(bias, np.float64)
    out = np.empty(batch * norm_size, dtype=np.float64)
    check(_lib.load().fth_layer_norm_forward_f64(_p(x), x.size, _p(weight), _p(bias), batch, norm_size, eps, _p(out), out.size))
    return out


def add_layer_norm_forward_f32(a, b, weight, bias, batch, norm_size, eps):
    a, b = _slice(a, np.float32), _slice(b, np.float32)
    weight, bias = _opt(weight, np.float32), _opt(bias, np.float32)
    out = np.empty(batch * norm_size, dtype=np.float32)
    check(_lib.load().fth_add_layer_norm_forward_f32(_p(a), _p(b), min(a.size, b.size), _p(weight), _p(bias), batch,
                                                     norm_size, eps, _p(out), out.size))
    return out


def rms_norm_forward_f32(x, weight, batch, norm_size, eps):
    x, weight = _slice(x, np.float32), _opt(weight, np.float32)
    out = np.empty(batch * norm_size, dtype=np.float32)
    check(_lib.load().fth_rms_norm_forward_f32(_p(x), x.size, _p(weight), batch, norm_size, eps, _p(out), out.size))
    return out


def rms_norm_forward_f64(x, weight, batch, norm_size, eps):
    x, weight = _slice(x, np.float64), _opt(weight, np.float64)
    out = np.empty(batch * norm_size, dtype=np.float64)
    check(_lib.load().fth_rms_norm_forward_f64(_p(x), x.size, _p(weight), batch, norm_size, eps, _p(out), out.size))
    return out


def _layer_norm_backward(sfx, dtype, dy, x, weight, batch, norm_size, eps):
    dy, x, weight = _slice(dy, dtype), _slice(x, dtype), _slice(weight, dtype)
    dx = np.empty(batch * norm_size, dtype=dtype)
    dw, db = np.empty(norm_size, dtype=dtype), np.empty(norm_size, dtype=dtype)
    check(getattr(_lib.load(), "fth_layer_norm_backward_" + sfx)(_p(dy), dy.size, _p(x), x.size, _p(weight), batch, norm_size, eps,
                                                                 _p(dx), dx.size, _p(dw), dw.size, _p(db), db.size))
    return dx, dw, db


def layer_norm_backward_f32(dy, x, weight, batch, norm_size, eps):
    """(dx, dweight, dbias), crates/ft-kernel-cpu/src/lib.rs:6189."""
    return _layer_norm_backward("f32", np.float32, dy, x, weight, batch, norm_size, eps)


def layer_norm_backward_f64(dy, x, weight, batch, norm_size, eps):
    return _layer_norm_backward("f64", np.float64, dy, x, weight, batch, norm_size, eps)


def _rms_norm_backward(sfx, dtype, dy, x, weight, batch, norm_size, eps):
    dy, x, weight = _slice(dy, dtype), _slice(x, dtype), _opt(weight, dtype)
    dx = np.empty(batch * norm_size, dtype=dtype)
    dw = None if weight is None else np.empty(norm_size, dtype=dtype)
    check(getattr(_lib.load(), "fth_rms_norm_backward_" + sfx)(_p(dy), dy.size, _p(x), x.size, _p(weight), batch, norm_size, eps,
                                                               _p(dx), dx.size, _p(dw), 0 if dw is None else dw.size))
    return dx, dw


def rms_norm_backward_f32(dy, x, weight, batch, norm_size, eps):
    """(dx, Option<dweight>), crates/ft-kernel-cpu/src/lib.rs:6574."""
    return _rms_norm_backward("f32", np.float32, dy, x, weight, batch, norm_size, eps)


def rms_norm_backward_f64(dy, x, weight, batch, norm_size, eps):
    return _rms_norm_backward("f64", np.float64, dy, x, weight, batch, norm_size, eps)


def _linear_backward(sfx, dtype, dy, x, weight, batch, in_features, out_features, need_bias):
    dy, x, weight = _slice(dy, dtype), _slice(x, dtype), _slice(weight, dtype)
    dx = np.empty(batch * in_features, dtype=dtype)
    dw = np.empty(out_features * in_features, dtype=dtype)
    db = np.empty(out_features, dtype=dtype) if need_bias else None
    check(getattr(_lib.load(), "fth_linear_backward_" + sfx)(_p(dy), dy.size, _p(x), x.size, _p(weight), weight.size, batch, in_features,
                                                             out_features, 1 if need_bias else 0, _p(dx), dx.size, _p(dw), dw.size,
                                                             _p(db), 0 if db is None else db.size))
    return dx, dw, db


def linear_backward_f64(dy, x, weight, batch, in_features, out_features, need_bias):
    """(dx, dweight, Option<dbias>), crates/ft-kernel-cpu/src/lib.rs:17226."""
    return _linear_backward("f64", np.float64, dy, x, weight, batch, in_features, out_features, need_bias)


def linear_backward_f32(dy, x, weight, batch, in_features, out_features, need_bias):
    return _linear_backward("f32", np.float32, dy, x, weight, batch, in_features, out_features, need_bias)


def _sdpa_backward(sfx, dtype, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    q, k, v, dout = _slice(q, dtype), _slice(k, dtype), _slice(v, dtype), _slice(dout, dtype)
    dq = np.empty(num_bh * seq_q * d_k, dtype=dtype)
    dk = np.empty(num_bh * seq_k * d_k, dtype=dtype)
    dv = np.empty(num_bh * seq_k * d_v, dtype=dtype)
    check(getattr(_lib.load(), "fth_sdpa_backward_" + sfx)(_p(q), q.size, _p(k), k.size, _p(v), v.size, _p(dout), dout.size, num_bh, seq_q,
                                                           seq_k, d_k, d_v, scale, 1 if causal else 0, _p(dq), dq.size, _p(dk), dk.size,
                                                           _p(dv), dv.size))
    return dq, dk, dv


def sdpa_backward_f32(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    """(dq, dk, dv), crates/ft-kernel-cpu/src/lib.rs:5539."""
    return _sdpa_backward("f32", np.float32, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal)


def sdpa_backward_f64(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    return _sdpa_backward("f64", np.float64, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal)


def sdpa_backward_f32_unit_dout(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    """(dq, dk, dv) for dout = ones([num_bh, seq_q, d_v]) without that tensor, crates/ft-kernel-cpu/src/lib.rs:5662."""
    q, k, v = _slice(q, np.float32), _slice(k, np.float32), _slice(v, np.float32)
    dq = np.empty(num_bh * seq_q * d_k, dtype=np.float32)
    dk = np.empty(num_bh * seq_k * d_k, dtype=np.float32)
    dv = np.empty(num_bh * seq_k * d_v, dtype=np.float32)
    check(_lib.load().fth_sdpa_backward_f32_unit_dout(_p(q), q.size, _p(k), k.size, _p(v), v.size, num_bh, seq_q, seq_k, d_k, d_v, scale,
                                                      1 if causal else 0, _p(dq), dq.size, _p(dk), dk.size, _p(dv), dv.size))
    return dq, dk, dv


def _sdpa_backward_masked(sfx, dtype, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    q, k, v, dout, mask = _slice(q, dtype), _slice(k, dtype), _slice(v, dtype), _slice(dout, dtype), _slice(mask, dtype)
    dq = np.empty(num_bh * seq_q * d_k, dtype=dtype)
    dk = np.empty(num_bh * seq_k * d_k, dtype=dtype)
    dv = np.empty(num_bh * seq_k * d_v, dtype=dtype)
    check(getattr(_lib.load(), "fth_sdpa_backward_masked_" + sfx)(_p(q), q.size, _p(k), k.size, _p(v), v.size, _p(dout), dout.size, num_bh,
                                                                  seq_q, seq_k, d_k, d_v, scale, _p(mask), mask.size, mask_bh_stride, _p(dq),
                                                                  dq.size, _p(dk), dk.size, _p(dv), dv.size))
    return dq, dk, dv


def sdpa_backward_masked_f64(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    """(dq, dk, dv) with P = softmax(scale * Q.K^T + mask), crates/ft-kernel-cpu/src/lib.rs:5423."""
    return _sdpa_backward_masked("f64", np.float64, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride)


def sdpa_backward_masked_f32(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    """The f32 twin of sdpa_backward_masked_f64 (the reference has the masked backward in f64 only)."""
    return _sdpa_backward_masked("f32", np.float32, q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride)


def _sdpa(name, dtype, q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    q, k, v = _slice(q, dtype), _slice(k, dtype), _slice(v, dtype)
    out = np.empty(num_bh * seq_q * d_v, dtype=dtype)
    check(getattr(_lib.load(), name)(_p(q), q.size, _p(k), k.size, _p(v), v.size, num_bh, seq_q, seq_k, d_k, d_v, scale,
                                     1 if causal else 0, _p(out), out.size))
    return out


def _quantize_i8(name, w, rows, cols):
    w = _slice(w, np.float32)
    q, scales = np.empty(rows * cols, np.int8), np.empty(rows, np.float32)
    check(getattr(_lib.load(), name)(_p(w), w.size, rows, cols, _p(q), q.size, _p(scales), scales.size))
    return q, scales


def quantize_per_output_channel_i8(w, out, in_):
    """(w_i8, scales), crates/ft-kernel-cpu/src/lib.rs:37836."""
    return _quantize_i8("fth_quantize_per_output_channel_i8", w, out, in_)


def quantize_rows_i8(x, m, k):
    """(x_i8, a_scales), crates/ft-kernel-cpu/src/lib.rs:37879."""
    return _quantize_i8("fth_quantize_rows_i8", x, m, k)


def linear_int8_dynamic_f32(x, m, k, w_i8, w_scales, n, bias=None):
    """crates/ft-kernel-cpu/src/lib.rs:37966."""
    x, w_scales = _slice(x, np.float32), _slice(w_scales, np.float32)
    w_i8 = np.ascontiguousarray(w_i8, dtype=np.int8).reshape(-1)
    bias = None if bias is None else _slice(bias, np.float32)
    out = np.empty(m * n, np.float32)
    check(_lib.load().fth_linear_int8_dynamic_f32(_p(x), x.size, m, k, _p(w_i8), w_i8.size, _p(w_scales), w_scales.size, n,
                                                  _p(bias), 0 if bias is None else bias.size, _p(out), out.size))
    return out


def _sdpa_masked(sfx, dtype, q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    q, k, v, mask = _slice(q, dtype), _slice(k, dtype), _slice(v, dtype), _slice(mask, dtype)
    out = np.empty(batch * h_q * seq_q * d_v, dtype=dtype)
    check(getattr(_lib.load(), "fth_sdpa_forward_masked_gqa_" + sfx)(_p(q), q.size, _p(k), k.size, _p(v), v.size, batch, h_q, h_kv, seq_q,
                                                                     seq_k, d_k, d_v, scale, _p(mask), mask.size, mask_bh_stride,
                                                                     _p(out), out.size))
    return out


def sdpa_forward_masked_f64(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    """crates/ft-kernel-cpu/src/lib.rs:4661."""
    q, k, v, mask = _slice(q, np.float64), _slice(k, np.float64), _slice(v, np.float64), _slice(mask, np.float64)
    out = np.empty(num_bh * seq_q * d_v, dtype=np.float64)
    check(_lib.load().fth_sdpa_forward_masked_f64(_p(q), q.size, _p(k), k.size, _p(v), v.size, num_bh, seq_q, seq_k, d_k, d_v, scale,
                                                  _p(mask), mask.size, mask_bh_stride, _p(out), out.size))
    return out


def sdpa_forward_masked_f32(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    """The f32 twin of sdpa_forward_masked_f64 (the reference has the f64 form only)."""
    q, k, v, mask = _slice(q, np.float32), _slice(k, np.float32), _slice(v, np.float32), _slice(mask, np.float32)
    out = np.empty(num_bh * seq_q * d_v, dtype=np.float32)
    check(_lib.load().fth_sdpa_forward_masked_f32(_p(q), q.size, _p(k), k.size, _p(v), v.size, num_bh, seq_q, seq_k, d_k, d_v, scale,
                                                  _p(mask), mask.size, mask_bh_stride, _p(out), out.size))
    return out


def sdpa_forward_masked_gqa_f64(q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    """crates/ft-kernel-cpu/src/lib.rs:4777."""
    return _sdpa_masked("f64", np.float64, q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride)


def sdpa_forward_masked_gqa_f32(q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride):
    return _sdpa_masked("f32", np.float32, q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride)


def sdpa_forward_f32(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    return _sdpa("fth_sdpa_forward_f32", np.float32, q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal)


def sdpa_forward_f64(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal):
    return _sdpa("fth_sdpa_forward_f64", np.float64, q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal)


def _transpose(name, dtype, src, batch, rows, cols, batched):
    src = _slice(src, dtype)
    total = batch * rows * cols
    out = np.empty(total if total < 2 ** 62 else 0, dtype=dtype)  # an overflowing extent is for the library to report
    fn = getattr(_lib.load(), name)
    if batched:
        check(fn(_p(src), src.size, batch, rows, cols, _p(out), out.size))
    else:
        check(fn(_p(src), src.size, _p(out), out.size, rows, cols))
    return out


def transpose_2d_f32(src, rows, cols):
    """src [rows, cols] -> [cols, rows] (transpose_2d_f32 / transpose_2d_into_f32, crates/ft-kernel-cpu/src/lib.rs:42406-42439)."""
    return _transpose("fth_transpose_2d_into_f32", np.float32, src, 1, rows, cols, False)


def transpose_2d_f64(src, rows, cols):
    return _transpose("fth_transpose_2d_into_f64", np.float64, src, 1, rows, cols, False)


def transpose_batched_materialize_f32(src, batch, rows, cols):
    """src [batch, rows, cols] -> [batch, cols, rows] (crates/ft-kernel-cpu/src/lib.rs:42526-42556)."""
    return _transpose("fth_transpose_batched_materialize_f32", np.float32, src, batch, rows, cols, True)


def transpose_batched_materialize_f64(src, batch, rows, cols):
    return _transpose("fth_transpose_batched_materialize_f64", np.float64, src, batch, rows, cols, True)
