"""Resident-tensor tier, the shape of `ft_kernel_metal::fused`: `HipTensor` (GpuTensor), `Batch`,
`EncoderHip` (EncoderGpu) and the GPT-2-shaped `Gpt2Hip`. Activations stay in HBM between ops;
`Batch.finish()` / `download()` are the only synchronisation points
(crates/ft-kernel-metal/src/fused.rs:540-933, 986-1190).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import numpy as np

from . import _lib
from .core import check
from .device import DeviceBuffer, is_available  # noqa: F401  (re-exported: fused::is_available)

LAYER_KEYS = ("ln1_w", "ln1_b", "wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "ln2_w", "ln2_b", "w1", "b1", "w2", "b2")


class HipTensor:
    """A resident f32 [rows, cols] matrix (GpuTensor, fused.rs:540-580)."""

    def __init__(self, handle: int):
        self._h = handle

    @classmethod
    def upload(cls, data, rows: Optional[int] = None, cols: Optional[int] = None) -> "HipTensor":
        a = np.ascontiguousarray(data, dtype=np.float32)
        if rows is None or cols is None:
            if a.ndim == 1:
                rows, cols = 1, a.size
            else:
                rows, cols = int(np.prod(a.shape[:-1], dtype=np.int64)), a.shape[-1]
        if rows * cols != a.size:
            raise ValueError("upload: %d elements do not fill [%d, %d]" % (a.size, rows, cols))
        h = C.c_void_p()
        check(_lib.load().fth_tensor_upload(a.ctypes.data, rows, cols, C.byref(h)))
        return cls(h.value)

    @property
    def shape(self):
        r, c = C.c_int64(), C.c_int64()
        check(_lib.load().fth_tensor_shape(self._h, C.byref(r), C.byref(c)))
        return (r.value, c.value)

    @property
    def data_ptr(self) -> int:
        return _lib.load().fth_tensor_data(self._h) or 0

    def download(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=np.float32)
        check(_lib.load().fth_tensor_download(self._h, out.ctypes.data, out.size))
        return out

    def free(self) -> None:
        if self._h:
            _lib.load().fth_tensor_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _h(t: Optional[HipTensor]):
    return None if t is None else t._h


class Batch:
    """Stream-ordered op batch (Batch, fused.rs:676-932). Each op returns a fresh resident tensor."""

    def __init__(self):
        h = C.c_void_p()
        check(_lib.load().fth_batch_new(C.byref(h)))
        self._b = h.value

    def _op(self, fn, *args) -> HipTensor:
        out = C.c_void_p()
        check(fn(self._b, *args, C.byref(out)))
        return HipTensor(out.value)

    def matmul_bias(self, a: HipTensor, w: HipTensor, bias: Optional[HipTensor] = None) -> HipTensor:
        """a[m,k] . w[n,k]^T (+ bias[n]); w in nn.Linear's [out, in] layout."""
        return self._op(_lib.load().fth_batch_linear, _h(a), _h(w), _h(bias))

    def matmul(self, a: HipTensor, rhs: HipTensor) -> HipTensor:
        return self._op(_lib.load().fth_batch_matmul, _h(a), _h(rhs))

    def layernorm(self, x, gamma, beta, eps: float) -> HipTensor:
        return self._op(_lib.load().fth_batch_layernorm, _h(x), _h(gamma), _h(beta), eps)

    def rmsnorm(self, x, gamma, eps: float) -> HipTensor:
        return self._op(_lib.load().fth_batch_rmsnorm, _h(x), _h(gamma), eps)

    def gelu(self, x) -> HipTensor:
        return self._op(_lib.load().fth_batch_gelu, _h(x))

    def gelu_tanh(self, x) -> HipTensor:
        return self._op(_lib.load().fth_batch_gelu_tanh, _h(x))

    def add(self, a, b) -> HipTensor:
        return self._op(_lib.load().fth_batch_add, _h(a), _h(b))

    def softmax(self, x) -> HipTensor:
        return self._op(_lib.load().fth_batch_softmax, _h(x))

    def mha(self, q, k, v, n_heads: int, batch: int = 1, causal: bool = False) -> HipTensor:
        return self._op(_lib.load().fth_batch_mha, _h(q), _h(k), _h(v), n_heads, batch, 1 if causal else 0)

    def finish(self) -> None:
        check(_lib.load().fth_batch_finish(self._b))

    def __del__(self):
        try:
            _lib.load().fth_batch_free(self._b)
        except Exception:
            pass


def _pack_layers(layers: Sequence[dict]):
    arr = (_lib.LayerWeights * max(1, len(layers)))()
    keep = []
    for i, lw in enumerate(layers):
        for key in LAYER_KEYS:
            v = lw.get(key)
            if v is None:
                setattr(arr[i], key, None)
            else:
                a = np.ascontiguousarray(v, dtype=np.float32)
                keep.append(a)
                setattr(arr[i], key, a.ctypes.data)
    return arr, keep


class EncoderHip:
    """Pre-LN transformer stack with resident weights (EncoderGpu, fused.rs:1024-1190)."""

    def __init__(self, d_model: int, n_heads: int, d_ff: int, layers: Sequence[dict], ln_eps: float = 1e-5,
                 causal: bool = True, gelu_tanh: bool = False):
        """gelu_tanh: the tanh form the Metal encoder computes (fused.rs:301-313) in place of ft-kernel-cpu's erf form."""
        self.d_model, self.n_heads, self.d_ff = d_model, n_heads, d_ff
        arr, keep = _pack_layers(layers)
        h = C.c_void_p()
        check(_lib.load().fth_encoder_new(d_model, n_heads, d_ff, ln_eps, 1 if causal else 0, arr, len(layers), C.byref(h)))
        self._e = h.value
        del keep
        if gelu_tanh:
            check(_lib.load().fth_encoder_set_activation(self._e, 1))

    def forward(self, x, batch: int, seq: int) -> np.ndarray:
        """Host in, host out."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty((batch * seq, self.d_model), dtype=np.float32)
        check(_lib.load().fth_encoder_forward(self._e, x.ctypes.data, batch, seq, out.ctypes.data, out.size))
        return out

    def forward_dev(self, x: DeviceBuffer, out: DeviceBuffer, batch: int, seq: int, stream=None, graph: bool = False):
        """Resident in, resident out, no synchronisation; graph=True replays a captured HIP graph."""
        fn = _lib.load().fth_encoder_forward_graph if graph else _lib.load().fth_encoder_forward_dev
        check(fn(self._e, x.ptr, batch, seq, out.ptr, stream))

    def __del__(self):
        try:
            _lib.load().fth_encoder_free(self._e)
        except Exception:
            pass


class Gpt2Hip:
    """GPT-2-shaped decoder: learned positions, pre-LN causal blocks, final LN, tied LM head."""

    def __init__(self, wte, wpe, layers: Sequence[dict], lnf_w, lnf_b, n_heads: int, ln_eps: float = 1e-5,
                 gelu_tanh: bool = False):
        wte = np.ascontiguousarray(wte, dtype=np.float32)
        wpe = np.ascontiguousarray(wpe, dtype=np.float32)
        self.vocab, self.d_model = wte.shape
        self.max_pos = wpe.shape[0]
        d_ff = layers[0]["w1"].shape[0] if layers else self.d_model
        arr, keep = _pack_layers(layers)
        lw = None if lnf_w is None else np.ascontiguousarray(lnf_w, dtype=np.float32)
        lb = None if lnf_b is None else np.ascontiguousarray(lnf_b, dtype=np.float32)
        h = C.c_void_p()
        check(_lib.load().fth_gpt2_new(self.vocab, self.max_pos, self.d_model, n_heads, d_ff, ln_eps, wte.ctypes.data,
                                       wpe.ctypes.data, arr, len(layers), None if lw is None else lw.ctypes.data,
                                       None if lb is None else lb.ctypes.data, C.byref(h)))
        self._g = h.value
        del keep
        if gelu_tanh:  # GPT-2 checkpoints were trained with the tanh form
            check(_lib.load().fth_gpt2_set_activation(self._g, 1))

    @classmethod
    def from_safetensors(cls, source, n_heads: int, ln_eps: float = 1e-5, gelu_tanh: bool = True) -> "Gpt2Hip":
        """A GPT-2 checkpoint (path, bytes or an open serialize.SafeTensorsFile) straight into resident buffers: Conv1D
        weights are transposed and F16 / BF16 / F64 tensors converted on the GPU while loading."""
        from .serialize import SafeTensorsFile

        f = source if isinstance(source, SafeTensorsFile) else SafeTensorsFile(source)
        h = C.c_void_p()
        check(_lib.load().fth_gpt2_from_safetensors(f._h, n_heads, ln_eps, 1 if gelu_tanh else 0, C.byref(h)))
        self = cls.__new__(cls)
        self._g = h.value
        dims = [C.c_int64() for _ in range(6)]
        check(_lib.load().fth_gpt2_dims(self._g, *[C.byref(d) for d in dims]))
        self.vocab, self.max_pos, self.d_model, self.n_heads, self.d_ff, self.n_layers = (d.value for d in dims)
        return self

    @classmethod
    def from_state_dict(cls, source, n_heads: int, ln_eps: float = 1e-5, gelu_tanh: bool = True) -> "Gpt2Hip":
        """The same from a native state-dict container ("FTSV"; path, bytes or an open serialize.StateDictFile)."""
        from .serialize import StateDictFile

        return cls.from_safetensors(source if isinstance(source, StateDictFile) else StateDictFile(source), n_heads, ln_eps, gelu_tanh)

    def forward_dev(self, ids: DeviceBuffer, batch: int, seq: int, logits: Optional[DeviceBuffer],
                    argmax: Optional[DeviceBuffer], stream=None) -> None:
        check(_lib.load().fth_gpt2_forward_dev(self._g, ids.ptr, batch, seq, None if logits is None else logits.ptr,
                                               None if argmax is None else argmax.ptr, stream))

    def hidden(self, tokens: int) -> np.ndarray:
        """Final hidden state [tokens, d_model] of the last forward (synchronises)."""
        out = np.empty((tokens, self.d_model), dtype=np.float32)
        ptr = _lib.load().fth_gpt2_hidden_dev(self._g)
        check(_lib.load().fth_memcpy_d2h(out.ctypes.data, ptr, out.nbytes))
        return out

    def bad_index(self) -> int:
        pos = C.c_int64()
        check(_lib.load().fth_gpt2_bad_index(self._g, C.byref(pos)))
        return pos.value

    def __del__(self):
        try:
            _lib.load().fth_gpt2_free(self._g)
        except Exception:
            pass
