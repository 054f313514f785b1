"""Seeded random sweep of the host-slice entry points (the ft_kernel_cpu-named functions) against float64 numpy restatements:
random ranks, reduce dims, storage offsets and trailing storage, both dtypes. Each case is printed before it runs."""
import math

import numpy as np
import pytest
from scipy.special import erf

from frankentorch_amd.core import DType, TensorMeta

pytestmark = pytest.mark.gpu


def rel(a, b):
    a = np.asarray(a).ravel()
    d = np.max(np.abs(a.astype(np.float64) - np.asarray(b).ravel())) if a.size else 0.0
    return d / max(1.0, np.max(np.abs(b)) if np.asarray(b).size else 1.0)


def meta(shape, off, dt):
    strides = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
    return TensorMeta.from_shape_and_strides(shape, strides, off, DType.F32 if dt == np.float32 else DType.F64)


def store(rng, shape, off, dt, lo=-1.0, hi=1.0):
    """A storage slice with `off` leading and a few trailing elements around the tensor, and the tensor in float64."""
    n = int(np.prod(shape))
    s = rng.uniform(lo, hi, off + n + int(rng.integers(0, 5))).astype(dt)
    return s, s[off:off + n].reshape(shape).astype(np.float64)


@pytest.mark.parametrize("seed", [51, 52])
def test_host_slice_entry_points_random_shapes_and_offsets(hip, seed):
    from frankentorch_amd import kernel_hip as K

    rng = np.random.default_rng(seed)
    for _ in range(40):
        dt = np.float32 if rng.random() < 0.6 else np.float64
        sfx = "f32" if dt == np.float32 else "f64"
        tol = 2e-5 if dt == np.float32 else 1e-12
        off1, off2, off3 = (int(rng.integers(0, 4)) * int(rng.integers(0, 2)) for _ in range(3))
        m, n, k = (int(rng.integers(1, 90)) for _ in range(3))
        b = int(rng.integers(1, 12))
        print("host", dict(dt=sfx, m=m, n=n, k=k, b=b, offs=(off1, off2, off3)), flush=True)
        A, a = store(rng, (m, k), off1, dt)
        B, b_ = store(rng, (k, n), off2, dt)
        assert rel(getattr(K, "matmul_tensor_contiguous_" + sfx)(A, B, meta((m, k), off1, dt), meta((k, n), off2, dt)), a @ b_) <= tol
        A3, a3 = store(rng, (b, m, k), off1, dt)
        B3, b3 = store(rng, (b, k, n), off2, dt)
        assert rel(getattr(K, "bmm_tensor_contiguous_" + sfx)(A3, B3, meta((b, m, k), off1, dt), meta((b, k, n), off2, dt)), a3 @ b3) <= tol
        two_d = rng.random() < 0.5
        ishape = (m, n) if two_d else (n,)
        I, i_ = store(rng, ishape, off3, dt)
        beta, alpha = float(rng.choice([1.0, 0.0, 0.5, -1.5])), float(rng.choice([1.0, 0.0, 2.0]))
        got = getattr(K, "addmm_tensor_contiguous_" + sfx)(I, A, B, meta(ishape, off3, dt), meta((m, k), off1, dt), meta((k, n), off2, dt), beta, alpha)
        assert rel(got, beta * np.broadcast_to(i_, (m, n)) + alpha * (a @ b_)) <= 2 * tol
        W, w = store(rng, (n, k), 0, dt)
        bias = rng.uniform(-1, 1, n).astype(dt)
        use_bias = rng.random() < 0.5
        got = getattr(K, "linear_tensor_" + sfx)(A[off1:off1 + m * k], W[:n * k], bias if use_bias else None, m, k, n)
        assert rel(got, a @ w.T + (bias.astype(np.float64) if use_bias else 0)) <= tol
        assert rel(getattr(K, "matmul_rhs_transposed_contiguous_" + sfx)(m, k, n, A[off1:off1 + m * k], W[:n * k]), a @ w.T) <= tol
        # ops over one dim of a rank-1..4 tensor
        shape = [int(rng.integers(1, 9)) for _ in range(int(rng.integers(1, 5)))]
        if rng.random() < 0.3:
            shape[int(rng.integers(0, len(shape)))] = int(rng.integers(30, 300))
        dim = int(rng.integers(0, len(shape)))
        X, x = store(rng, shape, off1, dt, -3, 3)
        print("dimops", dict(dt=sfx, shape=shape, dim=dim, off=off1), flush=True)
        e = np.exp(x - x.max(dim, keepdims=True))
        sm = e / e.sum(dim, keepdims=True)
        rtol = 1e-5 if dt == np.float32 else 1e-12
        mt = meta(shape, off1, dt)
        assert rel(getattr(K, "softmax_dim_tensor_contiguous_" + sfx)(X, mt, dim), sm) <= rtol
        assert rel(getattr(K, "log_softmax_dim_tensor_contiguous_" + sfx)(X, mt, dim), np.log(sm)) <= 4 * rtol
        xs = X[off1:off1 + int(np.prod(shape))].reshape(shape)
        got = np.asarray(getattr(K, "argmax_dim_tensor_contiguous_" + sfx)(X, mt, dim), dtype=np.float64)
        assert np.array_equal(got, xs.argmax(dim).ravel().astype(np.float64))
        idx = rng.integers(0, shape[dim], int(rng.integers(0, 20))).astype(np.float64)
        got = getattr(K, "index_select_tensor_contiguous_" + sfx)(X, mt, dim, idx)
        assert np.array_equal(np.asarray(got), np.take(xs, idx.astype(np.int64), axis=dim).ravel())
        assert rel(getattr(K, "gelu_tensor_contiguous_" + sfx)(X, mt), 0.5 * x * (1 + erf(x / math.sqrt(2)))) <= rtol
        tanh_ref = 0.5 * x * (1 + np.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x**3)))
        assert rel(getattr(K, "gelu_tanh_tensor_contiguous_" + sfx)(X, mt), tanh_ref) <= rtol
        Y, _ = store(rng, shape, off2, dt)
        got = getattr(K, "add_tensor_contiguous_" + sfx)(X, Y, mt, meta(shape, off2, dt))
        assert np.array_equal(np.asarray(got), (xs + Y[off2:off2 + xs.size].reshape(shape)).ravel())


@pytest.mark.parametrize("seed", [61])
def test_resident_batch_ops_random_shapes(hip, seed):
    """The stream-ordered batch of resident tensors (the ft_kernel_metal::fused surface): random shapes through a chain
    x -> LayerNorm -> linear(+bias) -> GELU -> linear -> add -> softmax, and multi-head attention over [batch * seq, d_model] rows
    with random head counts, against float64 numpy restatements."""
    from frankentorch_amd.fused import Batch, HipTensor

    rng = np.random.default_rng(seed)
    for _ in range(25):
        m, d, f = int(rng.integers(1, 200)), int(rng.choice([8, 24, 64, 100, 256])), int(rng.choice([16, 40, 128, 300]))
        print("batch chain", dict(m=m, d=d, f=f), flush=True)
        x = rng.normal(size=(m, d)).astype(np.float32)
        g, be = rng.uniform(0.5, 1.5, d).astype(np.float32), rng.normal(size=d).astype(np.float32)
        w1, b1 = (rng.normal(size=(f, d)) * 0.2).astype(np.float32), rng.normal(size=f).astype(np.float32)
        w2 = (rng.normal(size=(d, f)) * 0.2).astype(np.float32)
        bt = Batch()
        tx = HipTensor.upload(x)
        h = bt.layernorm(tx, HipTensor.upload(g, 1, d), HipTensor.upload(be, 1, d), 1e-5)
        h = bt.gelu(bt.matmul_bias(h, HipTensor.upload(w1), HipTensor.upload(b1, 1, f)))
        y = bt.softmax(bt.add(bt.matmul_bias(h, HipTensor.upload(w2)), tx))
        bt.finish()
        x64 = x.astype(np.float64)
        r = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5) * g + be
        r = r @ w1.T.astype(np.float64) + b1
        r = 0.5 * r * (1 + erf(r / math.sqrt(2)))
        r = r @ w2.T.astype(np.float64) + x64
        e = np.exp(r - r.max(1, keepdims=True))
        assert rel(y.download(), e / e.sum(1, keepdims=True)) <= 4e-5

        heads = int(rng.choice([1, 2, 4]))
        hd = int(rng.choice([16, 32, 64]))
        batch, seq = int(rng.integers(1, 4)), int(rng.integers(1, 150))
        causal = bool(rng.random() < 0.5)
        print("batch mha", dict(heads=heads, hd=hd, batch=batch, seq=seq, causal=causal), flush=True)
        dm = heads * hd
        q, k, v = (rng.normal(size=(batch * seq, dm)).astype(np.float32) for _ in range(3))
        bt = Batch()
        o = bt.mha(HipTensor.upload(q), HipTensor.upload(k), HipTensor.upload(v), heads, batch, causal)
        bt.finish()
        split = lambda t: t.astype(np.float64).reshape(batch, seq, heads, hd).transpose(0, 2, 1, 3)
        sc = np.einsum("bhqd,bhkd->bhqk", split(q), split(k)) / math.sqrt(hd)
        if causal:
            sc = np.where(np.arange(seq)[None, None, None, :] <= np.arange(seq)[None, None, :, None], sc, -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        ref = np.einsum("bhqk,bhkd->bhqd", p, split(v)).transpose(0, 2, 1, 3).reshape(batch * seq, dm)
        assert rel(o.download(), ref) <= 2e-5
