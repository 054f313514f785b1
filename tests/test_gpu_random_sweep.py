"""Seeded random sweeps of the device entry points against float64 numpy restatements of the textbook operations.

The shapes, pitches, batch strides, offsets, epilogues and dtypes are drawn at random (fixed seeds), which reaches
combinations the hand-picked parity cases do not: odd pitches with padding between batches, [k, m] operands, every
epilogue with alpha != 1, sequence lengths on both sides of every kernel-selection threshold. The sweeps also check
that nothing outside the [m, n] window of a pitched output is written. Each case is printed before it runs.
"""
import math

import numpy as np
import pytest
from scipy.special import erf

from frankentorch_amd import device as D
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def rel(a, b):
    d = np.max(np.abs(a.astype(np.float64) - b)) if a.size else 0.0
    return d / max(1.0, np.max(np.abs(b)) if b.size else 1.0)


def dims(rng, lo, hi, mult=1):
    c = rng.integers(0, 4)
    if c == 0:
        v = int(rng.integers(lo, max(lo, min(hi, 40)) + 1))
    elif c == 1:
        v = int(rng.choice([32, 64, 96, 128, 192, 256, 384, 512, 768, 1024]))
    else:
        v = int(rng.integers(lo, hi + 1))
    v = min(v, hi)
    return max(mult, v // mult * mult)


def strided(flat, offset, rows, pitch):
    return np.lib.stride_tricks.as_strided(flat[offset:], (rows, pitch), (pitch * flat.itemsize, flat.itemsize))


@pytest.mark.parametrize("seed", [11, 12])
def test_gemm_random_shapes_pitches_and_epilogues(hip, seed):
    rng = np.random.default_rng(seed)
    for _ in range(60):
        dt = np.float32 if rng.random() < 0.7 else np.float64
        m, n, k = dims(rng, 1, 700), dims(rng, 1, 700), dims(rng, 1, 900)
        if rng.random() < 0.4:
            m, n, k = dims(rng, 1, 700, 4), dims(rng, 1, 700, 4), dims(rng, 1, 900, 32)
        batch = int(rng.choice([1, 1, 1, 2, 3, 9]))
        ta = bool(rng.random() < 0.25)
        tb = (not ta) and bool(rng.random() < 0.5)
        pad = lambda: int(rng.choice([0, 0, 4, 1, 7]))
        lda, ldb, ldc = (m if ta else k) + pad(), (k if tb else n) + pad(), n + pad()
        ra, rb = (k if ta else m), (n if tb else k)
        sa, sb, sc = ra * lda + pad(), rb * ldb + pad(), m * ldc + pad()
        epi = int(rng.choice([0, 0, 1, 3, 5, 9, 4, 7]))
        alpha = float(rng.choice([1.0, 1.0, 0.5, -2.0]))
        print("gemm", dict(dt=dt.__name__, m=m, n=n, k=k, batch=batch, ta=ta, tb=tb, lda=lda, ldb=ldb, ldc=ldc, sa=sa, sb=sb, sc=sc, epi=epi,
                           alpha=alpha), flush=True)
        A = rng.uniform(-1, 1, batch * sa + 8).astype(dt)
        B = rng.uniform(-1, 1, batch * sb + 8).astype(dt)
        bias = rng.uniform(-1, 1, n).astype(dt)
        res = rng.uniform(-1, 1, batch * sc + 8).astype(dt)
        c0 = np.full(batch * sc + 8, 777.0, dt)
        dA, dB, dC, dbias, dres = (DeviceBuffer.from_host(t) for t in (A, B, c0, bias, res))
        d = D.gemm_desc(m, n, k, trans_b=tb, batch=batch, epilogue=epi, lda=lda, ldb=ldb, ldc=ldc, stride_a=sa, stride_b=sb, stride_c=sc,
                        trans_a=ta)
        hip.gemm(d, dA, dB, dC, bias=dbias if epi & 1 else None, residual=dres if epi & 4 else None, alpha=alpha)
        ref = c0.astype(np.float64).copy()
        for b in range(batch):
            a2 = strided(A, b * sa, ra, lda)[:, : (m if ta else k)].astype(np.float64)
            b2 = strided(B, b * sb, rb, ldb)[:, : (k if tb else n)].astype(np.float64)
            r = alpha * ((a2.T if ta else a2) @ (b2.T if tb else b2))
            if epi & 1:
                r = r + bias.astype(np.float64)
            if epi & 2:
                r = 0.5 * r * (1 + erf(r / math.sqrt(2)))
            if epi & 8:
                r = 0.5 * r * (1 + np.tanh(math.sqrt(2 / math.pi) * (r + 0.044715 * r**3)))
            if epi & 4:
                r = r + strided(res, b * sc, m, ldc)[:, :n].astype(np.float64)
            strided(ref, b * sc, m, ldc)[:, :n] = r
        # the 777 fill outside the [m, n] windows must survive: err covers the whole buffer
        assert rel(dC.to_host(), ref) <= (2e-5 if dt == np.float32 else 1e-12) * max(1.0, math.sqrt(k) / 4)


@pytest.mark.parametrize("seed", [21, 22])
def test_sdpa_forward_and_backward_random_shapes(hip, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        dt = np.float32 if rng.random() < 0.6 else np.float64
        bh = int(rng.integers(1, 7)) if rng.random() < 0.6 else int(rng.integers(20, 60))  # few / many query blocks: both fp32 kernels
        sq = dims(rng, 1, 600)
        sk = sq if rng.random() < 0.6 else dims(rng, 1, 600)
        dk = int(rng.choice([32, 64, 128, 16, 40, 8, 96]))
        dv = dk if rng.random() < 0.7 else int(rng.choice([32, 64, 128, 24]))
        causal, masked = bool(rng.random() < 0.5), bool(rng.random() < 0.3)
        print("sdpa", dict(dt=dt.__name__, bh=bh, sq=sq, sk=sk, dk=dk, dv=dv, causal=causal, masked=masked), flush=True)
        q = rng.normal(size=(bh, sq, dk)).astype(dt)
        k = rng.normal(size=(bh, sk, dk)).astype(dt)
        v = rng.normal(size=(bh, sk, dv)).astype(dt)
        s = 1 / math.sqrt(dk)
        sc = np.einsum("bqd,bkd->bqk", q.astype(np.float64), k.astype(np.float64)) * s
        mask = None
        if masked:
            mask = np.where(rng.random((bh, sq, sk)) < 0.2, -np.inf, rng.normal(size=(bh, sq, sk))).astype(dt)
            mask[:, :, 0] = 0  # no fully hidden row
            sc = sc + mask.astype(np.float64)
        if causal:
            sc = np.where(np.arange(sk)[None, None, :] <= np.arange(sq)[None, :, None], sc, -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        p = p / p.sum(-1, keepdims=True)
        tol = 2e-5 if dt == np.float32 else 1e-12
        dq_, dk_, dv_ = (DeviceBuffer.from_host(t) for t in (q, k, v))
        o = DeviceBuffer((bh, sq, dv), dt)
        d = D.sdpa_desc_contiguous(bh, sq, sk, dk, dv, causal)
        if masked:
            hip.sdpa_forward_masked(d, s, dq_, dk_, dv_, DeviceBuffer.from_host(mask), sq * sk, o)
        else:
            hip.sdpa_forward(d, s, dq_, dk_, dv_, o)
        assert rel(o.to_host(), np.einsum("bqk,bkd->bqd", p, v.astype(np.float64))) <= tol
        if not masked and rng.random() < 0.5:
            do = rng.normal(size=(bh, sq, dv)).astype(dt)
            dP = np.einsum("bqd,bkd->bqk", do.astype(np.float64), v.astype(np.float64))
            dU = p * (dP - (p * dP).sum(-1, keepdims=True))
            refs = (s * np.einsum("bqk,bkd->bqd", dU, k.astype(np.float64)), s * np.einsum("bqk,bqd->bkd", dU, q.astype(np.float64)),
                    np.einsum("bqk,bqd->bkd", p, do.astype(np.float64)))
            gq, gk, gv = DeviceBuffer(q.shape, dt), DeviceBuffer(k.shape, dt), DeviceBuffer(v.shape, dt)
            hip.sdpa_backward(dq_, dk_, dv_, DeviceBuffer.from_host(do), bh, sq, sk, dk, dv, s, causal, gq, gk, gv)
            for g, r in zip((gq, gk, gv), refs):
                assert rel(g.to_host(), r) <= 2 * tol


@pytest.mark.parametrize("seed", [31])
def test_row_and_loss_kernels_random_shapes(hip, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        dt = np.float32 if rng.random() < 0.7 else np.float64
        rows = dims(rng, 1, 200)
        cols = dims(rng, 1, 9000) if rng.random() < 0.7 else int(rng.integers(9000, 140000))
        if rows * cols > 2e7:
            rows = max(1, int(2e7 // cols))
        print("rows", dict(dt=dt.__name__, rows=rows, cols=cols), flush=True)
        x = (rng.normal(size=(rows, cols)) * 2).astype(dt)
        w = rng.uniform(0.5, 1.5, cols).astype(dt)
        b = rng.normal(size=cols).astype(dt)
        x64 = x.astype(np.float64)
        dx, dw, db = (DeviceBuffer.from_host(t) for t in (x, w, b))
        y = DeviceBuffer((rows, cols), dt)
        tol = 1e-5 if dt == np.float32 else 1e-12
        hip.softmax_lastdim(dx, y, rows, cols)
        e = np.exp(x64 - x64.max(1, keepdims=True))
        assert rel(y.to_host(), e / e.sum(1, keepdims=True)) <= tol
        hip.layer_norm(dx, dw, db, y, rows, cols, 1e-5)
        assert rel(y.to_host(), (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5) * w + b) <= 4 * tol
        hip.rms_norm(dx, dw, y, rows, cols, 1e-6)
        assert rel(y.to_host(), x64 / np.sqrt((x64**2).mean(1, keepdims=True) + 1e-6) * w) <= 4 * tol
        hip.bias_residual_add(dx, db, dx, y, rows, cols)
        assert np.array_equal(y.to_host(), (x + b) + x)
        out = DeviceBuffer((rows,), dt)
        hip.argmax(dx, rows, cols, 1, out)
        assert np.array_equal(out.to_host(), x.argmax(1).astype(dt))
        tgt = rng.integers(0, cols, rows).astype(np.int64)
        g = rng.normal(size=rows).astype(dt)
        dtg, dg, loss = DeviceBuffer.from_host(tgt), DeviceBuffer.from_host(g), DeviceBuffer((rows,), dt)
        m = x64.max(1, keepdims=True)
        lse = m + np.log(np.exp(x64 - m).sum(1, keepdims=True))
        hip.log_softmax_strided(dx, y, rows, cols, 1)
        assert rel(y.to_host(), x64 - lse) <= tol
        hip.cross_entropy_forward(dx, dtg, rows, cols, loss)
        assert rel(loss.to_host(), lse[:, 0] - x64[np.arange(rows), tgt]) <= tol
        hip.cross_entropy_backward(dx, dtg, dg, rows, cols, y)
        r = np.exp(x64 - lse)
        r[np.arange(rows), tgt] -= 1
        assert rel(y.to_host(), r * g.astype(np.float64)[:, None]) <= tol


@pytest.mark.parametrize("seed", [41])
def test_int8_linear_random_shapes_bit_exact(hip, seed):
    rng = np.random.default_rng(seed)
    for _ in range(50):
        m, n = dims(rng, 1, 600), dims(rng, 1, 600)
        k = dims(rng, 1, 1200) if rng.random() < 0.5 else dims(rng, 64, 1280, 64)
        print("int8", dict(m=m, n=n, k=k), flush=True)
        x = rng.normal(size=(m, k)).astype(np.float32)
        wq = rng.integers(-127, 128, (n, k), dtype=np.int8)
        ws = rng.uniform(0.001, 0.02, n).astype(np.float32)
        bias = rng.normal(size=n).astype(np.float32)
        amax = np.abs(x).max(1)
        sc = np.where(amax > 0, amax / np.float32(127), np.float32(1)).astype(np.float32)
        xq = np.clip(np.rint(x / sc[:, None]), -127, 127).astype(np.int32)
        ref = ((xq @ wq.astype(np.int32).T).astype(np.float32) * sc[:, None]) * ws[None, :] + bias
        out = DeviceBuffer((m, n))
        hip.linear_int8_dynamic(DeviceBuffer.from_host(x), m, k, DeviceBuffer.from_host(wq), DeviceBuffer.from_host(ws), n,
                                DeviceBuffer.from_host(bias), out)
        assert np.array_equal(out.to_host().view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("seed", [71])
def test_small_problem_kernels_random_shapes(hip, seed):
    """The latency-oriented kernels: key-split attention (few query blocks, up to 4096 keys, head size 32 / 64) and the
    16 x 16-tile GEMM for reductions of 512 and more, NT and NN, batched, with every epilogue."""
    rng = np.random.default_rng(seed)
    for _ in range(40):
        bh, sq = int(rng.integers(1, 5)), int(rng.integers(1, 300))
        sk = int(rng.integers(1, 4097)) if rng.random() < 0.5 else sq
        dk, causal = int(rng.choice([32, 64])), bool(rng.random() < 0.5)
        print("sdpa_small", dict(bh=bh, sq=sq, sk=sk, d=dk, causal=causal), flush=True)
        q, k, v = (rng.normal(size=(bh, n, dk)).astype(np.float32) for n in (sq, sk, sk))
        s = 1 / math.sqrt(dk)
        sc = np.einsum("bqd,bkd->bqk", q.astype(np.float64), k.astype(np.float64)) * s
        if causal:
            sc = np.where(np.arange(sk)[None, None, :] <= np.arange(sq)[None, :, None], sc, -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        o = DeviceBuffer((bh, sq, dk))
        hip.sdpa_forward(D.sdpa_desc_contiguous(bh, sq, sk, dk, dk, causal), s, DeviceBuffer.from_host(q), DeviceBuffer.from_host(k),
                         DeviceBuffer.from_host(v), o)
        assert rel(o.to_host(), np.einsum("bqk,bkd->bqd", p, v.astype(np.float64))) <= 2e-5
    for _ in range(60):
        m, n, k = int(rng.integers(1, 300)), int(rng.integers(1, 300)), int(rng.integers(32, 257)) * 16
        tb = bool(rng.random() < 0.6)
        if not tb:
            n = max(4, n // 4 * 4)
        if 2.0 * m * n * k > 4e8:
            continue
        batch, epi = int(rng.choice([1, 1, 2, 5])), int(rng.choice([0, 1, 3, 5, 9]))
        print("gemm_small16", dict(m=m, n=n, k=k, tb=tb, batch=batch, epi=epi), flush=True)
        A = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (batch, n, k) if tb else (batch, k, n)).astype(np.float32)
        bias, res = rng.uniform(-1, 1, n).astype(np.float32), rng.uniform(-1, 1, (batch, m, n)).astype(np.float32)
        c = DeviceBuffer((batch, m, n))
        hip.gemm(D.gemm_desc(m, n, k, trans_b=tb, batch=batch, epilogue=epi), DeviceBuffer.from_host(A), DeviceBuffer.from_host(B), c,
                 bias=DeviceBuffer.from_host(bias) if epi & 1 else None, residual=DeviceBuffer.from_host(res) if epi & 4 else None)
        r = A.astype(np.float64) @ (np.swapaxes(B, 1, 2) if tb else B).astype(np.float64)
        if epi & 1:
            r = r + bias
        if epi & 2:
            r = 0.5 * r * (1 + erf(r / math.sqrt(2)))
        if epi & 8:
            r = 0.5 * r * (1 + np.tanh(math.sqrt(2 / math.pi) * (r + 0.044715 * r**3)))
        if epi & 4:
            r = r + res
        assert rel(c.to_host(), r) <= 2e-5 * max(1.0, math.sqrt(k) / 4)


@pytest.mark.parametrize("seed", [81])
def test_linear_argmax_random_shapes_equal_the_plain_argmax(hip, seed):
    """Shapes on both sides of every condition of the one-pass path (tile count against the compute units, K a multiple of
    32 or not, ragged last tiles, one row), small-integer operands so that equal logits are the rule, and a few rows that
    carry inf / NaN through the product: the indices must be those of the plain argmax kernel on the logits written."""
    rng = np.random.default_rng(seed)
    for it in range(24):
        big = it % 3 != 2
        k = int(rng.choice([32, 64, 96, 160, 256])) if rng.random() < 0.8 else int(rng.integers(1, 200))
        if big:
            rows = int(rng.integers(300, 2600))
            n_lo = 128 * -(-256 // -(-rows // 128))  # where a 256-compute-unit part has one 128 x 128 tile per unit
            n = int(rng.integers(n_lo - 600, n_lo + 3000))
        else:
            rows, n = int(rng.integers(1, 300)), int(rng.integers(1, 3000))
        print("linear_argmax", dict(rows=rows, n=n, k=k), flush=True)
        x = rng.integers(-1, 2, size=(rows, k)).astype(np.float32)
        w = rng.integers(-1, 2, size=(n, k)).astype(np.float32)
        for r in rng.integers(0, rows, size=min(rows, 6)):
            x[r, rng.integers(0, k)] = rng.choice(np.array([np.inf, -np.inf, np.nan, 3e38], np.float32))
        nws = hip.linear_argmax_workspace_floats(rows, n)
        ws = DeviceBuffer.from_host(np.full(nws, 4321.0, np.float32))
        dx, dw = DeviceBuffer.from_host(x), DeviceBuffer.from_host(w)
        logits, idx, ref_idx = DeviceBuffer((rows, n)), DeviceBuffer((rows,)), DeviceBuffer((rows,))
        hip.linear_argmax(dx, dw, rows, n, k, logits, idx, workspace=ws)
        hip.argmax(logits, rows, n, 1, ref_idx)
        assert np.array_equal(idx.to_host(), ref_idx.to_host())
        got = logits.to_host()
        plain = DeviceBuffer((rows, n))
        hip.gemm(hip.gemm_desc(rows, n, k, trans_b=True), dx, dw, plain)
        assert np.array_equal(got, plain.to_host(), equal_nan=True)
        took_one_pass = not np.all(ws.to_host() == 4321.0)
        tiles = -(-rows // 128) * -(-n // 128)
        assert took_one_pass == (tiles >= hip.device_info()["compute_units"] and k % 32 == 0), (tiles, k)
