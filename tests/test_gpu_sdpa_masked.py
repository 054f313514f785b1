"""Masked and grouped-query SDPA against the CPU checker: softmax(scale * q k^T + mask) v with an additive mask shared
by all heads or given per head, K/V heads shared by groups of query heads. fp32 <= 2e-5, fp64 <= 1e-12."""
import math

import numpy as np
import pytest

from conftest import TOL_F64, TOL_GEMM_F32, rel_err
from frankentorch_amd import kernel_hip as K
from frankentorch_amd import synth
from frankentorch_amd.core import HipError
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def _inputs(seed, batch, h_q, h_kv, sq, sk, dk, dv, dtype):
    q = synth.normal(seed, "q", (batch, h_q, sq, dk), 0.0, 1.0).astype(dtype)
    k = synth.normal(seed, "k", (batch, h_kv, sk, dk), 0.0, 1.0).astype(dtype)
    v = synth.normal(seed, "v", (batch, h_kv, sk, dv), 0.0, 1.0).astype(dtype)
    return q, k, v


def _mask(seed, kind, num_bh, sq, sk, dtype):
    """shared / per-head additive masks: a soft bias everywhere, with some keys hidden by -inf."""
    shape = (sq, sk) if kind == "shared" else (num_bh, sq, sk)
    m = synth.normal(seed, "mask", shape, 0.0, 0.5).astype(dtype)
    hide = synth.uniform(seed, "hide", shape) < 0.3
    hide[..., 0] = False  # keep one key per row visible
    m[hide] = -np.inf
    return m


def _run(hip, q, k, v, scale, mask, causal=False):
    batch, h_q, sq, dk = q.shape
    h_kv, sk, dv = k.shape[1], k.shape[2], v.shape[3]
    bufs = [DeviceBuffer.from_host(t) for t in (q, k, v, mask)]
    out = DeviceBuffer((batch, h_q, sq, dv), q.dtype)
    desc = hip.sdpa_desc_gqa(batch, h_q, h_kv, sq, sk, dk, dv, causal)
    hip.sdpa_forward_masked(desc, scale, bufs[0], bufs[1], bufs[2], bufs[3], 0 if mask.ndim == 2 else sq * sk, out)
    return out.to_host()


# (batch, h_q, h_kv, seq_q, seq_k, d_k, d_v): MFMA head sizes with and without grouping, ragged tails, seq_k not a
# multiple of four (scalar mask reads), and shapes that take the generic kernel
SHAPES = [(2, 8, 2, 40, 40, 64, 64), (1, 4, 4, 130, 77, 64, 64), (2, 6, 3, 100, 100, 128, 128), (1, 8, 1, 77, 130, 32, 32),
          (2, 4, 2, 129, 131, 128, 128), (2, 8, 2, 40, 40, 16, 16), (1, 2, 1, 33, 50, 48, 24), (1, 16, 8, 256, 256, 64, 64)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("kind", ["shared", "per_head"])
def test_masked_gqa_f32_matches_oracle(hip, oracle, shape, kind):
    batch, h_q, h_kv, sq, sk, dk, dv = shape
    q, k, v = _inputs(7, *shape, np.float32)
    mask = _mask(7, kind, batch * h_q, sq, sk, np.float32)
    scale = np.float32(1.0 / math.sqrt(dk))
    got = _run(hip, q, k, v, scale, mask)
    assert rel_err(got, oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask)) <= TOL_GEMM_F32
    assert np.array_equal(got.view(np.uint32), _run(hip, q, k, v, scale, mask).view(np.uint32))


@pytest.mark.parametrize("shape", [(2, 8, 2, 40, 40, 16, 16), (1, 4, 2, 70, 45, 64, 64), (1, 2, 2, 33, 33, 128, 128)])
@pytest.mark.parametrize("kind", ["shared", "per_head"])
def test_masked_gqa_f64_matches_oracle(hip, oracle, shape, kind):
    batch, h_q, h_kv, sq, sk, dk, dv = shape
    q, k, v = _inputs(8, *shape, np.float64)
    mask = _mask(8, kind, batch * h_q, sq, sk, np.float64)
    scale = 1.0 / math.sqrt(dk)
    assert rel_err(_run(hip, q, k, v, scale, mask), oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask)) <= TOL_F64


def test_reference_gqa_case_and_expand_identity(hip, oracle):
    """The inputs of sdpa_masked_gqa_f64_matches_expand_then_masked_bit_exact (crates/ft-kernel-cpu/src/lib.rs:45160):
    grouped equals the masked kernel on K/V heads repeated `group` times, bit for bit, in f64 and f32."""
    batch, h_q, h_kv, sq, sk, dk, dv = 2, 8, 2, 40, 40, 16, 16
    i = lambda n: np.arange(n, dtype=np.float64)
    q = (np.sin(i(batch * h_q * sq * dk) * 0.017 + 0.3) * 0.2).reshape(batch, h_q, sq, dk)
    k = (np.sin(i(batch * h_kv * sk * dk) * 0.013 + 1.1) * 0.2).reshape(batch, h_kv, sk, dk)
    v = (np.cos(i(batch * h_kv * sk * dv) * 0.011 + 2.2) * 0.2).reshape(batch, h_kv, sk, dv)
    mask2d = np.where(np.arange(sq * sk) % 3 == 0, -0.5, 0.0).reshape(sq, sk)
    mask3d = np.where(np.arange(batch * h_q * sq * sk) % 5 == 0, -0.7, 0.0).reshape(batch * h_q, sq, sk)
    scale = 1.0 / math.sqrt(dk)
    group = h_q // h_kv
    k_rep, v_rep = np.repeat(k, group, axis=1), np.repeat(v, group, axis=1)
    for dt, tol in ((np.float64, TOL_F64), (np.float32, TOL_GEMM_F32)):
        for mask in (mask2d, mask3d):
            a = [t.astype(dt) for t in (q, k, v, k_rep, v_rep, mask)]
            grouped = _run(hip, a[0], a[1], a[2], dt(scale), a[5])
            expanded = _run(hip, a[0], a[3], a[4], dt(scale), a[5])
            assert np.array_equal(grouped.view(np.uint8), expanded.view(np.uint8))
            assert rel_err(grouped, oracle.sdpa_forward_masked_gqa(a[0], a[1], a[2], dt(scale), a[5])) <= tol
    # host-slice entry points with the reference's argument lists
    got = K.sdpa_forward_masked_gqa_f64(q, k, v, batch, h_q, h_kv, sq, sk, dk, dv, scale, mask3d, sq * sk)
    assert rel_err(got, oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask3d).ravel()) <= TOL_F64
    got = K.sdpa_forward_masked_f64(q, k_rep, v_rep, batch * h_q, sq, sk, dk, dv, scale, mask2d, 0)
    assert rel_err(got, oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask2d).ravel()) <= TOL_F64
    got = K.sdpa_forward_masked_gqa_f32(q, k, v, batch, h_q, h_kv, sq, sk, dk, dv, scale, mask2d, 0)
    assert got.dtype == np.float32 and rel_err(got, oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask2d).ravel()) <= TOL_GEMM_F32
    with pytest.raises(HipError):  # a mask shorter than the shape reads: a slice-index panic in the reference
        K.sdpa_forward_masked_gqa_f64(q, k, v, batch, h_q, h_kv, sq, sk, dk, dv, scale, mask3d.ravel()[:-1], sq * sk)
    with pytest.raises(HipError):
        K.sdpa_forward_masked_gqa_f64(q, k, v, batch, h_q, 3, sq, sk, dk, dv, scale, mask2d, 0)


@pytest.mark.parametrize("dk", [64, 16])
def test_mask_reduces_to_the_unmasked_and_causal_kernels(hip, oracle, dk):
    batch, h, sq, sk = 2, 4, 150, 150
    q, k, v = _inputs(9, batch, h, h, sq, sk, dk, dk, np.float32)
    scale = np.float32(1.0 / math.sqrt(dk))
    flat = lambda t: t.reshape(batch * h, t.shape[2], t.shape[3])
    zero = np.zeros((sq, sk), np.float32)
    assert rel_err(_run(hip, q, k, v, scale, zero).reshape(batch * h, sq, dk), oracle.sdpa_forward(flat(q), flat(k), flat(v), scale, False)) <= TOL_GEMM_F32
    tri = np.where(np.arange(sk)[None, :] > np.arange(sq)[:, None], -np.inf, 0.0).astype(np.float32)
    want = oracle.sdpa_forward(flat(q), flat(k), flat(v), scale, True)
    assert rel_err(_run(hip, q, k, v, scale, tri).reshape(batch * h, sq, dk), want) <= TOL_GEMM_F32
    # the causal flag and a mask together: the mask adds to what the flag leaves visible
    assert rel_err(_run(hip, q, k, v, scale, zero, causal=True).reshape(batch * h, sq, dk), want) <= TOL_GEMM_F32


@pytest.mark.parametrize("dk", [64, 24])
def test_hidden_leading_keys_and_fully_hidden_rows(hip, oracle, dk):
    """A sliding window hides the first keys of late rows (whole leading tiles for the MFMA kernel); rows with every key
    hidden are NaN as in the reference, and only those."""
    batch, h, sq, sk = 1, 2, 200, 200
    q, k, v = _inputs(10, batch, h, h, sq, sk, dk, dk, np.float32)
    rows, cols = np.arange(sq)[:, None], np.arange(sk)[None, :]
    mask = np.where((cols > rows) | (cols < rows - 20), -np.inf, 0.0).astype(np.float32)
    mask[[5, 150], :] = -np.inf
    scale = np.float32(1.0 / math.sqrt(dk))
    got, ref = _run(hip, q, k, v, scale, mask), oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask)
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.all(np.isnan(got[:, :, [5, 150]]))
    ok = ~np.isnan(ref)
    assert rel_err(got[ok], ref[ok]) <= TOL_GEMM_F32


def test_masked_gqa_at_a_serving_shape(hip, oracle):
    """B2, 32 query heads on 8 K/V heads, S 2048, D 128, fp32, shared causal-window mask: sampled heads against the
    checker, and the whole output against the expand-then-masked identity."""
    batch, h_q, h_kv, s, d = 2, 32, 8, 2048, 128
    q, k, v = _inputs(11, batch, h_q, h_kv, s, s, d, d, np.float32)
    rows, cols = np.arange(s)[:, None], np.arange(s)[None, :]
    mask = np.where((cols > rows) | (cols < rows - 1023), -np.inf, 0.0).astype(np.float32)
    scale = np.float32(1.0 / math.sqrt(d))
    got = _run(hip, q, k, v, scale, mask)
    for b, hq in ((0, 0), (1, 13), (1, 31)):
        kv = hq // (h_q // h_kv)
        ref = oracle.sdpa_forward_masked(q[b, hq][None], k[b, kv][None], v[b, kv][None], scale, mask)
        assert rel_err(got[b, hq], ref[0]) <= TOL_GEMM_F32
    expanded = _run(hip, q, np.repeat(k, h_q // h_kv, axis=1), np.repeat(v, h_q // h_kv, axis=1), scale, mask)
    assert np.array_equal(got.view(np.uint32), expanded.view(np.uint32))
