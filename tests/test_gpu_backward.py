"""Backward kernels against the CPU checker: fp32 row work <= 1e-5, fp32 products <= 2e-5, fp64 <= 1e-12
(max|d| / max|ref|), bitwise repeatable, and a size-independent property at the benchmark shape."""
import math

import numpy as np
import pytest

from conftest import NORM_COLSUM_TOL_FACTOR, TOL_F64, TOL_GEMM_F32, TOL_ROW_F32, rel_err
from frankentorch_amd import synth
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def _up(*arrays):
    return [None if a is None else DeviceBuffer.from_host(a) for a in arrays]


# register-resident path (cols a vector multiple, up to 16 vectors per thread), ragged / long rows (streaming path)
NORM_SHAPES = [(64, 256), (37, 768), (300, 4096), (5, 7), (3, 16), (9, 16384), (4, 20000), (130, 1026), (1, 4)]


@pytest.mark.parametrize("rows,cols", NORM_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_layer_norm_backward(hip, oracle, rows, cols, dtype):
    tol = TOL_ROW_F32 if dtype == np.float32 else TOL_F64
    x = synth.normal(11, "x", (rows, cols), dtype=dtype)
    dy = synth.normal(11, "dy", (rows, cols), dtype=dtype)
    w = synth.uniform(11, "w", (cols,), 0.5, 1.5, dtype=dtype)
    dx_r, dw_r, db_r = oracle.layer_norm_backward(dy, x, w, dtype(1e-5))
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((rows, cols), dtype), DeviceBuffer((cols,), dtype), DeviceBuffer((cols,), dtype)
    hip.layer_norm_backward(ddy, dx_, dw_, ddx, ddw, ddb, rows, cols, 1e-5)
    got = (ddx.to_host(), ddw.to_host(), ddb.to_host())
    assert rel_err(got[0], dx_r) <= tol and rel_err(got[1], dw_r) <= tol * NORM_COLSUM_TOL_FACTOR and rel_err(got[2], db_r) <= tol * NORM_COLSUM_TOL_FACTOR
    hip.layer_norm_backward(ddy, dx_, dw_, ddx, ddw, ddb, rows, cols, 1e-5)
    for a, b in zip(got, (ddx.to_host(), ddw.to_host(), ddb.to_host())):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("rows,cols", NORM_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("with_weight", [True, False])
def test_rms_norm_backward(hip, oracle, rows, cols, dtype, with_weight):
    tol = TOL_ROW_F32 if dtype == np.float32 else TOL_F64
    x = synth.normal(12, "x", (rows, cols), dtype=dtype)
    dy = synth.normal(12, "dy", (rows, cols), dtype=dtype)
    w = synth.uniform(12, "w", (cols,), 0.5, 1.5, dtype=dtype) if with_weight else None
    dx_r, dw_r = oracle.rms_norm_backward(dy, x, w, dtype(1e-6))
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx = DeviceBuffer((rows, cols), dtype)
    ddw = DeviceBuffer((cols,), dtype) if with_weight else None
    hip.rms_norm_backward(ddy, dx_, dw_, ddx, ddw, rows, cols, 1e-6)
    assert rel_err(ddx.to_host(), dx_r) <= tol
    if with_weight:
        assert rel_err(ddw.to_host(), dw_r) <= tol * NORM_COLSUM_TOL_FACTOR


@pytest.mark.parametrize("batch,in_f,out_f", [(96, 40, 72), (128, 256, 1024), (200, 300, 100), (1024, 768, 2304), (1, 5, 3), (33, 64, 64)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_linear_backward(hip, oracle, batch, in_f, out_f, dtype):
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    dy = synth.normal(13, "dy", (batch, out_f), dtype=dtype)
    x = synth.normal(13, "x", (batch, in_f), dtype=dtype)
    w = synth.normal(13, "w", (out_f, in_f), dtype=dtype)
    dx_r, dw_r, db_r = oracle.linear_backward(dy, x, w, True)
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((batch, in_f), dtype), DeviceBuffer((out_f, in_f), dtype), DeviceBuffer((out_f,), dtype)
    hip.linear_backward(ddy, dx_, dw_, ddx, ddw, ddb, batch, in_f, out_f)
    assert rel_err(ddx.to_host(), dx_r) <= tol and rel_err(ddw.to_host(), dw_r) <= tol and rel_err(ddb.to_host(), db_r) <= tol
    # need_bias = false
    ddb2 = DeviceBuffer.from_host(np.full((out_f,), 7, dtype))
    hip.linear_backward(ddy, dx_, dw_, ddx, ddw, None, batch, in_f, out_f)
    assert np.all(ddb2.to_host() == 7)


def test_linear_backward_at_the_benchmark_shape_sampled(hip, oracle):
    """Batch 8192, 768 -> 3072 (the FC1 layer of the GPT-2 shape): dx = dy . W is an 8192 x 768 x 3072 product with W stored
    [k, n], which runs on 128 x 96 tiles (512 whole tiles, one per resident workgroup); dweight splits its 8192-deep reduction
    across workgroups. Sampled rows of both against the checker's GEMM, dbias against its column sum, and a bitwise repeat."""
    batch, in_f, out_f = 8192, 768, 3072
    dy = synth.normal(33, "dy", (batch, out_f))
    x = synth.normal(33, "x", (batch, in_f))
    w = synth.normal(33, "w", (out_f, in_f), 0.0, 0.02)
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((batch, in_f)), DeviceBuffer((out_f, in_f)), DeviceBuffer((out_f,))
    hip.linear_backward(ddy, dx_, dw_, ddx, ddw, ddb, batch, in_f, out_f)
    gx, gw, gb = ddx.to_host(), ddw.to_host(), ddb.to_host()
    rows = np.unique(np.concatenate([np.arange(3, batch, 131), [0, 127, 128, batch - 1]]))
    assert rel_err(gx[rows], oracle.gemm(dy[rows], w, False)) <= TOL_GEMM_F32
    outs = np.unique(np.concatenate([np.arange(5, out_f, 67), [0, 95, 96, out_f - 1]]))
    assert rel_err(gw[outs], oracle.gemm(np.ascontiguousarray(dy[:, outs].T), x, False)) <= TOL_GEMM_F32
    assert rel_err(gb, oracle.gemm(np.ones((1, batch), np.float32), dy, False)[0]) <= TOL_GEMM_F32
    hip.linear_backward(ddy, dx_, dw_, ddx, ddw, ddb, batch, in_f, out_f)
    for a, b in zip((gx, gw, gb), (ddx.to_host(), ddw.to_host(), ddb.to_host())):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


def test_linear_backward_reference_test_inputs(hip, oracle):
    """The inputs of the reference's own dweight test (crates/ft-kernel-cpu/src/lib.rs:43862-43911), fp64."""
    batch, in_f, out_f = 96, 40, 72
    dy = ((np.arange(batch * out_f) % 101) * 0.01 - 0.5).reshape(batch, out_f)
    x = ((np.arange(batch * in_f) % 89) * 0.02 - 0.7).reshape(batch, in_f)
    w = ((np.arange(out_f * in_f) % 53) * 0.03 - 0.4).reshape(out_f, in_f)
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((batch, in_f), np.float64), DeviceBuffer((out_f, in_f), np.float64), DeviceBuffer((out_f,), np.float64)
    hip.linear_backward(ddy, dx_, dw_, ddx, ddw, ddb, batch, in_f, out_f)
    assert np.allclose(ddw.to_host(), dy.T @ x, rtol=0, atol=1e-11)
    assert np.allclose(ddb.to_host(), dy.sum(0), rtol=0, atol=1e-12)


# The last four shapes are square and long enough for the causal form to take the block-causal products
# (blocks of 256 rows; 640 and 1152 end in a partial block).
# Head sizes 64 and 128 with sequence lengths of at least 32 take the fused path (statistics pass, key-owned
# kernel, dQ product; intermediates in whole 32 x 32 tiles); the ragged ones among them end in partial query tiles and
# partial key blocks: a single tile, fewer keys than a key block holds, more queries than keys, odd lengths.
@pytest.mark.parametrize("bh,sq,sk,dk,dv", [(2, 64, 64, 64, 64), (3, 100, 70, 32, 48), (4, 128, 128, 128, 128), (1, 5, 6, 4, 3), (2, 33, 200, 16, 16),
                                            (2, 512, 512, 64, 64), (1, 640, 640, 32, 48), (3, 1024, 1024, 64, 64), (2, 1152, 1152, 128, 128),
                                            (2, 100, 76, 64, 64), (1, 36, 260, 128, 128), (2, 256, 384, 64, 64), (2, 388, 132, 128, 128),
                                            (1, 32, 32, 64, 64), (2, 132, 36, 128, 128), (1, 580, 68, 64, 64),
                                            (2, 101, 77, 64, 64), (1, 45, 131, 128, 128), (2, 333, 333, 64, 64)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sdpa_backward(hip, oracle, bh, sq, sk, dk, dv, causal, dtype):
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    s = 1.0 / math.sqrt(dk)
    q = synth.normal(14, "q", (bh, sq, dk), dtype=dtype)
    k = synth.normal(14, "k", (bh, sk, dk), dtype=dtype)
    v = synth.normal(14, "v", (bh, sk, dv), dtype=dtype)
    do = synth.normal(14, "do", (bh, sq, dv), dtype=dtype)
    ref = oracle.sdpa_backward(q, k, v, do, dtype(s), causal)
    dq_, dk_, dv_, ddo = _up(q, k, v, do)
    gq, gk, gv = DeviceBuffer(q.shape, dtype), DeviceBuffer(k.shape, dtype), DeviceBuffer(v.shape, dtype)
    hip.sdpa_backward(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, s, causal, gq, gk, gv)
    got = (gq.to_host(), gk.to_host(), gv.to_host())
    for g, r in zip(got, ref):
        assert rel_err(g, r) <= tol
    hip.sdpa_backward(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, s, causal, gq, gk, gv)
    for a, b in zip(got, (gq.to_host(), gk.to_host(), gv.to_host())):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("bh,sq,sk,dk,dv", [(2, 64, 64, 64, 64), (3, 100, 70, 32, 48), (1, 5, 6, 4, 3), (2, 33, 203, 16, 16), (2, 512, 384, 128, 128)])
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sdpa_backward_masked(hip, oracle, bh, sq, sk, dk, dv, shared, dtype):
    """sdpa_backward_masked_f64 (crates/ft-kernel-cpu/src/lib.rs:5423-5530) and its f32 twin: soft additive masks with hidden keys,
    one mask for all heads or one per head; seq_k = 203 and the one-element offset below take the unvectorised row pass."""
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    s = 1.0 / math.sqrt(dk)
    q = synth.normal(24, "q", (bh, sq, dk), dtype=dtype)
    k = synth.normal(24, "k", (bh, sk, dk), dtype=dtype)
    v = synth.normal(24, "v", (bh, sk, dv), dtype=dtype)
    do = synth.normal(24, "do", (bh, sq, dv), dtype=dtype)
    mshape = (sq, sk) if shared else (bh, sq, sk)
    mask = synth.normal(24, "mask", mshape, dtype=dtype)
    mask = np.where(synth.uniform(24, "hide", mshape, 0, 1) < 0.25, -np.inf, mask).astype(dtype)
    mask[..., 0] = 0  # every row keeps one key
    ref = oracle.sdpa_backward_masked(q, k, v, do, dtype(s), mask)
    dq_, dk_, dv_, ddo, dmask = _up(q, k, v, do, mask)
    gq, gk, gv = DeviceBuffer(q.shape, dtype), DeviceBuffer(k.shape, dtype), DeviceBuffer(v.shape, dtype)
    stride = 0 if shared else sq * sk
    hip.sdpa_backward_masked(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, s, dmask, stride, gq, gk, gv)
    got = (gq.to_host(), gk.to_host(), gv.to_host())
    for g, r in zip(got, ref):
        assert rel_err(g, r) <= tol
    hip.sdpa_backward_masked(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, s, dmask, stride, gq, gk, gv)
    for a, b in zip(got, (gq.to_host(), gk.to_host(), gv.to_host())):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    if shared:  # a mask that starts one element into its buffer: unaligned rows
        pad = DeviceBuffer.from_host(np.concatenate([np.zeros(1, dtype), mask.ravel()]))
        hip.sdpa_backward_masked(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, s, pad.view(1), 0, gq, gk, gv)
        for g, r in zip((gq.to_host(), gk.to_host(), gv.to_host()), ref):
            assert rel_err(g, r) <= tol


@pytest.mark.parametrize("bh,sq,sk,dk,dv", [(2, 5, 6, 4, 3), (3, 100, 70, 32, 48), (2, 640, 640, 64, 64), (2, 99, 71, 64, 64)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sdpa_backward_unit_dout(hip, oracle, bh, sq, sk, dk, dv, causal, dtype):
    """sdpa_backward_f32_unit_dout (crates/ft-kernel-cpu/src/lib.rs:5662-5770): against the checker's restatement and against the
    general backward given a materialised ones tensor (the reference's own test, :45119-45155); 640 takes the block-causal path."""
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    s = 1.0 / math.sqrt(dk)
    q, k, v = (synth.normal(27, t, shp, dtype=dtype) for t, shp in (("q", (bh, sq, dk)), ("k", (bh, sk, dk)), ("v", (bh, sk, dv))))
    ref = oracle.sdpa_backward_unit_dout(q, k, v, dtype(s), causal)
    dq_, dk_, dv_ = _up(q, k, v)
    gq, gk, gv = DeviceBuffer(q.shape, dtype), DeviceBuffer(k.shape, dtype), DeviceBuffer(v.shape, dtype)
    hip.sdpa_backward_unit_dout(dq_, dk_, dv_, bh, sq, sk, dk, dv, s, causal, gq, gk, gv)
    got = (gq.to_host(), gk.to_host(), gv.to_host())
    for g, r in zip(got, ref):
        assert rel_err(g, r) <= tol
    assert np.all(got[2] == got[2][:, :, :1])  # every value lane of a key gets the same gradient, bit for bit
    hq, hk, hv = DeviceBuffer(q.shape, dtype), DeviceBuffer(k.shape, dtype), DeviceBuffer(v.shape, dtype)
    hip.sdpa_backward(dq_, dk_, dv_, DeviceBuffer.from_host(np.ones((bh, sq, dv), dtype)), bh, sq, sk, dk, dv, s, causal, hq, hk, hv)
    for a, b in zip(got, (hq.to_host(), hk.to_host(), hv.to_host())):
        assert rel_err(a, b) <= tol


def test_sdpa_backward_masked_reduces_to_the_unmasked_and_causal_forms(hip):
    bh, sq, sk, dk, dv = 2, 96, 96, 32, 32
    q, k, v, do = (synth.normal(25, t, (bh, sq, dk)) for t in ("q", "k", "v", "do"))
    dq_, dk_, dv_, ddo = _up(q, k, v, do)
    outs = []
    for mask, causal in ((np.zeros((sq, sk), np.float32), False), (np.where(np.arange(sk)[None, :] <= np.arange(sq)[:, None], 0.0, -np.inf).astype(np.float32), True)):
        gq, gk, gv = DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)
        hq, hk, hv = DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)
        hip.sdpa_backward_masked(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, 0.2, DeviceBuffer.from_host(mask), 0, gq, gk, gv)
        hip.sdpa_backward(dq_, dk_, dv_, ddo, bh, sq, sk, dk, dv, 0.2, causal, hq, hk, hv)
        for a, b in zip((gq, gk, gv), (hq, hk, hv)):
            assert rel_err(a.to_host(), b.to_host()) <= TOL_GEMM_F32


@pytest.mark.parametrize("bh,sq,sk,d,causal", [(4, 2048, 2048, 128, True), (2, 1024, 1536, 64, False), (3, 1100, 1100, 64, True), (96, 1024, 1024, 64, True)])
def test_fused_sdpa_backward_against_the_materialising_path_at_full_length(hip, bh, sq, sk, d, causal):
    """Head sizes 64 / 128 without a mask take the fused three-pass backward (scores + statistics, key-owned pass,
    query-owned pass); the same problem with its mask passed explicitly takes the materialising path (five batched GEMMs
    around two row passes). Two independent implementations, compared at the benchmark's sequence length and at a
    ragged one, plus linearity of the fused path in dOut (no checker involved)."""
    s = 1.0 / math.sqrt(d)
    q, k, v, do = (synth.normal(31, t, (bh, n, d), 0.0, 1.0) for t, n in (("q", sq), ("k", sk), ("v", sk), ("do", sq)))
    dq_, dk_, dv_, ddo = _up(q, k, v, do)
    mask = np.where(np.arange(sk)[None, :] <= np.arange(sq)[:, None], 0.0, -np.inf).astype(np.float32) if causal else np.zeros((sq, sk), np.float32)
    fused = [DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)]
    mat = [DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)]
    ws = hip.sdpa_backward(dq_, dk_, dv_, ddo, bh, sq, sk, d, d, s, causal, *fused)
    hip.sdpa_backward_masked(dq_, dk_, dv_, ddo, bh, sq, sk, d, d, s, DeviceBuffer.from_host(mask), 0, *mat)
    f = [b.to_host() for b in fused]
    for a, b in zip(f, mat):
        assert rel_err(a, b.to_host()) <= TOL_GEMM_F32
    # linearity: backward(2 dOut + dOut') = 2 backward(dOut) + backward(dOut')
    do2 = synth.normal(32, "do2", (bh, sq, d))
    g2 = [DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)]
    g3 = [DeviceBuffer(q.shape), DeviceBuffer(k.shape), DeviceBuffer(v.shape)]
    hip.sdpa_backward(dq_, dk_, dv_, DeviceBuffer.from_host(do2), bh, sq, sk, d, d, s, causal, *g2, workspace=ws)
    hip.sdpa_backward(dq_, dk_, dv_, DeviceBuffer.from_host(2.0 * do + do2), bh, sq, sk, d, d, s, causal, *g3, workspace=ws)
    for a, b, c in zip(f, g2, g3):
        assert rel_err(2.0 * a + b.to_host(), c.to_host()) <= TOL_GEMM_F32


def test_host_slice_sdpa_backward_masked_and_its_errors(oracle):
    from frankentorch_amd import kernel_hip as K
    from frankentorch_amd.core import HipError, KernelError

    bh, sq, sk, dk, dv = 2, 17, 23, 16, 8
    q, k, v = synth.normal(26, "q", (bh, sq, dk), dtype=np.float64), synth.normal(26, "k", (bh, sk, dk), dtype=np.float64), synth.normal(26, "v", (bh, sk, dv), dtype=np.float64)
    do = synth.normal(26, "do", (bh, sq, dv), dtype=np.float64)
    mask = synth.normal(26, "m", (bh, sq, sk), dtype=np.float64)
    got = K.sdpa_backward_masked_f64(q.ravel(), k.ravel(), v.ravel(), do.ravel(), bh, sq, sk, dk, dv, 0.25, mask.ravel(), sq * sk)
    for g, r in zip(got, oracle.sdpa_backward_masked(q, k, v, do, 0.25, mask)):
        assert rel_err(g, r.ravel()) <= 2 * TOL_F64
    got = K.sdpa_backward_f32_unit_dout(q.astype(np.float32).ravel(), k.astype(np.float32).ravel(), v.astype(np.float32).ravel(), bh, sq, sk, dk,
                                        dv, 0.25, True)
    for g, r in zip(got, oracle.sdpa_backward_unit_dout(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), np.float32(0.25), True)):
        assert rel_err(g, r.ravel()) <= 2 * TOL_GEMM_F32
    with pytest.raises((KernelError, HipError)):  # a mask slice shorter than num_bh planes
        K.sdpa_backward_masked_f64(q.ravel(), k.ravel(), v.ravel(), do.ravel(), bh, sq, sk, dk, dv, 0.25, mask.ravel()[:-1], sq * sk)
    with pytest.raises((KernelError, HipError)):  # a per-head stride smaller than one plane
        K.sdpa_backward_masked_f64(q.ravel(), k.ravel(), v.ravel(), do.ravel(), bh, sq, sk, dk, dv, 0.25, mask.ravel(), 5)


def test_norm_backward_at_the_row_op_benchmark_shape(hip, oracle):
    """fp32 [8192, 4096]: sampled rows against the checker, column sums against an f64 numpy sum, and the
    property that dx rows of LayerNorm sum to zero."""
    rows, cols = 8192, 4096
    x = synth.normal(1, "x", (rows, cols))
    dy = synth.normal(1, "dyb", (rows, cols))
    w = synth.uniform(1, "gamma", (cols,), 0.5, 1.5)
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((rows, cols)), DeviceBuffer((cols,)), DeviceBuffer((cols,))
    hip.layer_norm_backward(ddy, dx_, dw_, ddx, ddw, ddb, rows, cols, 1e-5)
    dx = ddx.to_host()
    pick = np.arange(3, rows, 509)
    dx_r, _, _ = oracle.layer_norm_backward(dy[pick], x[pick], w, np.float32(1e-5))
    assert rel_err(dx[pick], dx_r) <= TOL_ROW_F32
    assert np.max(np.abs(dx.astype(np.float64).sum(1))) <= 1e-3
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    xhat = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    assert rel_err(ddw.to_host(), (dy64 * xhat).sum(0)) <= 4 * TOL_ROW_F32
    assert rel_err(ddb.to_host(), dy64.sum(0)) <= 4 * TOL_ROW_F32
    hip.rms_norm_backward(ddy, dx_, dw_, ddx, ddw, rows, cols, 1e-6)
    dxr, _ = oracle.rms_norm_backward(dy[pick], x[pick], w, np.float32(1e-6))
    assert rel_err(ddx.to_host()[pick], dxr) <= TOL_ROW_F32
    rstd = 1.0 / np.sqrt((x64 * x64).mean(1, keepdims=True) + 1e-6)
    assert rel_err(ddw.to_host(), (dy64 * x64 * rstd).sum(0)) <= 4 * TOL_ROW_F32


@pytest.mark.parametrize("rows,cols", [(8192, 4096), (8192, 768), (3000, 1024)])
def test_column_sums_are_no_further_from_the_f64_sum_than_the_serial_f32_sum_is(hip, oracle, rows, cols):
    """What NORM_COLSUM_TOL_FACTOR stands on. dweight / dbias are sums over the batch; the reference adds the rows in one
    serial fp32 chain, the kernels add (rows of a workgroup) then (workgroups). Both are fp32 roundings of the same exact
    sum, so the fair question is not how far they are from each other but how far each is from the float64 sum of the
    same terms: the GPU's re-associated sum must not be the worse of the two."""
    x = synth.normal(41, "x", (rows, cols))
    dy = synth.normal(41, "dy", (rows, cols))
    w = synth.uniform(41, "w", (cols,), 0.5, 1.5)
    _, dw_o, db_o = oracle.layer_norm_backward(dy, x, w, np.float32(1e-5))   # the reference's serial fp32 sums
    ddy, dx_, dw_ = _up(dy, x, w)
    ddx, ddw, ddb = DeviceBuffer((rows, cols)), DeviceBuffer((cols,)), DeviceBuffer((cols,))
    hip.layer_norm_backward(ddy, dx_, dw_, ddx, ddw, ddb, rows, cols, 1e-5)
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    xhat = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    for name, gpu, serial, truth in (("dweight", ddw.to_host(), dw_o, (dy64 * xhat).sum(0)), ("dbias", ddb.to_host(), db_o, dy64.sum(0))):
        e_gpu, e_serial = rel_err(gpu, truth), rel_err(serial, truth)
        assert e_gpu <= max(e_serial, 1e-6), "%s: GPU %.3g from the f64 sum, the serial fp32 sum %.3g" % (name, e_gpu, e_serial)
        assert e_gpu <= TOL_ROW_F32  # and against the truth the plain row-op bar holds, without the factor
        assert rel_err(gpu, serial) <= TOL_ROW_F32 * NORM_COLSUM_TOL_FACTOR


def test_host_slice_backward_entry_points(oracle):
    """The ft_kernel_cpu-named functions on host slices (upload, kernels, download), and their error statuses."""
    from frankentorch_amd import kernel_hip as K
    from frankentorch_amd.core import HipError, KernelError

    rows, cols = 33, 96
    x, dy = synth.normal(21, "x", (rows, cols)), synth.normal(21, "dy", (rows, cols))
    w = synth.uniform(21, "w", (cols,), 0.5, 1.5)
    dx, dw, db = K.layer_norm_backward_f32(dy.ravel(), x.ravel(), w, rows, cols, 1e-5)
    rx, rw, rb = oracle.layer_norm_backward(dy, x, w, np.float32(1e-5))
    assert rel_err(dx, rx.ravel()) <= TOL_ROW_F32 and rel_err(dw, rw) <= 4 * TOL_ROW_F32 and rel_err(db, rb) <= 4 * TOL_ROW_F32
    dx, dw = K.rms_norm_backward_f64(dy.astype(np.float64).ravel(), x.astype(np.float64).ravel(), None, rows, cols, 1e-6)
    assert dw is None
    assert rel_err(dx, oracle.rms_norm_backward(dy.astype(np.float64), x.astype(np.float64), None, 1e-6)[0].ravel()) <= TOL_F64
    batch, in_f, out_f = 40, 24, 56
    dyl, xl, wl = synth.normal(22, "dy", (batch, out_f)), synth.normal(22, "x", (batch, in_f)), synth.normal(22, "w", (out_f, in_f))
    gx, gw, gb = K.linear_backward_f32(dyl.ravel(), xl.ravel(), wl.ravel(), batch, in_f, out_f, True)
    ox, ow, ob = oracle.linear_backward(dyl, xl, wl, True)
    assert rel_err(gx, ox.ravel()) <= TOL_GEMM_F32 and rel_err(gw, ow.ravel()) <= TOL_GEMM_F32 and rel_err(gb, ob) <= TOL_GEMM_F32
    assert K.linear_backward_f32(dyl.ravel(), xl.ravel(), wl.ravel(), batch, in_f, out_f, False)[2] is None
    bh, sq, sk, dk, dv = 2, 17, 23, 16, 8
    q, k, v = synth.normal(23, "q", (bh, sq, dk)), synth.normal(23, "k", (bh, sk, dk)), synth.normal(23, "v", (bh, sk, dv))
    do = synth.normal(23, "do", (bh, sq, dv))
    got = K.sdpa_backward_f32(q.ravel(), k.ravel(), v.ravel(), do.ravel(), bh, sq, sk, dk, dv, 0.25, True)
    for g, r in zip(got, oracle.sdpa_backward(q, k, v, do, np.float32(0.25), True)):
        assert rel_err(g, r.ravel()) <= 2 * TOL_GEMM_F32
    with pytest.raises((KernelError, HipError)):  # a slice shorter than batch * norm_size
        K.layer_norm_backward_f32(dy.ravel()[:10], x.ravel(), w, rows, cols, 1e-5)
