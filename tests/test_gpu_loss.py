"""log-softmax and the fused softmax-cross-entropy kernels against the CPU checker: fp32 <= 1e-5, fp64 <= 1e-12
(max|d| / max|ref|), the reference's golden bits, bad-target reporting, bitwise repeatability, and closed-form
properties at the GPT-2 vocabulary width."""
import numpy as np
import pytest

from conftest import TOL_F64, TOL_ROW_F32, rel_err
from frankentorch_amd import kernel_hip as K
from frankentorch_amd import synth
from frankentorch_amd.core import DType, HipError, TensorMeta, contiguous_strides
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu

# ragged, unaligned, shorter than a workgroup, one element, the GPT-2 vocabulary, the longest register-resident rows
# (fp32 65536, fp64 32768) and rows beyond them (the streaming kernels)
ROW_SHAPES = [(7, 5), (64, 256), (33, 1000), (3, 1), (1, 50257), (19, 50257), (130, 1026), (5, 4099), (6, 16384), (3, 32768), (2, 65536), (2, 70001)]


def _tol(dtype):
    return TOL_ROW_F32 if dtype == np.float32 else TOL_F64


def _targets(seed, rows, cols):
    return synth.token_ids(seed, "target", (rows,), cols).astype(np.int64)


@pytest.mark.parametrize("rows,cols", ROW_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_log_softmax_rows(hip, oracle, rows, cols, dtype):
    x = synth.normal(21, "x", (rows, cols), dtype=dtype) * dtype(3.0)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer((rows, cols), dtype)
    hip.log_softmax_strided(dx, dy, rows, cols, 1)
    got = dy.to_host()
    assert rel_err(got, oracle.log_softmax(x, 1)) <= _tol(dtype)
    hip.log_softmax_strided(dx, dy, rows, cols, 1)
    assert np.array_equal(got.view(np.uint8), dy.to_host().view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_log_softmax_strided_dims(hip, oracle, dtype):
    x = synth.normal(22, "x", (6, 37, 19), dtype=dtype)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer(x.shape, dtype)
    hip.log_softmax_strided(dx, dy, 6, 37, 19)
    assert rel_err(dy.to_host(), oracle.log_softmax(x, 1)) <= _tol(dtype)
    hip.log_softmax_strided(dx, dy, 1, 6, 37 * 19)
    assert rel_err(dy.to_host(), oracle.log_softmax(x, 0)) <= _tol(dtype)


def test_log_softmax_golden_bits_and_specials(hip, oracle, vectors):
    b = vectors["golden_text"]["softmax_parallel_bits"]
    rows = b["meta"]["fast_rows"]
    # the reference's golden run: [8192, 1] of 3.0 over dim 1, and [4096, 1, 2] of 7.0 over dim 1 -> +0.0 everywhere
    for dt, bits_t, key in ((np.float32, np.uint32, "f32"), (np.float64, np.uint64, "f64")):
        dx, dy = DeviceBuffer.from_host(np.full((rows, 1), 3.0, dt)), DeviceBuffer((rows, 1), dt)
        hip.log_softmax_strided(dx, dy, rows, 1, 1)
        bits = dy.to_host().ravel().view(bits_t)
        for i, v in b["bits"][key + "_log_softmax_fast_bits"].items():
            assert bits[int(i)] == int(v, 16)
        so = b["meta"]["strided_outer"]
        dx, dy = DeviceBuffer.from_host(np.full((so, 1, 2), 7.0, dt)), DeviceBuffer((so, 1, 2), dt)
        hip.log_softmax_strided(dx, dy, so, 1, 2)
        bits = dy.to_host().ravel().view(bits_t)
        for i, v in b["bits"][key + "_log_softmax_strided_bits"].items():
            assert bits[int(i)] == int(v, 16)
    inf, nan = np.float32(np.inf), np.float32(np.nan)
    x = np.array([[1, nan, 2, 3], [-inf, 0, 1, -inf], [inf, 1, 2, 3], [-inf, -inf, -inf, -inf], [1e30, -1e30, 0, 5]], np.float32)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer(x.shape, np.float32)
    hip.log_softmax_strided(dx, dy, x.shape[0], x.shape[1], 1)
    got, ref = dy.to_host(), oracle.log_softmax(x, 1)
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(np.isinf(got[ok]), np.isinf(ref[ok]))
    fin = ok & np.isfinite(ref)
    assert rel_err(got[fin], ref[fin]) <= TOL_ROW_F32


@pytest.mark.parametrize("cols", [1, 63, 64, 1000, 1025, 24577, 50257])
@pytest.mark.parametrize("in_off,out_off", [(1, 1), (3, 2), (0, 63), (5, 0)])
def test_resident_rows_at_odd_element_offsets(hip, oracle, cols, in_off, out_off):
    """Rows that start anywhere (operands at odd element offsets inside larger buffers, input and output aligned differently):
    log-softmax, softmax and the loss gradient write exactly their rows -- the elements in front of the first row, between
    the output's end and the buffer's end, stay as they were -- and match the checker."""
    rows = 5
    x = synth.normal(31, "x", (rows, cols)) * np.float32(2.5)
    pad = 70
    xin = np.full(rows * cols + 2 * pad, 7.0, np.float32)
    xin[in_off:in_off + rows * cols] = x.ravel()
    dxin = DeviceBuffer.from_host(xin)
    guard = np.float32(-123.25)

    def run(fn, ref):
        dout = DeviceBuffer.from_host(np.full(rows * cols + 2 * pad, guard, np.float32))
        fn(dxin.view(in_off), dout.view(out_off))
        got = dout.to_host()
        assert np.all(got[:out_off] == guard) and np.all(got[out_off + rows * cols:] == guard)
        assert rel_err(got[out_off:out_off + rows * cols].reshape(rows, cols), ref) <= TOL_ROW_F32

    run(lambda a, b: hip.log_softmax_strided(a, b, rows, cols, 1), oracle.log_softmax(x, 1))
    run(lambda a, b: hip.softmax_lastdim(a, b, rows, cols), oracle.softmax(x, 1))
    target = _targets(31, rows, cols)
    dloss = synth.normal(31, "dloss", (rows,))
    dt, dg = DeviceBuffer.from_host(target), DeviceBuffer.from_host(dloss)
    run(lambda a, b: hip.cross_entropy_backward(a, dt, dg, rows, cols, b), oracle.cross_entropy_backward(x, target, dloss))


def test_log_softmax_empty_is_a_no_op(hip):
    d = DeviceBuffer((4,))
    hip.log_softmax_strided(d, d, 0, 4, 1)
    hip.log_softmax_strided(d, d, 4, 0, 1)
    hip.log_softmax_strided(d, d, 2, 2, 0)


@pytest.mark.parametrize("rows,cols", ROW_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_cross_entropy_forward_backward(hip, oracle, rows, cols, dtype):
    logits = synth.normal(23, "logits", (rows, cols), dtype=dtype) * dtype(2.0)
    target = _targets(23, rows, cols)
    dloss = synth.normal(23, "dloss", (rows,), dtype=dtype)
    dl, dt, dg = DeviceBuffer.from_host(logits), DeviceBuffer.from_host(target), DeviceBuffer.from_host(dloss)
    loss, dlogits = DeviceBuffer((rows,), dtype), DeviceBuffer((rows, cols), dtype)
    bad = DeviceBuffer((1,), np.int64)
    hip.cross_entropy_forward(dl, dt, rows, cols, loss, bad)
    assert int(bad.to_host()[0]) == -1
    got_loss = loss.to_host()
    assert rel_err(got_loss, oracle.cross_entropy_forward(logits, target)) <= _tol(dtype)
    hip.cross_entropy_backward(dl, dt, dg, rows, cols, dlogits, bad)
    assert int(bad.to_host()[0]) == -1
    got_d = dlogits.to_host()
    assert rel_err(got_d, oracle.cross_entropy_backward(logits, target, dloss)) <= _tol(dtype)
    # every row of dlogits sums to zero times dloss: softmax sums to one, the one-hot takes one away
    assert np.max(np.abs(got_d.astype(np.float64).sum(axis=1))) <= (1e-4 if dtype == np.float32 else 1e-12) * max(1.0, np.abs(dloss).max())
    hip.cross_entropy_forward(dl, dt, rows, cols, loss)
    hip.cross_entropy_backward(dl, dt, dg, rows, cols, dlogits)
    assert np.array_equal(got_loss.view(np.uint8), loss.to_host().view(np.uint8))
    assert np.array_equal(got_d.view(np.uint8), dlogits.to_host().view(np.uint8))


@pytest.mark.parametrize("cols", [8192, 8229, 20003])
def test_cross_entropy_forward_long_rows_specials(hip, oracle, cols):
    """fp32 rows of 8192 classes and more take the one-pass loss kernel (running maximum and rescaled sum per lane). Rows that
    start at every 4-byte offset inside a 16-byte vector (odd class counts), targets in the scalar head, body and tail, and the
    special values: -inf entries (weight zero), a row whose maximum comes last, huge spreads, NaN, +inf and a row of nothing
    but -inf (NaN in the reference's two-pass form as well)."""
    rows = 12
    logits = synth.normal(41, "logits", (rows, cols)) * np.float32(3.0)
    logits[1, ::3] = -np.inf
    logits[2, -1] = 60.0                      # the maximum is the last element (tail)
    logits[3, 0] = 75.0                       # ... or the first (head)
    logits[4] = np.linspace(-80.0, 80.0, cols, dtype=np.float32)   # ascending: every batch raises the maximum
    logits[5] = np.linspace(80.0, -80.0, cols, dtype=np.float32)
    logits[6, 5] = np.nan
    logits[7, cols // 2] = np.inf
    logits[8] = -np.inf
    logits[9] = -3.0e38                        # every value below any practical start of a running maximum
    logits[10, : cols - 1] = -np.inf          # one finite value, in the tail
    target = np.array([0, 1, cols - 1, 3, cols // 2, 2, 7, 9, 4, cols - 2, cols - 1, 5], np.int64)
    dl, dt = DeviceBuffer.from_host(logits), DeviceBuffer.from_host(target)
    loss, bad = DeviceBuffer((rows,)), DeviceBuffer((1,), np.int64)
    hip.cross_entropy_forward(dl, dt, rows, cols, loss, bad)
    assert int(bad.to_host()[0]) == -1
    got, ref = loss.to_host(), oracle.cross_entropy_forward(logits, target)
    assert np.array_equal(np.isnan(got), np.isnan(ref)), (got, ref)
    assert np.isnan(ref[[6, 7, 8]]).all()
    ok = ~np.isnan(ref)
    assert np.array_equal(np.isinf(got[ok]), np.isinf(ref[ok])) and np.array_equal(got[ok][np.isinf(ref[ok])], ref[ok][np.isinf(ref[ok])])
    fin = ok & np.isfinite(ref)
    assert np.max(np.abs(got[fin] - ref[fin])) <= TOL_ROW_F32 * np.max(np.abs(ref[fin]))
    hip.cross_entropy_forward(dl, dt, rows, cols, loss)
    assert np.array_equal(got.view(np.uint8), loss.to_host().view(np.uint8))


def test_cross_entropy_reports_the_first_bad_target(hip, oracle):
    rows, cols = 40, 33
    logits = synth.normal(24, "logits", (rows, cols))
    target = _targets(24, rows, cols)
    target[31], target[17], target[5] = cols, -1, cols + 7
    with pytest.raises(IndexError):
        oracle.cross_entropy_forward(logits, target)
    dl, dt = DeviceBuffer.from_host(logits), DeviceBuffer.from_host(target)
    sentinel = np.full(rows, -77.0, np.float32)
    loss, bad = DeviceBuffer.from_host(sentinel), DeviceBuffer((1,), np.int64)
    hip.cross_entropy_forward(dl, dt, rows, cols, loss, bad)
    assert int(bad.to_host()[0]) == 5
    got = loss.to_host()
    good = np.ones(rows, bool)
    good[[5, 17, 31]] = False
    assert np.all(got[~good] == -77.0)
    fixed = target.copy()
    fixed[~good] = 0
    assert rel_err(got[good], oracle.cross_entropy_forward(logits, fixed)[good]) <= TOL_ROW_F32
    dg = DeviceBuffer.from_host(np.ones(rows, np.float32))
    dlog = DeviceBuffer((rows, cols))
    hip.cross_entropy_backward(dl, dt, dg, rows, cols, dlog, bad)
    assert int(bad.to_host()[0]) == 5
    # the host-slice entry point refuses before any launch and names the row
    with pytest.raises(HipError) as e:
        K.cross_entropy_forward_f32(logits, np.where(target < 0, 2**63, target).astype(np.uint64), rows, cols)
    assert e.value.kind == "InvalidArgument" and "row 5" in e.value.message


def test_cross_entropy_uniform_rows_closed_form(hip):
    # uniform logits: loss = ln(classes) for any target, dlogits = dloss * (1/classes - onehot)
    rows, cols = 64, 50257
    for dtype in (np.float32, np.float64):
        logits = np.full((rows, cols), 1.25, dtype)
        target = _targets(25, rows, cols)
        dl, dt = DeviceBuffer.from_host(logits), DeviceBuffer.from_host(target)
        loss, dlog = DeviceBuffer((rows,), dtype), DeviceBuffer((rows, cols), dtype)
        dg = DeviceBuffer.from_host(np.full(rows, 2.0, dtype))
        hip.cross_entropy_forward(dl, dt, rows, cols, loss)
        hip.cross_entropy_backward(dl, dt, dg, rows, cols, dlog)
        assert rel_err(loss.to_host(), np.full(rows, np.log(float(cols)))) <= _tol(dtype)
        want = np.full((rows, cols), 2.0 / cols)
        want[np.arange(rows), target] -= 2.0
        assert np.max(np.abs(dlog.to_host() - want)) <= _tol(dtype) * 2.0


def test_loss_kernels_at_the_gpt2_logits_shape(hip, oracle):
    """[8192, 50257] fp32 logits made on the device by the LM-head product of the benchmark's forward.
    Sampled rows against the checker, and over the whole tensor: exp(log_softmax) sums to one per row,
    loss = -log_softmax[target], dlogits = softmax - onehot."""
    rows, cols, width = 8192, 50257, 768
    h = synth.normal(5, "hidden", (rows, width)) * np.float32(0.25)
    wte = synth.normal(5, "wte", (cols, width))
    target = _targets(5, rows, cols)
    dh, dw, dt = DeviceBuffer.from_host(h), DeviceBuffer.from_host(wte), DeviceBuffer.from_host(target)
    x, y, d = DeviceBuffer((rows, cols)), DeviceBuffer((rows, cols)), DeviceBuffer((rows, cols))
    loss, ones = DeviceBuffer((rows,)), DeviceBuffer.from_host(np.ones(rows, np.float32))
    hip.gemm(hip.gemm_desc(rows, cols, width, trans_b=True), dh, dw, x)
    hip.log_softmax_strided(x, y, rows, cols, 1)
    hip.cross_entropy_forward(x, dt, rows, cols, loss)
    hip.cross_entropy_backward(x, dt, ones, rows, cols, d)
    xs, ys, ds, ls = x.to_host(), y.to_host(), d.to_host(), loss.to_host()
    pick = np.arange(0, rows, 257)
    assert rel_err(ys[pick], oracle.log_softmax(xs[pick], 1)) <= TOL_ROW_F32
    assert rel_err(ls[pick], oracle.cross_entropy_forward(xs[pick], target[pick])) <= TOL_ROW_F32
    # The reference adds the 50 257 exponentials of a row one after another in fp32, so on these peaked rows its own
    # softmax is ~1e-5 away from the fp64 result; the kernel's tree sum is held to the fp64 result at the stated
    # tolerance and to the fp32 checker at that tolerance plus the checker's own distance from fp64.
    one = np.ones(pick.size, np.float32)
    d32 = oracle.cross_entropy_backward(xs[pick], target[pick], one)
    d64 = oracle.cross_entropy_backward(xs[pick].astype(np.float64), target[pick], one.astype(np.float64))
    assert rel_err(ds[pick], d64) <= TOL_ROW_F32
    assert rel_err(ds[pick], d32) <= TOL_ROW_F32 + rel_err(d32, d64)
    worst_sum = worst_d = 0.0
    for r0 in range(0, rows, 512):
        sm = np.exp(ys[r0:r0 + 512])
        worst_sum = max(worst_sum, float(np.abs(sm.sum(axis=1, dtype=np.float64) - 1.0).max()))
        sm[np.arange(sm.shape[0]), target[r0:r0 + 512]] -= 1.0
        worst_d = max(worst_d, float(np.abs(ds[r0:r0 + 512] - sm).max()))
    assert worst_sum <= 2e-5 and worst_d <= 1e-5
    assert np.max(np.abs(ls + ys[np.arange(rows), target])) <= 1e-5 * np.max(np.abs(ls))


def _m(shape, dtype):
    return TensorMeta.from_shape_and_strides(shape, contiguous_strides(shape), 0, DType.F32 if dtype == np.float32 else DType.F64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_host_slice_entry_points(hip, oracle, dtype):
    x = synth.normal(26, "x", (5, 11, 3), dtype=dtype)
    fn = K.log_softmax_dim_tensor_contiguous_f32 if dtype == np.float32 else K.log_softmax_dim_tensor_contiguous_f64
    for dim in range(3):
        got = fn(x.ravel(), _m(x.shape, dtype), dim)
        assert got.dtype == dtype and rel_err(got, oracle.log_softmax(x, dim).ravel()) <= _tol(dtype)
    with pytest.raises(Exception):
        fn(x.ravel(), _m(x.shape, dtype), 3)
    rows, cols = 9, 70
    logits = synth.normal(27, "logits", (rows, cols), dtype=dtype)
    target = _targets(27, rows, cols)
    dloss = synth.normal(27, "dloss", (rows,), dtype=dtype)
    sfx = "f32" if dtype == np.float32 else "f64"
    loss = getattr(K, "cross_entropy_forward_" + sfx)(logits, target, rows, cols)
    assert loss.dtype == dtype and rel_err(loss, oracle.cross_entropy_forward(logits, target)) <= _tol(dtype)
    d = getattr(K, "cross_entropy_backward_" + sfx)(logits, target, dloss, rows, cols)
    assert rel_err(d, oracle.cross_entropy_backward(logits, target, dloss).ravel()) <= _tol(dtype)
    assert getattr(K, "cross_entropy_forward_" + sfx)(logits[:0], target[:0], 0, cols).size == 0
    with pytest.raises(HipError):
        getattr(K, "cross_entropy_forward_" + sfx)(logits.ravel()[:-1], target, rows, cols)
