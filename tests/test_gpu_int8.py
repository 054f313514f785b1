"""Int8 dynamic-quantised linear: bit-exact against the CPU checker (integer accumulation has no order, the three float
operations of the dequantisation are kept apart), on the reference's test inputs and on larger seeded shapes."""
import numpy as np
import pytest

from frankentorch_amd import kernel_hip as K
from frankentorch_amd import synth
from frankentorch_amd.core import HipError
from frankentorch_amd.device import DeviceBuffer
from test_oracle_backward import _lcg_matrices

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _quantize(hip, x):
    rows, cols = x.shape
    dx, dq, ds = DeviceBuffer.from_host(x), DeviceBuffer((rows, cols), np.int8), DeviceBuffer((rows,), np.float32)
    hip.quantize_rows_i8(dx, rows, cols, dq, ds)
    return dq.to_host(), ds.to_host()


# vector kernel (cols a multiple of 4 up to 8192, every registers-per-thread variant), scalar kernel (ragged or longer rows)
@pytest.mark.parametrize("rows,cols", [(1, 8), (7, 200), (64, 384), (33, 4099), (300, 768), (5, 1), (40, 1028), (9, 2048), (17, 4096), (6, 8192),
                                       (3, 8196), (5, 12288)])
def test_quantize_rows_is_exact(hip, oracle, rows, cols):
    x = synth.normal(41, "x", (rows, cols), 0.0, 2.0)
    x[0, 0] = 0.0
    if rows > 3:
        x[2] = 0.0          # an all-zero row: scale 1
        x[3, 0] = np.nan    # NaN quantises to 0 and does not move the scale
    q, s = _quantize(hip, x)
    qr, sr = oracle.quantize_rows_i8(x)
    assert np.array_equal(q, qr) and np.array_equal(_bits(s), _bits(sr))


def test_round_ties_to_even_like_the_reference(hip):
    # int8_quantizers_round_signed_ties_to_even, crates/ft-kernel-cpu/src/lib.rs:43721-43740
    ties = np.array([[-127.0, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 127.0]], np.float32)
    q, s = _quantize(hip, ties)
    assert q.tolist() == [[-127, -2, -2, 0, 0, 2, 2, 127]] and s.tolist() == [1.0]
    q, s = K.quantize_per_output_channel_i8(ties, 1, 8)
    assert q.tolist() == [-127, -2, -2, 0, 0, 2, 2, 127] and s.tolist() == [1.0]
    q, s = K.quantize_rows_i8(ties, 1, 8)
    assert q.tolist() == [-127, -2, -2, 0, 0, 2, 2, 127] and s.tolist() == [1.0]


def _linear(hip, x, w_i8, w_scales, bias):
    m, k = x.shape
    n = w_i8.shape[0]
    bufs = [DeviceBuffer.from_host(t) for t in (x, w_i8, w_scales)]
    db = None if bias is None else DeviceBuffer.from_host(bias)
    out = DeviceBuffer((m, n), np.float32)
    hip.linear_int8_dynamic(bufs[0], m, k, bufs[1], bufs[2], n, db, out)
    return out.to_host()


# the reference's three test shapes (k = 200 takes the plain kernel), matrix-core shapes with ragged m / n, K of one stage,
# and two shapes with enough 256 x 256 tiles for the large-tile kernel (ragged edges; K of one, two and five stages)
SHAPES = [(8, 384, 384), (4, 384, 1536), (7, 200, 53), (128, 64, 128), (130, 768, 300), (257, 1024, 129), (1, 64, 1), (512, 3072, 768),
          (4100, 128, 4100), (4096, 64, 4096), (8200, 320, 2050)]


@pytest.mark.parametrize("m,k,n", SHAPES)
@pytest.mark.parametrize("with_bias", [True, False])
def test_linear_int8_dynamic_is_bit_exact(hip, oracle, m, k, n, with_bias):
    if m * k * n <= 8 * 384 * 1536:
        x, w, bias = _lcg_matrices(m, k, n)  # the reference's generator for its own shapes
    else:
        x, w, bias = synth.normal(42, "x", (m, k), 0.0, 3.0), synth.normal(42, "w", (n, k), 0.0, 0.5), synth.normal(42, "b", (n,))
    w_i8, w_scales = oracle.quantize_rows_i8(w)
    b = bias if with_bias else None
    got = _linear(hip, x, w_i8, w_scales, b)
    assert np.array_equal(_bits(got), _bits(oracle.linear_int8_dynamic(x, w_i8, w_scales, b)))
    # the reference's accuracy bound against the f32 product
    if with_bias:
        ref = x.astype(np.float64) @ w.astype(np.float64).T + bias
        y = got.astype(np.float64)
        assert (ref * y).sum() / np.sqrt((ref * ref).sum() * (y * y).sum()) > 0.999


def test_extreme_integers_do_not_overflow(hip, oracle):
    """Every product +-127 * +-127 with the same sign over K = 4096: |acc| = 66 064 384, far inside int32."""
    m, k, n = 64, 4096, 128
    x = np.full((m, k), 5.0, np.float32)
    w = np.full((n, k), -0.25, np.float32)
    w[::2] *= -1
    w_i8, w_scales = oracle.quantize_rows_i8(w)
    got = _linear(hip, x, w_i8, w_scales, None)
    assert np.array_equal(_bits(got), _bits(oracle.linear_int8_dynamic(x, w_i8, w_scales)))
    assert np.allclose(got[:, 0], 5.0 * 0.25 * k, rtol=1e-6) and np.allclose(got[:, 1], -5.0 * 0.25 * k, rtol=1e-6)


def test_host_slice_entry_points(hip, oracle):
    m, k, n = 6, 384, 384  # linear_int8_dynamic_is_deterministic, crates/ft-kernel-cpu/src/lib.rs:43710-43719
    x = (((np.arange(m * k) % 17).astype(np.float32) - 8.0) * np.float32(0.1)).reshape(m, k)
    w = (((np.arange(n * k) % 13).astype(np.float32) - 6.0) * np.float32(0.05)).reshape(n, k)
    w_i8, w_scales = K.quantize_per_output_channel_i8(w, n, k)
    wr, sr = oracle.quantize_rows_i8(w)
    assert np.array_equal(w_i8.reshape(n, k), wr) and np.array_equal(_bits(w_scales), _bits(sr))
    a = K.linear_int8_dynamic_f32(x, m, k, w_i8, w_scales, n)
    assert np.array_equal(_bits(a), _bits(K.linear_int8_dynamic_f32(x, m, k, w_i8, w_scales, n)))
    assert np.array_equal(_bits(a), _bits(oracle.linear_int8_dynamic(x, wr, sr).ravel()))
    for bad in (lambda: K.linear_int8_dynamic_f32(x.ravel()[:-1], m, k, w_i8, w_scales, n),   # the reference's assert_eq!s
                lambda: K.linear_int8_dynamic_f32(x, m, k, w_i8[:-1], w_scales, n),
                lambda: K.linear_int8_dynamic_f32(x, m, k, w_i8, w_scales[:-1], n),
                lambda: K.linear_int8_dynamic_f32(x, m, k, w_i8, w_scales, n, np.zeros(n - 1, np.float32))):
        with pytest.raises(HipError):
            bad()
    assert K.linear_int8_dynamic_f32(x[:0], 0, k, w_i8, w_scales, n).size == 0
