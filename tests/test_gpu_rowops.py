"""Parity of the HIP row kernels with the CPU checker, through the device-pointer C ABI.

fp32 row ops: max|d| / max|ref| <= 1e-5; fp64: <= 1e-12; add / bias add: bit-exact.
"""
import numpy as np
import pytest

from conftest import TOL_F64, TOL_ROW_F32, rel_err
from frankentorch_amd import synth
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu

# register-resident one-wave rows, four-wave rows, streaming rows, ragged / unaligned lengths
SHAPES = [(1, 1), (3, 7), (64, 256), (33, 768), (5, 1024), (16, 4100), (9, 4096), (8, 16384), (3, 20000), (4, 50257), (7, 513),
          (2, 40000), (2, 65536), (2, 65541)]  # beyond 8192 vectors: the register-and-LDS resident rows, then the sweeping kernel


def _inputs(rows, cols, dtype, seed=11):
    x = synth.normal(seed, "x", (rows, cols)).astype(dtype)
    w = synth.uniform(seed, "gamma", (cols,), 0.5, 1.5).astype(dtype)
    b = synth.normal(seed, "beta", (cols,), 0.0, 0.1).astype(dtype)
    r = synth.normal(seed, "res", (rows, cols)).astype(dtype)
    return x, w, b, r


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_row_ops_match_oracle(hip, oracle, rows, cols, dtype):
    tol = TOL_ROW_F32 if dtype == np.float32 else TOL_F64
    x, w, b, r = _inputs(rows, cols, dtype)
    dx, dw, db, dr = (DeviceBuffer.from_host(a) for a in (x, w, b, r))
    dy = DeviceBuffer(x.shape, dtype)
    hip.softmax_lastdim(dx, dy, rows, cols)
    assert rel_err(dy.to_host(), oracle.softmax(x, 1)) <= tol
    hip.layer_norm(dx, dw, db, dy, rows, cols, 1e-5)
    assert rel_err(dy.to_host(), oracle.layer_norm(x, w, b, 1e-5)) <= tol
    hip.layer_norm(dx, None, None, dy, rows, cols, 1e-5)
    assert rel_err(dy.to_host(), oracle.layer_norm(x, None, None, 1e-5)) <= tol
    hip.layer_norm(dx, dw, None, dy, rows, cols, 1e-5)
    assert rel_err(dy.to_host(), oracle.layer_norm(x, w, None, 1e-5)) <= tol
    hip.rms_norm(dx, dw, dy, rows, cols, 1e-6)
    assert rel_err(dy.to_host(), oracle.rms_norm(x, w, 1e-6)) <= tol
    hip.rms_norm(dx, None, dy, rows, cols, 1e-6)
    assert rel_err(dy.to_host(), oracle.rms_norm(x, None, 1e-6)) <= tol
    hip.gelu(dx, dy, rows * cols)
    assert rel_err(dy.to_host(), oracle.gelu(x)) <= tol
    hip.add(dx, dr, dy, rows * cols)
    assert np.array_equal(dy.to_host(), oracle.add(x, r))  # exact IEEE
    hip.bias_add(dx, db, dy, rows, cols)
    assert np.array_equal(dy.to_host(), oracle.bias_add(x, b))
    hip.bias_residual_add(dx, db, dr, dy, rows, cols)
    assert np.array_equal(dy.to_host(), oracle.bias_add(x, b, r))
    if dtype == np.float32:
        hip.add_layer_norm(dx, dr, dw, db, dy, rows, cols, 1e-5)
        assert rel_err(dy.to_host(), oracle.add_layer_norm(x, r, w, b, 1e-5)) <= tol
    else:
        with pytest.raises(TypeError):  # add_layer_norm_forward_f32 has no f64 twin
            hip.add_layer_norm(dx, dr, dw, db, dy, rows, cols, 1e-5)


def test_unaligned_pointers_take_the_scalar_path(hip, oracle):
    """A storage offset of one element breaks 16-byte alignment: results must not change class."""
    rows, cols = 6, 1024
    x, w, b, r = _inputs(rows, cols + 0, np.float32)
    pad = np.concatenate([np.zeros(1, np.float32), x.ravel()])
    dpad = DeviceBuffer.from_host(pad)
    dy = DeviceBuffer((rows * cols + 1,), np.float32)
    dw, db = DeviceBuffer.from_host(w), DeviceBuffer.from_host(b)
    hip.softmax_lastdim(dpad.view(1), dy.view(1), rows, cols)
    assert rel_err(dy.to_host()[1:].reshape(rows, cols), oracle.softmax(x, 1)) <= TOL_ROW_F32
    hip.layer_norm(dpad.view(1), dw, db, dy.view(1), rows, cols, 1e-5)
    assert rel_err(dy.to_host()[1:].reshape(rows, cols), oracle.layer_norm(x, w, b, 1e-5)) <= TOL_ROW_F32
    hip.gelu(dpad.view(1), dy.view(1), rows * cols)
    assert rel_err(dy.to_host()[1:].reshape(rows, cols), oracle.gelu(x)) <= TOL_ROW_F32
    hip.bias_add(dpad.view(1), db, dy.view(1), rows, cols)
    assert np.array_equal(dy.to_host()[1:].reshape(rows, cols), x + b)


def test_softmax_strided_dims(hip, oracle):
    x = synth.normal(5, "s", (6, 37, 19))
    dx = DeviceBuffer.from_host(x)
    dy = DeviceBuffer(x.shape)
    hip.softmax_strided(dx, dy, 6, 37, 19)
    assert rel_err(dy.to_host(), oracle.softmax(x, 1)) <= TOL_ROW_F32
    hip.softmax_strided(dx, dy, 1, 6, 37 * 19)
    assert rel_err(dy.to_host(), oracle.softmax(x, 0)) <= TOL_ROW_F32
    x64 = x.astype(np.float64)
    dx64, dy64 = DeviceBuffer.from_host(x64), DeviceBuffer(x.shape, np.float64)
    hip.softmax_strided(dx64, dy64, 6, 37, 19)
    assert rel_err(dy64.to_host(), oracle.softmax(x64, 1)) <= TOL_F64


def test_softmax_special_values(hip, oracle, vectors):
    """inf -> all-NaN row, NaN -> all-NaN row, finite extremes -> exact 0 and 1, uniform -> exact 0.5
    (crates/ft-kernel-cpu/src/lib.rs:65294-65317; golden bits 0x3f000000)."""
    cols = 8
    x = np.zeros((6, cols), np.float32)
    x[0, 2] = np.inf
    x[1, 3] = np.nan
    x[2] = [-1000.0, 0.0, 1000.0, 0, 0, 0, 0, 0]
    x[3] = -np.inf
    x[4] = 5.0
    x[5, 0] = -np.inf
    dx = DeviceBuffer.from_host(x)
    dy = DeviceBuffer(x.shape)
    hip.softmax_lastdim(dx, dy, 6, cols)
    y = dy.to_host()
    ref = oracle.softmax(x, 1)
    assert np.all(np.isnan(y[0])) and np.all(np.isnan(y[1])) and np.all(np.isnan(y[3]))
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert y[2, 0] == 0.0 and y[2, 2] == 1.0
    assert np.all(y[4].view(np.uint32) == 0x3E000000)  # 1/8 exactly
    assert y[5, 0] == 0.0 and rel_err(y[5, 1:], ref[5, 1:]) <= TOL_ROW_F32
    b = vectors["golden_text"]["softmax_parallel_bits"]
    rows, c2 = b["meta"]["fast_rows"], b["meta"]["fast_cols"]
    dz = DeviceBuffer.from_host(np.zeros((rows, c2), np.float32))
    dzo = DeviceBuffer((rows, c2))
    hip.softmax_lastdim(dz, dzo, rows, c2)
    bits = dzo.to_host().ravel().view(np.uint32)
    for i, v in b["bits"]["f32_softmax_fast_bits"].items():
        assert bits[int(i)] == int(v, 16)


@pytest.mark.parametrize("cols", [5, 1023, 50257, 40000])
def test_softmax_ragged_and_long_rows_special_values(hip, oracle, cols):
    """Rows that are no multiple of a 128-bit vector, or longer than 8192 vectors, take the resident-row kernel: the same
    special cases as the short rows (an infinity or a NaN poisons its row only, -inf elements weigh nothing), and every
    finite row sums to one."""
    x = synth.normal(77, "x", (7, cols)) * np.float32(3.0)
    x[0, cols // 2] = np.inf
    x[1, cols - 1] = np.nan
    x[2] = -np.inf
    x[3, 0] = -np.inf
    x[3, cols - 1] = -np.inf
    x[4] = 5.0
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer(x.shape)
    hip.softmax_lastdim(dx, dy, 7, cols)
    y, ref = dy.to_host(), oracle.softmax(x, 1)
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert np.all(np.isnan(y[0])) and np.all(np.isnan(y[1])) and np.all(np.isnan(y[2]))
    assert y[3, 0] == 0.0 and y[3, cols - 1] == 0.0
    fin = [3, 4, 5, 6]
    assert rel_err(y[fin], ref[fin]) <= TOL_ROW_F32
    assert np.max(np.abs(y[fin].astype(np.float64).sum(axis=1) - 1.0)) <= 1e-5
    assert np.all(y[4] == y[4, 0])
    hip.softmax_lastdim(dx, dy, 7, cols)
    assert np.array_equal(y.view(np.uint32), dy.to_host().view(np.uint32))


def test_gelu_special_values_and_dense_accuracy(hip, oracle):
    """The branch-free erf form against the checker (libm erff) on the values where the two could part: zeros, infinities,
    NaN, the far tails (where 1 + erff is exactly 0 or 2), denormals; and its absolute error on a dense sweep of [-8, 8]
    against erf in double precision (the documented bound is 4e-7; a 1-ulp erff is at 3e-7 there)."""
    import math

    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 6.0, -6.0, 5.7, -5.7, 1e-30, -1e-30, 1e-40, -1e-40, 3.0, -3.0, 0.5, -0.5],
                 np.float32)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer(x.shape)
    hip.gelu(dx, dy, x.size)
    y, ref = dy.to_host(), oracle.gelu(x)
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    fin = ~np.isnan(ref)
    assert np.array_equal(np.isinf(y[fin]), np.isinf(ref[fin])) and np.array_equal(np.signbit(y[fin]), np.signbit(ref[fin]))
    ok = fin & ~np.isinf(ref)
    assert np.max(np.abs(y[ok].astype(np.float64) - ref[ok].astype(np.float64))) <= 5e-7
    assert y[5] == 6.0 and y[6] == 0.0 and y[0] == 0.0
    sweep = np.linspace(-8.0, 8.0, 1 << 20).astype(np.float32)
    ds, do = DeviceBuffer.from_host(sweep), DeviceBuffer(sweep.shape)
    hip.gelu(ds, do, sweep.size)
    exact = 0.5 * sweep.astype(np.float64) * (1.0 + np.vectorize(math.erf)(sweep.astype(np.float64) / math.sqrt(2.0)))
    assert np.max(np.abs(do.to_host().astype(np.float64) - exact)) <= 5e-7


def test_empty_inputs_are_no_ops(hip):
    dx = DeviceBuffer((4,))
    hip.softmax_lastdim(dx, dx, 0, 4)
    hip.softmax_lastdim(dx, dx, 4, 0)
    hip.layer_norm(dx, None, None, dx, 0, 16, 1e-5)
    hip.gelu(dx, dx, 0)
    hip.add(dx, dx, dx, 0)


def test_full_size_row_ops_parity_determinism_and_properties(hip, oracle):
    """Config 2: fp32 [8192, 4096], seed 1. Parity on the whole tensor, run-twice bitwise equality,
    and properties that do not need the oracle (rows sum to 1, zero mean / unit variance, linearity)."""
    rows, cols = 8192, 4096
    x = synth.normal(1, "x", (rows, cols))
    gamma = synth.uniform(1, "gamma", (cols,), 0.5, 1.5)
    beta = synth.normal(1, "beta", (cols,), 0.0, 0.1)
    bias = synth.normal(1, "bias", (cols,), 0.0, 0.1)
    res = synth.normal(1, "residual", (rows, cols))
    dx, dg, dbt, dbi, dr = (DeviceBuffer.from_host(a) for a in (x, gamma, beta, bias, res))
    dy, dy2 = DeviceBuffer(x.shape), DeviceBuffer(x.shape)

    def twice(launch):
        launch(dy)
        launch(dy2)
        a, b = dy.to_host(), dy2.to_host()
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), "repeated runs differ bitwise"
        return a

    y = twice(lambda out: hip.softmax_lastdim(dx, out, rows, cols))
    assert rel_err(y, oracle.softmax(x, 1)) <= TOL_ROW_F32
    assert np.max(np.abs(y.sum(axis=1, dtype=np.float64) - 1.0)) < 1e-5 and y.min() >= 0 and y.max() <= 1
    y = twice(lambda out: hip.layer_norm(dx, dg, dbt, out, rows, cols, 1e-5))
    assert rel_err(y, oracle.layer_norm(x, gamma, beta, 1e-5)) <= TOL_ROW_F32
    hip.layer_norm(dx, None, None, dy, rows, cols, 1e-5)
    z = dy.to_host().astype(np.float64)
    assert np.max(np.abs(z.mean(axis=1))) < 1e-5 and np.max(np.abs(z.var(axis=1) - 1.0)) < 1e-3
    y = twice(lambda out: hip.rms_norm(dx, dg, out, rows, cols, 1e-6))
    assert rel_err(y, oracle.rms_norm(x, gamma, 1e-6)) <= TOL_ROW_F32
    y = twice(lambda out: hip.gelu(dx, out, rows * cols))
    assert rel_err(y, oracle.gelu(x)) <= TOL_ROW_F32
    y = twice(lambda out: hip.bias_residual_add(dx, dbi, dr, out, rows, cols))
    assert np.array_equal(y, (x + bias) + res)
    y = twice(lambda out: hip.add_layer_norm(dx, dr, dg, dbt, out, rows, cols, 1e-5))
    assert rel_err(y, oracle.add_layer_norm(x, res, gamma, beta, 1e-5)) <= TOL_ROW_F32


def test_layer_norm_row_pairs_give_the_bits_of_single_rows(hip):
    """Batches with rows enough run LayerNorm with two rows side by side per row group (gamma / beta fetched once per
    pair); smaller batches run one row per group. Per row the arithmetic and the reduction tree are the same, so a batch
    normalised in one call equals the same rows normalised in calls too small for the paired kernel, bit for bit -
    also with an odd number of rows, where the last pair has a single live row."""
    for rows, cols, piece in ((4097, 4096, 1024), (8192, 768, 1000), (5001, 2048, 512)):
        x = synth.normal(21, "x", (rows, cols))
        g = synth.uniform(21, "g", (cols,), 0.5, 1.5)
        b = synth.normal(21, "b", (cols,), 0.0, 0.1)
        dx, dg, db = DeviceBuffer.from_host(x), DeviceBuffer.from_host(g), DeviceBuffer.from_host(b)
        whole, parts = DeviceBuffer((rows, cols)), DeviceBuffer((rows, cols))
        hip.layer_norm(dx, dg, db, whole, rows, cols, 1e-5)
        for r0 in range(0, rows, piece):
            n = min(piece, rows - r0)
            hip.layer_norm(dx.view(r0 * cols), dg, db, parts.view(r0 * cols), n, cols, 1e-5)
        assert np.array_equal(whole.to_host().view(np.uint32), parts.to_host().view(np.uint32))
