"""tanh-form GELU (the activation of the reference's fused GPU encoder and of GELU::tanh()): the elementwise kernel, the
GEMM epilogue and the encoder option against the CPU checker; fp32 row work <= 1e-5, products <= 2e-5, fp64 <= 1e-12."""
import numpy as np
import pytest

from conftest import TOL_F64, TOL_GEMM_F32, TOL_ROW_F32, rel_err
from frankentorch_amd import fused
from frankentorch_amd import kernel_hip as K
from frankentorch_amd import synth
from frankentorch_amd.core import DType, TensorMeta, contiguous_strides
from frankentorch_amd.device import EPI_BIAS, EPI_GELU, EPI_GELU_TANH, DeviceBuffer
from test_gpu_resident import make_layer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 7, 1000, 4096 * 33 + 5])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_elementwise_matches_oracle(hip, oracle, n, dtype):
    x = synth.normal(31, "x", (n,), 0.0, 3.0, dtype=dtype)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer((n,), dtype)
    hip.gelu_tanh(dx, dy, n)
    got = dy.to_host()
    assert rel_err(got, oracle.gelu_tanh(x)) <= (TOL_ROW_F32 if dtype == np.float32 else TOL_F64)
    hip.gelu_tanh(dx, dx, n)  # in place
    assert np.array_equal(dx.to_host().view(np.uint8), got.view(np.uint8))


def test_golden_values_and_saturation(hip, vectors):
    c = {v["name"]: v for v in vectors["in_source"]}["gelu_tanh_module_matches_torch"]
    x = np.array(c["input"], np.float64)
    meta = lambda dt, n: TensorMeta.from_shape_and_strides([n], contiguous_strides([n]), 0, DType.F32 if dt == np.float32 else DType.F64)
    got = K.gelu_tanh_tensor_contiguous_f64(x, meta(np.float64, x.size))
    assert np.max(np.abs(got - np.array(c["expected_output"]))) <= c["abs_tol"]
    got32 = K.gelu_tanh_tensor_contiguous_f32(x, meta(np.float32, x.size))
    assert got32.dtype == np.float32 and np.max(np.abs(got32 - np.array(c["expected_output"]))) <= 2e-7
    # the fused module's clamp: x >= 10 passes through, x <= -10 gives 0; inf and NaN behave
    edge = np.array([10.0, 12.5, 1e30, np.inf, -10.0, -50.0, -1e30, -np.inf, 0.0, -0.0, np.nan], np.float32)
    y = K.gelu_tanh_tensor_contiguous_f32(edge, meta(np.float32, edge.size))
    assert np.array_equal(y[:4], edge[:4]) and np.all(y[4:10] == 0.0) and np.isnan(y[10])
    # distinct from the erf form at the reference's example point: 0.84119 vs 0.84134
    e = K.gelu_tensor_contiguous_f64(np.array([1.0]), meta(np.float64, 1))[0]
    t = K.gelu_tanh_tensor_contiguous_f64(np.array([1.0]), meta(np.float64, 1))[0]
    assert abs(t - 0.8411919906082768) < 1e-12 and abs(e - t) > 1e-4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(150, 200, 96), (512, 3072, 768), (37, 53, 41)])
def test_gemm_epilogue(hip, oracle, dtype, shape):
    """bias + tanh-GELU in the epilogue (the direct-to-LDS kernel, the split-K fix-up and the generic kernel) against the
    checker's linear followed by its tanh-GELU."""
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    m, n, k = shape
    a = synth.uniform(32, "a", (m, k), -1, 1, dtype=dtype)
    w = synth.uniform(32, "w", (n, k), -1, 1, dtype=dtype)
    bias = synth.normal(32, "bias", (n,), dtype=dtype)
    da, dw, db, dc = DeviceBuffer.from_host(a), DeviceBuffer.from_host(w), DeviceBuffer.from_host(bias), DeviceBuffer((m, n), dtype)
    hip.gemm(hip.gemm_desc(m, n, k, trans_b=True, epilogue=EPI_BIAS | EPI_GELU_TANH), da, dw, dc, bias=db)
    got = dc.to_host()
    ref = oracle.gelu_tanh(oracle.linear(a, w, bias))
    assert rel_err(got, ref) <= tol
    hip.gemm(hip.gemm_desc(m, n, k, trans_b=True, epilogue=EPI_BIAS | EPI_GELU_TANH), da, dw, dc, bias=db)
    assert np.array_equal(got.view(np.uint8), dc.to_host().view(np.uint8))
    with pytest.raises(Exception):  # both forms at once
        hip.gemm(hip.gemm_desc(m, n, k, trans_b=True, epilogue=EPI_BIAS | EPI_GELU | EPI_GELU_TANH), da, dw, dc, bias=db)


def test_encoder_and_batch_with_the_tanh_form(hip, oracle):
    batch, seq, d, heads, f = 2, 64, 256, 4, 1024
    layers = [make_layer(5, 0, d, f, biases_zero=False), make_layer(5, 1, d, f, biases_zero=False)]
    x = synth.normal(5, "x", (batch * seq, d))
    enc = fused.EncoderHip(d, heads, f, layers, 1e-5, causal=True, gelu_tanh=True)
    got = enc.forward(x, batch, seq)
    ref = x
    for layer in layers:
        ref = oracle.encoder_layer(layer, ref, batch, seq, heads, 1e-5, True, gelu_tanh=True)
    assert rel_err(got, ref) <= TOL_GEMM_F32
    erf_ref = x
    for layer in layers:
        erf_ref = oracle.encoder_layer(layer, erf_ref, batch, seq, heads, 1e-5, True)
    assert rel_err(got, erf_ref) > TOL_GEMM_F32  # the two activations are told apart at this tolerance
    b = fused.Batch()
    t = b.gelu_tanh(fused.HipTensor.upload(x))
    b.finish()
    assert rel_err(t.download(), oracle.gelu_tanh(x)) <= TOL_ROW_F32
