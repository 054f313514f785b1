"""The `ft_kernel_cpu`-shaped entry points (host arrays in, host array out) on the GPU: the
reference's own fixtures and in-source known answers, then seeded parity with the CPU checker."""
import math

import numpy as np
import pytest

from conftest import TOL_F64, TOL_GEMM_F32, TOL_ROW_F32, rel_err
from frankentorch_amd import kernel_hip as K
from frankentorch_amd import synth
from frankentorch_amd.core import DType, TensorMeta, contiguous_strides

pytestmark = pytest.mark.gpu


def _m(shape, dtype, off=0):
    return TensorMeta.from_shape_and_strides(shape, contiguous_strides(shape), off, DType.F32 if dtype == np.float32 else DType.F64)


def _f(vals):
    return np.array([float(v) for v in vals], dtype=np.float64)


def test_conformance_fixtures(hip, vectors):
    for c in vectors["conformance"]:
        tol = max(c.get("tolerance", 0.0), 0.0)
        exp = _f(c["expected_output"])
        for dt, extra in ((np.float64, 0.0), (np.float32, 1e-6)):
            if c["op"] == "gelu":
                got = K.gelu_tensor_contiguous_f64(_f(c["input"]), _m(c["shape"], dt)) if dt == np.float64 else \
                    K.gelu_tensor_contiguous_f32(_f(c["input"]), _m(c["shape"], dt))
            elif c["op"] == "softmax":
                fn = K.softmax_dim_tensor_contiguous_f64 if dt == np.float64 else K.softmax_dim_tensor_contiguous_f32
                got = fn(_f(c["input"]), _m(c["shape"], dt), c["dim"])
            elif c["op"] == "log_softmax":
                fn = K.log_softmax_dim_tensor_contiguous_f64 if dt == np.float64 else K.log_softmax_dim_tensor_contiguous_f32
                got = fn(_f(c["input"]), _m(c["shape"], dt), c["dim"])
            elif c["op"] == "add":
                fn = K.add_tensor_contiguous_f64 if dt == np.float64 else K.add_tensor_contiguous_f32
                got = fn(_f(c["lhs"]), _f(c["rhs"]), _m(c["shape"], dt), _m(c["shape"], dt))
            elif c["op"] == "matmul":
                fn = K.matmul_tensor_contiguous_f64 if dt == np.float64 else K.matmul_tensor_contiguous_f32
                got = fn(_f(c["lhs"]), _f(c["rhs"]), _m(c.get("lhs_shape", c.get("shape")), dt), _m(c.get("rhs_shape", c.get("shape")), dt))
            elif c["op"] == "index_select":
                fn = K.index_select_tensor_contiguous_f64 if dt == np.float64 else K.index_select_tensor_contiguous_f32
                got = fn(_f(c["input"]), _m(c["input_shape"], dt), c["dim"], _f(c["index"]))
            else:
                raise AssertionError("unhandled fixture op " + c["op"])
            assert got.dtype == dt and got.shape == exp.shape, c["name"]
            assert np.max(np.abs(got - exp)) <= tol + extra, (c["name"], dt)


def test_in_source_known_answers(hip, vectors):
    by = {c["name"]: c for c in vectors["in_source"]}
    c = by["bmm_respects_storage_offsets_and_batch_order"]
    for dt, fn in ((np.float64, K.bmm_tensor_contiguous_f64), (np.float32, K.bmm_tensor_contiguous_f32)):
        got = fn(_f(c["lhs"]), _f(c["rhs"]), _m(c["lhs_shape"], dt, c["lhs_offset"]), _m(c["rhs_shape"], dt, c["rhs_offset"]))
        assert got.tolist() == [float(v) for v in c["expected_output"]]
    c = by["bmm_f32_4x4_with_offsets"]
    batch, lo, ro = c["batch"], c["lhs_offset"], c["rhs_offset"]
    lhs = np.full(lo + batch * 16, c["lhs_fill"], np.float32)
    rhs = np.full(ro + batch * 16, c["rhs_fill"], np.float32)
    i = np.arange(batch * 16)
    lhs[lo:] = (i % 7) - 3.0
    rhs[ro:] = (i % 11) - 5.0
    got = K.bmm_tensor_contiguous_f32(lhs, rhs, _m([batch, 4, 4], np.float32, lo), _m([batch, 4, 4], np.float32, ro))
    exp = np.einsum("bij,bjk->bik", lhs[lo:].reshape(batch, 4, 4), rhs[ro:].reshape(batch, 4, 4))
    assert np.array_equal(got.reshape(batch, 4, 4), exp)  # small integers: exact in any order
    for name in ("addmm_accepts_contiguous_operands", "addmm_alpha_zero_f64", "addmm_alpha_zero_f32"):
        c = by[name]
        dt = np.float32 if c["dtype"] == "f32" else np.float64
        fn = K.addmm_tensor_contiguous_f32 if dt == np.float32 else K.addmm_tensor_contiguous_f64
        got = fn(_f(c["input"]), _f(c["mat1"]), _f(c["mat2"]), _m(c["input_shape"], dt), _m(c["mat1_shape"], dt), _m(c["mat2_shape"], dt),
                 c["beta"], c["alpha"])
        assert got.tolist() == [float(v) for v in c["expected_output"]], name
    c = by["inf_in_softmax_produces_nan"]
    assert np.all(np.isnan(K.softmax_dim_tensor_contiguous_f64(_f(c["input"]), _m(c["shape"], np.float64), 0)))
    c = by["softmax_with_finite_extremes"]
    got = K.softmax_dim_tensor_contiguous_f64(_f(c["input"]), _m(c["shape"], np.float64), 0)
    assert got[0] == 0.0 and got[2] == 1.0
    for name in ("argmax_dim_reduces_along_dim0", "argmax_dim_reduces_along_dim1", "argmax_dim_1d_reduces_to_scalar"):
        c = by[name]
        got = K.argmax_dim_tensor_contiguous_f64(_f(c["input"]), _m(c["shape"], np.float64), c["dim"])
        assert got.tolist() == [float(v) for v in c["expected_output"]], name
    c = by["gelu_returns_expected_values"]
    got = K.gelu_tensor_contiguous_f64(_f(c["input"]), _m([3], np.float64))
    assert all(abs(g - e) < t for g, e, t in zip(got, c["expected_near"], c["abs_tol"]))
    for row in vectors["golden_text"]["softmax_rows_pass10"]["rows"]:
        got = K.softmax_dim_tensor_contiguous_f64(_f(row["input"]), _m([1, 3], np.float64), 1)
        assert np.max(np.abs(got - _f(row["expected_output"]))) < 1e-12


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_seeded_parity_of_every_entry_point(hip, oracle, dtype):
    f32 = dtype == np.float32
    sfx = "f32" if f32 else "f64"
    trow, tgemm = (TOL_ROW_F32, TOL_GEMM_F32) if f32 else (TOL_F64, TOL_F64)
    g = lambda name: getattr(K, name + "_" + sfx)
    x = synth.normal(12, "x", (37, 260)).astype(dtype)
    w = synth.uniform(12, "w", (260,), 0.5, 1.5).astype(dtype)
    b = synth.normal(12, "b", (260,)).astype(dtype)
    r = synth.normal(12, "r", (37, 260)).astype(dtype)
    m2 = _m([37, 260], dtype)
    assert rel_err(g("softmax_dim_tensor_contiguous")(x, m2, 1).reshape(x.shape), oracle.softmax(x, 1)) <= trow
    assert rel_err(g("softmax_dim_tensor_contiguous")(x, m2, 0).reshape(x.shape), oracle.softmax(x, 0)) <= trow
    assert rel_err(g("layer_norm_forward")(x, w, b, 37, 260, 1e-5).reshape(x.shape), oracle.layer_norm(x, w, b, 1e-5)) <= trow
    assert rel_err(g("layer_norm_forward")(x, None, None, 37, 260, 1e-5).reshape(x.shape), oracle.layer_norm(x, None, None, 1e-5)) <= trow
    assert rel_err(g("rms_norm_forward")(x, w, 37, 260, 1e-6).reshape(x.shape), oracle.rms_norm(x, w, 1e-6)) <= trow
    assert rel_err(g("gelu_tensor_contiguous")(x, m2).reshape(x.shape), oracle.gelu(x)) <= trow
    assert np.array_equal(g("add_tensor_contiguous")(x, r, m2, m2).reshape(x.shape), x + r)
    if f32:
        assert rel_err(K.add_layer_norm_forward_f32(x, r, w, b, 37, 260, 1e-5).reshape(x.shape), oracle.add_layer_norm(x, r, w, b, 1e-5)) <= trow
    # storage offsets are honoured (crates/ft-kernel-cpu/src/lib.rs:37794-37795)
    padded = np.concatenate([np.full(5, 9.0, dtype), x.ravel()])
    assert rel_err(g("softmax_dim_tensor_contiguous")(padded, _m([37, 260], dtype, 5), 1).reshape(x.shape), oracle.softmax(x, 1)) <= trow
    a = synth.uniform(12, "A", (70, 130), -1, 1).astype(dtype)
    bm = synth.uniform(12, "B", (130, 50), -1, 1).astype(dtype)
    wt = np.ascontiguousarray(bm.T)
    bias = synth.normal(12, "bias", (50,)).astype(dtype)
    assert rel_err(g("matmul_tensor_contiguous")(a, bm, _m([70, 130], dtype), _m([130, 50], dtype)).reshape(70, 50), oracle.gemm(a, bm)) <= tgemm
    assert rel_err(g("matmul_rhs_transposed_contiguous")(70, 130, 50, a, wt).reshape(70, 50), oracle.gemm(a, bm)) <= tgemm
    assert rel_err(g("linear_tensor")(a, wt, bias, 70, 130, 50).reshape(70, 50), oracle.linear(a, wt, bias)) <= tgemm
    assert rel_err(g("linear_tensor")(a, wt, None, 70, 130, 50).reshape(70, 50), oracle.linear(a, wt, None)) <= tgemm
    inp = synth.normal(12, "inp", (70, 50)).astype(dtype)
    assert rel_err(g("addmm_tensor_contiguous")(inp, a, bm, _m([70, 50], dtype), _m([70, 130], dtype), _m([130, 50], dtype), 0.5, 2.0).reshape(70, 50),
                   oracle.addmm(inp, a, bm, 0.5, 2.0)) <= tgemm
    assert rel_err(g("addmm_tensor_contiguous")(bias, a, bm, _m([50], dtype), _m([70, 130], dtype), _m([130, 50], dtype), -1.0, 1.0).reshape(70, 50),
                   oracle.addmm(bias, a, bm, -1.0, 1.0)) <= tgemm
    a3 = synth.uniform(12, "A3", (9, 20, 30), -1, 1).astype(dtype)
    b3 = synth.uniform(12, "B3", (9, 30, 10), -1, 1).astype(dtype)
    assert rel_err(g("bmm_tensor_contiguous")(a3, b3, _m([9, 20, 30], dtype), _m([9, 30, 10], dtype)).reshape(9, 20, 10), oracle.bmm(a3, b3)) <= tgemm
    q = synth.normal(12, "q", (3, 40, 64), 0, 0.125).astype(dtype)
    k = synth.normal(12, "k", (3, 40, 64)).astype(dtype)
    v = synth.normal(12, "v", (3, 40, 64)).astype(dtype)
    got = g("sdpa_forward")(q, k, v, 3, 40, 40, 64, 64, 0.125, True).reshape(3, 40, 64)
    assert rel_err(got, oracle.sdpa_forward(q, k, v, 0.125, True)) <= tgemm
    t = synth.normal(12, "t", (11, 6, 4)).astype(dtype)
    idx = np.array([5.0, 0.0, 5.0, 2.0])
    assert np.array_equal(g("index_select_tensor_contiguous")(t, _m([11, 6, 4], dtype), 1, idx).reshape(11, 4, 4), oracle.index_select(t, 1, idx)[0])
    assert np.array_equal(g("argmax_dim_tensor_contiguous")(t, _m([11, 6, 4], dtype), 1).reshape(11, 4), oracle.argmax(t, 1))
    assert np.array_equal(g("argmax_dim_tensor_contiguous")(t, _m([11, 6, 4], dtype), 2).reshape(11, 6), oracle.argmax(t, 2))


def test_short_slices_are_errors_not_faults(hip):
    """The reference panics on a short slice in its infallible fused entry points; here that is a
    clean InvalidArgument before any launch."""
    from frankentorch_amd.core import HipError

    x = np.zeros(10, np.float32)
    with pytest.raises(HipError):
        K.layer_norm_forward_f32(x, None, None, 4, 4, 1e-5)
    with pytest.raises(HipError):
        K.linear_tensor_f32(x, x, None, 4, 4, 4)
    with pytest.raises(HipError):
        K.sdpa_forward_f32(x, x, x, 1, 4, 4, 4, 4, 1.0, True)
    with pytest.raises(HipError):
        K.rms_norm_forward_f32(x, None, 3, 4, 1e-6)


# ---- the staged transfer paths: operands of 1 MiB and more go through the pinned rings, row-wise ops run as an
# upload / kernel / download pipeline over chunks of rows (8 MiB chunks: the shapes below give 1, 3 and 7 chunks,
# with a ragged last chunk) ----
PIPE_SHAPES = [(300, 1000), (5001, 1000), (1237, 12288), (3, 1048576)]


@pytest.mark.parametrize("rows,cols", PIPE_SHAPES)
def test_row_pipeline_equals_the_device_tier_bit_for_bit(hip, oracle, rows, cols):
    """Chunking a row-wise op over the pipeline cannot change a bit: every row goes through the same kernel as in one
    launch over the resident tensor. Checked against the device tier, and against the CPU checker at the row-op bar."""
    from frankentorch_amd.device import DeviceBuffer

    x = synth.normal(41, "x", (rows, cols))
    r = synth.normal(41, "r", (rows, cols))
    g = synth.uniform(41, "g", (cols,), 0.5, 1.5)
    b = synth.normal(41, "b", (cols,), 0.0, 0.1)
    m = _m([rows, cols], np.float32)
    dx, dr, dg, db = (DeviceBuffer.from_host(a) for a in (x, r, g, b))
    dy = DeviceBuffer((rows, cols))

    def dev(fn):
        fn()
        return dy.to_host().reshape(-1)

    cases = [
        ("softmax", K.softmax_dim_tensor_contiguous_f32(x, m, 1), dev(lambda: hip.softmax_lastdim(dx, dy, rows, cols)), oracle.softmax(x, 1)),
        ("log_softmax", K.log_softmax_dim_tensor_contiguous_f32(x, m, 1), dev(lambda: hip.log_softmax_strided(dx, dy, rows, cols, 1)), None),
        ("layer_norm", K.layer_norm_forward_f32(x, g, b, rows, cols, 1e-5), dev(lambda: hip.layer_norm(dx, dg, db, dy, rows, cols, 1e-5)),
         oracle.layer_norm(x, g, b, 1e-5)),
        ("add_layer_norm", K.add_layer_norm_forward_f32(x, r, g, b, rows, cols, 1e-5), dev(lambda: hip.add_layer_norm(dx, dr, dg, db, dy, rows, cols, 1e-5)), None),
        ("rms_norm", K.rms_norm_forward_f32(x, g, rows, cols, 1e-6), dev(lambda: hip.rms_norm(dx, dg, dy, rows, cols, 1e-6)), oracle.rms_norm(x, g, 1e-6)),
        ("gelu", K.gelu_tensor_contiguous_f32(x, m), dev(lambda: hip.gelu(dx, dy, rows * cols)), oracle.gelu(x)),
        ("add", K.add_tensor_contiguous_f32(x, r, m, m), dev(lambda: hip.add(dx, dr, dy, rows * cols)), (x + r)),
    ]
    for name, got, resident, ref in cases:
        assert got.shape == (rows * cols,), name
        assert np.array_equal(got.view(np.uint32), resident.view(np.uint32)), name
        # rows of a million elements: the checker's serial fp32 sums (the reference's order) are themselves 2e-4 away from
        # the exact sums there, so only the bitwise comparison with the device tier applies
        if ref is not None and cols <= 65536:
            assert rel_err(got, np.asarray(ref).reshape(-1)) <= TOL_ROW_F32, name


def test_pinned_slices_take_the_direct_path_and_give_the_same_bits(hip):
    from frankentorch_amd.device import PinnedArray

    rows, cols = 4099, 1536
    x = synth.normal(42, "x", (rows, cols))
    m = _m([rows, cols], np.float32)
    ref = K.softmax_dim_tensor_contiguous_f32(x, m, 1)
    px, py = PinnedArray((rows * cols,)), PinnedArray((rows * cols,))
    px.array[:] = x.reshape(-1)
    py.array[:] = -1.0
    import ctypes as C

    from frankentorch_amd import _lib
    from frankentorch_amd.core import check

    mc, n_out = m.to_c(), C.c_size_t(0)
    check(_lib.load().fth_softmax_dim_tensor_contiguous_f32(px.ptr, rows * cols, C.byref(mc), 1, py.ptr, rows * cols, C.byref(n_out)))
    assert n_out.value == rows * cols
    assert np.array_equal(py.array.view(np.uint32), ref.view(np.uint32))
    # a pinned input with a pageable output, and the other way round
    out = np.full(rows * cols, -1.0, np.float32)
    check(_lib.load().fth_softmax_dim_tensor_contiguous_f32(px.ptr, rows * cols, C.byref(mc), 1, out.ctypes.data, out.size, C.byref(n_out)))
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32))
    py.array[:] = -1.0
    xin = np.ascontiguousarray(x.reshape(-1))
    check(_lib.load().fth_softmax_dim_tensor_contiguous_f32(xin.ctypes.data, xin.size, C.byref(mc), 1, py.ptr, rows * cols, C.byref(n_out)))
    assert np.array_equal(py.array.view(np.uint32), ref.view(np.uint32))
    px.free()
    py.free()


def test_staged_operands_of_a_product(hip, oracle):
    """Operands above 1 MiB are uploaded through the pinned rings (here 3 and 2 chunks) and the result comes back the same way."""
    m_, k_, n_ = 1500, 1400, 1100
    a = synth.uniform(43, "a", (m_, k_), -1, 1)
    b = synth.uniform(43, "b", (k_, n_), -1, 1)
    got = K.matmul_tensor_contiguous_f32(a, b, _m([m_, k_], np.float32), _m([k_, n_], np.float32))
    assert rel_err(got.reshape(m_, n_), oracle.gemm(a, b)) <= TOL_GEMM_F32
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    got = K.matmul_tensor_contiguous_f64(a64, b64, _m([m_, k_], np.float64), _m([k_, n_], np.float64))
    assert rel_err(got.reshape(m_, n_), oracle.gemm(a64, b64)) <= TOL_F64
    # and a second call right after: the rings are idle again and reusable
    got2 = K.matmul_tensor_contiguous_f64(a64, b64, _m([m_, k_], np.float64), _m([k_, n_], np.float64))
    assert np.array_equal(got.view(np.uint64), got2.view(np.uint64))
