"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, validates exactly as the reference does (validation never needs a GPU), and refuses to
compute without one (no CPU fallback)."""
import ctypes as C
import os

import numpy as np
import pytest

from frankentorch_amd import _lib, core, kernel_hip as K, synth
from frankentorch_amd.core import DType, Device, KernelError, TensorMeta


def test_library_exports_every_declared_symbol():
    protos = _lib.protos()
    assert len(protos) >= 100
    lib = _lib.load()
    missing = [n for n in protos if not hasattr(lib, n)]
    assert missing == []
    for family in ("fth_dev_gemm_f32", "fth_dev_sdpa_forward_f32", "fth_dev_softmax_lastdim_f32", "fth_matmul_tensor_contiguous_f32",
                   "fth_sdpa_forward_f64", "fth_tensor_upload", "fth_batch_mha", "fth_encoder_forward_graph", "fth_gpt2_forward_dev"):
        assert family in protos


def test_struct_layouts_match_the_header():
    assert C.sizeof(_lib.Meta) == 16 + 8 * 8 * 2 + 8
    assert C.sizeof(_lib.GemmDesc) == 10 * 8 + 16
    assert C.sizeof(_lib.SdpaDesc) == 18 * 8 + 8
    assert C.sizeof(_lib.LayerWeights) == 16 * 8
    assert C.sizeof(_lib.ErrorInfo) == 16 + 64 + 64 + 16 + 16 + 200


def test_status_names():
    lib = _lib.load()
    assert lib.fth_status_name(0) == b"Ok"
    assert lib.fth_status_name(3) == b"ShapeMismatch"
    assert lib.fth_status_name(100) == b"Unavailable"


def test_tensor_meta_contiguity_rules():
    m = TensorMeta.from_shape([2, 3, 4])
    assert m.strides == [12, 4, 1] and m.numel() == 24
    # size-1 dims are contiguous whatever their stride (crates/ft-core/src/lib.rs:580-607)
    a = np.zeros(6, np.float32)
    ok = TensorMeta.from_shape_and_strides([2, 1, 3], [3, 99, 1], 0)
    assert K.gelu_tensor_contiguous_f32.__name__  # surface exists
    out_len = C.c_size_t()
    mc = ok.to_c()
    assert _lib.load().fth_gelu_tensor_contiguous_f32(a.ctypes.data, a.size, C.byref(mc), None, 0, C.byref(out_len)) == 0
    assert out_len.value == 6
    bad = TensorMeta.from_shape_and_strides([2, 3], [1, 2], 0).to_c()
    assert _lib.load().fth_gelu_tensor_contiguous_f32(a.ctypes.data, a.size, C.byref(bad), None, 0, C.byref(out_len)) == 4


def _err(fn, *args):
    with pytest.raises(KernelError) as ei:
        fn(*args)
    return ei.value


def test_matmul_validation_order_and_payloads():
    """dtype -> device -> lhs layout -> rhs layout -> rank / inner dim -> storage
    (crates/ft-kernel-cpu/src/lib.rs:36935-36962, 37787-37793)."""
    a = np.zeros(6, np.float32)
    f32 = lambda s, **kw: TensorMeta.from_shape(s, DType.F32, kw.get("device", Device.Cpu))
    e = _err(K.matmul_tensor_contiguous_f32, a, a, TensorMeta.from_shape([2, 3], DType.F64), f32([3, 2]))
    assert e.kind == "Incompatible(DTypeMismatch)"
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([2, 3], device=Device.Cuda), f32([3, 2]))
    assert e.kind == "Incompatible(DeviceMismatch)"
    nc = TensorMeta.from_shape_and_strides([2, 3], [1, 2], 0)
    e = _err(K.matmul_tensor_contiguous_f32, a, a, nc, nc)
    assert e.kind == "UnsupportedLayout" and e.side == "lhs"
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([2, 3]), nc)
    assert e.kind == "UnsupportedLayout" and e.side == "rhs"
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([2, 3]), f32([2, 3]))
    assert e.kind == "ShapeMismatch" and e.lhs == [2, 3] and e.rhs == [2, 3]
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([6]), f32([6]))
    assert e.kind == "ShapeMismatch"
    off = TensorMeta.from_shape_and_strides([2, 3], [3, 1], 1)
    e = _err(K.matmul_tensor_contiguous_f32, a, a, off, f32([3, 2]))
    assert e.kind == "InsufficientStorage" and e.side == "lhs" and e.needed == 7 and e.available == 6
    # m * n overflows while each operand's own element count does not
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([2 ** 40, 1]), f32([1, 2 ** 40]))
    assert e.kind == "ShapeOverflow"
    # an operand whose own element count overflows is already non-contiguous (checked_mul in is_contiguous)
    e = _err(K.matmul_tensor_contiguous_f32, a, a, f32([2 ** 40, 2 ** 40]), f32([2 ** 40, 2 ** 40]))
    assert e.kind == "UnsupportedLayout" and e.side == "lhs"


def test_reference_error_cases(vectors):
    by = {c["name"]: c for c in vectors["in_source"]}
    c = by["addmm_alpha_zero_still_validates_mat1"]
    m = lambda shape, off=0: TensorMeta.from_shape_and_strides(shape, core.contiguous_strides(shape), off, DType.F64)
    e = _err(K.addmm_tensor_contiguous_f64, np.array(c["input"], float), np.array(c["mat1"], float), np.array(c["mat2"], float),
             m(c["input_shape"]), m(c["mat1_shape"], c["mat1_offset"]), m(c["mat2_shape"]), c["beta"], c["alpha"])
    assert e.kind == "InsufficientStorage" and e.side == "mat1" and e.needed == 7 and e.available == 6
    c = by["argmax_dim_invalid_dim"]
    e = _err(K.argmax_dim_tensor_contiguous_f64, np.array(c["input"], float), m(c["shape"]), c["dim"])
    assert e.kind == "InvalidDimension" and e.dim == 2 and e.ndim == 2
    c = by["argmax_over_empty_dim"]
    e = _err(K.argmax_dim_tensor_contiguous_f64, np.zeros(0), m(c["shape"]), c["dim"])
    assert e.kind == "EmptyReductionDim" and e.dim == 1
    for name in ("index_select_invalid_dim", "index_select_out_of_bounds", "index_select_nan_index", "index_select_huge_index",
                 "index_select_negative_index"):
        c = by[name]
        e = _err(K.index_select_tensor_contiguous_f64, np.array(c["input"], float), m(c["shape"]), c["dim"],
                 np.array([float(v) for v in c["index"]]))
        assert e.kind == "InvalidDimension", name
    # fractional index beyond f64::EPSILON is rejected, an exact integer value is accepted by validation
    e = _err(K.index_select_tensor_contiguous_f64, np.arange(6.0), m([3, 2]), 0, np.array([1.5]))
    assert e.kind == "InvalidDimension" and e.dim == 3 and e.ndim == 3


def test_add_and_addmm_shape_rules():
    a = np.zeros(6, np.float32)
    f32 = lambda s: TensorMeta.from_shape(s, DType.F32)
    e = _err(K.add_tensor_contiguous_f32, a, a, f32([2, 3]), f32([3, 2]))  # no broadcast
    assert e.kind == "ShapeMismatch"
    e = _err(K.addmm_tensor_contiguous_f32, a, a, a, f32([3]), f32([2, 3]), f32([3, 2]), 1.0, 1.0)
    assert e.kind == "ShapeMismatch" and e.lhs == [3] and e.rhs == [2, 2]
    e = _err(K.bmm_tensor_contiguous_f32, a, a, f32([1, 2, 3]), f32([2, 3, 1]))
    assert e.kind == "ShapeMismatch"
    e = _err(K.softmax_dim_tensor_contiguous_f32, a, f32([2, 3]), 2)
    assert e.kind == "InvalidDimension" and e.dim == 2 and e.ndim == 2


def test_fused_entry_points_check_slice_lengths_before_any_device_call():
    """The reference's fused kernels panic on short slices (plain indexing); the C ABI reports InvalidArgument instead, and does
    so before it needs a device, for the forward, backward, masked and loss forms alike."""
    bh, sq, sk, dk, dv = 2, 5, 6, 4, 3
    q, k, v = np.zeros(bh * sq * dk), np.zeros(bh * sk * dk), np.zeros(bh * sk * dv)
    do, mask = np.zeros(bh * sq * dv), np.zeros(bh * sq * sk)
    for call in (
        lambda: K.sdpa_forward_f64(q[:-1], k, v, bh, sq, sk, dk, dv, 0.5, True),
        lambda: K.sdpa_backward_f64(q, k, v, do[:-1], bh, sq, sk, dk, dv, 0.5, False),
        lambda: K.sdpa_backward_masked_f64(q, k, v, do, bh, sq, sk, dk, dv, 0.5, mask[:-1], sq * sk),  # mask shorter than num_bh planes
        lambda: K.sdpa_backward_masked_f64(q, k, v, do, bh, sq, sk, dk, dv, 0.5, mask, 7),             # stride smaller than a plane
        lambda: K.sdpa_forward_masked_f64(q, k, v, bh, sq, sk, dk, dv, 0.5, mask[:-1], sq * sk),
        lambda: K.sdpa_backward_f32_unit_dout(q.astype(np.float32), k.astype(np.float32)[:-1], v.astype(np.float32), bh, sq, sk, dk, dv, 0.5, True),
        lambda: K.cross_entropy_forward_f64(np.zeros(11), np.zeros(3, np.int64), 3, 4),
        lambda: K.layer_norm_backward_f64(np.zeros(11), np.zeros(12), None, 3, 4, 1e-5),
    ):
        with pytest.raises((core.KernelError, core.HipError)) as ei:
            call()
        assert ei.value.kind != "Unavailable", "the length check must come before the device check"


def test_transposes_check_lengths_before_any_device_call():
    x = np.zeros(12, np.float32)
    assert K.transpose_2d_f32(np.zeros(0, np.float32), 0, 5).size == 0          # empty result: no device needed
    assert K.transpose_batched_materialize_f64(np.zeros(0), 3, 0, 4).size == 0
    with pytest.raises(core.HipError) as ei:
        K.transpose_2d_f32(x[:-1], 3, 4)                                          # source shorter than rows * cols
    assert ei.value.kind == "InvalidArgument"
    with pytest.raises(core.HipError) as ei:
        K.transpose_batched_materialize_f32(x, 2 ** 40, 2 ** 40, 2 ** 40)         # extent product overflows
    assert ei.value.kind == "InvalidArgument"
    out = np.zeros(11, np.float32)
    rc = _lib.load().fth_transpose_2d_into_f32(x.ctypes.data, x.size, out.ctypes.data, out.size, 3, 4)
    assert _lib.load().fth_status_name(rc) == b"OutputTooSmall"


def test_graph_replay_is_refused_under_a_profiler_tool(env={"LD_PRELOAD": "/nonexistent/librocprofiler-sdk-tool.so"}):
    """fth_encoder_forward_graph returns Unavailable, with its own message, whenever a rocprofiler tool library is named in
    the process environment; the check precedes any device call, so a child process without a GPU can show it (the dynamic
    loader only warns about a preload it cannot find; naming a missing file in ROCP_TOOL_LIBRARIES, the other trigger, makes
    the HIP runtime itself abort at load, so that one is not exercised here). The handle and the two buffers are never
    dereferenced before the check."""
    import subprocess
    import sys

    code = (
        "import ctypes as C, sys\n"
        "sys.path.insert(0, %r)\n"
        "from frankentorch_amd import _lib\n"
        "L = _lib.load()\n"
        "rc = L.fth_encoder_forward_graph(C.c_void_p(4096), C.c_void_p(8192), 1, 8, C.c_void_p(12288), None)\n"
        "print(rc, _lib.last_error().message.decode())\n" % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    )
    child_env = dict(os.environ)
    child_env.update(env)
    out = subprocess.run([sys.executable, "-c", code], env=child_env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    rc, message = out.stdout.strip().split(" ", 1)
    assert int(rc) == 100 and "rocprofiler tool" in message and "fth_encoder_forward_dev" in message
    # without the variable the same call gets as far as the device check (or, on a GPU box, would run): not this message
    clean = {k: v for k, v in os.environ.items() if k not in ("ROCP_TOOL_LIBRARIES",) and not (k == "LD_PRELOAD" and "rocprofiler" in v)}
    if not os.path.exists("/dev/kfd"):
        out = subprocess.run([sys.executable, "-c", code], env=clean, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
        assert out.returncode == 0 and out.stdout.startswith("100 ") and "rocprofiler tool" not in out.stdout


def test_empty_results_need_no_device():
    f32 = lambda s: TensorMeta.from_shape(s, DType.F32)
    z = np.zeros(0, np.float32)
    assert K.matmul_tensor_contiguous_f32(z, z, f32([0, 3]), f32([3, 0])).size == 0
    assert K.softmax_dim_tensor_contiguous_f32(z, f32([0, 4]), 1).size == 0
    assert K.gelu_tensor_contiguous_f32(z, f32([0])).size == 0
    assert K.index_select_tensor_contiguous_f32(np.zeros(6, np.float32), f32([2, 3]), 0, np.zeros(0)).size == 0
    assert K.linear_tensor_f32(z, z, None, 0, 4, 0).size == 0


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present: the unavailable stub is not in effect")
def test_no_gpu_means_unavailable_not_a_cpu_fallback():
    """Mirrors the non-macOS stub test of ft-kernel-metal (crates/ft-kernel-metal/src/lib.rs:343-352)."""
    from frankentorch_amd import device, fused

    assert device.is_available() is False
    a = np.ones(6, np.float32)
    f32 = lambda s: TensorMeta.from_shape(s, DType.F32)
    with pytest.raises(core.HipError) as ei:
        K.matmul_tensor_contiguous_f32(a, a, f32([2, 3]), f32([3, 2]))
    assert ei.value.kind == "Unavailable"
    with pytest.raises(core.HipError) as ei:
        fused.HipTensor.upload(a, 2, 3)
    assert ei.value.kind == "Unavailable"
    with pytest.raises(core.HipError):
        K.layer_norm_forward_f32(a, None, None, 2, 3, 1e-5)


def test_synthetic_inputs_are_reproducible_and_shaped():
    a = synth.normal(1, "x", (64, 33))
    b = synth.normal(1, "x", (64, 33))
    assert a.dtype == np.float32 and np.array_equal(a, b)
    assert not np.array_equal(a, synth.normal(2, "x", (64, 33)))
    assert not np.array_equal(a, synth.normal(1, "y", (64, 33)))
    # any slice of a stream can be generated independently of the rest
    assert np.array_equal(synth.normal(1, "x", (64 * 33,))[:100], a.ravel()[:100])
    big = synth.normal(3, "n", (400000,))
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1.0) < 0.01
    u = synth.uniform(2, "u", (100000,), -1.0, 1.0)
    assert u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 0.02
    ids = synth.token_ids(4, "ids", (8, 128), 50257)
    assert ids.dtype == np.float64 and ids.min() >= 0 and ids.max() < 50257 and np.all(ids == np.floor(ids))
