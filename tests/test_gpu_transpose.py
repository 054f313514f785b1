"""2-D and batched transposes and the streaming copy: pure data movement, so every case is bit-exact against numpy
(transpose_2d_into_f32 / transpose_batched_materialize_f32, crates/ft-kernel-cpu/src/lib.rs:42415-42439, 42526-42556).
NaN payloads and signed zeros must come through untouched, hence the comparisons on the raw bytes."""
import numpy as np
import pytest

from frankentorch_amd import kernel_hip as K, synth
from frankentorch_amd.core import HipError
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def _planes(seed, batch, rows, cols, dtype):
    x = synth.normal(seed, "t%dx%dx%d" % (batch, rows, cols), (batch, rows, cols)).astype(dtype)
    flat = x.reshape(-1)
    if flat.size > 6:
        flat[1], flat[3], flat[5] = np.nan, -0.0, np.inf
    return x


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rows,cols", [(1, 1), (1, 7), (7, 1), (3, 5), (32, 32), (33, 31), (64, 64), (64, 68), (100, 260),
                                       (128, 4096), (768, 2304), (1026, 514), (4096, 11008)])
def test_transpose_2d_is_exact(hip, dtype, rows, cols):
    x = _planes(11, 1, rows, cols, dtype)[0]
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer((cols, rows), dtype)
    hip.transpose_2d(dx, dy, rows, cols)
    assert np.array_equal(_bits(dy.to_host()), _bits(x.T))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("batch,rows,cols", [(1, 8, 8), (3, 5, 9), (32, 512, 128), (96, 1024, 64), (7, 130, 66), (2, 64, 4)])
def test_transpose_batched_is_exact(hip, dtype, batch, rows, cols):
    x = _planes(12, batch, rows, cols, dtype)
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer((batch, cols, rows), dtype)
    hip.transpose_batched(dx, dy, batch, rows, cols)
    assert np.array_equal(_bits(dy.to_host()), _bits(x.transpose(0, 2, 1)))


def test_transpose_of_an_unaligned_view_takes_the_element_path(hip):
    rows, cols = 64, 128
    x = _planes(13, 1, rows, cols, np.float32)[0]
    pad = np.concatenate([np.zeros(1, np.float32), x.ravel()])
    dpad, dy = DeviceBuffer.from_host(pad), DeviceBuffer((cols, rows))
    hip.transpose_2d(dpad.view(1), dy, rows, cols)
    assert np.array_equal(_bits(dy.to_host()), _bits(x.T))


def test_transpose_twice_is_the_identity_at_the_rectangle_of_config_3(hip):
    rows, cols = 4096, 11008
    x = synth.uniform(2, "B2", (rows, cols), -1, 1)
    dx, dt, dback = DeviceBuffer.from_host(x), DeviceBuffer((cols, rows)), DeviceBuffer((rows, cols))
    hip.transpose_2d(dx, dt, rows, cols)
    hip.transpose_2d(dt, dback, cols, rows)
    assert np.array_equal(_bits(dback.to_host()), _bits(x))


def test_empty_extents_and_aliasing(hip):
    one = DeviceBuffer((4,))
    hip.transpose_2d(one, one, 0, 5)      # nothing to do: returns before looking at the pointers
    hip.transpose_batched(one, one, 0, 2, 2)
    with pytest.raises(HipError) as exc:
        hip.transpose_2d(one, one, 2, 2)
    assert exc.value.kind == "InvalidArgument"


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_host_slice_transposes(hip, dtype):
    sfx = "f32" if dtype == np.float32 else "f64"
    x = _planes(14, 5, 37, 20, dtype)
    got = getattr(K, "transpose_batched_materialize_" + sfx)(x, 5, 37, 20)
    assert np.array_equal(_bits(got.reshape(5, 20, 37)), _bits(x.transpose(0, 2, 1)))
    got = getattr(K, "transpose_2d_" + sfx)(x[0], 37, 20)
    assert np.array_equal(_bits(got.reshape(20, 37)), _bits(x[0].T))
    big = _planes(15, 1, 1024, 768, dtype)[0]   # above the staged-copy threshold of the host-slice tier
    got = getattr(K, "transpose_2d_" + sfx)(big, 1024, 768)
    assert np.array_equal(_bits(got.reshape(768, 1024)), _bits(big.T))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [0, 1, 3, 4, 1023, 4096, 1 << 20, (1 << 20) + 3])
def test_streaming_copy_is_exact(hip, dtype, n):
    x = synth.normal(16, "c%d" % n, (max(n, 1),)).astype(dtype)[:n]
    if n > 2:
        x[1], x[2] = np.nan, -0.0
    dx, dy = DeviceBuffer.from_host(x), DeviceBuffer((n,), dtype)
    hip.copy(dx, dy, n)
    assert np.array_equal(_bits(dy.to_host()), _bits(x))
