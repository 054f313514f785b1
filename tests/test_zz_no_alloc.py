"""The allocation-free LayerNorm backward against the workspace form of the same entry point: bit for bit, on two calls in a
row (the second on a smaller input, so the shared scratch still holds the first call's partial sums), and its size limit."""
import numpy as np
import pytest

from frankentorch_amd import synth
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def _both(hip, rows, cols, seed):
    x = synth.normal(seed, "x", (rows, cols))
    dy = synth.normal(seed, "dy", (rows, cols))
    w = synth.uniform(seed, "w", (cols,), 0.5, 1.5)
    ddy, dx_, dw_ = (DeviceBuffer.from_host(a) for a in (dy, x, w))
    ref = [DeviceBuffer((rows, cols)), DeviceBuffer((cols,)), DeviceBuffer((cols,))]
    got = [DeviceBuffer((rows, cols)), DeviceBuffer((cols,)), DeviceBuffer((cols,))]
    hip.layer_norm_backward(ddy, dx_, dw_, ref[0], ref[1], ref[2], rows, cols, 1e-5)
    hip.layer_norm_backward_noalloc(ddy, dx_, dw_, got[0], got[1], got[2], rows, cols, 1e-5)
    hip.synchronize()
    return [b.to_host() for b in ref], [b.to_host() for b in got]


def test_no_alloc_layer_norm_backward_equals_the_workspace_form(hip, oracle):
    # first call: the benchmark shape (register-resident kernel, 8.1 MiB of the 24 MiB scratch)
    for rows, cols, seed in ((8192, 4096, 31), (300, 1024, 32), (37, 1026, 33), (5, 7, 34)):
        ref, got = _both(hip, rows, cols, seed)
        for name, a, b in zip(("dx", "dweight", "dbias"), ref, got):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (rows, cols, name)
    # and against the CPU checker on the last small shapes, at the row-op tolerance
    rows, cols = 300, 1024
    x, dy = synth.normal(32, "x", (rows, cols)), synth.normal(32, "dy", (rows, cols))
    w = synth.uniform(32, "w", (cols,), 0.5, 1.5)
    dx_r, dw_r, db_r = oracle.layer_norm_backward(dy, x, w, np.float32(1e-5))
    ref, got = _both(hip, rows, cols, 32)
    from conftest import NORM_COLSUM_TOL_FACTOR, TOL_ROW_F32, rel_err

    assert rel_err(got[0], dx_r) <= TOL_ROW_F32
    assert rel_err(got[1], dw_r) <= TOL_ROW_F32 * NORM_COLSUM_TOL_FACTOR and rel_err(got[2], db_r) <= TOL_ROW_F32 * NORM_COLSUM_TOL_FACTOR


def test_no_alloc_call_allocates_nothing(hip):
    """The property the entry point exists for: after a first call (which looks the scratch array's address up), a call
    changes neither the library pool's block and byte counts nor the device's free memory, for the register-resident shape
    and for a streaming one (columns not a multiple of the vector width)."""
    import ctypes as C

    from frankentorch_amd import _lib

    def pool():
        used, cached = C.c_uint64(), C.c_uint64()
        assert _lib.load().fth_pool_stats(C.byref(used), C.byref(cached)) == 0
        return used.value, cached.value

    for rows, cols in ((4096, 4096), (700, 1026)):
        x = synth.normal(35, "x", (rows, cols))
        dy = synth.normal(35, "dy", (rows, cols))
        w = synth.uniform(35, "w", (cols,), 0.5, 1.5)
        ddy, dx_, dw_ = (DeviceBuffer.from_host(a) for a in (dy, x, w))
        out = [DeviceBuffer((rows, cols)), DeviceBuffer((cols,)), DeviceBuffer((cols,))]
        hip.layer_norm_backward_noalloc(ddy, dx_, dw_, out[0], out[1], out[2], rows, cols, 1e-5)  # warm-up
        hip.synchronize()
        before = (pool(), hip.memory_info()[0])
        for _ in range(3):
            hip.layer_norm_backward_noalloc(ddy, dx_, dw_, out[0], out[1], out[2], rows, cols, 1e-5)
        hip.synchronize()
        assert (pool(), hip.memory_info()[0]) == before, (rows, cols)


def test_no_alloc_rejects_shapes_beyond_the_scratch(hip):
    from frankentorch_amd.core import HipError

    cap = hip.layer_norm_backward_noalloc_max_bytes()
    assert cap == 24 << 20
    rows, cols = 32768, 8192  # 512 workgroups (64 rows each) x 8192 columns x 2 arrays x 4 bytes = 32 MiB of partial sums
    assert hip.norm_backward_workspace_bytes(rows, cols, np.float32) > cap
    one = DeviceBuffer((1,))
    with pytest.raises(HipError) as exc:
        hip.layer_norm_backward_noalloc(one, one, one, one, one, one, rows, cols, 1e-5)
    assert exc.value.kind == "BufferTooLarge" and "scratch" in exc.value.message
