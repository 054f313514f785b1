"""fp32 / fp64 MFMA GEMM against the wide-accumulation CPU checker.
fp32: max|d| / max|ref| <= 2e-5; fp64: <= 1e-12."""
import numpy as np
import pytest

from conftest import TOL_F64, TOL_GEMM_F32, rel_err
from frankentorch_amd import synth
from frankentorch_amd.device import EPI_BIAS, EPI_GELU, EPI_RESIDUAL, DeviceBuffer

pytestmark = pytest.mark.gpu


def _run(hip, a, b, trans_b, bias=None, residual=None, epilogue=0, alpha=1.0):
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    da, db = DeviceBuffer.from_host(a), DeviceBuffer.from_host(b)
    dc = DeviceBuffer((m, n), a.dtype)
    dbias = None if bias is None else DeviceBuffer.from_host(bias)
    dres = None if residual is None else DeviceBuffer.from_host(residual)
    hip.gemm(hip.gemm_desc(m, n, k, trans_b=trans_b, epilogue=epilogue), da, db, dc, dbias, dres, alpha)
    return dc.to_host()


# full tiles, ragged edges in every dimension, k not a multiple of the vector width, tiny, skinny
SHAPES = [(128, 128, 64), (256, 384, 128), (200, 300, 100), (77, 50, 33), (1, 1, 1), (5, 1000, 7), (1000, 5, 7), (130, 130, 513),
          (64, 64, 4096), (512, 768, 256), (3, 129, 2)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gemm_matches_oracle(hip, oracle, m, n, k, trans_b, dtype):
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    a = synth.uniform(2, "a", (m, k), -1, 1, dtype=dtype)
    b = synth.uniform(2, "b", (n, k) if trans_b else (k, n), -1, 1, dtype=dtype)
    got = _run(hip, a, b, trans_b)
    assert rel_err(got, oracle.gemm(a, b, trans_b)) <= tol


# K a whole number of 128-byte K-tiles with 16-byte aligned rows: the global->LDS direct kernels.
# Ragged m / n (clamped edge rows and columns), one-row and one-vector extents, tile counts that
# leave every workgroup a mix of whole and split tiles (several tiles per workgroup, K split 2-3 ways), and the GPT-2
# O-projection shape at a short K, which the [n, k] fp32 form runs on 128 x 96 tiles (512 whole tiles, none split).
DIRECT_SHAPES = [(200, 300, 96), (77, 52, 64), (130, 132, 512), (1, 4, 32), (1000, 8, 32), (129, 257 * 4, 160),
                 (2048, 2304, 768), (4096, 3072, 256), (2050, 1540, 288), (8192, 768, 64)]


@pytest.mark.parametrize("m,n,k", DIRECT_SHAPES)
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_direct_to_lds_kernels(hip, oracle, m, n, k, trans_b, dtype):
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    a = synth.uniform(2, "da", (m, k), -1, 1, dtype=dtype)
    b = synth.uniform(2, "db", (n, k) if trans_b else (k, n), -1, 1, dtype=dtype)
    bias = synth.normal(2, "dbias", (n,), dtype=dtype)
    res = synth.normal(2, "dres", (m, n), dtype=dtype)
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 37)), [m - 1]]))
    ref = oracle.gemm(a[rows], b, trans_b)
    plain = _run(hip, a, b, trans_b)
    assert rel_err(plain[rows], ref) <= tol
    again = _run(hip, a, b, trans_b)
    assert np.array_equal(plain.view(np.uint8), again.view(np.uint8))          # fixed summation order
    got = _run(hip, a, b, trans_b, bias, res, EPI_BIAS | EPI_RESIDUAL)
    assert np.array_equal(got, (plain + bias) + res)                             # same roundings as the separate ops
    got = _run(hip, a, b, trans_b, bias, None, EPI_BIAS | EPI_GELU)
    assert rel_err(got[rows], oracle.gelu(ref + bias)) <= tol


# A stored [k, m] (gemm::sgemm_tb / dgemm_tb): direct-to-LDS shapes, a ragged shape that goes through
# the transposed copy, scaled (alpha) and batched.
@pytest.mark.parametrize("m,n,k", [(256, 384, 128), (200, 300, 96), (72, 40, 96), (77, 50, 33), (1024, 2304, 512), (4, 8, 16)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gemm_with_a_stored_k_by_m(hip, oracle, m, n, k, dtype):
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    at = synth.uniform(2, "ta", (k, m), -1, 1, dtype=dtype)
    b = synth.uniform(2, "tb", (k, n), -1, 1, dtype=dtype)
    da, db = DeviceBuffer.from_host(at), DeviceBuffer.from_host(b)
    dc = DeviceBuffer((m, n), dtype)
    hip.gemm(hip.gemm_desc(m, n, k, trans_a=True), da, db, dc)
    ref = oracle.gemm(np.ascontiguousarray(at.T), b)
    got = dc.to_host()
    assert rel_err(got, ref) <= tol
    hip.gemm(hip.gemm_desc(m, n, k, trans_a=True), da, db, dc, alpha=0.25)
    assert np.array_equal(dc.to_host(), dtype(0.25) * got)
    # batched with a shared right operand
    at3 = synth.uniform(2, "ta3", (3, k, m), -1, 1, dtype=dtype)
    da3, dc3 = DeviceBuffer.from_host(at3), DeviceBuffer((3, m, n), dtype)
    hip.gemm(hip.gemm_desc(m, n, k, trans_a=True, batch=3, stride_b=0), da3, db, dc3)
    assert rel_err(dc3.to_host()[2], oracle.gemm(np.ascontiguousarray(at3[2].T), b)) <= tol


def test_gemm_workspace_growth_is_bounded(hip, oracle):
    """Ragged [k, m] operands go through a transposed copy in a workspace that only grows; an outgrown block is retired
    (queued kernels or a captured graph may still address it), and because blocks grow geometrically what has been retired
    stays below what is live. fth_gemm_workspace_info reports both."""
    live0, ret0 = hip.gemm_workspace_info()
    for m, k in ((33, 77), (130, 301), (515, 1201), (1030, 4803), (2055, 9607)):
        n = 24
        at = synth.uniform(9, "wa", (k, m), -1, 1)
        b = synth.uniform(9, "wb", (k, n), -1, 1)
        da, db, dc = DeviceBuffer.from_host(at), DeviceBuffer.from_host(b), DeviceBuffer((m, n))
        hip.gemm(hip.gemm_desc(m, n, k, trans_a=True), da, db, dc)
        assert rel_err(dc.to_host(), oracle.gemm(np.ascontiguousarray(at.T), b)) <= TOL_GEMM_F32
        live, ret = hip.gemm_workspace_info()
        assert live >= m * k * 4
        assert ret - ret0 < live, (m, k, live, ret)
    assert live >= live0 and ret >= ret0
    again = hip.gemm_workspace_info()
    hip.gemm(hip.gemm_desc(m, n, k, trans_a=True), da, db, dc)  # a request that fits allocates and retires nothing
    assert hip.gemm_workspace_info() == again


def test_direct_to_lds_kernels_with_row_pitch_and_batches(hip, oracle):
    """Sub-blocks of larger buffers (pitch > row, 16-byte aligned offsets) and a batched problem whose
    tiles straddle workgroup ranges, through the direct kernels."""
    big_a = synth.uniform(2, "qa", (300, 264), -1, 1)
    big_b = synth.uniform(2, "qb", (280, 200), -1, 1)
    dA, dB = DeviceBuffer.from_host(big_a), DeviceBuffer.from_host(big_b)
    dC = DeviceBuffer.from_host(np.zeros((300, 212), np.float32))
    # A sub-block [290, 256] at element offset 4 (pitch 264); B^T sub-block [270, 256]... stored [n, k] with pitch 200 would
    # not hold k = 256, so B is taken as [k, n] = [256, 196] at offset 4 with pitch 200.
    hip.gemm(hip.gemm_desc(290, 196, 256, lda=264, ldb=200, ldc=212), dA.view(4), dB.view(4), dC.view(8))
    a_sub = big_a.ravel()[4:][: 290 * 264].reshape(290, 264)[:, :256]
    b_sub = big_b.ravel()[4:][: 256 * 200].reshape(256, 200)[:, :196]
    got = dC.to_host().ravel()[8:][: 290 * 212].reshape(290, 212)[:, :196]
    assert rel_err(got, oracle.gemm(np.ascontiguousarray(a_sub), np.ascontiguousarray(b_sub))) <= TOL_GEMM_F32
    untouched = dC.to_host().ravel()[8:][: 290 * 212].reshape(290, 212)[:, 196:]
    assert np.all(untouched == 0.0)
    a = synth.uniform(2, "qba", (24, 384, 96), -1, 1)
    w = synth.uniform(2, "qbw", (24, 320, 96), -1, 1)
    da, dw = DeviceBuffer.from_host(a), DeviceBuffer.from_host(w)
    dc = DeviceBuffer((24, 384, 320))
    hip.gemm(hip.gemm_desc(384, 320, 96, batch=24, trans_b=True), da, dw, dc)
    assert rel_err(dc.to_host(), oracle.bmm(a, np.ascontiguousarray(w.transpose(0, 2, 1)))) <= TOL_GEMM_F32


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_epilogues_keep_their_own_roundings(hip, oracle, dtype):
    """bias, GELU and residual applied in the epilogue equal the separate ops applied to the
    GEMM's own rounded output, bit for bit."""
    tol = TOL_GEMM_F32 if dtype == np.float32 else TOL_F64
    m, n, k = 150, 200, 96
    a = synth.uniform(2, "a", (m, k), -1, 1, dtype=dtype)
    w = synth.uniform(2, "w", (n, k), -1, 1, dtype=dtype)
    bias = synth.normal(2, "bias", (n,), dtype=dtype)
    res = synth.normal(2, "res", (m, n), dtype=dtype)
    plain = _run(hip, a, w, True)
    got = _run(hip, a, w, True, bias, None, EPI_BIAS)
    assert np.array_equal(got, plain + bias)
    assert rel_err(got, oracle.linear(a, w, bias)) <= tol
    got = _run(hip, a, w, True, bias, res, EPI_BIAS | EPI_RESIDUAL)
    assert np.array_equal(got, (plain + bias) + res)
    got = _run(hip, a, w, True, bias, None, EPI_BIAS | EPI_GELU)
    assert rel_err(got, oracle.gelu(oracle.linear(a, w, bias))) <= tol
    got = _run(hip, a, w, True, None, None, 0, alpha=0.5)
    assert np.array_equal(got, dtype(0.5) * plain)


def test_degenerate_extents(hip):
    a = np.ones((4, 0), np.float32)
    b = np.ones((0, 6), np.float32)
    bias = np.arange(6, dtype=np.float32)
    da, db, dbias = DeviceBuffer((1,)), DeviceBuffer((1,)), DeviceBuffer.from_host(bias)
    dc = DeviceBuffer.from_host(np.full((4, 6), 7.0, np.float32))
    hip.gemm(hip.gemm_desc(4, 6, 0), da, db, dc)           # k == 0: zeros (overwrite, beta = 0)
    assert np.all(dc.to_host() == 0.0)
    hip.gemm(hip.gemm_desc(4, 6, 0, epilogue=EPI_BIAS), da, db, dc, dbias)
    assert np.array_equal(dc.to_host(), np.tile(bias, (4, 1)))
    dc = DeviceBuffer.from_host(np.full((4, 6), 7.0, np.float32))
    hip.gemm(hip.gemm_desc(0, 6, 3), da, db, dc)           # m == 0: returns at once, C untouched
    hip.gemm(hip.gemm_desc(4, 0, 3), da, db, dc)
    assert np.all(dc.to_host() == 7.0)


def test_batched_and_strided(hip, oracle):
    """Config 3 batched case [32,512,128] @ [32,128,512], plus a shared (stride 0) right operand."""
    a = synth.uniform(2, "ba", (32, 512, 128), -1, 1)
    b = synth.uniform(2, "bb", (32, 128, 512), -1, 1)
    da, db = DeviceBuffer.from_host(a), DeviceBuffer.from_host(b)
    dc = DeviceBuffer((32, 512, 512))
    hip.gemm(hip.gemm_desc(512, 512, 128, batch=32), da, db, dc)
    got = dc.to_host()
    assert rel_err(got, oracle.bmm(a, b)) <= TOL_GEMM_F32
    hip.gemm(hip.gemm_desc(512, 512, 128, batch=32, stride_b=0), da, db, dc)
    assert rel_err(dc.to_host()[5], oracle.gemm(a[5], b[0])) <= TOL_GEMM_F32
    # row pitches larger than the rows: operate on a sub-block of larger buffers
    big_a = synth.uniform(2, "pa", (70, 200), -1, 1)
    big_b = synth.uniform(2, "pb", (90, 150), -1, 1)
    dA, dB = DeviceBuffer.from_host(big_a), DeviceBuffer.from_host(big_b)
    dC = DeviceBuffer.from_host(np.zeros((70, 130), np.float32))
    hip.gemm(hip.gemm_desc(60, 100, 80, lda=200, ldb=150, ldc=130), dA.view(3), dB.view(7), dC.view(5))
    ref = oracle.gemm(np.ascontiguousarray(big_a.ravel()[3:].reshape(-1)[: 60 * 200].reshape(60, 200)[:, :80]),
                      np.ascontiguousarray(big_b.ravel()[7:][: 80 * 150].reshape(80, 150)[:, :100]))
    got = dC.to_host().ravel()[5:][: 60 * 130].reshape(60, 130)[:, :100]
    assert rel_err(got, ref) <= TOL_GEMM_F32


def test_reference_f64_checksums_on_the_gpu(hip, vectors):
    """The reference's stored sums of its own dgemm outputs (sin/cos inputs), 12 decimals."""
    for s in vectors["golden_text"]["gemm_f64_checksums"]["sums"]:
        m, k, n = s["m"], s["k"], s["n"]
        a = np.sin(np.arange(m * k, dtype=np.float64) * 0.001).reshape(m, k)
        b = np.cos(np.arange(n * k, dtype=np.float64) * 0.0017).reshape((n, k) if s["bt"] else (k, n))
        got = _run(hip, a, b, bool(s["bt"]))
        total = float(np.sum(got.ravel().tolist()))
        assert abs(total - s["sum"]) <= 5e-11 * max(1.0, abs(s["sum"])), (s, total)


def test_known_answers_and_precision_contract(hip, vectors):
    by = {c["name"]: c for c in vectors["in_source"]}
    c = by["matmul_tensor_contiguous_returns_expected_values"]
    for dt in (np.float32, np.float64):
        a = np.array(c["lhs"], dt).reshape(c["lhs_shape"])
        b = np.array(c["rhs"], dt).reshape(c["rhs_shape"])
        assert _run(hip, a, b, False).ravel().tolist() == [float(v) for v in c["expected_output"]]
    c = by["matmul_unit_vector_dot_k10001"]
    r = 1.0 / np.sqrt(c["k"])
    got = _run(hip, np.full((1, c["k"]), r), np.full((c["k"], 1), r), False)
    # The reference pins its pairwise dgemm to 1e-14 here; the MFMA kernel sums k sequentially
    # (K/4 dependent steps) and is held to the fp64 tolerance of this backend, 1e-12.
    assert abs(got[0, 0] - 1.0) < TOL_F64


def test_config3_shapes_whole_outputs_and_determinism(hip, oracle):
    """4096^3, [4096,4096]@[4096,11008]+bias in fp32 and 4096^3 in fp64. The WHOLE fp32 square output, in both layouts of
    B, is compared with the wide-accumulation truth (a few seconds of CPU work); 512 rows of the rectangle and 256 of the
    fp64 square, spread over every tile row; the whole output is compared bitwise between two runs; linearity
    (A.(B1+B2) vs A.B1 + A.B2) is checked without the oracle."""
    a = synth.uniform(2, "A", (4096, 4096), -1, 1)
    b = synth.uniform(2, "B", (4096, 4096), -1, 1)
    da, db = DeviceBuffer.from_host(a), DeviceBuffer.from_host(b)
    dc, dc2 = DeviceBuffer((4096, 4096)), DeviceBuffer((4096, 4096))
    rows = np.arange(3, 4096, 8)  # 512 rows, four in every 128-row tile
    for trans_b in (False, True):
        d = hip.gemm_desc(4096, 4096, 4096, trans_b=trans_b)
        hip.gemm(d, da, db, dc)
        hip.gemm(d, da, db, dc2)
        c = dc.to_host()
        assert np.array_equal(c.view(np.uint32), dc2.to_host().view(np.uint32))
        ref = oracle.gemm(a, b, trans_b)
        assert rel_err(c, ref) <= TOL_GEMM_F32
        # per 128 x 128 output tile as well: an error confined to one tile must not hide behind the global maximum
        tile_err = np.abs(c.astype(np.float64) - ref).reshape(32, 128, 32, 128).max(axis=(1, 3))
        tile_ref = np.abs(ref).reshape(32, 128, 32, 128).max(axis=(1, 3))
        assert np.all(tile_err <= TOL_GEMM_F32 * tile_ref)
        del ref
    # rectangular with bias
    b2 = synth.uniform(2, "B2", (4096, 11008), -1, 1)
    bias = synth.uniform(2, "bias2", (11008,), -1, 1)
    db2, dbias = DeviceBuffer.from_host(b2), DeviceBuffer.from_host(bias)
    dr = DeviceBuffer((4096, 11008))
    hip.gemm(hip.gemm_desc(4096, 11008, 4096, epilogue=EPI_BIAS), da, db2, dr, dbias)
    c = dr.to_host()
    assert rel_err(c[rows], oracle.gemm(a[rows], b2) + bias) <= TOL_GEMM_F32
    del dr, db2, c
    # fp64 square
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    da64, db64 = DeviceBuffer.from_host(a64), DeviceBuffer.from_host(b64)
    dc64 = DeviceBuffer((4096, 4096), np.float64)
    hip.gemm(hip.gemm_desc(4096, 4096, 4096), da64, db64, dc64)
    c64 = dc64.to_host()
    r64 = rows[::2]
    assert rel_err(c64[r64], oracle.gemm(a64[r64], b64)) <= TOL_F64
    # linearity in B, fp64, no oracle: A.(B + B^T-ish perturbation) == A.B + A.P within rounding
    p = np.roll(b64, 17, axis=1)
    dp, dsum = DeviceBuffer.from_host(p), DeviceBuffer.from_host(b64 + p)
    dcp, dcs = DeviceBuffer((4096, 4096), np.float64), DeviceBuffer((4096, 4096), np.float64)
    hip.gemm(hip.gemm_desc(4096, 4096, 4096), da64, dp, dcp)
    hip.gemm(hip.gemm_desc(4096, 4096, 4096), da64, dsum, dcs)
    assert rel_err(dcs.to_host(), c64 + dcp.to_host()) <= 1e-12
