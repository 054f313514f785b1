"""Integer-exact kernels: argmax, index_select / embedding gather, head split-merge permute.
Bit-exact against the CPU checker."""
import numpy as np
import pytest

from frankentorch_amd import synth
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_argmax_semantics_ties_nan_and_all_neg_inf(hip, oracle, dtype):
    x = synth.normal(7, "am", (41, 50257)).astype(dtype)
    x[3, 100] = np.nan
    x[3, 40000] = np.nan          # the FIRST NaN wins
    x[4, :] = -np.inf             # nothing is > -inf: index 0
    x[5, 9000] = x[5, 7] = x[5].max() + 1  # tie: the first index wins
    x[6, 50256] = 1e9             # last element
    x[7, 0] = 1e9
    x[8, 12] = np.inf
    x[9, 5] = np.nan
    x[9, 4] = np.inf              # a NaN beats +inf even when it comes later
    dx = DeviceBuffer.from_host(x)
    dy = DeviceBuffer((41,), dtype)
    hip.argmax(dx, 41, 50257, 1, dy)
    got = dy.to_host()
    assert np.array_equal(got, oracle.argmax(x, 1))
    assert got[3] == 100 and got[4] == 0 and got[5] == 7 and got[6] == 50256 and got[7] == 0 and got[8] == 12 and got[9] == 5


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("cols", [1, 2, 3, 4, 5, 7, 9, 33, 1027, 4099])
def test_argmax_last_dim_short_and_unaligned_rows_with_ties(hip, oracle, cols, dtype):
    """Rows whose scalar head, vector body and scalar tail are empty or a few elements long, every starting alignment
    (odd row length, plus a base one element into the buffer), heavy ties and NaNs: first maximum / first NaN must win."""
    rows = 37
    x = np.round(synth.normal(9, "am3", (rows, cols)) * 1.5).astype(dtype)
    if cols > 4:
        x[5, cols // 2] = np.nan
        x[6, cols - 1] = np.nan
        x[7, 0] = np.nan
    pad = np.concatenate([np.zeros(1, dtype), x.ravel()])
    dpad = DeviceBuffer.from_host(pad)
    dy = DeviceBuffer((rows,), dtype)
    hip.argmax(dpad.view(1), rows, cols, 1, dy)
    assert np.array_equal(dy.to_host(), oracle.argmax(x, 1))
    hip.argmax(DeviceBuffer.from_host(x), rows, cols, 1, dy)
    assert np.array_equal(dy.to_host(), oracle.argmax(x, 1))


@pytest.mark.parametrize("shape,dim", [((5, 17, 9), 1), ((64, 3), 0), ((2, 300, 4), 1), ((1, 7), 1), ((3, 1, 5), 1)])
def test_argmax_any_dim(hip, oracle, shape, dim):
    x = np.round(synth.normal(8, "am2", shape) * 2)  # many ties
    x.ravel()[::13] = np.nan
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    inner = int(np.prod(shape[dim + 1:], dtype=np.int64))
    dx = DeviceBuffer.from_host(x)
    dy = DeviceBuffer((outer * inner,))
    hip.argmax(dx, outer, shape[dim], inner, dy)
    assert np.array_equal(dy.to_host().reshape(oracle.argmax(x, dim).shape), oracle.argmax(x, dim))


def test_argmax_empty_reduce_dim_is_an_error(hip):
    from frankentorch_amd.core import KernelError

    dx = DeviceBuffer((4,))
    with pytest.raises(KernelError) as ei:
        hip.argmax(dx, 3, 0, 1, dx)
    assert ei.value.kind == "EmptyReductionDim"
    hip.argmax(dx, 0, 0, 1, dx)  # empty output: nothing to do, as in the reference


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_index_select_rows_and_general(hip, oracle, dtype):
    table = synth.normal(9, "tab", (1000, 768)).astype(dtype)
    ids = synth.token_ids(9, "ids", (513,), 1000)
    dt, di = DeviceBuffer.from_host(table), DeviceBuffer.from_host(ids)
    do = DeviceBuffer((513, 768), dtype)
    bad = DeviceBuffer((1,), np.int64)
    hip.index_select(dt, 1, 1000, 768, di, 513, do, bad)
    ref, rbad = oracle.index_select(table, 0, ids)
    assert rbad == -1 and bad.to_host()[0] == -1
    assert np.array_equal(do.to_host(), ref)
    # middle dim, odd inner (scalar copy path)
    t3 = synth.normal(9, "t3", (4, 11, 7)).astype(dtype)
    idx = np.array([10.0, 0.0, 3.0, 3.0])
    d3, di3 = DeviceBuffer.from_host(t3), DeviceBuffer.from_host(idx)
    o3 = DeviceBuffer((4, 4, 7), dtype)
    hip.index_select(d3, 4, 11, 7, di3, 4, o3, bad)
    assert np.array_equal(o3.to_host(), oracle.index_select(t3, 1, idx)[0])


def test_index_select_reports_first_invalid_index(hip, oracle):
    table = synth.normal(9, "tab", (10, 8))
    dt = DeviceBuffer.from_host(table)
    bad = DeviceBuffer((1,), np.int64)
    for idx, want in (([1.0, 2.5, 3.0], 1), ([1.0, 2.0, 10.0], 2), ([-1.0, 99.0], 0), ([np.nan], 0), ([1e300], 0), ([np.inf], 0)):
        sentinel = np.full((len(idx), 8), 123.0, np.float32)
        do = DeviceBuffer.from_host(sentinel)
        di = DeviceBuffer.from_host(np.array(idx))
        hip.index_select(dt, 1, 10, 8, di, len(idx), do, bad)
        assert bad.to_host()[0] == want == oracle.index_select(table, 0, idx)[1]
        out = do.to_host()
        assert np.all(out[want] == 123.0)  # rows with an invalid index are left untouched


def test_embedding_add_and_permute(hip, oracle):
    vocab, maxpos, d, batch, seq = 777, 40, 768, 3, 32
    wte = synth.normal(4, "wte", (vocab, d), 0.0, 0.02)
    wpe = synth.normal(4, "wpe", (maxpos, d), 0.0, 0.02)
    ids = synth.token_ids(4, "ids", (batch * seq,), vocab)
    dwte, dwpe, dids = DeviceBuffer.from_host(wte), DeviceBuffer.from_host(wpe), DeviceBuffer.from_host(ids)
    out = DeviceBuffer((batch * seq, d))
    bad = DeviceBuffer((1,), np.int64)
    hip.embedding_add(dwte, vocab, dwpe, maxpos, dids, batch * seq, seq, d, out, bad)
    ref = wte[ids.astype(int)] + np.tile(wpe[:seq], (batch, 1))
    assert np.array_equal(out.to_host(), ref) and bad.to_host()[0] == -1
    for shape in ((2, 5, 3, 8), (3, 128, 12, 64), (1, 7, 2, 3)):
        x = synth.normal(6, "perm", shape)
        dx = DeviceBuffer.from_host(x)
        dy = DeviceBuffer((shape[0], shape[2], shape[1], shape[3]))
        hip.permute_0213(dx, dy, *shape)
        assert np.array_equal(dy.to_host(), oracle.permute_0213(x))
        back = DeviceBuffer(shape)
        hip.permute_0213(dy, back, shape[0], shape[2], shape[1], shape[3])
        assert np.array_equal(back.to_host(), x)  # split then merge is the identity


def _linear_argmax_case(rows, n, k, seed):
    """Integer-valued operands (every logit is exact and ties abound) with rows that drive the special values through the
    product: NaN from inf * 0, +-inf from inf * w and from overflow, an all -inf row, an all-zero row."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-1, 2, size=(rows, k)).astype(np.float32)
    w = rng.integers(-1, 2, size=(n, k)).astype(np.float32)
    w[:, 1] = rng.choice(np.array([-2, -1, 1, 2], np.float32), size=n)  # never zero
    w[:, 3] = rng.integers(1, 4, size=n).astype(np.float32)              # positive
    w[:, 4] = 1.0
    late = n - n // 5
    w[late, 4] = 0.0                                                     # the one zero of column 4
    special = {}
    r = rows // 7
    x[r] = 0; x[r, 0] = np.inf; special["nan_from_inf_times_zero"] = r          # NaN wherever w[:, 0] == 0: the first wins
    r = rows // 5
    x[r] = 0; special["all_zero_row"] = r                                       # all ties: index 0
    r = rows // 3
    x[r] = 0; x[r, 1] = np.inf; special["inf_no_nan"] = r                       # +-inf only: the first +inf
    r = rows // 2
    x[r] = 0; x[r, 2] = 3e38; w[:, 2] = rng.integers(-3, 4, size=n)             # overflow to +-inf through finite operands
    special["overflow"] = r
    r = rows - 2
    x[r] = 0; x[r, 3] = -np.inf; special["all_neg_inf"] = r                     # every logit -inf: index 0
    r = rows - 1
    x[r] = 0; x[r, 4] = np.inf; special["one_late_nan"] = r                     # +inf everywhere, one NaN late in the row
    return x, w, special, late


@pytest.mark.parametrize("rows,n,k", [(1500, 12901, 64), (1100, 16384, 32), (2100, 8200, 96), (40, 40000, 64)])
def test_linear_argmax_fused_equals_gemm_then_argmax(hip, oracle, rows, n, k):
    """The product that records group maxima in its epilogue and the argmax that reads them give, bit for bit, the indices
    of the plain argmax kernel on the same logits, and the logits of the plain product; tiles the product splits over
    several workgroups, ragged last tiles and rows of NaN / +-inf go through the element-by-element branch."""
    x, w, special, late = _linear_argmax_case(rows, n, k, seed=rows + n)
    dx, dw = DeviceBuffer.from_host(x), DeviceBuffer.from_host(w)
    nws = hip.linear_argmax_workspace_floats(rows, n)
    assert nws == rows * 2 * ((n + 127) // 128)
    sentinel = np.full(nws, 12345.0, np.float32)
    ws = DeviceBuffer.from_host(sentinel)
    logits, idx = DeviceBuffer((rows, n), np.float32), DeviceBuffer((rows,), np.float32)
    hip.linear_argmax(dx, dw, rows, n, k, logits, idx, workspace=ws)
    got_logits, got = logits.to_host(), idx.to_host()
    gm = ws.to_host().reshape(-1, rows)
    assert not np.any(gm == 12345.0), "the product kernel with the row-maximum epilogue did not run"
    # the recorded maxima are right wherever they claim to be known
    known = ~np.isnan(gm)
    assert known.mean() > 0.3 and (~known).sum() > 0
    pad = np.full((rows, gm.shape[0] * 64), -np.inf, np.float32)
    pad[:, :n] = np.where(np.isnan(got_logits), np.inf, got_logits)
    true_gm = pad.reshape(rows, -1, 64).max(axis=2).T
    assert np.array_equal(gm[known], true_gm[known])
    # logits: the plain product's, bit for bit (both are exact here where finite)
    plain = DeviceBuffer((rows, n), np.float32)
    hip.gemm(hip.gemm_desc(rows, n, k, trans_b=True), dx, dw, plain)
    assert np.array_equal(got_logits, plain.to_host(), equal_nan=True)
    ordinary = np.ones(rows, bool)
    ordinary[list(special.values())] = False
    assert np.array_equal(got_logits[ordinary], (x[ordinary].astype(np.float64) @ w.T.astype(np.float64)).astype(np.float32))
    # indices: the plain kernel's on the same logits, and the checker's
    ref_idx = DeviceBuffer((rows,), np.float32)
    hip.argmax(logits, rows, n, 1, ref_idx)
    assert np.array_equal(got, ref_idx.to_host())
    assert np.array_equal(got, oracle.argmax(got_logits, 1))
    assert got[special["all_zero_row"]] == 0 and got[special["all_neg_inf"]] == 0 and got[special["one_late_nan"]] == late
    assert got[special["nan_from_inf_times_zero"]] == np.flatnonzero(w[:, 0] == 0)[0]
    assert got[special["inf_no_nan"]] == np.flatnonzero(w[:, 1] > 0)[0]
    assert got[special["overflow"]] == np.flatnonzero(w[:, 2] >= 2)[0]  # 3e38 * 1 is finite, * 2 is +inf
    # without a workspace: the two separate kernels, same answers
    idx2, logits2 = DeviceBuffer((rows,), np.float32), DeviceBuffer((rows, n), np.float32)
    hip.linear_argmax(dx, dw, rows, n, k, logits2, idx2)
    assert np.array_equal(idx2.to_host(), got) and np.array_equal(logits2.to_host(), got_logits, equal_nan=True)


def test_linear_argmax_random_logits_and_small_shapes(hip, oracle):
    """Normal operands at the vocabulary width (no exact ties), and shapes the large-tile kernel does not take, which fall
    back to the two kernels with the workspace left untouched."""
    rows, n, k = 1024, 50257, 128
    x = synth.normal(11, "la.x", (rows, k)).astype(np.float32)
    w = synth.normal(12, "la.w", (n, k)).astype(np.float32)
    dx, dw = DeviceBuffer.from_host(x), DeviceBuffer.from_host(w)
    ws = DeviceBuffer((hip.linear_argmax_workspace_floats(rows, n),), np.float32)
    logits, idx, ref_idx = DeviceBuffer((rows, n), np.float32), DeviceBuffer((rows,), np.float32), DeviceBuffer((rows,), np.float32)
    hip.linear_argmax(dx, dw, rows, n, k, logits, idx, workspace=ws)
    hip.argmax(logits, rows, n, 1, ref_idx)
    got_logits = logits.to_host()
    assert np.array_equal(idx.to_host(), ref_idx.to_host())
    assert np.array_equal(idx.to_host(), oracle.argmax(got_logits, 1))
    ref = x.astype(np.float64) @ w.T.astype(np.float64)
    assert np.abs(got_logits - ref).max() / np.abs(ref).max() <= 2e-5
    for rows, n, k in [(3, 700, 64), (300, 1000, 40), (1, 20000, 96)]:
        x = synth.normal(13, "la.x2", (rows, k)).astype(np.float32)
        w = synth.normal(14, "la.w2", (n, k)).astype(np.float32)
        nws = hip.linear_argmax_workspace_floats(rows, n)
        ws = DeviceBuffer.from_host(np.full(nws, 7.0, np.float32))
        logits, idx = DeviceBuffer((rows, n), np.float32), DeviceBuffer((rows,), np.float32)
        hip.linear_argmax(DeviceBuffer.from_host(x), DeviceBuffer.from_host(w), rows, n, k, logits, idx, workspace=ws)
        assert np.all(ws.to_host() == 7.0)
        got_logits = logits.to_host()
        assert np.array_equal(idx.to_host(), oracle.argmax(got_logits, 1))
        ref = x.astype(np.float64) @ w.T.astype(np.float64)
        assert np.abs(got_logits - ref).max() / np.abs(ref).max() <= 2e-5
