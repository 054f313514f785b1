"""Pins the CPU checker's backward functions without running the reference: central differences of
the already pinned forward functions in f64 (a dropped term, a wrong sign or a transposed operand
fails them), the identities the reference's own tests assert, and its test inputs
(crates/ft-kernel-cpu/src/lib.rs:43862-43911, 64200-64360)."""
import numpy as np
import pytest


def _num_grad(f, x, dy, h=1e-6):
    """d/dx sum(dy * f(x)) by central differences, f64."""
    g = np.zeros_like(x)
    flat, gf = x.reshape(-1), g.reshape(-1)
    for i in range(flat.size):
        old = flat[i]
        flat[i] = old + h
        up = float(np.sum(dy * f(x)))
        flat[i] = old - h
        dn = float(np.sum(dy * f(x)))
        flat[i] = old
        gf[i] = (up - dn) / (2 * h)
    return g


def test_layer_norm_backward_is_the_gradient_of_the_forward(oracle):
    rng = np.random.default_rng(5)
    batch, n, eps = 4, 9, 1e-5
    x, dy = rng.standard_normal((batch, n)), rng.standard_normal((batch, n))
    w, b = rng.uniform(0.5, 1.5, n), rng.standard_normal(n)
    dx, dw, db = oracle.layer_norm_backward(dy, x, w, eps)
    assert np.allclose(dx, _num_grad(lambda t: oracle.layer_norm(t, w, b, eps), x.copy(), dy), atol=1e-7)
    assert np.allclose(dw, _num_grad(lambda t: oracle.layer_norm(x, t, b, eps), w.copy(), dy), atol=1e-7)
    assert np.allclose(db, _num_grad(lambda t: oracle.layer_norm(x, w, t, eps), b.copy(), dy), atol=1e-7)
    assert np.array_equal(db, np.add.reduce(dy, axis=0))  # serial sum over the rows in row order
    assert np.allclose(dx.sum(1), 0, atol=1e-12)  # a shift of the whole row leaves the output unchanged


def test_layer_norm_backward_reference_test_inputs(oracle):
    """Inputs of layer_norm_f32_unit_dy_matches_general_reference_bits (KC:64300-64360): with dy = 1 the
    shortcut the reference takes must equal the general formula, i.e. dbias = batch and
    dweight = sum of xhat over the rows."""
    for batch, n in [(5, 7), (3, 16)]:
        i = np.arange(batch * n)
        x = (((i % 23).astype(np.float32) - 11.0) * np.float32(0.03125) + i.astype(np.float32) * np.float32(0.00091)).reshape(batch, n)
        w = (0.75 + (np.arange(n) % 5) * 0.046875).astype(np.float32)
        dy = np.ones_like(x)
        dx, dw, db = oracle.layer_norm_backward(dy, x, w, np.float32(1e-5))
        assert np.all(db == np.float32(batch))
        x64 = x.astype(np.float64)
        xhat = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
        assert np.allclose(dw, xhat.sum(0), atol=2e-5)
        dx64, _, _ = oracle.layer_norm_backward(dy.astype(np.float64), x64, w.astype(np.float64), 1e-5)
        assert np.allclose(dx, dx64, atol=2e-5)


def test_rms_norm_backward_is_the_gradient_of_the_forward(oracle):
    rng = np.random.default_rng(6)
    batch, n, eps = 3, 8, 1e-6
    x, dy, w = rng.standard_normal((batch, n)), rng.standard_normal((batch, n)), rng.uniform(0.5, 1.5, n)
    dx, dw = oracle.rms_norm_backward(dy, x, w, eps)
    assert np.allclose(dx, _num_grad(lambda t: oracle.rms_norm(t, w, eps), x.copy(), dy), atol=1e-7)
    assert np.allclose(dw, _num_grad(lambda t: oracle.rms_norm(x, t, eps), w.copy(), dy), atol=1e-7)
    dx1, dw1 = oracle.rms_norm_backward(dy, x, None, eps)
    assert dw1 is None
    assert np.allclose(dx1, _num_grad(lambda t: oracle.rms_norm(t, None, eps), x.copy(), dy), atol=1e-7)


def test_linear_backward_reference_test_inputs_and_gradient(oracle):
    """Inputs of linear_backward_dgemm_tb_dweight_matches_materialized_transpose_bit_exact (KC:43862-43911):
    dweight must equal dy^T . x computed through an explicit transpose, dbias the column sums of dy."""
    batch, in_f, out_f = 96, 40, 72
    dy = ((np.arange(batch * out_f) % 101) * 0.01 - 0.5).reshape(batch, out_f)
    x = ((np.arange(batch * in_f) % 89) * 0.02 - 0.7).reshape(batch, in_f)
    w = ((np.arange(out_f * in_f) % 53) * 0.03 - 0.4).reshape(out_f, in_f)
    dx, dw, db = oracle.linear_backward(dy, x, w, True)
    assert np.allclose(dw, oracle.gemm(np.ascontiguousarray(dy.T), x), rtol=0, atol=1e-12)
    assert np.allclose(dw, dy.T @ x, atol=1e-11) and np.allclose(dx, dy @ w, atol=1e-11)
    ref_db = np.zeros(out_f)
    for b in range(batch):
        ref_db += dy[b]
    assert np.array_equal(db, ref_db)
    # gradient of the forward on a small case
    rng = np.random.default_rng(7)
    xs, ws, bs, dys = rng.standard_normal((3, 4)), rng.standard_normal((5, 4)), rng.standard_normal(5), rng.standard_normal((3, 5))
    dxs, dws, dbs = oracle.linear_backward(dys, xs, ws, True)
    assert np.allclose(dxs, _num_grad(lambda t: oracle.linear(t, ws, bs), xs.copy(), dys), atol=1e-8)
    assert np.allclose(dws, _num_grad(lambda t: oracle.linear(xs, t, bs), ws.copy(), dys), atol=1e-8)
    assert np.allclose(dbs, _num_grad(lambda t: oracle.linear(xs, ws, t), bs.copy(), dys), atol=1e-8)
    assert oracle.linear_backward(dys, xs, ws, False)[2] is None


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_backward_is_the_gradient_of_the_forward(oracle, causal):
    rng = np.random.default_rng(8)
    bh, sq, sk, dk, dv = 2, 5, 6, 4, 3
    q, k, v = rng.standard_normal((bh, sq, dk)), rng.standard_normal((bh, sk, dk)), rng.standard_normal((bh, sk, dv))
    dout = rng.standard_normal((bh, sq, dv))
    scale = 0.37
    dq, dk_, dv_ = oracle.sdpa_backward(q, k, v, dout, scale, causal)
    assert np.allclose(dq, _num_grad(lambda t: oracle.sdpa_forward(t, k, v, scale, causal), q.copy(), dout), atol=1e-7)
    assert np.allclose(dk_, _num_grad(lambda t: oracle.sdpa_forward(q, t, v, scale, causal), k.copy(), dout), atol=1e-7)
    assert np.allclose(dv_, _num_grad(lambda t: oracle.sdpa_forward(q, k, t, scale, causal), v.copy(), dout), atol=1e-7)
    if causal:  # a key no query can see gets no gradient
        assert np.all(dk_[:, sq:, :] == 0) and np.all(dv_[:, sq:, :] == 0)
    # f32 twin agrees with f64 to f32 rounding
    f = np.float32
    dq32, dk32, dv32 = oracle.sdpa_backward(q.astype(f), k.astype(f), v.astype(f), dout.astype(f), f(scale), causal)
    assert np.allclose(dq32, dq, atol=2e-5) and np.allclose(dk32, dk_, atol=2e-5) and np.allclose(dv32, dv_, atol=2e-5)


def test_sdpa_backward_unit_dout_matches_dense_ones_on_the_reference_inputs(oracle):
    """The reference's own test (crates/ft-kernel-cpu/src/lib.rs:45119-45155): its inputs, its bound 2e-4 + 2e-4 |want|."""
    num_bh, seq_q, seq_k, d_k, d_v = 2, 5, 6, 4, 3
    f = np.float32
    q = (((np.arange(num_bh * seq_q * d_k) % 11).astype(f) - f(5.0)) * f(0.07)).reshape(num_bh, seq_q, d_k)
    k = (((np.arange(num_bh * seq_k * d_k) % 13).astype(f) - f(6.0)) * f(0.05)).reshape(num_bh, seq_k, d_k)
    v = (((np.arange(num_bh * seq_k * d_v) % 7).astype(f) - f(3.0)) * f(0.09)).reshape(num_bh, seq_k, d_v)
    scale = f(1.0) / np.sqrt(f(d_k))
    for causal in (False, True):
        want = oracle.sdpa_backward(q, k, v, np.ones((num_bh, seq_q, d_v), f), scale, causal)
        got = oracle.sdpa_backward_unit_dout(q, k, v, scale, causal)
        for a, b in zip(got, want):
            assert np.all(np.abs(a - b) <= 2.0e-4 + 2.0e-4 * np.abs(b))
            assert np.allclose(a, b, atol=2e-6)  # in fact far closer
        # every value lane of a key gets the same gradient
        assert np.all(got[2] == got[2][:, :, :1])
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    for a, b in zip(oracle.sdpa_backward_unit_dout(q64, k64, v64, 0.5, True), oracle.sdpa_backward(q64, k64, v64, np.ones((num_bh, seq_q, d_v)), 0.5, True)):
        assert np.allclose(a, b, atol=1e-14)


@pytest.mark.parametrize("shared", [True, False])
def test_sdpa_backward_masked_is_the_gradient_of_the_masked_forward(oracle, shared):
    """sdpa_backward_masked_f64 (crates/ft-kernel-cpu/src/lib.rs:5423-5530) has no test of its own in the reference: it is pinned by
    central differences of the pinned masked forward, by its reduction to the unmasked and causal backward for a zero and a
    -inf-triangle mask, and by an einsum restatement of the textbook formulas."""
    rng = np.random.default_rng(18)
    bh, sq, sk, dk, dv = 3, 5, 6, 4, 3
    q, k, v = rng.standard_normal((bh, sq, dk)), rng.standard_normal((bh, sk, dk)), rng.standard_normal((bh, sk, dv))
    dout = rng.standard_normal((bh, sq, dv))
    scale = 0.41
    mask = rng.standard_normal((sq, sk) if shared else (bh, sq, sk))
    mask[..., 1, 2] = -np.inf  # a hidden key in a row that keeps others
    dq, dk_, dv_ = oracle.sdpa_backward_masked(q, k, v, dout, scale, mask)
    assert np.allclose(dq, _num_grad(lambda t: oracle.sdpa_forward_masked(t, k, v, scale, mask), q.copy(), dout), atol=1e-7)
    assert np.allclose(dk_, _num_grad(lambda t: oracle.sdpa_forward_masked(q, t, v, scale, mask), k.copy(), dout), atol=1e-7)
    assert np.allclose(dv_, _num_grad(lambda t: oracle.sdpa_forward_masked(q, k, t, scale, mask), v.copy(), dout), atol=1e-7)
    # einsum restatement
    m3 = np.broadcast_to(mask, (bh, sq, sk))
    sc = np.einsum("bqd,bkd->bqk", q, k) * scale + m3
    p = np.exp(sc - sc.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    dp = np.einsum("bqd,bkd->bqk", dout, v)
    du = p * (dp - (p * dp).sum(-1, keepdims=True))
    assert np.allclose(dq, scale * np.einsum("bqk,bkd->bqd", du, k), atol=1e-12)
    assert np.allclose(dk_, scale * np.einsum("bqk,bqd->bkd", du, q), atol=1e-12)
    assert np.allclose(dv_, np.einsum("bqk,bqd->bkd", p, dout), atol=1e-12)
    # zero mask = unmasked; -inf above the diagonal = causal
    for got, ref in zip(oracle.sdpa_backward_masked(q, k, v, dout, scale, np.zeros((sq, sk))), oracle.sdpa_backward(q, k, v, dout, scale, False)):
        assert np.array_equal(got, ref)
    tri = np.where(np.arange(sk)[None, :] <= np.arange(sq)[:, None], 0.0, -np.inf)
    for got, ref in zip(oracle.sdpa_backward_masked(q, k, v, dout, scale, tri), oracle.sdpa_backward(q, k, v, dout, scale, True)):
        assert np.allclose(got, ref, atol=1e-14)
    f = np.float32
    g32 = oracle.sdpa_backward_masked(q.astype(f), k.astype(f), v.astype(f), dout.astype(f), f(scale), mask.astype(f))
    for a, b in zip(g32, (dq, dk_, dv_)):
        assert np.allclose(a, b, atol=2e-5)


def test_log_softmax_reference_fixtures_and_identity(oracle, vectors):
    cases = [c for c in vectors["conformance"] if c["op"] == "log_softmax"]
    assert len(cases) == 2
    for c in cases:
        x = np.array(c["input"], np.float64).reshape(c["shape"])
        got = oracle.log_softmax(x, c["dim"])
        assert np.allclose(got.ravel(), c["expected_output"], rtol=0, atol=c["tolerance"])
        assert np.allclose(oracle.log_softmax(x.astype(np.float32), c["dim"]).ravel(), c["expected_output"], atol=1e-6)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 7, 5)) * 4
    for dim in (0, 1, 2):
        assert np.allclose(oracle.log_softmax(x, dim), np.log(oracle.softmax(x, dim)), atol=1e-12)
        assert np.allclose(np.exp(oracle.log_softmax(x, dim)).sum(dim), 1.0, atol=1e-12)


def test_cross_entropy_is_minus_log_softmax_at_the_target_and_its_gradient(oracle):
    rng = np.random.default_rng(10)
    batch, classes = 6, 11
    logits = rng.standard_normal((batch, classes)) * 3
    target = rng.integers(0, classes, batch)
    loss = oracle.cross_entropy_forward(logits, target)
    assert np.allclose(loss, -oracle.log_softmax(logits, 1)[np.arange(batch), target], atol=1e-12)
    dloss = rng.standard_normal(batch)
    g = oracle.cross_entropy_backward(logits, target, dloss)
    num = _num_grad(lambda t: oracle.cross_entropy_forward(t, target), logits.copy(), dloss)
    assert np.allclose(g, num, atol=1e-7)
    assert np.allclose(g.sum(1), 0, atol=1e-12)  # softmax sums to one, the one-hot too
    l32 = oracle.cross_entropy_forward(logits.astype(np.float32), target)
    assert np.allclose(l32, loss, atol=2e-6)
    with pytest.raises(IndexError):
        oracle.cross_entropy_forward(logits, np.full(batch, classes))


def _reference_gqa_inputs():
    """The inputs of sdpa_masked_gqa_f64_matches_expand_then_masked_bit_exact (crates/ft-kernel-cpu/src/lib.rs:45160-45183)."""
    batch, h_q, h_kv, seq_q, seq_k, d_k, d_v = 2, 8, 2, 40, 40, 16, 16
    i = lambda n: np.arange(n, dtype=np.float64)
    q = (np.sin(i(batch * h_q * seq_q * d_k) * 0.017 + 0.3) * 0.2).reshape(batch, h_q, seq_q, d_k)
    k = (np.sin(i(batch * h_kv * seq_k * d_k) * 0.013 + 1.1) * 0.2).reshape(batch, h_kv, seq_k, d_k)
    v = (np.cos(i(batch * h_kv * seq_k * d_v) * 0.011 + 2.2) * 0.2).reshape(batch, h_kv, seq_k, d_v)
    mask2d = np.where(np.arange(seq_q * seq_k) % 3 == 0, -0.5, 0.0).reshape(seq_q, seq_k)
    mask3d = np.where(np.arange(batch * h_q * seq_q * seq_k) % 5 == 0, -0.7, 0.0).reshape(batch * h_q, seq_q, seq_k)
    return q, k, v, mask2d, mask3d, 1.0 / np.sqrt(d_k)


def test_masked_gqa_sdpa_restatement_is_pinned(oracle):
    q, k, v, mask2d, mask3d, scale = _reference_gqa_inputs()
    batch, h_q, seq_q, d_k = q.shape
    h_kv, seq_k = k.shape[1], k.shape[2]
    group = h_q // h_kv
    k_rep, v_rep = np.repeat(k, group, axis=1), np.repeat(v, group, axis=1)  # head hq reads kv head hq // group
    for mask in (mask2d, mask3d):
        grouped = oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask)
        # the reference's own assertion: bit-exact with expand-then-masked
        expanded = oracle.sdpa_forward_masked(q.reshape(batch * h_q, seq_q, d_k), k_rep.reshape(batch * h_q, seq_k, d_k),
                                              v_rep.reshape(batch * h_q, seq_k, -1), scale, mask)
        assert np.array_equal(grouped.reshape(expanded.shape).view(np.uint64), expanded.view(np.uint64))
        # independent of the restatement: softmax(scale * q k^T + mask) v in numpy
        s = np.einsum("bhqd,bhkd->bhqk", q, k_rep) * scale + mask.reshape((-1, h_q, seq_q, seq_k) if mask.ndim == 3 else (1, 1, seq_q, seq_k))
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        assert np.allclose(grouped, np.einsum("bhqk,bhkd->bhqd", p, v_rep), rtol=0, atol=1e-14)
    # a zero mask is the unmasked kernel, a -inf upper triangle the causal one (both pinned by the reference's fixtures)
    qf, kf, vf = (t.reshape(batch * h_q, seq_q, -1) for t in (q, k_rep, v_rep))
    zero = np.zeros((seq_q, seq_k))
    assert np.allclose(oracle.sdpa_forward_masked(qf, kf, vf, scale, zero), oracle.sdpa_forward(qf, kf, vf, scale, False), atol=1e-15)
    tri = np.where(np.arange(seq_k)[None, :] > np.arange(seq_q)[:, None], -np.inf, 0.0)
    assert np.allclose(oracle.sdpa_forward_masked(qf, kf, vf, scale, tri), oracle.sdpa_forward(qf, kf, vf, scale, True), atol=1e-15)
    # a fully masked row is NaN, as exp(-inf - -inf) makes it in the reference
    tri[3, :] = -np.inf
    out = oracle.sdpa_forward_masked(qf, kf, vf, scale, tri)
    assert np.all(np.isnan(out[:, 3, :])) and not np.any(np.isnan(np.delete(out, 3, axis=1)))
    # f32 instantiation agrees to f32 rounding
    f = np.float32
    o32 = oracle.sdpa_forward_masked_gqa(q.astype(f), k.astype(f), v.astype(f), f(scale), mask2d.astype(f))
    assert np.allclose(o32, oracle.sdpa_forward_masked_gqa(q, k, v, scale, mask2d), atol=2e-6)


def test_gelu_tanh_restatement_is_pinned(oracle, vectors):
    c = {v["name"]: v for v in vectors["in_source"]}["gelu_tanh_module_matches_torch"]
    x = np.array(c["input"], np.float64)
    assert np.max(np.abs(oracle.gelu_tanh(x) - np.array(c["expected_output"]))) <= c["abs_tol"]
    assert np.max(np.abs(oracle.gelu_tanh(x.astype(np.float32)) - np.array(c["expected_output"]))) <= 2e-7
    # a library routine for the rest of the range: torch's CPU kernel of the same approximation
    import torch

    xs = np.linspace(-12.0, 12.0, 4801)
    want = torch.nn.functional.gelu(torch.from_numpy(xs), approximate="tanh").numpy()
    assert np.max(np.abs(oracle.gelu_tanh(xs) - want)) <= 1e-14
    want32 = torch.nn.functional.gelu(torch.from_numpy(xs.astype(np.float32)), approximate="tanh").numpy()
    assert np.max(np.abs(oracle.gelu_tanh(xs.astype(np.float32)) - want32)) <= 1e-6
    # equals x * sigmoid(2u), the form the GEMM epilogue computes
    u = 0.7978845608028654 * (xs + 0.044715 * xs ** 3)
    assert np.max(np.abs(oracle.gelu_tanh(xs) - xs / (1.0 + np.exp(-2.0 * u)))) <= 1e-14


def _lcg_matrices(m, k, n):
    """The generator of linear_int8_dynamic_matches_f32_reference (crates/ft-kernel-cpu/src/lib.rs:43650-43662)."""
    state = [0x123456789ABCDEF0 ^ (m * 131 + k * 17 + n)]

    def lcg():
        state[0] = (state[0] * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        return np.float32(np.float32(state[0] >> 33) / np.float32(1 << 31)) - np.float32(1.0)

    x = np.array([lcg() * np.float32(3.0) for _ in range(m * k)], np.float32).reshape(m, k)
    w = np.array([lcg() * np.float32(0.5) for _ in range(n * k)], np.float32).reshape(n, k)
    bias = np.array([lcg() for _ in range(n)], np.float32)
    return x, w, bias


def test_int8_dynamic_linear_restatement_is_pinned(oracle):
    # int8_quantizers_round_signed_ties_to_even (:43721-43740): exact expected bytes and scale
    ties = np.array([[-127.0, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 127.0]], np.float32)
    q, scales = oracle.quantize_rows_i8(ties)
    assert q.tolist() == [[-127, -2, -2, 0, 0, 2, 2, 127]] and scales.tolist() == [1.0]
    # an all-zero row keeps scale 1; NaN quantises to 0 and does not move the scale; the scale is amax / 127
    q, scales = oracle.quantize_rows_i8(np.array([[0.0, 0.0, -0.0], [np.nan, 2.0, -4.0], [1e-3, 5e-4, 0.0]], np.float32))
    assert scales[0] == 1.0 and q[0].tolist() == [0, 0, 0]
    assert scales[1] == np.float32(4.0) / np.float32(127.0) and q[1].tolist() == [0, 64, -127]  # 63.5 rounds to the even 64
    assert scales[2] == np.float32(1e-3) / np.float32(127.0) and q[2].tolist() == [127, 64, 0]
    # linear_int8_dynamic_matches_f32_reference (:43645-43708): the reference's shapes, inputs and bounds
    for m, k, n in ((8, 384, 384), (4, 384, 1536), (7, 200, 53)):
        x, w, bias = _lcg_matrices(m, k, n)
        w_i8, w_scales = oracle.quantize_rows_i8(w)
        y = oracle.linear_int8_dynamic(x, w_i8, w_scales, bias).astype(np.float64)
        ref = (x.astype(np.float64) @ w.astype(np.float64).T + bias).astype(np.float32).astype(np.float64)
        cos = (ref * y).sum() / np.sqrt((ref * ref).sum() * (y * y).sum())
        assert cos > 0.999 and np.abs(ref - y).max() / np.abs(ref).max() < 0.05
        # independent of the restatement: the same integers through numpy
        xq, a_scales = oracle.quantize_rows_i8(x)
        acc = xq.astype(np.int64) @ w_i8.astype(np.int64).T
        want = (acc.astype(np.float32) * a_scales[:, None]) * w_scales[None, :] + bias[None, :]
        assert np.array_equal(oracle.linear_int8_dynamic(x, w_i8, w_scales, bias).view(np.uint32), want.astype(np.float32).view(np.uint32))
    # linear_int8_dynamic_is_deterministic (:43710-43719)
    m, k, n = 6, 384, 384
    x = (((np.arange(m * k) % 17).astype(np.float32) - 8.0) * np.float32(0.1)).reshape(m, k)
    w = (((np.arange(n * k) % 13).astype(np.float32) - 6.0) * np.float32(0.05)).reshape(n, k)
    w_i8, w_scales = oracle.quantize_rows_i8(w)
    assert np.array_equal(oracle.linear_int8_dynamic(x, w_i8, w_scales), oracle.linear_int8_dynamic(x, w_i8, w_scales))
