"""Pins the CPU checker (oracle/ft_oracle.cpp) before anything trusts it.

Each function of the oracle is checked against (a) the reference's own fixtures and in-source
known answers (tests/golden/reference_vectors.json), and (b) what the mathematics fixes
independently of the oracle's formula: library routines (numpy / scipy / torch CPU), closed forms,
invariants and brute force, chosen so a dropped term, a wrong sign / index or a transposed operand
fails at least one check.
"""
import math

import numpy as np
import pytest
import scipy.special

from conftest import rel_err


def _f(vals):
    return np.array([float(v) for v in vals], dtype=np.float64)


# ---------------------------------------------------------------- reference fixtures
def test_conformance_fixtures(oracle, vectors):
    seen = set()
    for c in vectors["conformance"]:
        tol = c.get("tolerance", 0.0)
        exp = _f(c["expected_output"])
        if c["op"] == "gelu":
            got = oracle.gelu(_f(c["input"]))
        elif c["op"] == "softmax":
            got = oracle.softmax(_f(c["input"]).reshape(c["shape"]), c["dim"]).ravel()
        elif c["op"] == "log_softmax":
            got = oracle.log_softmax(_f(c["input"]).reshape(c["shape"]), c["dim"]).ravel()
        elif c["op"] == "add":
            got = oracle.add(_f(c["lhs"]), _f(c["rhs"]))
        elif c["op"] == "matmul":
            ls = c.get("lhs_shape", c.get("shape"))
            rs = c.get("rhs_shape", c.get("shape"))
            got = oracle.gemm(_f(c["lhs"]).reshape(ls), _f(c["rhs"]).reshape(rs)).ravel()
        elif c["op"] == "index_select":
            got, bad = oracle.index_select(_f(c["input"]).reshape(c["input_shape"]), c["dim"], c["index"])
            assert bad == -1
            got = got.ravel()
        else:
            raise AssertionError("unhandled fixture op " + c["op"])
        assert got.shape == exp.shape, c["name"]
        assert np.max(np.abs(got - exp)) <= tol, c["name"]
        seen.add(c["op"])
    assert seen == {"gelu", "softmax", "log_softmax", "add", "matmul", "index_select"}


def test_in_source_known_answers(oracle, vectors):
    by = {c["name"]: c for c in vectors["in_source"]}
    c = by["matmul_tensor_contiguous_returns_expected_values"]
    for dt in (np.float64, np.float32):
        got = oracle.gemm(_f(c["lhs"]).reshape(c["lhs_shape"]).astype(dt), _f(c["rhs"]).reshape(c["rhs_shape"]).astype(dt))
        assert got.ravel().tolist() == [float(v) for v in c["expected_output"]]
    c = by["bmm_respects_storage_offsets_and_batch_order"]
    for dt in (np.float64, np.float32):
        lhs = _f(c["lhs"])[c["lhs_offset"]:][:8].reshape(2, 2, 2).astype(dt)
        rhs = _f(c["rhs"])[c["rhs_offset"]:][:8].reshape(2, 2, 2).astype(dt)
        assert oracle.bmm(lhs, rhs).ravel().tolist() == [float(v) for v in c["expected_output"]]
    assert vectors["golden_text"]["bmm_batch_pass13"]["values"] == [float(v) for v in c["expected_output"]]
    for name in ("addmm_accepts_contiguous_operands", "addmm_alpha_zero_f64", "addmm_alpha_zero_f32"):
        c = by[name]
        dt = np.float32 if c["dtype"] == "f32" else np.float64
        got = oracle.addmm(_f(c["input"]).reshape(c["input_shape"]).astype(dt), _f(c["mat1"]).reshape(c["mat1_shape"]).astype(dt),
                           _f(c["mat2"]).reshape(c["mat2_shape"]).astype(dt), c["beta"], c["alpha"])
        assert got.ravel().tolist() == [float(v) for v in c["expected_output"]], name
    c = by["gelu_returns_expected_values"]
    got = oracle.gelu(_f(c["input"]))
    for g, e, t in zip(got, c["expected_near"], c["abs_tol"]):
        assert abs(g - e) < t
    c = by["inf_in_softmax_produces_nan"]
    assert np.all(np.isnan(oracle.softmax(_f(c["input"]), 0)))
    assert np.all(np.isnan(oracle.softmax(_f(c["input"]).astype(np.float32), 0)))
    c = by["softmax_with_finite_extremes"]
    got = oracle.softmax(_f(c["input"]), 0)
    assert got[0] == 0.0 and got[2] == 1.0 and abs(got.sum() - 1.0) < 1e-10
    for name in ("argmax_dim_reduces_along_dim0", "argmax_dim_reduces_along_dim1", "argmax_dim_1d_reduces_to_scalar"):
        c = by[name]
        got = oracle.argmax(_f(c["input"]).reshape(c["shape"]), c["dim"])
        assert got.ravel().tolist() == [float(v) for v in c["expected_output"]], name
    for name in ("index_select_out_of_bounds", "index_select_nan_index", "index_select_huge_index", "index_select_negative_index"):
        c = by[name]
        _, bad = oracle.index_select(_f(c["input"]).reshape(c["shape"]), c["dim"], _f(c["index"]))
        assert bad == 0, name
    c = by["matmul_unit_vector_dot_k10001"]
    r = 1.0 / math.sqrt(c["k"])
    got = oracle.gemm(np.full((1, c["k"]), r), np.full((c["k"], 1), r))
    assert abs(got[0, 0] - c["expected"]) < c["abs_tol"]


def test_golden_text_files(oracle, vectors):
    g = vectors["golden_text"]
    for row in g["softmax_rows_pass10"]["rows"]:
        got = oracle.softmax(_f(row["input"]).reshape(1, -1), 1).ravel()
        assert np.max(np.abs(got - _f(row["expected_output"]))) < 1e-15
    # uniform rows: every output is exactly 0.5, f64 bits 0x3fe0..., f32 bits 0x3f000000
    b = g["softmax_parallel_bits"]
    rows, cols = b["meta"]["fast_rows"], b["meta"]["fast_cols"]
    y64 = oracle.softmax(np.zeros((rows, cols)), 1).ravel()
    y32 = oracle.softmax(np.zeros((rows, cols), dtype=np.float32), 1).ravel()
    for i, bits in b["bits"]["f64_softmax_fast_bits"].items():
        assert y64[int(i)].view(np.uint64) == int(bits, 16)
    for i, bits in b["bits"]["f32_softmax_fast_bits"].items():
        assert y32[int(i)].view(np.uint32) == int(bits, 16)
    so, sr, si = b["meta"]["strided_outer"], b["meta"]["strided_reduce"], b["meta"]["strided_inner"]
    s32 = oracle.softmax(np.zeros((so, sr, si), dtype=np.float32), 1).ravel()
    for i, bits in b["bits"]["f32_softmax_strided_bits"].items():
        assert s32[int(i)].view(np.uint32) == int(bits, 16)
    assert oracle.add(_f([0.5, 1.5, 2.5, 3.5]), _f([1.0, 2.0, 3.0, 4.0])).tolist() == g["elementwise_simd_pass7"]["add_f64"]
    assert g["gemm_crossover"]["f32_2x3_times_3x2"] == [58.0, 64.0, 139.0, 154.0]


def test_gemm_f64_checksums_from_reference_artifacts(oracle, vectors):
    """Stored sums of matmul / matmul-with-[n,k]-rhs outputs for sin/cos inputs, 12 decimals."""
    for s in vectors["golden_text"]["gemm_f64_checksums"]["sums"]:
        m, k, n = s["m"], s["k"], s["n"]
        a = np.sin(np.arange(m * k, dtype=np.float64) * 0.001).reshape(m, k)
        if s["bt"]:
            b = np.cos(np.arange(n * k, dtype=np.float64) * 0.0017).reshape(n, k)
        else:
            b = np.cos(np.arange(k * n, dtype=np.float64) * 0.0017).reshape(k, n)
        total = float(np.sum(oracle.gemm(a, b, bool(s["bt"])).ravel().tolist()))
        assert "%.12e" % total == "%.12e" % s["sum"], s


# ---------------------------------------------------------------- independent mathematics
def test_softmax_vs_scipy_and_invariants(oracle):
    rng = np.random.default_rng(0)
    for dt, tol in ((np.float64, 1e-15), (np.float32, 3e-7)):
        x = rng.standard_normal((37, 301)).astype(dt)
        for dim in (0, 1):
            y = oracle.softmax(x, dim)
            assert rel_err(y, scipy.special.softmax(x.astype(np.float64), axis=dim)) < tol
            assert np.all((y >= 0) & (y <= 1))
            assert np.allclose(y.sum(axis=dim), 1.0, atol=1e-5)
        # shift invariance (crates/ft-kernel-cpu/src/lib.rs:57181) and order preservation
        assert rel_err(oracle.softmax(x + dt(3.0), 1), oracle.softmax(x, 1)) < 10 * tol
        assert np.array_equal(np.argsort(x[0], kind="stable"), np.argsort(oracle.softmax(x, 1)[0], kind="stable"))
    x3 = rng.standard_normal((3, 5, 7))
    assert rel_err(oracle.softmax(x3, 1), scipy.special.softmax(x3, axis=1)) < 1e-15


def test_layer_norm_rms_norm_closed_forms(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((9, 257))
    w = rng.uniform(0.5, 1.5, 257)
    b = rng.standard_normal(257) * 0.1
    mu = x.mean(-1, keepdims=True)
    var = x.var(-1, keepdims=True)  # population variance
    ref = (x - mu) / np.sqrt(var + 1e-5) * w + b
    assert rel_err(oracle.layer_norm(x, w, b, 1e-5), ref) < 1e-14
    assert rel_err(oracle.layer_norm(x, None, None, 1e-5), (x - mu) / np.sqrt(var + 1e-5)) < 1e-14
    assert rel_err(oracle.layer_norm(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32), 1e-5), ref) < 2e-6
    # a sample-variance (n-1) mistake or a missing eps would exceed these tolerances
    bad = (x - mu) / np.sqrt(x.var(-1, keepdims=True, ddof=1) + 1e-5) * w + b
    assert rel_err(oracle.layer_norm(x, w, b, 1e-5), bad) > 1e-4
    r = rng.standard_normal((9, 257)).astype(np.float32)
    xa = x.astype(np.float32)
    assert np.array_equal(oracle.add_layer_norm(xa, r, w.astype(np.float32), b.astype(np.float32), 1e-5),
                          oracle.layer_norm(xa + r, w.astype(np.float32), b.astype(np.float32), 1e-5))
    rms = np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
    assert rel_err(oracle.rms_norm(x, w, 1e-6), x / rms * w) < 1e-14
    assert rel_err(oracle.rms_norm(x.astype(np.float32), None, 1e-6), x / rms) < 2e-6
    # torch CPU as an independent library routine
    import torch

    t = torch.nn.functional.layer_norm(torch.from_numpy(x), (257,), torch.from_numpy(w), torch.from_numpy(b), 1e-5)
    assert rel_err(oracle.layer_norm(x, w, b, 1e-5), t.numpy()) < 1e-14


def test_gelu_add_bias(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(1001) * 3
    ref = 0.5 * x * (1 + scipy.special.erf(x / np.sqrt(2)))
    assert rel_err(oracle.gelu(x), ref) < 1e-15
    assert rel_err(oracle.gelu(x.astype(np.float32)), ref) < 3e-7
    # the tanh approximation is a different op and must NOT match at this tolerance
    tanh_form = 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3)))
    assert rel_err(oracle.gelu(x), tanh_form) > 1e-5
    a = rng.standard_normal((5, 33)).astype(np.float32)
    r = rng.standard_normal((5, 33)).astype(np.float32)
    bias = rng.standard_normal(33).astype(np.float32)
    assert np.array_equal(oracle.add(a, r), a + r)
    assert np.array_equal(oracle.bias_add(a, bias), a + bias)
    assert np.array_equal(oracle.bias_add(a, bias, r), (a + bias) + r)


def test_gemm_linear_against_numpy(oracle):
    rng = np.random.default_rng(3)
    for dt, tol in ((np.float64, 1e-14), (np.float32, 2e-7)):
        a = rng.uniform(-1, 1, (23, 41)).astype(dt)
        b = rng.uniform(-1, 1, (41, 17)).astype(dt)
        ref = a.astype(np.float64) @ b.astype(np.float64)
        assert rel_err(oracle.gemm(a, b), ref) < tol
        assert rel_err(oracle.gemm(a, np.ascontiguousarray(b.T), True), ref) < tol
        # a transposed-operand mistake shows on a non-square shape
        assert oracle.gemm(a, b).shape == (23, 17)
        bias = rng.standard_normal(17).astype(dt)
        assert rel_err(oracle.linear(a, np.ascontiguousarray(b.T), bias), ref + bias) < tol
        inp = rng.standard_normal((23, 17)).astype(dt)
        assert rel_err(oracle.addmm(inp, a, b, 0.5, 2.0), 0.5 * inp + 2.0 * ref) < 2 * tol
        assert rel_err(oracle.addmm(bias, a, b, 0.5, 2.0), 0.5 * bias + 2.0 * ref) < 2 * tol
    a = rng.uniform(-1, 1, (3, 7, 5)).astype(np.float32)
    b = rng.uniform(-1, 1, (3, 5, 4)).astype(np.float32)
    assert rel_err(oracle.bmm(a, b), np.einsum("bij,bjk->bik", a.astype(np.float64), b.astype(np.float64))) < 2e-7
    big_a = rng.uniform(-1, 1, (64, 300)).astype(np.float32)
    big_b = rng.uniform(-1, 1, (300, 50)).astype(np.float32)
    fast = oracle.sgemm_blocked(big_a, big_b)
    if fast is not None:
        assert rel_err(fast, big_a.astype(np.float64) @ big_b.astype(np.float64)) < 2e-6


def _textbook_attention(q, k, v, scale, causal):
    q, k, v = (t.astype(np.float64) for t in (q, k, v))
    s = np.einsum("bqd,bkd->bqk", q, k) * scale
    if causal:
        sq, sk = s.shape[1:]
        mask = np.arange(sk)[None, :] > np.arange(sq)[:, None]
        s = np.where(mask[None], -np.inf, s)
    p = scipy.special.softmax(s, axis=-1)
    return np.einsum("bqk,bkd->bqd", p, v)


def test_sdpa_against_textbook_attention(oracle):
    rng = np.random.default_rng(4)
    for (bh, sq, sk, dk, dv, causal) in [(3, 17, 17, 8, 8, True), (2, 9, 14, 16, 5, False), (2, 14, 9, 4, 6, True)]:
        q = rng.standard_normal((bh, sq, dk))
        k = rng.standard_normal((bh, sk, dk))
        v = rng.standard_normal((bh, sk, dv))
        scale = 1 / math.sqrt(dk)
        ref = _textbook_attention(q, k, v, scale, causal)
        assert rel_err(oracle.sdpa_forward(q, k, v, scale, causal), ref) < 1e-14
        assert rel_err(oracle.sdpa_forward(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), scale, causal), ref) < 2e-6
    # causal independence (crates/ft-nn/src/lib.rs:24403): changing later keys cannot move earlier rows
    q = rng.standard_normal((1, 12, 8))
    k = rng.standard_normal((1, 12, 8))
    v = rng.standard_normal((1, 12, 8))
    base = oracle.sdpa_forward(q, k, v, 0.3, True)
    k2, v2 = k.copy(), v.copy()
    k2[:, 7:] += 5.0
    v2[:, 7:] -= 3.0
    assert np.array_equal(oracle.sdpa_forward(q, k2, v2, 0.3, True)[:, :7], base[:, :7])
    # torch CPU attention as an independent library routine
    import torch

    t = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), is_causal=True,
                                                         scale=0.3)
    assert rel_err(base, t.numpy()) < 1e-13


def test_argmax_index_permute_semantics(oracle):
    x = np.array([[1.0, 7.0, 7.0, 2.0], [np.nan, 9.0, 1.0, np.nan], [-np.inf] * 4, [3.0, np.nan, 9.0, 9.0]])
    assert oracle.argmax(x, 1).tolist() == [1.0, 0.0, 0.0, 1.0]  # first max, first NaN, all -inf -> 0
    assert oracle.argmax(x.astype(np.float32), 1).tolist() == [1.0, 0.0, 0.0, 1.0]
    rng = np.random.default_rng(5)
    y = rng.standard_normal((4, 6, 5))
    for d in range(3):
        assert np.array_equal(oracle.argmax(y, d), np.argmax(y, axis=d).astype(np.float64))
    t = rng.standard_normal((7, 3, 2))
    out, bad = oracle.index_select(t, 1, [2.0, 0.0, 2.0])
    assert bad == -1 and np.array_equal(out, t[:, [2, 0, 2], :])
    _, bad = oracle.index_select(t, 1, [1.0, 1.5])
    assert bad == 1
    p = rng.standard_normal((2, 3, 4, 5))
    assert np.array_equal(oracle.permute_0213(p), p.transpose(0, 2, 1, 3))


def _rand_layer(rng, d, f):
    n = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float32)
    return {"ln1_w": (1 + 0.1 * rng.standard_normal(d)).astype(np.float32), "ln1_b": n(d), "wq": n(d, d), "bq": n(d), "wk": n(d, d),
            "bk": n(d), "wv": n(d, d), "bv": n(d), "wo": n(d, d), "bo": n(d),
            "ln2_w": (1 + 0.1 * rng.standard_normal(d)).astype(np.float32), "ln2_b": n(d), "w1": n(f, d), "b1": n(f), "w2": n(d, f), "b2": n(d)}


def test_block_and_gpt2_composition_against_numpy(oracle):
    """The composite oracles equal the textbook pre-LN block / decoder written out in numpy f64."""
    rng = np.random.default_rng(6)
    d, f, heads, batch, seq, vocab = 16, 32, 4, 2, 6, 37
    L = [_rand_layer(rng, d, f) for _ in range(2)]
    x = rng.standard_normal((batch * seq, d)).astype(np.float32)

    def ln(z, w, b):
        mu = z.mean(-1, keepdims=True)
        return (z - mu) / np.sqrt(z.var(-1, keepdims=True) + 1e-5) * w + b

    def block(z, w):
        z = z.astype(np.float64)
        h = ln(z, w["ln1_w"], w["ln1_b"])
        q, k, v = (h @ w[n].T.astype(np.float64) + w[bn] for n, bn in (("wq", "bq"), ("wk", "bk"), ("wv", "bv")))
        hd = d // heads
        sp = lambda t: t.reshape(batch, seq, heads, hd).transpose(0, 2, 1, 3).reshape(batch * heads, seq, hd)
        ctx = _textbook_attention(sp(q), sp(k), sp(v), 1 / math.sqrt(hd), True)
        ctx = ctx.reshape(batch, heads, seq, hd).transpose(0, 2, 1, 3).reshape(batch * seq, d)
        z = z + ctx @ w["wo"].T.astype(np.float64) + w["bo"]
        h = ln(z, w["ln2_w"], w["ln2_b"])
        u = h @ w["w1"].T.astype(np.float64) + w["b1"]
        u = 0.5 * u * (1 + scipy.special.erf(u / np.sqrt(2)))
        return z + u @ w["w2"].T.astype(np.float64) + w["b2"]

    assert rel_err(oracle.encoder_layer(L[0], x, batch, seq, heads, 1e-5, True), block(x, L[0])) < 5e-6
    wte = (0.02 * rng.standard_normal((vocab, d))).astype(np.float32)
    wpe = (0.02 * rng.standard_normal((seq + 2, d))).astype(np.float32)
    lnf_w = np.ones(d, np.float32)
    lnf_b = np.zeros(d, np.float32)
    ids = rng.integers(0, vocab, (batch, seq)).astype(np.float64)
    out = oracle.gpt2_forward(wte, wpe, L, lnf_w, lnf_b, ids, batch, seq, heads, 1e-5)
    z = wte[ids.astype(int).ravel()].astype(np.float64) + np.tile(wpe[:seq].astype(np.float64), (batch, 1))
    for w in L:
        z = block(z, w)
    hidden = ln(z, lnf_w, lnf_b)
    logits = hidden @ wte.T.astype(np.float64)
    assert out["bad"] == -1
    assert rel_err(out["hidden"], hidden) < 1e-5
    assert rel_err(out["logits"], logits) < 1e-5
    assert np.array_equal(out["argmax"], np.argmax(out["logits"], axis=1).astype(np.float32))
    bad = oracle.gpt2_forward(wte, wpe, L, lnf_w, lnf_b, np.where(np.arange(batch * seq) == 3, float(vocab), ids.ravel()), batch, seq, heads, 1e-5)
    assert bad["bad"] == 3
