"""Resident tier: HipTensor / Batch ops, the pre-LN block (config 1) and the GPT-2-shaped forward
(config 5, plus a small instance compared end to end) against the CPU checker."""
import math

import numpy as np
import pytest

from conftest import TOL_GEMM_F32, TOL_ROW_F32, rel_err
from frankentorch_amd import fused, synth
from frankentorch_amd.device import DeviceBuffer

pytestmark = pytest.mark.gpu


def make_layer(seed, li, d, f, biases_zero=True):
    """Weights N(0, 0.02), biases zero, LayerNorm gamma 1 / beta 0 (the configured initialisation);
    biases_zero=False perturbs every vector so that a dropped bias or affine term is visible."""
    n = lambda tag, *s: synth.normal(seed, "L%d.%s" % (li, tag), s, 0.0, 0.02)
    vec = (lambda tag, m, base: np.full(m, base, np.float32)) if biases_zero else \
        (lambda tag, m, base: (base + synth.normal(seed, "L%d.%s" % (li, tag), (m,), 0.0, 0.1)).astype(np.float32))
    return {"ln1_w": vec("ln1_w", d, 1.0), "ln1_b": vec("ln1_b", d, 0.0), "wq": n("wq", d, d), "bq": vec("bq", d, 0.0),
            "wk": n("wk", d, d), "bk": vec("bk", d, 0.0), "wv": n("wv", d, d), "bv": vec("bv", d, 0.0), "wo": n("wo", d, d),
            "bo": vec("bo", d, 0.0), "ln2_w": vec("ln2_w", d, 1.0), "ln2_b": vec("ln2_b", d, 0.0), "w1": n("w1", f, d),
            "b1": vec("b1", f, 0.0), "w2": n("w2", d, f), "b2": vec("b2", d, 0.0)}


def test_tensor_round_trip_and_pool(hip):
    a = synth.normal(1, "rt", (37, 19))
    t = fused.HipTensor.upload(a)
    assert t.shape == (37, 19) and np.array_equal(t.download(), a)
    with pytest.raises(ValueError):
        fused.HipTensor.upload(a, 5, 5)
    t.free()


def test_batch_ops_match_oracle(hip, oracle):
    m, k, n = 130, 96, 200
    x = synth.normal(2, "x", (m, k))
    w = synth.normal(2, "w", (n, k), 0.0, 0.1)
    bias = synth.normal(2, "b", (n,))
    gamma = synth.uniform(2, "g", (n,), 0.5, 1.5)
    beta = synth.normal(2, "be", (n,), 0.0, 0.1)
    b = fused.Batch()
    tx, tw, tb, tg, tbe = (fused.HipTensor.upload(a) for a in (x, w, bias, gamma, beta))
    y = b.matmul_bias(tx, tw, tb)
    ln = b.layernorm(y, tg, tbe, 1e-5)
    rn = b.rmsnorm(y, tg, 1e-6)
    ge = b.gelu(y)
    ad = b.add(y, ge)
    sm = b.softmax(y)
    mm = b.matmul(tx, fused.HipTensor.upload(np.ascontiguousarray(w.T)))
    b.finish()
    ref_y = oracle.linear(x, w, bias)
    got_y = y.download()
    assert rel_err(got_y, ref_y) <= TOL_GEMM_F32
    # downstream ops are compared on the GPU's own y so that only the op under test contributes
    assert rel_err(ln.download(), oracle.layer_norm(got_y, gamma, beta, 1e-5)) <= TOL_ROW_F32
    assert rel_err(rn.download(), oracle.rms_norm(got_y, gamma, 1e-6)) <= TOL_ROW_F32
    assert rel_err(ge.download(), oracle.gelu(got_y)) <= TOL_ROW_F32
    assert np.array_equal(ad.download(), got_y + ge.download())
    assert rel_err(sm.download(), oracle.softmax(got_y, 1)) <= TOL_ROW_F32
    assert rel_err(mm.download(), oracle.gemm(x, np.ascontiguousarray(w.T))) <= TOL_GEMM_F32


def test_batch_mha_matches_split_heads_oracle(hip, oracle):
    batch, seq, heads, hd = 2, 70, 4, 64
    d = heads * hd
    q, k, v = (synth.normal(3, t, (batch * seq, d), 0.0, 0.5) for t in "qkv")
    b = fused.Batch()
    out = b.mha(fused.HipTensor.upload(q), fused.HipTensor.upload(k), fused.HipTensor.upload(v), heads, batch, causal=True)
    b.finish()
    split = lambda t: oracle.permute_0213(t.reshape(batch, seq, heads, hd)).reshape(batch * heads, seq, hd)
    ctx = oracle.sdpa_forward(split(q), split(k), split(v), 1 / math.sqrt(hd), True)
    ref = oracle.permute_0213(ctx.reshape(batch, heads, seq, hd)).reshape(batch * seq, d)
    assert rel_err(out.download(), ref) <= TOL_GEMM_F32


def test_config1_block_forward_eager_graph_and_determinism(hip, oracle):
    """Config 1: batch 1, seq 128, d_model 256, 4 heads, FFN 1024, causal, fp32, seed 0."""
    batch, seq, d, heads, f = 1, 128, 256, 4, 1024
    layer = make_layer(0, 0, d, f)
    x = synth.normal(0, "x", (batch * seq, d))
    enc = fused.EncoderHip(d, heads, f, [layer], 1e-5, causal=True)
    got = enc.forward(x, batch, seq)
    ref = oracle.encoder_layer(layer, x, batch, seq, heads, 1e-5, True)
    assert rel_err(got, ref) <= TOL_GEMM_F32
    assert np.array_equal(got, enc.forward(x, batch, seq))  # bitwise repeatable
    # HIP-graph replay: every replay equals the eager result, with eager work in between
    dx, dout = DeviceBuffer.from_host(x), DeviceBuffer((batch * seq, d))
    scratch = DeviceBuffer((batch * seq, d))
    for _ in range(4):
        enc.forward_dev(dx, dout, batch, seq, graph=True)
        replay = dout.to_host()
        assert np.array_equal(replay, got)
        enc.forward_dev(dx, scratch, batch, seq)  # eager launch between replays
        hip.gelu(scratch, scratch, batch * seq * d)
        hip.synchronize()
    # a non-trivial layer (non-zero biases, non-unit gamma) so no term can be dropped unnoticed
    layer2 = make_layer(0, 1, d, f, biases_zero=False)
    enc2 = fused.EncoderHip(d, heads, f, [layer2], 1e-5, causal=True)
    assert rel_err(enc2.forward(x, batch, seq), oracle.encoder_layer(layer2, x, batch, seq, heads, 1e-5, True)) <= TOL_GEMM_F32
    # non-causal, batch > 1, two layers
    enc3 = fused.EncoderHip(d, heads, f, [layer, layer2], 1e-5, causal=False)
    x3 = synth.normal(0, "x3", (3 * 40, d))
    ref3 = oracle.encoder_layer(layer2, oracle.encoder_layer(layer, x3, 3, 40, heads, 1e-5, False), 3, 40, heads, 1e-5, False)
    assert rel_err(enc3.forward(x3, 3, 40), ref3) <= TOL_GEMM_F32


def test_small_gpt2_forward_matches_oracle(hip, oracle):
    vocab, maxpos, d, heads, f, nl, batch, seq = 1003, 48, 128, 4, 512, 3, 2, 40
    wte = synth.normal(4, "wte", (vocab, d), 0.0, 0.02)
    wpe = synth.normal(4, "wpe", (maxpos, d), 0.0, 0.02)
    layers = [make_layer(4, i, d, f, biases_zero=(i == 0)) for i in range(nl)]
    lnf_w = (1.0 + synth.normal(4, "lnf_w", (d,), 0.0, 0.1)).astype(np.float32)
    lnf_b = synth.normal(4, "lnf_b", (d,), 0.0, 0.1)
    ids = synth.token_ids(4, "ids", (batch * seq,), vocab)
    model = fused.Gpt2Hip(wte, wpe, layers, lnf_w, lnf_b, heads, 1e-5)
    dids = DeviceBuffer.from_host(ids)
    dlog, dam = DeviceBuffer((batch * seq, vocab)), DeviceBuffer((batch * seq,))
    model.forward_dev(dids, batch, seq, dlog, dam)
    logits, am = dlog.to_host(), dam.to_host()
    ref = oracle.gpt2_forward(wte, wpe, layers, lnf_w, lnf_b, ids, batch, seq, heads, 1e-5)
    assert model.bad_index() == -1 and ref["bad"] == -1
    assert rel_err(model.hidden(batch * seq), ref["hidden"]) <= TOL_GEMM_F32
    assert rel_err(logits, ref["logits"]) <= TOL_GEMM_F32
    assert np.array_equal(am, np.argmax(logits, axis=1).astype(np.float32))  # argmax kernel is exact on its own input
    assert np.array_equal(am, ref["argmax"])
    # argmax only (logits kept internal) gives the same indices
    dam2 = DeviceBuffer((batch * seq,))
    model.forward_dev(dids, batch, seq, None, dam2)
    assert np.array_equal(dam2.to_host(), am)
    # an out-of-range id is reported, not wrapped
    bad_ids = ids.copy()
    bad_ids[7] = float(vocab)
    model.forward_dev(DeviceBuffer.from_host(bad_ids), batch, seq, None, dam2)
    assert model.bad_index() == 7


def test_config5_gpt2_small_shape_logits_and_argmax(hip, oracle):
    """Config 5: 12 layers, d 768, 12 heads, FFN 3072, vocab 50257, batch 8, seq 1024, seed 4.
    The full CPU forward is too slow for a test, so the pipeline is pinned in three steps:
    (1) the first 16 tokens of sequence 0 are causal-closed, so the oracle runs the whole model on
    that prefix and must reproduce the GPU's final hidden rows; (2) on sampled rows of the GPU's
    final hidden state the oracle's tied LM head gives the logits and the argmax, which must be
    IDENTICAL unless the oracle's own top-2 gap is below the fp32 rounding of the product
    (reported, never silently accepted); (3) the whole logits tensor is bitwise repeatable."""
    vocab, maxpos, d, heads, f, nl, batch, seq = 50257, 1024, 768, 12, 3072, 12, 8, 1024
    wte = synth.normal(4, "wte", (vocab, d), 0.0, 0.02)
    wpe = synth.normal(4, "wpe", (maxpos, d), 0.0, 0.02)
    layers = [make_layer(4, i, d, f) for i in range(nl)]
    ids = synth.token_ids(4, "ids", (batch * seq,), vocab)
    model = fused.Gpt2Hip(wte, wpe, layers, None, None, heads, 1e-5)
    T = batch * seq
    dids = DeviceBuffer.from_host(ids)
    dlog, dam = DeviceBuffer((T, vocab)), DeviceBuffer((T,))
    model.forward_dev(dids, batch, seq, dlog, dam)
    am = dam.to_host()
    hidden = model.hidden(T)
    assert model.bad_index() == -1
    # (1) causal prefix through the whole model
    P = 16
    ref = oracle.gpt2_forward(wte, wpe, layers, np.ones(d, np.float32), np.zeros(d, np.float32), ids[:P], 1, P, heads, 1e-5,
                              want_logits=False)
    assert rel_err(hidden[:P], ref["hidden"]) <= TOL_GEMM_F32
    # (2) LM head + argmax on sampled rows
    rows = np.concatenate([np.arange(P), np.arange(97, T, 257)])
    ref_logits = oracle.gemm(hidden[rows], wte, trans_b=True)
    logits_rows = np.empty((rows.size, vocab), np.float32)
    full = dlog.to_host()
    logits_rows[:] = full[rows]
    assert rel_err(logits_rows, ref_logits) <= TOL_GEMM_F32
    ref_am = np.argmax(ref_logits, axis=1)
    assert np.array_equal(am[rows], np.argmax(logits_rows, axis=1).astype(np.float32))
    mism = np.nonzero(am[rows] != ref_am)[0]
    for i in mism:
        top2 = np.sort(ref_logits[i])[-2:]
        gap = float(top2[1] - top2[0])
        print("argmax differs at row %d: oracle %d gpu %d, oracle top-2 gap %.3e" % (rows[i], ref_am[i], am[rows][i], gap))
        assert gap <= 4 * np.finfo(np.float32).eps * float(np.max(np.abs(ref_logits[i]))), "argmax differs beyond rounding"
    # (3) bitwise repeatability of the whole forward
    dlog2 = DeviceBuffer((T, vocab))
    model.forward_dev(dids, batch, seq, dlog2, None)
    assert np.array_equal(full.view(np.uint32), dlog2.to_host().view(np.uint32))
