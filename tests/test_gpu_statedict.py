"""Weights from the reference's native state-dict container ("FTSV") straight into resident buffers: device reads with
conversion and transposition on the GPU, and a GPT-2-shaped checkpoint loaded into the resident decoder, which must give
the logits and the argmax of the model built from the same host arrays, bit for bit."""
import numpy as np
import pytest

from conftest import TOL_GEMM_F32, rel_err
from frankentorch_amd import fused, synth
from frankentorch_amd import serialize as S
from frankentorch_amd.core import HipError
from frankentorch_amd.device import DeviceBuffer
from test_gpu_ingest import _bf16, _checkpoint, _logits, _small_model

pytestmark = pytest.mark.gpu


def test_device_reads_convert_and_transpose(hip, oracle):
    rng = np.random.default_rng(21)
    m32 = rng.standard_normal((70, 45)).astype(np.float32)
    m16 = (rng.standard_normal((33, 130)) * 3).astype(np.float16)
    m16[0, :4] = [6e-8, -6e-5, np.inf, 65504.0]
    m64 = rng.standard_normal((5, 7))
    vec = rng.standard_normal(1000).astype(np.float32)
    mbf = rng.standard_normal((64, 64)).astype(np.float32)
    data = oracle.encode_state_dict({"m32": m32, "m16": m16, "m64": m64, "vec": vec, "mbf": (_bf16(mbf), "bf16")})
    f = S.StateDictFile(data)
    assert f.names() == ["m16", "m32", "m64", "mbf", "vec"]
    bf_exact = S.bf16_to_f32(_bf16(mbf)).reshape(mbf.shape)
    for name, want in (("m32", m32), ("m16", m16.astype(np.float32)), ("m64", m64.astype(np.float32)), ("mbf", bf_exact)):
        for transpose in (False, True):
            ref = want.T if transpose else want
            dst = DeviceBuffer(ref.shape, np.float32)
            f.read_dev(name, dst, transpose=transpose)
            assert np.array_equal(dst.to_host().view(np.uint32), np.ascontiguousarray(ref).view(np.uint32)), (name, transpose)
            d64 = DeviceBuffer(ref.shape, np.float64)
            f.read_dev(name, d64, transpose=transpose)
            want64 = (m64.T if transpose else m64) if name == "m64" else ref.astype(np.float64)
            assert np.array_equal(d64.to_host(), want64), (name, transpose)
    dv = DeviceBuffer((1000,), np.float32)
    f.read_dev("vec", dv)   # payloads sit at arbitrary byte offsets in this container: nothing may assume alignment
    assert np.array_equal(dv.to_host(), vec)
    with pytest.raises(HipError):
        f.read_dev("vec", dv, transpose=True)
    with pytest.raises(HipError):
        f.read_dev("absent", dv)


def test_gpt2_shaped_state_dict_equals_the_model_built_from_host_arrays(hip, oracle, tmp_path):
    vocab, heads, wte, wpe, layers, lnf_w, lnf_b = _small_model()
    batch, seq = 2, 40
    ids = synth.token_ids(6, "ids", (batch * seq,), vocab)
    p = tmp_path / "gpt2.ftsv"
    p.write_bytes(oracle.encode_state_dict(_checkpoint(wte, wpe, layers, lnf_w, lnf_b)))
    loaded = fused.Gpt2Hip.from_state_dict(p, heads, 1e-5, gelu_tanh=False)
    assert (loaded.vocab, loaded.max_pos, loaded.d_model, loaded.n_heads, loaded.d_ff, loaded.n_layers) == (vocab, 48, 128, heads, 512, 3)
    direct = fused.Gpt2Hip(wte, wpe, layers, lnf_w, lnf_b, heads, 1e-5, gelu_tanh=False)
    got = _logits(loaded, ids, batch, seq, vocab)
    assert np.array_equal(got.view(np.uint32), _logits(direct, ids, batch, seq, vocab).view(np.uint32))
    am_l, am_d = DeviceBuffer((batch * seq,)), DeviceBuffer((batch * seq,))
    dids = DeviceBuffer.from_host(ids)
    loaded.forward_dev(dids, batch, seq, None, am_l)
    direct.forward_dev(dids, batch, seq, None, am_d)
    ref = oracle.gpt2_forward(wte, wpe, layers, lnf_w, lnf_b, ids, batch, seq, heads, 1e-5)
    assert np.array_equal(am_l.to_host(), am_d.to_host()) and np.array_equal(am_l.to_host(), ref["argmax"])
    assert rel_err(got, ref["logits"]) <= TOL_GEMM_F32
    # half-precision payloads widen on the GPU; a missing tensor is reported by name
    ck16 = _checkpoint(wte, wpe, layers, lnf_w, lnf_b, dtype=np.float16)
    half = fused.Gpt2Hip.from_state_dict(oracle.encode_state_dict(ck16), heads)
    r = lambda a: np.asarray(a, np.float16).astype(np.float32)
    rl = [{k: r(v) for k, v in L.items()} for L in layers]
    direct16 = fused.Gpt2Hip(r(wte), r(wpe), rl, r(lnf_w), r(lnf_b), heads, 1e-5, gelu_tanh=True)
    assert np.array_equal(_logits(half, ids, batch, seq, vocab), _logits(direct16, ids, batch, seq, vocab))
    ck = _checkpoint(wte, wpe, layers, lnf_w, lnf_b)
    with pytest.raises(HipError) as e:
        fused.Gpt2Hip.from_state_dict(oracle.encode_state_dict({k: v for k, v in ck.items() if k != "h.2.ln_2.bias"}), heads)
    assert e.value.kind == "Corrupt" and "h.2.ln_2.bias" in e.value.message
