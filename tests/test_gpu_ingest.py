"""Weights from a safetensors container straight into resident buffers: device reads with conversion and transposition on
the GPU, and a GPT-2 checkpoint (Hugging Face tensor names, Conv1D [in, out] matrices) loaded into the resident decoder."""
import numpy as np
import pytest

from conftest import TOL_GEMM_F32, rel_err
from frankentorch_amd import fused, synth
from frankentorch_amd import serialize as S
from frankentorch_amd.core import HipError
from frankentorch_amd.device import DeviceBuffer
from test_gpu_resident import make_layer

pytestmark = pytest.mark.gpu
st = pytest.importorskip("safetensors")
from safetensors.numpy import save  # noqa: E402


def _bf16(a):
    return (np.asarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def _with_bf16(tensors, bf):
    """The crate's serializer for numpy types, plus hand-placed BF16 tensors (numpy has no such type)."""
    import json
    import struct

    hdr, payload = {}, b""
    for name, a in sorted(tensors.items()):
        dt = {np.dtype(np.float64): "F64", np.dtype(np.float32): "F32", np.dtype(np.float16): "F16"}[a.dtype]
        hdr[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [len(payload), len(payload) + a.nbytes]}
        payload += a.tobytes()
    for name, a in sorted(bf.items()):
        hdr[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [len(payload), len(payload) + a.size * 2]}
        payload += _bf16(a).tobytes()
    h = json.dumps(hdr).encode()
    return struct.pack("<Q", len(h)) + h + payload


def test_device_reads_convert_and_transpose(hip):
    rng = np.random.default_rng(1)
    m32 = rng.standard_normal((70, 45)).astype(np.float32)
    m16 = (rng.standard_normal((33, 130)) * 3).astype(np.float16)
    m16[0, :4] = [6e-8, -6e-5, np.inf, 65504.0]  # a subnormal, a small normal, infinity, the largest half
    m64 = rng.standard_normal((5, 7))
    vec = rng.standard_normal(1000).astype(np.float32)
    mbf = rng.standard_normal((64, 64)).astype(np.float32)
    f = S.SafeTensorsFile(_with_bf16({"m32": m32, "m16": m16, "m64": m64, "vec": vec}, {"mbf": mbf}))
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
    f.read_dev("vec", dv)
    assert np.array_equal(dv.to_host(), vec)
    with pytest.raises(HipError):
        f.read_dev("vec", dv, transpose=True)  # not a matrix
    with pytest.raises(HipError):
        f.read_dev("m32", DeviceBuffer((10,), np.float32))  # destination too small
    with pytest.raises(HipError):
        f.read_dev("absent", dv)


def test_a_tensor_larger_than_the_staging_buffers(hip, tmp_path):
    """80 MB (five fills of the 16 MiB pinned pair) from a memory-mapped file, plain and transposed + widened."""
    rng = np.random.default_rng(2)
    big = rng.standard_normal((5000, 4001)).astype(np.float32)
    half = big[:2500].astype(np.float16)
    p = tmp_path / "big.safetensors"
    p.write_bytes(save({"big": big, "half": half}))
    with S.SafeTensorsFile(p) as f:
        d = DeviceBuffer(big.shape, np.float32)
        f.read_dev("big", d)
        assert np.array_equal(d.to_host(), big)
        dt = DeviceBuffer((4001, 2500), np.float32)
        f.read_dev("half", dt, transpose=True)
        assert np.array_equal(dt.to_host(), half.astype(np.float32).T)


def _checkpoint(wte, wpe, layers, lnf_w, lnf_b, prefix="", dtype=np.float32):
    """Hugging Face GPT-2 tensor names; projections stored [in, out] as Conv1D keeps them."""
    t = {prefix + "wte.weight": wte, prefix + "wpe.weight": wpe, prefix + "ln_f.weight": lnf_w, prefix + "ln_f.bias": lnf_b}
    for i, L in enumerate(layers):
        h = "%sh.%d." % (prefix, i)
        t[h + "ln_1.weight"], t[h + "ln_1.bias"] = L["ln1_w"], L["ln1_b"]
        t[h + "attn.c_attn.weight"] = np.concatenate([L["wq"], L["wk"], L["wv"]], axis=0).T
        t[h + "attn.c_attn.bias"] = np.concatenate([L["bq"], L["bk"], L["bv"]])
        t[h + "attn.c_proj.weight"], t[h + "attn.c_proj.bias"] = L["wo"].T, L["bo"]
        t[h + "ln_2.weight"], t[h + "ln_2.bias"] = L["ln2_w"], L["ln2_b"]
        t[h + "mlp.c_fc.weight"], t[h + "mlp.c_fc.bias"] = L["w1"].T, L["b1"]
        t[h + "mlp.c_proj.weight"], t[h + "mlp.c_proj.bias"] = L["w2"].T, L["b2"]
        t[h + "attn.bias"] = np.tril(np.ones((1, 1, 8, 8), np.float32))  # the mask buffer real checkpoints carry: ignored
    return {k: np.ascontiguousarray(v, dtype=dtype) for k, v in t.items()}


def _small_model():
    vocab, maxpos, d, heads, f, nl = 1003, 48, 128, 4, 512, 3
    wte = synth.normal(6, "wte", (vocab, d), 0.0, 0.02)
    wpe = synth.normal(6, "wpe", (maxpos, d), 0.0, 0.02)
    layers = [make_layer(6, i, d, f, biases_zero=False) for i in range(nl)]
    lnf_w = (1.0 + synth.normal(6, "lnf_w", (d,), 0.0, 0.1)).astype(np.float32)
    lnf_b = synth.normal(6, "lnf_b", (d,), 0.0, 0.1)
    return vocab, heads, wte, wpe, layers, lnf_w, lnf_b


def _logits(model, ids, batch, seq, vocab):
    out = DeviceBuffer((batch * seq, vocab))
    model.forward_dev(DeviceBuffer.from_host(ids), batch, seq, out, None)
    return out.to_host()


@pytest.mark.parametrize("prefix", ["", "transformer."])
def test_gpt2_checkpoint_equals_the_model_built_from_host_arrays(hip, oracle, tmp_path, prefix):
    vocab, heads, wte, wpe, layers, lnf_w, lnf_b = _small_model()
    batch, seq = 2, 40
    ids = synth.token_ids(6, "ids", (batch * seq,), vocab)
    p = tmp_path / "gpt2.safetensors"
    p.write_bytes(save(_checkpoint(wte, wpe, layers, lnf_w, lnf_b, prefix), metadata={"format": "pt"}))
    for tanh in (False, True):
        loaded = fused.Gpt2Hip.from_safetensors(p, heads, 1e-5, gelu_tanh=tanh)
        assert (loaded.vocab, loaded.max_pos, loaded.d_model, loaded.n_heads, loaded.d_ff, loaded.n_layers) == (vocab, 48, 128, heads, 512, 3)
        direct = fused.Gpt2Hip(wte, wpe, layers, lnf_w, lnf_b, heads, 1e-5, gelu_tanh=tanh)
        got = _logits(loaded, ids, batch, seq, vocab)
        assert np.array_equal(got.view(np.uint32), _logits(direct, ids, batch, seq, vocab).view(np.uint32))
        if not tanh:
            ref = oracle.gpt2_forward(wte, wpe, layers, lnf_w, lnf_b, ids, batch, seq, heads, 1e-5)
            assert rel_err(got, ref["logits"]) <= TOL_GEMM_F32


def test_gpt2_checkpoint_in_half_precision_and_damaged_checkpoints(hip, tmp_path):
    vocab, heads, wte, wpe, layers, lnf_w, lnf_b = _small_model()
    batch, seq = 1, 16
    ids = synth.token_ids(7, "ids", (batch * seq,), vocab)
    ck16 = _checkpoint(wte, wpe, layers, lnf_w, lnf_b, dtype=np.float16)
    loaded = fused.Gpt2Hip.from_safetensors(save(ck16), heads)
    r = lambda a: np.asarray(a, np.float16).astype(np.float32)  # the model a half-precision file describes
    rl = [{k: r(v) for k, v in L.items()} for L in layers]
    direct = fused.Gpt2Hip(r(wte), r(wpe), rl, r(lnf_w), r(lnf_b), heads, 1e-5, gelu_tanh=True)
    assert np.array_equal(_logits(loaded, ids, batch, seq, vocab), _logits(direct, ids, batch, seq, vocab))
    ck = _checkpoint(wte, wpe, layers, lnf_w, lnf_b)
    missing = {k: v for k, v in ck.items() if k != "h.1.mlp.c_proj.bias"}
    with pytest.raises(HipError) as e:
        fused.Gpt2Hip.from_safetensors(save(missing), heads)
    assert e.value.kind == "Corrupt" and "h.1.mlp.c_proj.bias" in e.value.message
    wrong = dict(ck)
    wrong["h.0.attn.c_attn.weight"] = np.zeros((128, 300), np.float32)
    with pytest.raises(HipError) as e:
        fused.Gpt2Hip.from_safetensors(save(wrong), heads)
    assert e.value.kind == "Corrupt"
    with pytest.raises(HipError):
        fused.Gpt2Hip.from_safetensors(save(ck), 5)  # 128 is not divisible by 5 heads
