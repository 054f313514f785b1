"""The safetensors reader on the host (no GPU needed): the reference's own loader tests restated
(crates/ft-serialize/src/lib.rs:4769-5133), its fuzz-corpus seeds, and a seeded differential run against the
`safetensors` package 0.8.0 -- the Python binding of the very crate version the reference pins (Cargo.lock:2081-2084)."""
import json
import random
import struct

import numpy as np
import pytest

from frankentorch_amd import serialize as S
from frankentorch_amd.core import HipError

st = pytest.importorskip("safetensors")
from safetensors import deserialize  # noqa: E402
from safetensors.numpy import save  # noqa: E402

READABLE = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2}


def _container(header: dict, payload: bytes) -> bytes:
    h = json.dumps(header).encode()
    return struct.pack("<Q", len(h)) + h + payload


def _malformed(dtype, shape, payload):
    """malformed_safetensors_bytes, crates/ft-serialize/src/lib.rs:5062-5076."""
    return _container({"bad": {"dtype": dtype, "shape": shape, "data_offsets": [0, len(payload)]}}, bytes(payload))


def test_round_trips_of_the_reference(tmp_path):
    # safetensors_round_trip_f64 / _f32 / _f16 (:4769-4870), written by the crate's own serializer
    p = tmp_path / "w.safetensors"
    p.write_bytes(save({"weight": np.array([[1.0, 2.0], [3.0, 4.0]])}))
    got = S.load_safetensors(p)
    assert list(got) == ["weight"] and got["weight"].dtype == np.float64 and got["weight"].tolist() == [[1.0, 2.0], [3.0, 4.0]]
    got = S.load_safetensors_from_bytes(save({"w": np.array([1.0, 2.0, 3.0], np.float32)}))
    assert got["w"].dtype == np.float32 and got["w"].tolist() == [1.0, 2.0, 3.0]
    got = S.load_safetensors_from_bytes(save({"h": np.array([1.0, 2.0, 3.0], np.float16)}))
    assert got["h"].dtype == np.float16 and got["h"].tolist() == [1.0, 2.0, 3.0]
    # safetensors_round_trip_bf16 (:4872): 1, 2, 3 in bfloat16 are the top halves of the f32 patterns
    bits = (np.array([1.0, 2.0, 3.0], np.float32).view(np.uint32) >> 16).astype(np.uint16)
    got = S.load_safetensors_from_bytes(_container({"b": {"dtype": "BF16", "shape": [3], "data_offsets": [0, 6]}}, bits.tobytes()))
    assert got["b"].dtype == np.uint16 and S.bf16_to_f32(got["b"]).tolist() == [1.0, 2.0, 3.0]
    # safetensors_empty_state_dict (:4894), safetensors_multiple_tensors (:4974): name order, mixed types
    assert S.load_safetensors_from_bytes(save({})) == {}
    many = {"b.weight": np.arange(6, dtype=np.float32).reshape(2, 3), "a.bias": np.array([0.5, -1.5]), "c": np.zeros((3, 0, 5), np.float32)}
    got = S.load_safetensors_from_bytes(save(many))
    assert list(got) == sorted(many)
    for k, v in many.items():
        assert got[k].dtype == v.dtype and got[k].shape == v.shape and np.array_equal(got[k], v)


def test_bit_patterns_survive(tmp_path):
    """prop_safetensors_f32/f64_roundtrip_preserves_all_bit_patterns (:3543-3610): NaN payloads, infinities, subnormals."""
    rng = np.random.default_rng(3)
    b32 = rng.integers(0, 2 ** 32, 4096, dtype=np.uint64).astype(np.uint32)
    b64 = rng.integers(0, 2 ** 63, 4096, dtype=np.uint64) * 2 + rng.integers(0, 2, 4096, dtype=np.uint64)
    got = S.load_safetensors_from_bytes(save({"x": b32.view(np.float32), "y": b64.view(np.float64)}))
    assert np.array_equal(got["x"].view(np.uint32), b32) and np.array_equal(got["y"].view(np.uint64), b64)


def test_metadata(tmp_path):
    # safetensors_with_metadata / safetensors_no_metadata (:5009-5040)
    p = tmp_path / "m.safetensors"
    p.write_bytes(save({"w": np.ones(2, np.float32)}, metadata={"format": "pt", "author": "ü"}))
    md = S.load_safetensors_metadata(p)
    assert len(md) == 2 and md["format"] == "pt" and md.get("author") == "ü" and "missing" not in md
    p.write_bytes(save({"w": np.ones(2, np.float32)}))
    assert S.load_safetensors_metadata(p) is None


def test_rejections_of_the_reference(tmp_path):
    # safetensors_corrupt_bytes (:5057), the payload-width and dtype cases (:5079-5133)
    for data, needle in ((b"not a safetensors file", "safetensors"),
                         (_malformed("F32", [1], [0, 0, 128, 63, 255]), "safetensors"),
                         (_malformed("F16", [1], [0, 60, 1]), "safetensors"),
                         (_malformed("I64", [1], struct.pack("<q", 42)), "integer/bool SafeTensors dtype"),
                         (_malformed("BOOL", [1], [1]), "integer/bool SafeTensors dtype"),
                         (_malformed("U8", [2], [1, 2]), "unsupported SafeTensors dtype"),
                         (b"", "HeaderTooSmall")):
        with pytest.raises(HipError) as e:
            S.load_safetensors_from_bytes(data)
        assert e.value.kind == "Corrupt" and needle in e.value.message
    with pytest.raises(HipError) as e:
        S.load_safetensors(tmp_path / "does_not_exist.safetensors")
    assert e.value.kind == "Io"
    with pytest.raises(HipError) as e:
        S.load_safetensors(tmp_path)  # a directory
    assert e.value.kind == "Io"
    f = S.SafeTensorsFile(save({"w": np.ones(3, np.float32)}))
    with pytest.raises(HipError) as e:
        f.read("nope")
    assert e.value.kind == "InvalidArgument"


def test_container_rules():
    """Each rule of the container on its own: holes, overlaps, order, sizes, header bounds, JSON forms."""
    one = {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}
    ok = _container({"a": one, "b": {"dtype": "F16", "shape": [2, 1], "data_offsets": [8, 12]}}, bytes(12))
    assert list(S.load_safetensors_from_bytes(ok)) == ["a", "b"]
    bad = [
        _container({"a": one, "b": {"dtype": "F16", "shape": [2], "data_offsets": [9, 13]}}, bytes(13)),   # hole
        _container({"a": one, "b": {"dtype": "F16", "shape": [2], "data_offsets": [6, 10]}}, bytes(10)),   # overlap
        _container({"a": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, bytes(12)),             # does not start at 0
        _container({"a": {"dtype": "F32", "shape": [2], "data_offsets": [8, 0]}}, bytes(8)),               # end before begin
        _container({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, bytes(8)),               # numel * width != span
        _container({"a": one}, bytes(9)),                                                                   # trailing byte
        _container({"a": one}, bytes(7)),                                                                   # truncated buffer
        _container({"a": {"dtype": "F32", "shape": [2 ** 40, 2 ** 40], "data_offsets": [0, 8]}}, bytes(8)),  # element count overflows
        _container({"a": {"dtype": "F32", "shape": [2]}}, bytes(8)),                                        # missing field
        _container({"a": {"dtype": "F32", "shape": [2.0], "data_offsets": [0, 8]}}, bytes(8)),             # non-integer extent
        _container({"a": {"dtype": "F32", "shape": [-2], "data_offsets": [0, 8]}}, bytes(8)),
        _container({"a": {"dtype": "F33", "shape": [2], "data_offsets": [0, 8]}}, bytes(8)),               # unknown dtype name
        _container({"__metadata__": {"k": 1}}, b""),                                                        # metadata values are strings
        struct.pack("<Q", 5) + b"[1,2]",                                                                    # header is not an object
        struct.pack("<Q", 100_000_001) + b"{}",                                                             # header too large
        struct.pack("<Q", 50) + b"{}",                                                                      # header longer than the file
        struct.pack("<Q", 4) + b"{}\xff\xfe",                                                               # not UTF-8
        struct.pack("<Q", 2) + b"{}" + b"\x00",                                                             # bytes nobody owns
    ]
    for i, data in enumerate(bad):
        with pytest.raises(HipError) as e:
            S.load_safetensors_from_bytes(data)
        assert e.value.kind == "Corrupt", i
        with pytest.raises(Exception):
            deserialize(data)  # the crate agrees on every one of them
    # accepted forms: padding spaces after the header object, escapes in names, fields the record does not name
    h = json.dumps({"té\\n": {"dtype": "F64", "extra": {"x": [1, 2.5e3, None, True]}, "shape": [], "data_offsets": [0, 8]}}).encode() + b"   "
    data = struct.pack("<Q", len(h)) + h + struct.pack("<d", 2.5)
    got = S.load_safetensors_from_bytes(data)
    assert list(got) == ["té\\n"] and got["té\\n"].shape == () and float(got["té\\n"]) == 2.5
    assert [n for n, _ in deserialize(data)] == ["té\\n"]


def test_fuzz_corpus_seeds_match_the_crate(vectors):
    """fuzz_corpus_safetensors_does_not_panic (:4907-4942) reads these seeds; here every verdict, tensor list and byte is
    held to the crate's, with the loader's own restriction to four dtypes on top."""
    seeds = vectors["safetensors_corpus"]
    assert len(seeds) >= 15
    for c in seeds:
        _compare_with_crate(bytes.fromhex(c["hex"]), c["name"])


def _compare_with_crate(data, tag):
    try:
        ref = deserialize(data)
        want = sorted((n, d["dtype"], tuple(d["shape"]), bytes(d["data"])) for n, d in ref) if all(d["dtype"] in READABLE for _, d in ref) else None
    except Exception:
        want = None
    try:
        with S.SafeTensorsFile(data) as f:
            got = sorted((n, S.DTYPE_NAMES[f.info(n)[0]], f.info(n)[1], f.read(n).tobytes()) for n in f.names())
    except HipError as e:
        assert e.kind == "Corrupt", tag
        got = None
    assert got == want, tag


def test_differential_against_the_crate():
    """4000 seeded containers, valid and damaged (header bytes overwritten, lengths and offsets shifted, files cut or
    extended): same verdict, same tensors, same bytes as safetensors 0.8.0."""
    rng = random.Random(20250)
    for it in range(4000):
        hdr, off, payload = {}, 0, b""
        for i in range(rng.randint(0, 4)):
            dt = rng.choice(list(READABLE) + (["I64", "U8", "BOOL"] if rng.random() < 0.1 else []))
            w = READABLE.get(dt) or {"I64": 8, "U8": 1, "BOOL": 1}[dt]
            shape = [rng.randint(0, 4) for _ in range(rng.randint(0, 3))]
            nb = int(np.prod(shape, dtype=np.int64)) * w
            hdr["t%d" % i] = {"dtype": dt, "shape": shape, "data_offsets": [off, off + nb]}
            off += nb
            payload += bytes(rng.getrandbits(8) for _ in range(nb))
        if rng.random() < 0.3:
            hdr["__metadata__"] = {"k": "v", "é": "é\n"}
        h = json.dumps(hdr, ensure_ascii=rng.random() < 0.5).encode() + b" " * (rng.randint(1, 9) if rng.random() < 0.3 else 0)
        b = bytearray(struct.pack("<Q", len(h)) + h + payload)
        r = rng.random()
        if 0.25 <= r < 0.45 and h:
            for _ in range(rng.randint(1, 3)):
                b[8 + rng.randrange(len(h))] = rng.choice(b'{}[]",:0123456789 eE.-\\u' + bytes([rng.getrandbits(8)]))
        elif 0.45 <= r < 0.6:
            b = b[:rng.randrange(len(b) + 1)]
        elif 0.6 <= r < 0.7:
            b += bytes(rng.randint(1, 5))
        elif 0.7 <= r < 0.85:
            b[:8] = struct.pack("<Q", (struct.unpack("<Q", b[:8])[0] + rng.choice([-2, -1, 1, 2, 1 << 20, 1 << 40, 1 << 63])) % (1 << 64))
        elif r >= 0.85:
            digits = [i for i in range(8, 8 + len(h)) if 48 <= b[i] <= 57]
            if digits:
                i = rng.choice(digits)
                b[i] = 48 + (b[i] - 48 + rng.randint(1, 9)) % 10
        _compare_with_crate(bytes(b), "case %d" % it)
