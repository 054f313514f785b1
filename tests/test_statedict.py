"""The native state-dict ("FTSV") reader on the host (no GPU needed).

Three layers: (1) the checker's plain-Python restatement of load_state_dict_from_bytes (oracle.load_state_dict_from_bytes)
is pinned by what the reference itself holds: its golden encodings with the tensors they contain, its decode summary, and
the byte strings and error texts of its own unit tests (crates/ft-serialize/src/lib.rs:4105-4660, 5137-5290), each
rebuilt here byte by byte from the format description; (2) the library's reader must agree with those same known answers;
(3) the library and the checker must agree, verdict for verdict and byte for byte, on the reference's fuzz-corpus seeds
and on thousands of seeded damaged containers."""
import random
import struct

import numpy as np
import pytest

from frankentorch_amd import serialize as S
from frankentorch_amd.core import HipError

u64 = lambda v: struct.pack("<Q", v)
u32 = lambda v: struct.pack("<I", v)
HEAD = b"FTSV" + u32(1)
NP_OF = {"F64": (np.float64, np.uint64, 0), "F32": (np.float32, np.uint32, 1), "F16": (np.float16, np.uint16, 2), "BF16": (np.uint16, np.uint16, 3)}


def tensor(key: bytes, shape, tag: int, payload: bytes) -> bytes:
    return u64(len(key)) + key + u64(len(shape)) + b"".join(u64(d) for d in shape) + bytes([tag]) + payload


def lib_verdict(data):
    """("ok", {key: (tag, shape, bytes)}) or (kind, message) from the library, through the C ABI itself (a damaged
    container may hold a zero-element tensor with a dimension numpy cannot represent)."""
    import ctypes as C

    from frankentorch_amd import _lib

    L = _lib.load()
    try:
        with S.StateDictFile(data) as f:
            out = {}
            for n in f.names():
                info = S.TensorInfo()
                rc = L.fth_statedict_info(f._h, n.encode(), C.byref(info))
                if rc != 0:  # more than 8 dimensions: the info structure cannot hold the shape
                    out[n] = None
                    continue
                buf = C.create_string_buffer(max(int(info.byte_len), 1))
                assert L.fth_statedict_read(f._h, n.encode(), buf, int(info.byte_len)) == 0
                out[n] = (info.dtype, tuple(int(info.shape[i]) for i in range(info.ndim)), buf.raw[:int(info.byte_len)])
            return "ok", out
    except HipError as e:
        return e.kind, e.message


def oracle_verdict(oracle, data):
    try:
        return "ok", oracle.load_state_dict_from_bytes(data)
    except oracle.StateDictError as e:
        return e.kind, e.reason


def both(oracle, data):
    """Runs both readers, asserts that they agree, returns the common verdict."""
    ok, oo = lib_verdict(data), oracle_verdict(oracle, data)
    if oo[0] == "ok" and any("\0" in k for k in oo[1]):
        # the one documented deviation: a key with a NUL byte cannot be named through the C interface
        assert ok[0] == "Corrupt" and "NUL byte" in ok[1]
        return "Corrupt", ok[1]
    assert ok[0] == oo[0], (ok, oo)
    if ok[0] == "ok":
        assert list(ok[1]) == list(oo[1])
        for k in ok[1]:
            assert ok[1][k] is None and len(oo[1][k][1]) > 8 or ok[1][k] == oo[1][k], k
    elif ok[0] == "Corrupt":
        assert ok[1] == oo[1][:199].split("\0")[0] or "NUL byte" in ok[1]  # a C string: 199 characters at most, ends at a NUL
    return oo


# ---- (1) + (2): the reference's known answers ----------------------------------------------------
def test_golden_encodings_decode_to_the_tensors_the_reference_lists(vectors, oracle):
    for enc in vectors["native_state_dict"]["encodings"]:
        data = bytes.fromhex(enc["encoded_hex"])
        # (total_len is not checked: ft_serialize_f64_save_bulk_frankentorch-whlp.txt states 162 beside a 158-byte encoding,
        # the same bytes as its sibling file, which states 158)
        kind, got = both(oracle, data)
        assert kind == "ok" and list(got) == [t["key"] for t in enc["tensors"]], enc["source"]
        for t in enc["tensors"]:
            np_t, bits_t, tag = NP_OF[t["dtype"]]
            want = np.array([int(b, 16) for b in t["bits"]], dtype=bits_t)
            gtag, gshape, gbytes = got[t["key"]]
            assert gtag == tag and list(gshape) == t["shape"] and np.array_equal(np.frombuffer(gbytes, dtype=bits_t), want), (enc["source"], t["key"])
        # and the checker's writer reproduces the reference's bytes exactly (encode_state_dict_to_bytes, :4493-4510)
        rebuilt = {}
        for t in enc["tensors"]:
            np_t, bits_t, tag = NP_OF[t["dtype"]]
            arr = np.array([int(b, 16) for b in t["bits"]], dtype=bits_t).reshape(t["shape"])
            rebuilt[t["key"]] = (arr, "bf16") if t["dtype"] == "BF16" else arr.view(np_t)
        assert oracle.encode_state_dict(rebuilt) == data, enc["source"]


def test_decode_summary_of_many_small_tensors(vectors, oracle):
    # native_many_small_f64_payload(4, 4), crates/ft-serialize/src/lib.rs:3847-3870
    want = vectors["native_state_dict"]["decode_pass19"]["tensors"]
    data = HEAD + u64(4)
    for i in range(4):
        data += tensor(b"layer.%04d.weight" % i, [4], 0, np.arange(4 * i, 4 * i + 4, dtype=np.float64).tobytes())
    kind, got = both(oracle, data)
    assert kind == "ok" and list(got) == [t["key"] for t in want]
    for t in want:
        tag, shape, raw = got[t["key"]]
        assert tag == 0 and list(shape) == t["shape"] and np.frombuffer(raw, np.float64).tolist() == t["values"]
    host = S.load_state_dict_from_bytes(data)
    assert [host[t["key"]].tolist() for t in want] == [t["values"] for t in want]


def test_round_trips_of_the_reference(tmp_path, oracle):
    # save_load_empty_state_dict :4105, f16 scalar under an empty key :4174, mixed dtypes :5198, zero elements :5250, rank 6 :5266
    assert both(oracle, HEAD + u64(0)) == ("ok", {})
    kind, got = both(oracle, HEAD + u64(1) + tensor(b"", [], 2, np.float16(1.5).tobytes()))
    assert kind == "ok" and got[""] == (2, (), np.float16(1.5).tobytes())
    bf = (np.array([1.5, -2.0, 0.25], np.float32).view(np.uint32) >> 16).astype(np.uint16)   # save_load_bf16_tensor :4334
    mixed = {"w64": np.array([[1.0, -2.5], [3.25, 4.0]]), "w32": np.array([0.5, 1.5, -3.0], np.float32),
             "w16": np.array([1.0, -0.5], np.float16), "wb": (bf, "bf16"), "empty": np.zeros((3, 0, 2), np.float32),
             "deep": np.arange(64, dtype=np.float64).reshape(2, 2, 2, 2, 2, 2)}
    data = oracle.encode_state_dict(mixed)
    kind, got = both(oracle, data)
    assert kind == "ok" and list(got) == sorted(mixed)
    p = tmp_path / "state.ftsv"
    p.write_bytes(data)
    host = S.load_state_dict(p)
    assert list(host) == sorted(mixed)
    for k, v in mixed.items():
        arr = v[0] if isinstance(v, tuple) else v
        assert host[k].dtype == arr.dtype and host[k].shape == arr.shape and host[k].tobytes() == arr.tobytes(), k
    assert S.bf16_to_f32(host["wb"]).tolist() == [1.5, -2.0, 0.25]


def test_bit_patterns_survive(oracle):
    """prop_native_f64 / f32 / f16_bf16_roundtrip_preserves_all_bit_patterns (:3622-3720): NaN payloads, infinities, subnormals."""
    rng = np.random.default_rng(5)
    b64 = rng.integers(0, 2 ** 63, 2048, dtype=np.uint64) * 2 + rng.integers(0, 2, 2048, dtype=np.uint64)
    b32 = rng.integers(0, 2 ** 32, 2048, dtype=np.uint64).astype(np.uint32)
    b16 = rng.integers(0, 2 ** 16, 2048, dtype=np.uint64).astype(np.uint16)
    host = S.load_state_dict_from_bytes(oracle.encode_state_dict({"a": b64.view(np.float64), "b": b32.view(np.float32), "c": b16.view(np.float16), "d": (b16, "bf16")}))
    assert np.array_equal(host["a"].view(np.uint64), b64) and np.array_equal(host["b"].view(np.uint32), b32)
    assert np.array_equal(host["c"].view(np.uint16), b16) and np.array_equal(host["d"], b16)


def test_every_rejection_the_reference_tests(oracle):
    w = lambda payload, shape=(1,), tag=0, key=b"w": tensor(key, list(shape), tag, payload)
    one = np.float64(1.0).tobytes()
    cases = [
        (b"NOPE0000", "InvalidMagic", ""),                                                        # load_invalid_magic :4513
        (b"FTS", "InvalidMagic", ""),
        (b"", "InvalidMagic", ""),
        (b"FTSV", "Corrupt", "truncated u32"),                                                    # load_truncated_file :4520
        (b"FTSV" + u32(99), "UnsupportedVersion", ""),                                            # load_unsupported_version :4541
        (HEAD, "Corrupt", "truncated u64"),
        (HEAD + u64(1) + u64(5) + b"abcde" + u64(2), "Corrupt", "truncated shape data for tensor 'abcde'"),   # :4527
        (HEAD + u64(1) + w(b"\0" * 31, (4,)), "Corrupt", "truncated f64 data"),                    # :4316
        (HEAD + u64(1) + w(one) + b"junk", "Corrupt", "trailing bytes after state dict payload: remaining=4"),  # :4615
        (HEAD + u64(2) + b"\0" * 20, "Corrupt", "claimed 2 tensors but only 20 bytes remain (min 17 per tensor)"),  # :4628
        (HEAD + u64(2) + w(one) + w(np.float64(2.0).tobytes()), "Corrupt", "duplicate tensor key in native state dict: 'w'"),  # :4641
        (HEAD + u64(1) + tensor(b"x", [2 ** 64 - 1, 2], 0, b""), "Corrupt", "shape overflow in native state dict tensor 'x'"),  # :5137
        (HEAD + u64(2 ** 64 - 1), "Corrupt", "claimed 18446744073709551615 tensors but only 0 bytes remain (min 17 per tensor)"),  # :5161
        (HEAD + u64(1) + tensor(b"y", [(2 ** 64 - 1) // 4], 0, b""), "Corrupt", "byte count overflow for f64 tensor 'y'"),  # :5174
        # the remaining branches of the loader, one each
        (HEAD + u64(1) + u64(30) + b"k" * 20, "Corrupt", "truncated key data"),
        (HEAD + u64(1) + u64(2 ** 64 - 8) + b"k" * 24, "Corrupt", "key length overflow"),
        (HEAD + u64(1) + u64(2) + b"\xff\xfe" + u64(0) + b"\0", "Corrupt", "invalid UTF-8 in key"),
        (HEAD + u64(1) + u64(1) + b"k" + u64(1) + u64(1), "Corrupt", "truncated dtype"),
        (HEAD + u64(1) + w(one, tag=4), "Corrupt", "unknown dtype tag: 4"),
        (HEAD + u64(1) + w(b"\0" * 3, tag=1), "Corrupt", "truncated f32 data"),
        (HEAD + u64(1) + w(b"\0", tag=2), "Corrupt", "truncated f16 data"),
        (HEAD + u64(1) + w(b"\0", tag=3), "Corrupt", "truncated bf16 data"),
        (HEAD + u64(1) + u64(1) + b"k" + u64(3) + u64(1) * 2 + b"\0" * 7, "Corrupt", "truncated shape data for tensor 'k'"),
        (HEAD + u64(1) + u64(10) + b"k" * 10 + b"\0" * 3, "Corrupt", "truncated u64"),
    ]
    for data, kind, reason in cases:
        got = both(oracle, data)
        assert got[0] == kind, (data, got)
        if kind == "Corrupt":
            assert got[1] == reason, (data, got)
    # the payload of UnsupportedVersion
    with pytest.raises(HipError) as ei:
        S.StateDictFile(b"FTSV" + u32(99))
    assert ei.value.kind == "UnsupportedVersion" and "version 99 (max supported: 1)" in ei.value.message
    with pytest.raises(HipError) as ei:
        S.load_state_dict("/nonexistent/dir/state.ftsv")
    assert ei.value.kind == "Io"


def test_version_zero_is_accepted_and_a_later_count_guard_holds(oracle):
    # version <= FT_STATE_FORMAT_VERSION passes (:1018); the count guard uses the bytes AFTER the count field (:1029-1031)
    assert both(oracle, b"FTSV" + u32(0) + u64(0))[0] == "ok"
    assert both(oracle, HEAD + u64(1) + b"\0" * 16)[0] == "Corrupt"   # 16 bytes cannot hold one tensor header
    assert both(oracle, HEAD + u64(1) + tensor(b"", [], 2, b"\0\0"))[0] == "ok"  # the most compact tensor: 17 + 2 bytes


# ---- (3): differential runs ------------------------------------------------------------------------
def test_fuzz_corpus_seeds_of_the_reference(vectors, oracle):
    verdicts = [both(oracle, bytes.fromhex(s["hex"]))[0] for s in vectors["native_state_dict"]["fuzz_corpus"]]
    assert len(verdicts) == 18 and "ok" in verdicts and "Corrupt" in verdicts


def test_seeded_damage_gives_the_same_verdicts(oracle):
    rng = random.Random(20240607)
    nrng = np.random.default_rng(11)
    seeds = []
    for _ in range(40):
        tensors = {}
        for _ in range(rng.randrange(0, 5)):
            key = "".join(rng.choice("abcwé.0123") for _ in range(rng.randrange(0, 9)))
            shape = tuple(rng.randrange(0, 4) for _ in range(rng.randrange(0, 4)))
            kind = rng.randrange(4)
            if kind == 3:
                tensors[key] = (nrng.integers(0, 65536, shape).astype(np.uint16), "bf16")
            else:
                tensors[key] = nrng.standard_normal(shape).astype((np.float64, np.float32, np.float16)[kind])
        seeds.append(oracle.encode_state_dict(tensors))
    counts = {}
    for _ in range(4000):
        b = bytearray(rng.choice(seeds))
        for _ in range(rng.randrange(1, 4)):
            op = rng.randrange(5)
            if op == 0 and b:
                b[rng.randrange(len(b))] = rng.randrange(256)
            elif op == 1 and b:
                del b[rng.randrange(len(b)):]
            elif op == 2:
                b += bytes(rng.randrange(256) for _ in range(rng.randrange(1, 9)))
            elif op == 3 and len(b) > 8:
                i = rng.randrange(len(b) - 8)
                b[i:i + 8] = struct.pack("<Q", rng.choice([0, 1, 2, 17, 2 ** 32, 2 ** 61, 2 ** 63, 2 ** 64 - 1]))
            elif op == 4 and b:
                i = rng.randrange(len(b))
                b[i:i] = bytes([rng.randrange(256)])
        kind = both(oracle, bytes(b))[0]
        counts[kind] = counts.get(kind, 0) + 1
    assert counts.get("Corrupt", 0) > 1000 and counts.get("ok", 0) > 50, counts
