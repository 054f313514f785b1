"""Writes tests/golden/reference_vectors.json: the known-answer vectors the reference itself holds
for the transformer forward path, as DATA (inputs and expected outputs only).

Sources (read as text / JSON from the reference checkout; nothing is imported or executed):
  * crates/ft-conformance/fixtures/*.json          conformance cases (copied case by case)
  * artifacts/optimization/golden_outputs/*.txt    golden output text files (numbers parsed out)
  * artifacts/perf/frankentorch-kgs4.54/pass1_golden_gemm_bt.digest_lines   f64 GEMM checksums
  * fuzz/corpus/ft_serialize_safetensors/*         seed containers of the safetensors fuzz target (hex)
  * fuzz/corpus/ft_serialize_state_dict/*          seed containers of the native state-dict fuzz target (hex)
  * artifacts/optimization/golden_outputs/ft_serialize_*.txt   encoded native state dicts (hex) with their keys, dtypes,
                                                   shapes and value bit patterns
  * in-source #[test] literals of crates/ft-kernel-cpu/src/lib.rs, transcribed by hand below with
    their line numbers (the literal input vectors and the asserted outputs)

Run from the repo root in the build container: python tests/golden/make_fixtures.py
The JSON it writes is committed; tests never read the reference checkout.
"""
from __future__ import annotations

import json
import os
import re
import sys

REF = os.environ.get("FT_REFERENCE_ROOT", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "reference_vectors.json")

CONFORMANCE = {
    "tensor_unary_cases.json": ["tensor_gelu_basic"],
    "tensor_normalize_cases.json": ["softmax_1d_dim0", "softmax_2d_dim1", "log_softmax_1d_dim0", "log_softmax_2d_dim1"],
    "tensor_binary_cases.json": ["tensor_add_basic", "tensor_matmul_basic"],
    "tensor_linalg_cases.json": ["matmul_2x2", "matmul_2x3_3x2"],
    "tensor_indexing_cases.json": ["index_select_dim0", "index_select_dim1"],
}
KEEP_KEYS = ("name", "op", "input", "shape", "dim", "lhs", "rhs", "lhs_shape", "rhs_shape", "input_shape", "index",
             "index_shape", "expected_output", "expected_shape", "tolerance")

# Literals transcribed from #[test] bodies of crates/ft-kernel-cpu/src/lib.rs ("KC").
IN_SOURCE = [
    {"name": "matmul_tensor_contiguous_returns_expected_values", "source": "KC:55234-55243", "op": "matmul",
     "dtype": "f64", "lhs": [1, 2, 3, 4, 5, 6], "lhs_shape": [2, 3], "rhs": [7, 8, 9, 10, 11, 12], "rhs_shape": [3, 2],
     "expected_output": [58, 64, 139, 154]},
    {"name": "bmm_respects_storage_offsets_and_batch_order", "source": "KC:53365-53400", "op": "bmm", "dtype": "both",
     "lhs": [99, 1, 2, 3, 4, 5, 6, 7, 8], "lhs_shape": [2, 2, 2], "lhs_offset": 1,
     "rhs": [77, 88, 10, 11, 12, 13, 14, 15, 16, 17], "rhs_shape": [2, 2, 2], "rhs_offset": 2,
     "expected_output": [34, 37, 78, 85, 166, 177, 226, 241]},
    {"name": "bmm_f32_4x4_with_offsets", "source": "KC:53403-53437", "op": "bmm_pattern", "dtype": "f32", "batch": 260,
     "lhs_offset": 3, "rhs_offset": 5, "lhs_fill": 99.0, "rhs_fill": 77.0,
     "lhs_pattern": "(i % 7) - 3", "rhs_pattern": "(i % 11) - 5", "expected": "exact small-integer products"},
    {"name": "addmm_accepts_contiguous_operands", "source": "KC:55392-55415", "op": "addmm", "dtype": "f64",
     "input": [1, 1, 1, 1], "input_shape": [2, 2], "mat1": [1, 2, 3, 4], "mat1_shape": [2, 2], "mat2": [5, 6, 7, 8],
     "mat2_shape": [2, 2], "beta": 1.0, "alpha": 1.0, "expected_output": [20, 23, 44, 51]},
    {"name": "addmm_alpha_zero_f64", "source": "KC:55418-55437", "op": "addmm", "dtype": "f64", "input": [10, -4],
     "input_shape": [2], "mat1": [1, 2, 3, 4, 5, 6], "mat1_shape": [2, 3], "mat2": [7, 8, 9, 10, 11, 12],
     "mat2_shape": [3, 2], "beta": 0.5, "alpha": 0.0, "expected_output": [5, -2, 5, -2]},
    {"name": "addmm_alpha_zero_f32", "source": "KC:55462-55481", "op": "addmm", "dtype": "f32",
     "input": [1.0, -2.0, 3.5, -4.5], "input_shape": [2, 2], "mat1": [1, 1, 1, 1, 1, 1], "mat1_shape": [2, 3],
     "mat2": [2, 2, 2, 2, 2, 2], "mat2_shape": [3, 2], "beta": -2.0, "alpha": 0.0, "expected_output": [-2, 4, -7, 9]},
    {"name": "addmm_alpha_zero_still_validates_mat1", "source": "KC:55439-55460", "op": "addmm_error", "dtype": "f64",
     "input": [10, -4], "input_shape": [2], "mat1": [1, 2, 3, 4, 5, 6], "mat1_shape": [2, 3], "mat1_offset": 1,
     "mat2": [7, 8, 9, 10, 11, 12], "mat2_shape": [3, 2], "beta": 0.5, "alpha": 0.0,
     "expected_error": {"kind": "InsufficientStorage", "side": "mat1", "needed": 7, "available": 6}},
    {"name": "gelu_returns_expected_values", "source": "KC:58389-58396", "op": "gelu_bounds", "dtype": "f64",
     "input": [0.0, -5.0, 5.0], "expected_near": [0.0, 0.0, 5.0], "abs_tol": [1e-10, 0.01, 0.01]},
    {"name": "inf_in_softmax_produces_nan", "source": "KC:65294-65304", "op": "softmax_all_nan", "dtype": "f64",
     "input": ["-inf", 0.0, "inf"], "shape": [3], "dim": 0},
    {"name": "softmax_with_finite_extremes", "source": "KC:65307-65317", "op": "softmax_extremes", "dtype": "f64",
     "input": [-1000.0, 0.0, 1000.0], "shape": [3], "dim": 0, "expected_first": 0.0, "expected_last": 1.0},
    {"name": "argmax_dim_reduces_along_dim0", "source": "KC:56470-56477", "op": "argmax", "dtype": "f64",
     "input": [1, 5, 3, 4, 2, 6], "shape": [2, 3], "dim": 0, "expected_output": [1, 0, 1]},
    {"name": "argmax_dim_reduces_along_dim1", "source": "KC:56480-56487", "op": "argmax", "dtype": "f64",
     "input": [1, 5, 3, 4, 2, 6], "shape": [2, 3], "dim": 1, "expected_output": [1, 2]},
    {"name": "argmax_dim_1d_reduces_to_scalar", "source": "KC:56914-56919", "op": "argmax", "dtype": "f64",
     "input": [1, 4, 2, 3], "shape": [4], "dim": 0, "expected_output": [1]},
    {"name": "argmax_dim_invalid_dim", "source": "KC:56490-56498", "op": "argmax_error", "dtype": "f64",
     "input": [1, 2, 3, 4, 5, 6], "shape": [2, 3], "dim": 2,
     "expected_error": {"kind": "InvalidDimension", "dim": 2, "ndim": 2}},
    {"name": "argmax_over_empty_dim", "source": "KC:56501-56510", "op": "argmax_error", "dtype": "f64", "input": [],
     "shape": [3, 0], "dim": 1, "expected_error": {"kind": "EmptyReductionDim", "dim": 1}},
    {"name": "index_select_invalid_dim", "source": "KC:57834-57839", "op": "index_select_error", "dtype": "f64",
     "input": [1, 2, 3, 4, 5, 6], "shape": [2, 3], "dim": 5, "index": [0.0]},
    {"name": "index_select_out_of_bounds", "source": "KC:57842-57847", "op": "index_select_error", "dtype": "f64",
     "input": [1, 2, 3, 4, 5, 6], "shape": [2, 3], "dim": 0, "index": [5.0]},
    {"name": "index_select_nan_index", "source": "KC:57850-57855", "op": "index_select_error", "dtype": "f64",
     "input": [1, 2, 3, 4], "shape": [2, 2], "dim": 0, "index": ["nan"]},
    {"name": "index_select_huge_index", "source": "KC:57858-57863", "op": "index_select_error", "dtype": "f64",
     "input": [1, 2, 3, 4], "shape": [2, 2], "dim": 0, "index": [1.0e300]},
    {"name": "index_select_negative_index", "source": "KC:57866-57875", "op": "index_select_error", "dtype": "f64",
     "input": [1, 2, 3, 4, 5, 6], "shape": [3, 2], "dim": 0, "index": [-1.0]},
    {"name": "gelu_tanh_module_matches_torch", "source": "crates/ft-nn/src/lib.rs:21985-22004", "op": "gelu_tanh", "dtype": "f64",
     "input": [-1.0, 0.5, 1.0, 2.0],
     "expected_output": [-0.15880800939172324, 0.34571400982514394, 0.8411919906082768, 1.954597694087775], "abs_tol": 1e-9},
    {"name": "matmul_unit_vector_dot_k10001", "source": "KC:53274-53310", "op": "matmul_unit_dot", "dtype": "f64",
     "k": 10001, "expected": 1.0, "abs_tol": 1e-14},
]


def conformance_cases():
    out = []
    fx = os.path.join(REF, "crates", "ft-conformance", "fixtures")
    for fname, names in CONFORMANCE.items():
        data = json.load(open(os.path.join(fx, fname)))
        cases = data["cases"] if isinstance(data, dict) else data
        for c in cases:
            if c.get("name") in names:
                d = {k: c[k] for k in KEEP_KEYS if k in c}
                d["source"] = "crates/ft-conformance/fixtures/" + fname
                out.append(d)
    return out


def _floats(text):
    return [float(x) for x in re.findall(r"-?\d+\.\d+(?:e[+-]?\d+)?|-?\d+\.\d*", text)]


def golden_texts():
    g = os.path.join(REF, "artifacts", "optimization", "golden_outputs")
    out = {}
    t = open(os.path.join(g, "softmax_rows_pass10.txt")).read()
    rows = []
    for line in t.splitlines():
        m = re.match(r"row \d+ input \[(.*?)\] -> \[(.*?)\]", line)
        if m:
            rows.append({"input": _floats(m.group(1)), "expected_output": _floats(m.group(2))})
    out["softmax_rows_pass10"] = {"source": "artifacts/optimization/golden_outputs/softmax_rows_pass10.txt", "dtype": "f64",
                                  "rows": rows}
    t = open(os.path.join(g, "ft_kernel_cpu_softmax_parallel_frankentorch-wcoo.txt")).read()
    sec = {}
    cur = None
    meta = {}
    for line in t.splitlines():
        line = line.strip()
        m = re.match(r"(\w+)=(\d+)$", line)
        if m:
            meta[m.group(1)] = int(m.group(2))
        elif line.endswith("_bits:"):
            cur = line[:-1]
            sec[cur] = {}
        elif cur and re.match(r"\d+: 0x[0-9a-f]+", line):
            i, b = line.split(": ")
            sec[cur][i] = b
    out["softmax_parallel_bits"] = {"source": "artifacts/optimization/golden_outputs/ft_kernel_cpu_softmax_parallel_frankentorch-wcoo.txt",
                                    "note": "uniform rows: every softmax output is exactly 0.5", "meta": meta, "bits": sec}
    t = open(os.path.join(g, "bmm_batch_pass13.txt")).read()
    out["bmm_batch_pass13"] = {"source": "artifacts/optimization/golden_outputs/bmm_batch_pass13.txt",
                               "values": _floats(re.search(r"values=\[(.*?)\]", t).group(1))}
    t = open(os.path.join(g, "elementwise_simd_pass7.txt")).read()
    out["elementwise_simd_pass7"] = {"source": "artifacts/optimization/golden_outputs/elementwise_simd_pass7.txt",
                                     "add_f64": _floats(re.search(r"add_tensor_contiguous_f64 values: \[(.*?)\]", t).group(1)),
                                     "simd_tail_add_f64": _floats(re.search(r"simd_tail_add_f64 values: \[(.*?)\]", t).group(1))}
    t = open(os.path.join(g, "ft_kernel_cpu_gemm_crossover_frankentorch-kgs4-4.txt")).read()
    out["gemm_crossover"] = {"source": "artifacts/optimization/golden_outputs/ft_kernel_cpu_gemm_crossover_frankentorch-kgs4-4.txt",
                             "f64_2x3_times_3x2": _floats(re.search(r"f64_2x3_times_3x2=\[(.*?)\]", t).group(1)),
                             "f32_2x3_times_3x2": _floats(re.search(r"f32_2x3_times_3x2=\[(.*?)\]", t).group(1))}
    t = open(os.path.join(REF, "artifacts", "perf", "frankentorch-kgs4.54", "pass1_golden_gemm_bt.digest_lines")).read()
    sums = []
    for line in t.splitlines():
        m = re.match(r"(\d+)x(\d+)x(\d+) (bt_)?fnv1a=\w+ (?:bt_)?sum=(\S+)", line)
        if m:
            sums.append({"m": int(m.group(1)), "k": int(m.group(2)), "n": int(m.group(3)), "bt": bool(m.group(4)),
                         "sum": float(m.group(5))})
    out["gemm_f64_checksums"] = {
        "source": "artifacts/perf/frankentorch-kgs4.54/pass1_golden_gemm_bt.digest_lines",
        "generator": "crates/ft-kernel-cpu/examples/gemm_golden.rs:8-9: a[i] = sin(0.001 i) over m*k, b[i] = cos(0.0017 i) over k*n "
                     "(bt: the same b values read as [n, k]); sum = plain f64 sum of the output printed with 12 decimals",
        "sums": sums}
    return out


def safetensors_corpus():
    """The seed inputs of the reference's safetensors fuzz target (fuzz/corpus/ft_serialize_safetensors/*, which its unit
    test fuzz_corpus_safetensors_does_not_panic reads): small binary containers, kept as hex strings."""
    d = os.path.join(REF, "fuzz", "corpus", "ft_serialize_safetensors")
    return [{"name": n, "hex": open(os.path.join(d, n), "rb").read().hex()} for n in sorted(os.listdir(d))]


def native_state_dict():
    """Known answers for the native ("FTSV") state-dict container: the reference's golden encodings with the tensors
    they hold (artifacts/optimization/golden_outputs/ft_serialize_*save*.txt: `encoded_hex=` is the container, every
    `key=... dtype=... shape=[...] bits=a,b,...` line one tensor's raw element bit patterns), the decode summary of its
    generated many-small-tensors payload (ft_serialize_decode_pass19.txt; the payload itself is built by the test
    helper native_many_small_f64_payload, crates/ft-serialize/src/lib.rs:3847-3870, restated in the test that uses
    it), and the seed inputs of its fuzz target (fuzz/corpus/ft_serialize_state_dict/*, read by its unit test
    fuzz_corpus_state_dict_does_not_panic :4945-4971, which only asks for no panic)."""
    gdir = os.path.join(REF, "artifacts", "optimization", "golden_outputs")
    encodings = []
    for fn in sorted(os.listdir(gdir)):
        if not (fn.startswith("ft_serialize_") and "save" in fn):
            continue
        text = open(os.path.join(gdir, fn)).read()
        hexs = re.search(r"^encoded_hex=([0-9a-f]+)$", text, re.M).group(1)
        total = int(re.search(r"^total_len=(\d+)$", text, re.M).group(1))
        tensors = []
        for m in re.finditer(r"^key=(\S+) dtype=(\w+) shape=\[([^\]]*)\] bits=([0-9a-f,]*)$", text, re.M):
            shape = [int(v) for v in m.group(3).split(",") if v.strip()]
            tensors.append({"key": m.group(1), "dtype": m.group(2), "shape": shape, "bits": [b for b in m.group(4).split(",") if b]})
        encodings.append({"source": "artifacts/optimization/golden_outputs/" + fn, "total_len": total, "encoded_hex": hexs, "tensors": tensors})
    summary = open(os.path.join(gdir, "ft_serialize_decode_pass19.txt")).read()
    decoded = []
    for m in re.finditer(r"^key=(\S+) dtype=(\w+) shape=\[([^\]]*)\] values=\[([^\]]*)\]$", summary, re.M):
        decoded.append({"key": m.group(1), "dtype": m.group(2), "shape": [int(v) for v in m.group(3).split(",") if v.strip()],
                        "values": [float(v) for v in m.group(4).split(",") if v.strip()]})
    d = os.path.join(REF, "fuzz", "corpus", "ft_serialize_state_dict")
    corpus = [{"name": n, "hex": open(os.path.join(d, n), "rb").read().hex()} for n in sorted(os.listdir(d))]
    return {"encodings": encodings,
            "decode_pass19": {"source": "artifacts/optimization/golden_outputs/ft_serialize_decode_pass19.txt",
                              "generator": "4 tensors 'layer.%04d.weight', rank 1, width 4, F64, value = tensor_index * 4 + position",
                              "tensors": decoded},
            "fuzz_corpus": corpus}


def main():
    if not os.path.isdir(REF):
        sys.exit("reference checkout not found at %s" % REF)
    doc = {"conformance": conformance_cases(), "in_source": IN_SOURCE, "golden_text": golden_texts(),
           "safetensors_corpus": safetensors_corpus(), "native_state_dict": native_state_dict()}
    with open(OUT, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
