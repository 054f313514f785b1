#!/usr/bin/env python3
"""Writes the generated parts of the `ft-kernel-hip` crate from the two places the C side is defined:

    include/ft_kernel_hip.h            -> src/ffi.rs   (every constant, struct and `extern "C"` function)
    frankentorch_amd/build.py          -> build.rs     (the HIP translation units and hipcc flags)
    the wrapper table below            -> src/lib.rs   (one safe function per host-slice entry point, with the
                                                         signature of the `ft_kernel_cpu` function it stands in for)

    python rust/ft-kernel-hip/generate_bindings.py            # rewrite the files in place
    python rust/ft-kernel-hip/generate_bindings.py --check    # exit 1 if a committed file is out of date

The image this was written in has no Rust toolchain, so nothing here has been through rustc; tests/test_rust_crate.py
checks what can be checked without one: every header symbol is declared in ffi.rs with the header's arity, build.rs
lists exactly the translation units the Python build links, every host-slice entry point has a wrapper, and the
committed files are what this script writes today.
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
HEADER = os.path.join(ROOT, "include", "ft_kernel_hip.h")

# ------------------------------------------------------------------------------------------------
# header -> ffi.rs
# ------------------------------------------------------------------------------------------------
SCALAR = {"int8_t": "i8", "int32_t": "i32", "int64_t": "i64", "uint64_t": "u64", "size_t": "usize", "float": "f32",
          "double": "f64", "void": "c_void", "char": "c_char", "fth_stream": "fth_stream", "fth_event": "fth_event"}
RUST_KEYWORDS = {"in", "type", "fn", "ref", "match", "mod", "move", "use", "where", "impl", "loop", "box", "as"}


def strip_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def rust_type(decl: str, known_structs) -> str:
    """`const float *`, `fth_tensor **`, `size_t` ... -> the Rust spelling."""
    decl = decl.strip()
    stars = decl.count("*")
    core = decl.replace("*", " ").split()
    is_const = "const" in core
    core = [w for w in core if w not in ("const", "struct")]
    base = core[0]
    if base in SCALAR:
        rt = SCALAR[base]
    elif base in known_structs:
        rt = base
    else:
        raise ValueError("unknown C type %r" % decl)
    for level in range(stars):
        # only the innermost pointer level of `const T **` is const; handles are always mutable
        rt = ("*const " if (is_const and level == 0) else "*mut ") + rt
    return rt


def split_param(p: str):
    """`const float *x` -> (`const float *`, `x`)."""
    m = re.match(r"^(.*?)(\w+)\s*$", p.strip(), re.S)
    return m.group(1).strip(), m.group(2)


def parse_header(path: str = HEADER):
    raw = open(path).read()
    text = strip_comments(raw)
    consts = []
    for m in re.finditer(r"enum\s*\{(.*?)\}\s*;", text, re.S):
        for item in m.group(1).split(","):
            item = item.strip()
            if item:
                name, value = [s.strip() for s in item.split("=")]
                consts.append((name, int(value, 0)))
    for m in re.finditer(r"^\s*#define\s+(FTH_\w+)\s+(\d+)\s*$", text, re.M):
        consts.append((m.group(1), int(m.group(2))))
    structs, opaque, aliases = [], [], []
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*(\w+)\s*;", text, re.S):
        fields = []
        for stmt in m.group(2).split(";"):
            stmt = " ".join(stmt.split())
            if not stmt:
                continue
            # `int64_t m, n, k` / `const float *wq, *bq` / `uint64_t shape[FTH_MAX_DIMS]`
            tm = re.match(r"^((?:const\s+)?\w+)\s+(.*)$", stmt)
            base, rest = tm.group(1), tm.group(2)
            for item in rest.split(","):
                item = item.strip()
                stars = item.count("*")
                item = item.replace("*", "").strip()
                am = re.match(r"^(\w+)\s*\[\s*(\w+)\s*\]$", item)
                if am:
                    fields.append((am.group(1), base, stars, am.group(2)))
                else:
                    fields.append((item, base, stars, None))
        structs.append((m.group(3), fields))
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s+(\w+)\s*;", text):
        if m.group(1) == m.group(2):
            opaque.append(m.group(2))
        else:
            aliases.append((m.group(2), m.group(1)))
    funcs = []
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(fth_\w+)\s*\(([^;{}()]*)\)\s*;", text):
        ret, name, args = " ".join(m.group(1).split()), m.group(2), " ".join(m.group(3).split())
        if ret.startswith("typedef") or not ret:
            continue
        params = [] if args in ("", "void") else [split_param(a) for a in args.split(",")]
        funcs.append((name, ret, params))
    return consts, structs, opaque, aliases, funcs


def write_ffi(consts, structs, opaque, aliases, funcs) -> str:
    known = {s[0] for s in structs} | set(opaque) | {a[0] for a in aliases}
    const_value = dict(consts)
    out = ["// GENERATED by generate_bindings.py from include/ft_kernel_hip.h. Do not edit: change the header and regenerate.",
           "//", "// The C ABI of libft_kernel_hip.so, declaration for declaration: status codes and tags, the plain-data structs,",
           "// the opaque handles, and every exported function.", "",
           "#![allow(non_camel_case_types, non_snake_case, dead_code, clippy::too_many_arguments)]", "",
           "use std::os::raw::{c_char, c_void};", "",
           "/// A `hipStream_t`; null selects the library's own ordered stream.", "pub type fth_stream = *mut c_void;",
           "/// A `hipEvent_t`.", "pub type fth_event = *mut c_void;", ""]
    for name, value in consts:
        ty = "usize" if name == "FTH_MAX_DIMS" else "i32"
        out.append("pub const %s: %s = %d;" % (name, ty, value))
    out.append("")
    for name, fields in structs:
        out += ["#[repr(C)]", "#[derive(Debug, Clone, Copy)]", "pub struct %s {" % name]
        for fname, base, stars, dim in fields:
            rt = rust_type(base + " " + "*" * stars, known)
            if dim is not None:
                rt = "[%s; %d]" % (rt, const_value[dim] if dim in const_value else int(dim))
            out.append("    pub %s: %s," % (fname, rt))
        out += ["}", ""]
    for name in opaque:
        out += ["/// Opaque handle owned by the library.", "#[repr(C)]", "pub struct %s {" % name, "    _private: [u8; 0],", "}", ""]
    for alias, target in aliases:
        out += ["pub type %s = %s;" % (alias, target), ""]
    out.append('#[link(name = "ft_kernel_hip")]')
    out.append('extern "C" {')
    for name, ret, params in funcs:
        args = []
        for ctype, pname in params:
            if pname in RUST_KEYWORDS:
                pname += "_"
            args.append("%s: %s" % (pname, rust_type(ctype, known)))
        r = "" if ret == "void" else " -> " + rust_type(ret, known)
        out.append("    pub fn %s(%s)%s;" % (name, ", ".join(args), r))
    out += ["}", ""]
    return "\n".join(out)


# ------------------------------------------------------------------------------------------------
# build.py -> build.rs
# ------------------------------------------------------------------------------------------------
def build_lists():
    sys.path.insert(0, ROOT)
    from frankentorch_amd import build as B

    return list(B.HIP_SOURCES), list(B.HIPCC_FLAGS)


def write_build_rs(sources, flags) -> str:
    src_list = ", ".join('"%s"' % s for s in sources)
    flag_list = ", ".join('"%s"' % f for f in flags)
    return '''// GENERATED by generate_bindings.py from frankentorch_amd/build.py (HIP_SOURCES, HIPCC_FLAGS). Do not edit.
//
// Cross-compiles every HIP translation unit for gfx950 with hipcc and links libft_kernel_hip.so into OUT_DIR. No GPU is
// needed to build. `csrc/` and `include/` are the crate's copies of frankentorch_amd/csrc and include/.
use std::{env, path::PathBuf, process::Command};

const HIP_SOURCES: &[&str] = &[%s];
const HIPCC_FLAGS: &[&str] = &[%s];

fn main() {
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "hipcc".to_string());
    let (csrc, include) = (manifest.join("csrc"), manifest.join("include"));
    let mut objects = Vec::new();
    for src in HIP_SOURCES {
        let obj = out.join(src.replace(".hip", ".o"));
        let status = Command::new(&hipcc)
            .args(HIPCC_FLAGS)
            .arg("-I").arg(&include)
            .arg("-I").arg(&csrc)
            .arg("-c").arg(csrc.join(src))
            .arg("-o").arg(&obj)
            .status()
            .expect("hipcc not found: the gfx950 kernel library cannot be built");
        assert!(status.success(), "hipcc failed on {src}");
        objects.push(obj);
    }
    let lib = out.join("libft_kernel_hip.so");
    let status = Command::new(&hipcc)
        .args(["--offload-arch=gfx950", "-shared", "-fPIC", "-o"])
        .arg(&lib)
        .args(&objects)
        .args(["-Wl,-rpath,/opt/rocm/lib", "-Wl,--no-undefined"])
        .status()
        .expect("hipcc link");
    assert!(status.success(), "linking libft_kernel_hip.so failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=ft_kernel_hip");
    println!("cargo:rerun-if-changed=csrc");
    println!("cargo:rerun-if-changed=include");
    println!("cargo:rerun-if-env-changed=HIPCC");
}
''' % (src_list, flag_list)


# ------------------------------------------------------------------------------------------------
# wrapper table -> lib.rs
# ------------------------------------------------------------------------------------------------
# One entry per host-slice entry point of the header. `sig` is the argument list and return type of the ft_kernel_cpu
# function of the same name (crates/ft-kernel-cpu/src/lib.rs at `line`; None where the reference has no such function
# yet and the wrapper is new surface), `call` the C arguments before the output arguments, `outs` the outputs as
# (binding, element type, length expression), `ret` the returned expression. {T} is f32 / f64, {S} the suffix.
FALLIBLE_SIZED = "sized"  # C call ends with (out, out_cap, &mut out_len); validates and sizes with a null output first


def _twins(name, line32, line64, **kw):
    return [dict(name=name + "_f32", T="f32", line=line32, **kw), dict(name=name + "_f64", T="f64", line=line64, **kw)]


BINARY = dict(kind=FALLIBLE_SIZED, sig="lhs: &[{T}], rhs: &[{T}], lhs_meta: &TensorMeta, rhs_meta: &TensorMeta",
              ret_ty="Result<Vec<{T}>, KernelError>",
              pre="let (lm, rm) = (flatten(lhs_meta), flatten(rhs_meta));",
              call="lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), &lm, &rm")
UNARY_DIM = dict(kind=FALLIBLE_SIZED, sig="input: &[{T}], meta: &TensorMeta, dim: usize", ret_ty="Result<Vec<{T}>, KernelError>",
                 pre="let m = flatten(meta);", call="input.as_ptr(), input.len(), &m, dim")
UNARY = dict(kind=FALLIBLE_SIZED, sig="input: &[{T}], meta: &TensorMeta", ret_ty="Result<Vec<{T}>, KernelError>",
             pre="let m = flatten(meta);", call="input.as_ptr(), input.len(), &m")
SDPA_ARGS = "num_bh: usize, seq_q: usize, seq_k: usize, d_k: usize, d_v: usize"
SDPA_CALL = "q.as_ptr(), q.len(), k.as_ptr(), k.len(), v.as_ptr(), v.len()"

WRAPPERS = []
WRAPPERS += _twins("matmul_tensor_contiguous", 37752, 17355, **BINARY)
WRAPPERS += _twins("bmm_tensor_contiguous", 38496, 17785, **BINARY)
WRAPPERS += _twins("add_tensor_contiguous", 36870, 4476, **BINARY)
WRAPPERS += _twins("addmm_tensor_contiguous", 41562, 17514, kind=FALLIBLE_SIZED,
                   sig="input: &[{T}], mat1: &[{T}], mat2: &[{T}], input_meta: &TensorMeta, mat1_meta: &TensorMeta, mat2_meta: &TensorMeta, beta: {T}, alpha: {T}",
                   ret_ty="Result<Vec<{T}>, KernelError>",
                   pre="let (im, m1, m2) = (flatten(input_meta), flatten(mat1_meta), flatten(mat2_meta));",
                   call="input.as_ptr(), input.len(), mat1.as_ptr(), mat1.len(), mat2.as_ptr(), mat2.len(), &im, &m1, &m2, beta, alpha")
WRAPPERS += _twins("matmul_rhs_transposed_contiguous", 17408, 17381, kind=FALLIBLE_SIZED,
                   sig="m: usize, k: usize, n: usize, lhs: &[{T}], rhs_nk: &[{T}]", ret_ty="Result<Vec<{T}>, KernelError>",
                   pre="", call="m, k, n, lhs.as_ptr(), lhs.len(), rhs_nk.as_ptr(), rhs_nk.len()")
WRAPPERS += _twins("softmax_dim_tensor_contiguous", 39193, 18350, **UNARY_DIM)
WRAPPERS += _twins("log_softmax_dim_tensor_contiguous", 39298, 18504, **UNARY_DIM)
WRAPPERS += _twins("argmax_dim_tensor_contiguous", 39443, 18653, **UNARY_DIM)
WRAPPERS += _twins("gelu_tensor_contiguous", 37123, 3657, **UNARY)
WRAPPERS += _twins("gelu_tanh_tensor_contiguous", None, None, **UNARY)
WRAPPERS += _twins("index_select_tensor_contiguous", 40216, 20184, kind=FALLIBLE_SIZED,
                   sig="input: &[{T}], meta: &TensorMeta, dim: usize, indices: &[f64]", ret_ty="Result<Vec<{T}>, KernelError>",
                   pre="let m = flatten(meta);", call="input.as_ptr(), input.len(), &m, dim, indices.as_ptr(), indices.len()")
# Infallible fused entry points: the reference panics on short slices (plain indexing); so do these (`expect_ok`).
WRAPPERS += _twins("linear_tensor", 17306, 17162, kind="fixed",
                   sig="x: &[{T}], weight: &[{T}], bias: Option<&[{T}]>, batch: usize, in_features: usize, out_features: usize",
                   ret_ty="Vec<{T}>", pre="let mut n = 0usize;",
                   call="x.as_ptr(), x.len(), weight.as_ptr(), weight.len(), opt_ptr(bias), bias.map_or(0, <[{T}]>::len), batch, in_features, out_features",
                   outs=[("out", "{T}", "batch * out_features")], tail=", &mut n", ret="out")
WRAPPERS += _twins("layer_norm_forward", 5877, 5824, kind="fixed",
                   sig="x: &[{T}], weight: Option<&[{T}]>, bias: Option<&[{T}]>, batch: usize, norm_size: usize, eps: {T}", ret_ty="Vec<{T}>",
                   pre="", call="x.as_ptr(), x.len(), opt_ptr(weight), opt_ptr(bias), batch, norm_size, eps",
                   outs=[("out", "{T}", "batch * norm_size")], ret="out")
WRAPPERS += [dict(name="add_layer_norm_forward_f32", T="f32", line=5932, kind="fixed",
                  sig="a: &[f32], b: &[f32], weight: Option<&[f32]>, bias: Option<&[f32]>, batch: usize, norm_size: usize, eps: f32", ret_ty="Vec<f32>",
                  pre="", call="a.as_ptr(), b.as_ptr(), a.len().min(b.len()), opt_ptr(weight), opt_ptr(bias), batch, norm_size, eps",
                  outs=[("out", "f32", "batch * norm_size")], ret="out")]
WRAPPERS += _twins("rms_norm_forward", 6459, 6418, kind="fixed",
                   sig="x: &[{T}], weight: Option<&[{T}]>, batch: usize, norm_size: usize, eps: {T}", ret_ty="Vec<{T}>",
                   pre="", call="x.as_ptr(), x.len(), opt_ptr(weight), batch, norm_size, eps", outs=[("out", "{T}", "batch * norm_size")], ret="out")
WRAPPERS += _twins("sdpa_forward", 5200, 4572, kind="fixed",
                   sig="q: &[{T}], k: &[{T}], v: &[{T}], " + SDPA_ARGS + ", scale: {T}, causal: bool", ret_ty="Vec<{T}>", pre="",
                   call=SDPA_CALL + ", num_bh, seq_q, seq_k, d_k, d_v, scale, causal as i32", outs=[("out", "{T}", "num_bh * seq_q * d_v")], ret="out")
WRAPPERS += _twins("sdpa_forward_masked", None, 4661, kind="fixed",
                   sig="q: &[{T}], k: &[{T}], v: &[{T}], " + SDPA_ARGS + ", scale: {T}, mask: &[{T}], mask_bh_stride: usize", ret_ty="Vec<{T}>", pre="",
                   call=SDPA_CALL + ", num_bh, seq_q, seq_k, d_k, d_v, scale, mask.as_ptr(), mask.len(), mask_bh_stride",
                   outs=[("out", "{T}", "num_bh * seq_q * d_v")], ret="out")
WRAPPERS += _twins("sdpa_forward_masked_gqa", None, 4760, kind="fixed",
                   sig="q: &[{T}], k: &[{T}], v: &[{T}], batch: usize, h_q: usize, h_kv: usize, seq_q: usize, seq_k: usize, d_k: usize, d_v: usize, scale: {T}, mask: &[{T}], mask_bh_stride: usize",
                   ret_ty="Vec<{T}>", pre="",
                   call=SDPA_CALL + ", batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask.as_ptr(), mask.len(), mask_bh_stride",
                   outs=[("out", "{T}", "batch * h_q * seq_q * d_v")], ret="out")
WRAPPERS += _twins("cross_entropy_forward", 6717, 6649, kind="fixed", sig="logits: &[{T}], target: &[usize], batch: usize, classes: usize",
                   ret_ty="Vec<{T}>", pre="", call="logits.as_ptr(), logits.len(), target.as_ptr().cast::<u64>(), target.len(), batch, classes",
                   outs=[("loss", "{T}", "batch")], ret="loss")
WRAPPERS += _twins("cross_entropy_backward", 6745, 6679, kind="fixed",
                   sig="logits: &[{T}], target: &[usize], dloss: &[{T}], batch: usize, classes: usize", ret_ty="Vec<{T}>", pre="",
                   call="logits.as_ptr(), logits.len(), target.as_ptr().cast::<u64>(), target.len(), dloss.as_ptr(), dloss.len(), batch, classes",
                   outs=[("dlogits", "{T}", "batch * classes")], ret="dlogits")
WRAPPERS += _twins("layer_norm_backward", 6189, 6052, kind="fixed", sig="dy: &[{T}], x: &[{T}], weight: &[{T}], batch: usize, norm_size: usize, eps: {T}",
                   ret_ty="(Vec<{T}>, Vec<{T}>, Vec<{T}>)", pre="", call="dy.as_ptr(), dy.len(), x.as_ptr(), x.len(), weight.as_ptr(), batch, norm_size, eps",
                   outs=[("dx", "{T}", "batch * norm_size"), ("dweight", "{T}", "norm_size"), ("dbias", "{T}", "norm_size")], ret="(dx, dweight, dbias)")
WRAPPERS += _twins("rms_norm_backward", 6574, 6503, kind="fixed", sig="dy: &[{T}], x: &[{T}], weight: Option<&[{T}]>, batch: usize, norm_size: usize, eps: {T}",
                   ret_ty="(Vec<{T}>, Option<Vec<{T}>>)", pre="", call="dy.as_ptr(), dy.len(), x.as_ptr(), x.len(), opt_ptr(weight), batch, norm_size, eps",
                   outs=[("dx", "{T}", "batch * norm_size"), ("dweight", "{T}", "if weight.is_some() { norm_size } else { 0 }")],
                   ret="(dx, weight.map(|_| dweight))")
WRAPPERS += _twins("linear_backward", None, 17226, kind="fixed",
                   sig="dy: &[{T}], x: &[{T}], weight: &[{T}], batch: usize, in_features: usize, out_features: usize, need_bias: bool",
                   ret_ty="(Vec<{T}>, Vec<{T}>, Option<Vec<{T}>>)", pre="",
                   call="dy.as_ptr(), dy.len(), x.as_ptr(), x.len(), weight.as_ptr(), weight.len(), batch, in_features, out_features, need_bias as i32",
                   outs=[("dx", "{T}", "batch * in_features"), ("dweight", "{T}", "out_features * in_features"),
                         ("dbias", "{T}", "if need_bias { out_features } else { 0 }")],
                   ret="(dx, dweight, need_bias.then_some(dbias))")
SDPA_BWD_OUTS = [("dq", "{T}", "num_bh * seq_q * d_k"), ("dk", "{T}", "num_bh * seq_k * d_k"), ("dv", "{T}", "num_bh * seq_k * d_v")]
WRAPPERS += _twins("sdpa_backward", 5539, 5300, kind="fixed",
                   sig="q: &[{T}], k: &[{T}], v: &[{T}], dout: &[{T}], " + SDPA_ARGS + ", scale: {T}, causal: bool", ret_ty="(Vec<{T}>, Vec<{T}>, Vec<{T}>)", pre="",
                   call=SDPA_CALL + ", dout.as_ptr(), dout.len(), num_bh, seq_q, seq_k, d_k, d_v, scale, causal as i32", outs=SDPA_BWD_OUTS, ret="(dq, dk, dv)")
WRAPPERS += [dict(name="sdpa_backward_f32_unit_dout", T="f32", line=5662, kind="fixed",
                  sig="q: &[f32], k: &[f32], v: &[f32], " + SDPA_ARGS + ", scale: f32, causal: bool", ret_ty="(Vec<f32>, Vec<f32>, Vec<f32>)", pre="",
                  call=SDPA_CALL + ", num_bh, seq_q, seq_k, d_k, d_v, scale, causal as i32", outs=SDPA_BWD_OUTS, ret="(dq, dk, dv)")]
WRAPPERS += _twins("sdpa_backward_masked", None, 5423, kind="fixed",
                   sig="q: &[{T}], k: &[{T}], v: &[{T}], dout: &[{T}], " + SDPA_ARGS + ", scale: {T}, mask: &[{T}], mask_bh_stride: usize",
                   ret_ty="(Vec<{T}>, Vec<{T}>, Vec<{T}>)", pre="",
                   call=SDPA_CALL + ", dout.as_ptr(), dout.len(), num_bh, seq_q, seq_k, d_k, d_v, scale, mask.as_ptr(), mask.len(), mask_bh_stride",
                   outs=SDPA_BWD_OUTS, ret="(dq, dk, dv)")
WRAPPERS += [
    dict(name="quantize_per_output_channel_i8", T="f32", line=37836, kind="fixed", sig="w: &[f32], out: usize, in_: usize", ret_ty="(Vec<i8>, Vec<f32>)",
         pre="", call="w.as_ptr(), w.len(), out, in_", outs=[("q", "i8", "out * in_"), ("scales", "f32", "out")], ret="(q, scales)"),
    dict(name="quantize_rows_i8", T="f32", line=37879, kind="fixed", sig="x: &[f32], m: usize, k: usize", ret_ty="(Vec<i8>, Vec<f32>)",
         pre="", call="x.as_ptr(), x.len(), m, k", outs=[("q", "i8", "m * k"), ("scales", "f32", "m")], ret="(q, scales)"),
    dict(name="linear_int8_dynamic_f32", T="f32", line=37966, kind="fixed",
         sig="x: &[f32], m: usize, k: usize, w_i8: &[i8], w_scales: &[f32], n: usize, bias: Option<&[f32]>", ret_ty="Vec<f32>", pre="",
         call="x.as_ptr(), x.len(), m, k, w_i8.as_ptr(), w_i8.len(), w_scales.as_ptr(), w_scales.len(), n, opt_ptr(bias), bias.map_or(0, <[f32]>::len)",
         outs=[("out", "f32", "m * n")], ret="out"),
]
WRAPPERS += _twins("transpose_batched_materialize", 42526, 42490, kind="fixed", sig="src: &[{T}], batch: usize, rows: usize, cols: usize",
                   ret_ty="Vec<{T}>", pre="", call="src.as_ptr(), src.len(), batch, rows, cols", outs=[("out", "{T}", "batch * rows * cols")], ret="out")
WRAPPERS += _twins("transpose_2d_into", 42415, 42294, kind="into", sig="src: &[{T}], dst: &mut [{T}], rows: usize, cols: usize", ret_ty="()",
                   pre="", call="src.as_ptr(), src.len(), dst.as_mut_ptr(), dst.len(), rows, cols")


def fmt(s, w):
    return s.replace("{T}", w["T"])


def write_wrapper(w) -> str:
    name, T = w["name"], w["T"]
    ffi = "ffi::fth_" + name
    where = ("`ft_kernel_cpu::%s` (crates/ft-kernel-cpu/src/lib.rs:%d)" % (name, w["line"]) if w["line"]
             else "new surface: the reference has no `%s` yet; the signature follows its twin of the other precision" % name)
    lines = ["/// %s." % where]
    ret_ty = fmt(w["ret_ty"], w)
    lines.append("pub fn %s(%s)%s {" % (name, fmt(w["sig"], w), "" if ret_ty == "()" else " -> " + ret_ty))
    if w.get("pre"):
        lines.append("    " + fmt(w["pre"], w))
    call = fmt(w["call"], w)
    if w["kind"] == FALLIBLE_SIZED:
        lines += ["    let mut n = 0usize; // the first call validates and sizes; nothing is computed for a null output",
                  "    check(unsafe { %s(%s, std::ptr::null_mut(), 0, &mut n) })?;" % (ffi, call),
                  "    let mut out = Vec::<%s>::with_capacity(n); // every element is overwritten: no zero fill (build_uninit)" % T,
                  "    check(unsafe { %s(%s, out.as_mut_ptr(), n, &mut n) })?;" % (ffi, call),
                  "    unsafe { out.set_len(n) };", "    Ok(out)"]
    elif w["kind"] == "fixed":
        outs = [(b, fmt(t, w), fmt(l, w)) for b, t, l in w["outs"]]
        for b, t, l in outs:
            lines.append("    let mut %s = Vec::<%s>::with_capacity(%s);" % (b, t, l))
        out_args = ", ".join("%s.as_mut_ptr(), %s.capacity()" % (b, b) for b, _, _ in outs)
        lines.append("    expect_ok(unsafe { %s(%s, %s%s) }, \"%s\");" % (ffi, call, out_args, w.get("tail", ""), name))
        for b, _, l in outs:
            lines.append("    unsafe { %s.set_len(%s) };" % (b, l))
        lines.append("    " + fmt(w["ret"], w))
    elif w["kind"] == "into":
        lines.append("    expect_ok(unsafe { %s(%s) }, \"%s\");" % (ffi, call, name))
    lines.append("}")
    return "\n".join(lines)


LIB_HEAD = '''// GENERATED by generate_bindings.py (the wrapper table in that script). Do not edit: change the table and regenerate.
//
//! `ft-kernel-hip`: the MI355X (gfx950) kernel backend of FrankenTorch.
//!
//! Every function below has the name, the argument list and the return type of the `ft_kernel_cpu` function it stands
//! in for, so `ft-dispatch` routes `DispatchKey::HIP` to `ft_kernel_hip::<same name>` with the arguments it already
//! holds. Host slices go in, a freshly allocated `Vec` comes out; the work runs on the GPU through the host-slice tier
//! of `libft_kernel_hip.so` (`ffi`). There is no CPU fallback in this crate: `KernelError` has no variant for a missing
//! device, so without a usable gfx950 device these functions panic with the library's `Unavailable` message. The
//! dispatcher only selects `DispatchKey::HIP` for tensors on `Device::Hip`, which cannot be created without a device;
//! callers that want to probe first use `is_available()` (the contract of `ft_kernel_metal::fused::is_available`,
//! crates/ft-kernel-metal/src/fused.rs:631-633), and the `resident` tier reports `Error::Unavailable` as a value.
//!
//! `resident` holds the device-resident surface modelled on `ft_kernel_metal::fused` (GpuTensor / Batch / EncoderGpu).

pub mod ffi;
pub mod resident;

use ft_core::{DType, Device, TensorMeta};
pub use ft_kernel_cpu::KernelError;

/// `ft_kernel_metal::fused::is_available`: true when a gfx950 device can run the kernels.
#[must_use]
pub fn is_available() -> bool {
    unsafe { ffi::fth_is_available() != 0 }
}

/// Copies a `TensorMeta` (crates/ft-core/src/lib.rs:340-348) into the flat C struct.
fn flatten(meta: &TensorMeta) -> ffi::fth_meta {
    let mut m = ffi::fth_meta {
        ndim: meta.shape().len() as i32,
        dtype: match meta.dtype() {
            DType::F64 => ffi::FTH_DTYPE_F64,
            DType::F32 => ffi::FTH_DTYPE_F32,
            DType::F16 => ffi::FTH_DTYPE_F16,
            DType::BF16 => ffi::FTH_DTYPE_BF16,
            _ => -1, // refused by the library's dtype check, as the reference refuses it for these kernels
        },
        device: match meta.device() {
            Device::Cpu => ffi::FTH_DEVICE_CPU,
            Device::Cuda => ffi::FTH_DEVICE_CUDA,
            Device::Hip => ffi::FTH_DEVICE_HIP,
        },
        reserved: 0,
        shape: [0; ffi::FTH_MAX_DIMS],
        strides: [0; ffi::FTH_MAX_DIMS],
        storage_offset: meta.storage_offset() as u64,
    };
    assert!(meta.shape().len() <= ffi::FTH_MAX_DIMS, "ft-kernel-hip: tensors of more than 8 dimensions are not supported");
    for (i, (&d, &s)) in meta.shape().iter().zip(meta.strides()).enumerate() {
        m.shape[i] = d as u64;
        m.strides[i] = s as u64;
    }
    m
}

fn opt_ptr<T>(s: Option<&[T]>) -> *const T {
    s.map_or(std::ptr::null(), <[T]>::as_ptr)
}

fn last_error() -> ffi::fth_error_info {
    let mut info: ffi::fth_error_info = unsafe { std::mem::zeroed() };
    unsafe { ffi::fth_last_error(&mut info) };
    info
}

fn c_text(bytes: &[std::os::raw::c_char]) -> String {
    let end = bytes.iter().position(|&b| b == 0).unwrap_or(bytes.len());
    String::from_utf8_lossy(&bytes[..end].iter().map(|&b| b as u8).collect::<Vec<u8>>()).into_owned()
}

fn side_of(info: &ffi::fth_error_info) -> &'static str {
    match c_text(&info.side).as_str() {
        "lhs" => "lhs",
        "rhs" => "rhs",
        "mat1" => "mat1",
        "mat2" => "mat2",
        _ => "input",
    }
}

/// Status 1..9 are the `KernelError` variants one for one (crates/ft-kernel-cpu/src/lib.rs:1697-1733); the payload comes
/// from the calling thread's error slot. Anything else is a backend failure the reference has no variant for.
fn check(rc: i32) -> Result<(), KernelError> {
    if rc == ffi::FTH_OK {
        return Ok(());
    }
    let e = last_error();
    Err(match rc {
        ffi::FTH_ERR_DTYPE_MISMATCH => KernelError::Incompatible(ft_core::TensorCompatError::DTypeMismatch {
            lhs: dtype_of(e.a),
            rhs: dtype_of(e.b),
        }),
        ffi::FTH_ERR_DEVICE_MISMATCH => KernelError::Incompatible(ft_core::TensorCompatError::DeviceMismatch {
            lhs: device_of(e.a),
            rhs: device_of(e.b),
        }),
        ffi::FTH_ERR_SHAPE_MISMATCH => KernelError::ShapeMismatch {
            lhs: e.lhs_shape[..e.lhs_ndim as usize].iter().map(|&d| d as usize).collect(),
            rhs: e.rhs_shape[..e.rhs_ndim as usize].iter().map(|&d| d as usize).collect(),
        },
        ffi::FTH_ERR_UNSUPPORTED_LAYOUT => KernelError::UnsupportedLayout { side: side_of(&e) },
        ffi::FTH_ERR_STORAGE_SPAN_OVERFLOW => KernelError::StorageSpanOverflow {
            side: side_of(&e),
            storage_offset: e.a as usize,
            numel: e.b as usize,
        },
        ffi::FTH_ERR_INSUFFICIENT_STORAGE => KernelError::InsufficientStorage {
            side: side_of(&e),
            needed: e.a as usize,
            available: e.b as usize,
        },
        ffi::FTH_ERR_INVALID_DIMENSION => KernelError::InvalidDimension { dim: e.a as usize, ndim: e.b as usize },
        ffi::FTH_ERR_SHAPE_OVERFLOW => KernelError::ShapeOverflow { context: "ft-kernel-hip" },
        ffi::FTH_ERR_EMPTY_REDUCTION_DIM => KernelError::EmptyReductionDim { dim: e.a as usize },
        _ => panic!("ft-kernel-hip: backend failure {} ({})", rc, c_text(&e.message)),
    })
}

fn dtype_of(tag: u64) -> DType {
    match tag as i32 {
        ffi::FTH_DTYPE_F64 => DType::F64,
        ffi::FTH_DTYPE_F16 => DType::F16,
        ffi::FTH_DTYPE_BF16 => DType::BF16,
        _ => DType::F32,
    }
}

fn device_of(tag: u64) -> Device {
    match tag as i32 {
        ffi::FTH_DEVICE_CUDA => Device::Cuda,
        ffi::FTH_DEVICE_HIP => Device::Hip,
        _ => Device::Cpu,
    }
}

/// The reference's fused entry points are infallible and panic on a short slice (plain indexing, e.g.
/// crates/ft-kernel-cpu/src/lib.rs:5888); the C entry points report it as a status, which panics here with its message.
fn expect_ok(rc: i32, what: &str) {
    if rc != ffi::FTH_OK {
        let e = last_error();
        panic!("ft_kernel_hip::{what}: status {rc}: {}", c_text(&e.message));
    }
}

/// `matmul_tensor_contiguous_f32_into` (crates/ft-kernel-cpu/src/lib.rs:37780-37823): the product into a caller `Vec`,
/// resized without re-zeroing, as the reference does (:37798-37811).
pub fn matmul_tensor_contiguous_f32_into(out: &mut Vec<f32>, lhs: &[f32], rhs: &[f32], lhs_meta: &TensorMeta, rhs_meta: &TensorMeta) -> Result<(), KernelError> {
    let (lm, rm) = (flatten(lhs_meta), flatten(rhs_meta));
    let mut n = 0usize;
    check(unsafe { ffi::fth_matmul_tensor_contiguous_f32(lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), &lm, &rm, std::ptr::null_mut(), 0, &mut n) })?;
    out.clear();
    out.reserve(n);
    check(unsafe { ffi::fth_matmul_tensor_contiguous_f32(lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), &lm, &rm, out.as_mut_ptr(), n, &mut n) })?;
    unsafe { out.set_len(n) };
    Ok(())
}

/// `transpose_2d_f32` (crates/ft-kernel-cpu/src/lib.rs:42406-42411).
#[must_use]
pub fn transpose_2d_f32(src: &[f32], rows: usize, cols: usize) -> Vec<f32> {
    let mut dst = vec![0.0f32; rows * cols];
    transpose_2d_into_f32(src, &mut dst, rows, cols);
    dst
}

/// `transpose_2d_f64` (crates/ft-kernel-cpu/src/lib.rs:42286-42291).
#[must_use]
pub fn transpose_2d_f64(src: &[f64], rows: usize, cols: usize) -> Vec<f64> {
    let mut dst = vec![0.0f64; rows * cols];
    transpose_2d_into_f64(src, &mut dst, rows, cols);
    dst
}
'''

RESIDENT_RS = '''// Written by generate_bindings.py (static text). The device-resident surface, modelled on `ft_kernel_metal::fused`
// (crates/ft-kernel-metal/src/fused.rs:540-933, 986-1190): tensors live in HBM, every op enqueues on the batch's stream
// and returns a fresh resident tensor, `finish` is the only synchronisation.
use crate::ffi;

/// `ft_kernel_metal::Error` (crates/ft-kernel-metal/src/lib.rs:60-77) with the HIP backend's status codes behind it.
#[derive(Debug, Clone, PartialEq, Eq)]
pub enum Error {
    Unavailable,
    Kernel(String),
    SizeOverflow,
    BufferTooLarge,
    CommandBuffer(String),
}

fn check(rc: i32) -> Result<(), Error> {
    if rc == ffi::FTH_OK {
        return Ok(());
    }
    let mut info: ffi::fth_error_info = unsafe { std::mem::zeroed() };
    unsafe { ffi::fth_last_error(&mut info) };
    let end = info.message.iter().position(|&b| b == 0).unwrap_or(info.message.len());
    let text = String::from_utf8_lossy(&info.message[..end].iter().map(|&b| b as u8).collect::<Vec<u8>>()).into_owned();
    Err(match rc {
        ffi::FTH_ERR_UNAVAILABLE => Error::Unavailable,
        ffi::FTH_ERR_SIZE_OVERFLOW => Error::SizeOverflow,
        ffi::FTH_ERR_BUFFER_TOO_LARGE => Error::BufferTooLarge,
        ffi::FTH_ERR_STREAM => Error::CommandBuffer(text),
        _ => Error::Kernel(text),
    })
}

/// A resident f32 `[rows, cols]` matrix (`GpuTensor`, fused.rs:540-580): hipMalloc-backed, explicit copies.
pub struct HipTensor(*mut ffi::fth_tensor);
// The handle is only ever used through the library, which locks its own state (fused.rs:1018-1019 asserts the same).
unsafe impl Send for HipTensor {}
unsafe impl Sync for HipTensor {}

impl HipTensor {
    pub fn upload(host: &[f32], rows: usize, cols: usize) -> Result<Self, Error> {
        assert_eq!(host.len(), rows * cols);
        let mut t = std::ptr::null_mut();
        check(unsafe { ffi::fth_tensor_upload(host.as_ptr(), rows as i64, cols as i64, &mut t) })?;
        Ok(Self(t))
    }
    pub fn download(&self) -> Result<Vec<f32>, Error> {
        let (mut rows, mut cols) = (0i64, 0i64);
        check(unsafe { ffi::fth_tensor_shape(self.0, &mut rows, &mut cols) })?;
        let n = (rows * cols) as usize;
        let mut out = Vec::<f32>::with_capacity(n);
        check(unsafe { ffi::fth_tensor_download(self.0, out.as_mut_ptr(), n) })?;
        unsafe { out.set_len(n) };
        Ok(out)
    }
    pub(crate) fn raw(&self) -> *const ffi::fth_tensor {
        self.0
    }
}

impl Drop for HipTensor {
    fn drop(&mut self) {
        unsafe { ffi::fth_tensor_free(self.0) };
    }
}

/// A stream-ordered batch of ops (`Batch`, fused.rs:676-932).
pub struct Batch(*mut ffi::fth_batch);

impl Batch {
    pub fn new() -> Result<Self, Error> {
        let mut b = std::ptr::null_mut();
        check(unsafe { ffi::fth_batch_new(&mut b) })?;
        Ok(Self(b))
    }
    fn wrap(rc: i32, out: *mut ffi::fth_tensor) -> Result<HipTensor, Error> {
        check(rc).map(|()| HipTensor(out))
    }
    /// `y = a . w^T (+ bias)`, the weight in `nn.Linear`'s `[out, in]` layout (`Batch::matmul_bias`, fused.rs:676-762).
    pub fn linear(&mut self, a: &HipTensor, w: &HipTensor, bias: Option<&HipTensor>) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_linear(self.0, a.raw(), w.raw(), bias.map_or(std::ptr::null(), HipTensor::raw), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn matmul(&mut self, a: &HipTensor, rhs: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_matmul(self.0, a.raw(), rhs.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn layernorm(&mut self, x: &HipTensor, gamma: &HipTensor, beta: &HipTensor, eps: f32) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_layernorm(self.0, x.raw(), gamma.raw(), beta.raw(), eps, &mut out) };
        Self::wrap(rc, out)
    }
    pub fn rmsnorm(&mut self, x: &HipTensor, gamma: &HipTensor, eps: f32) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_rmsnorm(self.0, x.raw(), gamma.raw(), eps, &mut out) };
        Self::wrap(rc, out)
    }
    pub fn gelu(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_gelu(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn gelu_tanh(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_gelu_tanh(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn add(&mut self, x: &HipTensor, y: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_add(self.0, x.raw(), y.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    pub fn softmax(&mut self, x: &HipTensor) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_softmax(self.0, x.raw(), &mut out) };
        Self::wrap(rc, out)
    }
    /// Multi-head attention over `[batch * seq, d_model]` q / k / v (`Batch::mha`, fused.rs:861-925).
    pub fn mha(&mut self, q: &HipTensor, k: &HipTensor, v: &HipTensor, n_heads: usize, batch: usize, causal: bool) -> Result<HipTensor, Error> {
        let mut out = std::ptr::null_mut();
        let rc = unsafe { ffi::fth_batch_mha(self.0, q.raw(), k.raw(), v.raw(), n_heads as i64, batch as i64, causal as i32, &mut out) };
        Self::wrap(rc, out)
    }
    /// The only synchronisation (`Batch::finish`, fused.rs:929-932).
    pub fn finish(&mut self) -> Result<(), Error> {
        check(unsafe { ffi::fth_batch_finish(self.0) })
    }
}

impl Drop for Batch {
    fn drop(&mut self) {
        unsafe { ffi::fth_batch_free(self.0) };
    }
}

/// One layer's weights as host slices, `nn.Linear` layout `[out, in]` (`LayerWeightsRef`, fused.rs:986-1016).
pub struct LayerWeightsRef<'a> {
    pub ln1_w: &'a [f32], pub ln1_b: &'a [f32],
    pub wq: &'a [f32], pub bq: &'a [f32], pub wk: &'a [f32], pub bk: &'a [f32], pub wv: &'a [f32], pub bv: &'a [f32],
    pub wo: &'a [f32], pub bo: &'a [f32],
    pub ln2_w: &'a [f32], pub ln2_b: &'a [f32],
    pub w1: &'a [f32], pub b1: &'a [f32], pub w2: &'a [f32], pub b2: &'a [f32],
}

/// Pre-LN encoder with resident weights (`EncoderGpu`, fused.rs:1024-1190).
pub struct EncoderHip {
    handle: *mut ffi::fth_encoder,
    d_model: usize,
}
unsafe impl Send for EncoderHip {}
unsafe impl Sync for EncoderHip {}

impl EncoderHip {
    pub fn new(d_model: usize, n_heads: usize, d_ff: usize, ln_eps: f32, causal: bool, layers: &[LayerWeightsRef<'_>]) -> Result<Self, Error> {
        let flat: Vec<ffi::fth_layer_weights> = layers
            .iter()
            .map(|l| ffi::fth_layer_weights {
                ln1_w: l.ln1_w.as_ptr(), ln1_b: l.ln1_b.as_ptr(),
                wq: l.wq.as_ptr(), bq: l.bq.as_ptr(), wk: l.wk.as_ptr(), bk: l.bk.as_ptr(), wv: l.wv.as_ptr(), bv: l.bv.as_ptr(),
                wo: l.wo.as_ptr(), bo: l.bo.as_ptr(),
                ln2_w: l.ln2_w.as_ptr(), ln2_b: l.ln2_b.as_ptr(),
                w1: l.w1.as_ptr(), b1: l.b1.as_ptr(), w2: l.w2.as_ptr(), b2: l.b2.as_ptr(),
            })
            .collect();
        let mut handle = std::ptr::null_mut();
        check(unsafe { ffi::fth_encoder_new(d_model as i64, n_heads as i64, d_ff as i64, ln_eps, causal as i32, flat.as_ptr(), flat.len() as i64, &mut handle) })?;
        Ok(Self { handle, d_model })
    }
    /// Host in, host out (`EncoderGpu::forward`, fused.rs:1136-1146).
    pub fn forward(&self, input: &[f32], batch: usize, seq: usize) -> Result<Vec<f32>, Error> {
        let n = batch * seq * self.d_model;
        assert_eq!(input.len(), n);
        let mut out = Vec::<f32>::with_capacity(n);
        check(unsafe { ffi::fth_encoder_forward(self.handle, input.as_ptr(), batch as i64, seq as i64, out.as_mut_ptr(), n) })?;
        unsafe { out.set_len(n) };
        Ok(out)
    }
}

impl Drop for EncoderHip {
    fn drop(&mut self) {
        unsafe { ffi::fth_encoder_free(self.handle) };
    }
}
'''

CARGO_TOML = '''# Written by generate_bindings.py (static text).
[package]
name = "ft-kernel-hip"
version = "0.1.0"
edition = "2024"
license-file = "../../LICENSE"
description = "MI355X (gfx950) HIP kernels for FrankenTorch's transformer op set: the ft-kernel-cpu entry points over a C ABI, plus a device-resident tier."
repository = "https://github.com/Dicklesworthstone/frankentorch"
build = "build.rs"
links = "ft_kernel_hip"
include = ["src/**", "csrc/**", "include/**", "build.rs", "Cargo.toml"]

[lib]
name = "ft_kernel_hip"

[dependencies]
ft-core = { workspace = true }
# KernelError is ft-kernel-cpu's type, so that ft-dispatch keeps one error enum whichever backend ran.
ft-kernel-cpu = { workspace = true }
'''


def write_lib_rs() -> str:
    return LIB_HEAD + "\n" + "\n\n".join(write_wrapper(w) for w in WRAPPERS) + "\n"


def outputs():
    consts, structs, opaque, aliases, funcs = parse_header()
    sources, flags = build_lists()
    return {
        os.path.join(HERE, "src", "ffi.rs"): write_ffi(consts, structs, opaque, aliases, funcs),
        os.path.join(HERE, "build.rs"): write_build_rs(sources, flags),
        os.path.join(HERE, "src", "lib.rs"): write_lib_rs(),
        os.path.join(HERE, "src", "resident.rs"): RESIDENT_RS,
        os.path.join(HERE, "Cargo.toml"): CARGO_TOML,
    }


def main():
    check = "--check" in sys.argv[1:]
    stale = []
    for path, text in outputs().items():
        if check:
            if not os.path.exists(path) or open(path).read() != text:
                stale.append(os.path.relpath(path, ROOT))
        else:
            os.makedirs(os.path.dirname(path), exist_ok=True)
            with open(path, "w") as f:
                f.write(text)
            print("wrote", os.path.relpath(path, ROOT))
    if stale:
        sys.exit("out of date (run rust/ft-kernel-hip/generate_bindings.py): " + ", ".join(stale))


if __name__ == "__main__":
    main()
