"""The `ft-kernel-hip` crate files under rust/ are generated from the C header and the Python build recipe; with no Rust
toolchain in the image, this checks what can be checked without one: the committed files are what the generator writes
today, every header symbol is declared in ffi.rs with the header's arity and spelled types, build.rs lists exactly the
translation units the library is linked from, every host-slice entry point has a safe wrapper that calls it with the
right number of arguments, and the patches still name the reference lines they were cut against."""
import importlib.util
import os
import re

from frankentorch_amd import _lib
from frankentorch_amd import build as hip_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CRATE = os.path.join(ROOT, "rust", "ft-kernel-hip")


def _generator():
    spec = importlib.util.spec_from_file_location("generate_bindings", os.path.join(CRATE, "generate_bindings.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _read(*parts):
    return open(os.path.join(CRATE, *parts)).read()


def _split_args(text):
    """Top-level comma split of an argument list."""
    out, depth, cur = [], 0, ""
    for ch in text:
        if ch in "([{<":
            depth += 1
        elif ch in ")]}>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def _call_args(text, start):
    """The argument text of the call whose opening parenthesis is at `start`."""
    depth, i = 0, start
    while True:
        if text[i] == "(":
            depth += 1
        elif text[i] == ")":
            depth -= 1
            if depth == 0:
                return text[start + 1:i]
        i += 1


def test_committed_files_are_what_the_generator_writes():
    gen = _generator()
    for path, text in gen.outputs().items():
        assert os.path.exists(path), path
        assert open(path).read() == text, "%s is out of date: run rust/ft-kernel-hip/generate_bindings.py" % os.path.relpath(path, ROOT)


def test_ffi_declares_every_header_symbol_with_its_arity():
    ffi = _read("src", "ffi.rs")
    decls = {m.group(1): _split_args(m.group(2)) for m in re.finditer(r"pub fn (fth_\w+)\((.*?)\)(?: -> [^;]+)?;", ffi)}
    protos = _lib.protos()
    assert set(decls) == set(protos)
    for name, (restype, argtypes) in protos.items():
        assert len(decls[name]) == len(argtypes), name
    # spelled types of a few representative declarations
    assert "pub fn fth_dev_softmax_lastdim_f32(x: *const f32, y: *mut f32, rows: i64, cols: i64, s: fth_stream) -> i32;" in ffi
    assert "pub fn fth_tensor_upload(host: *const f32, rows: i64, cols: i64, out: *mut *mut fth_tensor) -> i32;" in ffi
    assert "pub fn fth_status_name(code: i32) -> *const c_char;" in ffi
    assert "pub fn fth_sdpa_desc_contiguous(d: *mut fth_sdpa_desc," in ffi and "causal: i32);" in ffi
    assert "pub fn fth_cross_entropy_forward_f32(logits: *const f32, logits_len: usize, target: *const u64," in ffi
    # struct layouts: the same field counts the ctypes mirror has
    for rust_name, ctypes_struct in (("fth_meta", _lib.Meta), ("fth_error_info", _lib.ErrorInfo), ("fth_gemm_desc", _lib.GemmDesc),
                                     ("fth_sdpa_desc", _lib.SdpaDesc), ("fth_layer_weights", _lib.LayerWeights)):
        body = re.search(r"pub struct %s \{(.*?)\}" % rust_name, ffi, re.S).group(1)
        assert len(re.findall(r"pub \w+:", body)) == len(ctypes_struct._fields_), rust_name
    assert "#[repr(C)]" in ffi and ffi.count("{") == ffi.count("}")


def test_build_rs_lists_the_translation_units_of_the_python_build():
    build_rs = _read("build.rs")
    listed = re.search(r"const HIP_SOURCES: &\[&str\] = &\[(.*?)\];", build_rs).group(1)
    assert [s.strip().strip('"') for s in listed.split(",")] == hip_build.HIP_SOURCES
    assert len(hip_build.HIP_SOURCES) == len([f for f in os.listdir(hip_build.CSRC) if f.endswith(".hip")])
    flags = re.search(r"const HIPCC_FLAGS: &\[&str\] = &\[(.*?)\];", build_rs).group(1)
    assert [s.strip().strip('"') for s in flags.split(",")] == hip_build.HIPCC_FLAGS
    assert "--offload-arch=gfx950" in flags and "-ffp-contract=off" in flags and "-packed-fp32-ops" in flags


def test_every_host_slice_entry_point_has_a_wrapper_that_calls_it_correctly():
    lib_rs = _read("src", "lib.rs")
    protos = _lib.protos()
    not_tier_a = re.compile(r"fth_(dev_|tensor_|batch_|encoder_|gpt2_|safetensors_|statedict_|pool_|stream_|event_|memcpy|memset|malloc|free|host_|"
                            r"device_|is_avail|last_error|status_name|sdpa_desc)")
    tier_a = [n for n in protos if not not_tier_a.match(n)]
    assert len(tier_a) >= 57
    for name in tier_a:
        rust_name = name[4:]
        assert re.search(r"^pub fn %s\(" % re.escape(rust_name), lib_rs, re.M), "no wrapper for " + name
        calls = [m.end() - 1 for m in re.finditer(r"ffi::%s\(" % re.escape(name), lib_rs)]
        assert calls, "wrapper does not call " + name
        for pos in calls:
            assert len(_split_args(_call_args(lib_rs, pos))) == len(protos[name][1]), name
    # the wrapper signatures are the reference's: spot checks against the argument lists of ft_kernel_cpu
    assert "pub fn sdpa_forward_f32(q: &[f32], k: &[f32], v: &[f32], num_bh: usize, seq_q: usize, seq_k: usize, d_k: usize, d_v: usize, scale: f32, causal: bool) -> Vec<f32> {" in lib_rs
    assert "pub fn layer_norm_backward_f32(dy: &[f32], x: &[f32], weight: &[f32], batch: usize, norm_size: usize, eps: f32) -> (Vec<f32>, Vec<f32>, Vec<f32>) {" in lib_rs
    assert "pub fn index_select_tensor_contiguous_f64(input: &[f64], meta: &TensorMeta, dim: usize, indices: &[f64]) -> Result<Vec<f64>, KernelError> {" in lib_rs
    assert "pub fn linear_tensor_f32(x: &[f32], weight: &[f32], bias: Option<&[f32]>, batch: usize, in_features: usize, out_features: usize) -> Vec<f32> {" in lib_rs
    for text in (lib_rs, _read("src", "resident.rs"), _read("build.rs")):
        assert text.count("{") == text.count("}") and text.count("(") == text.count(")")
    # the resident tier calls only functions the header declares, with their arity
    res = _read("src", "resident.rs")
    for m in re.finditer(r"ffi::(fth_\w+)\(", res):
        assert m.group(1) in protos, m.group(1)
        assert len(_split_args(_call_args(res, m.end() - 1))) == len(protos[m.group(1)][1]), m.group(1)


def test_patches_name_the_reference_files_and_add_the_hip_ids():
    pdir = os.path.join(ROOT, "rust", "patches")
    core, dev, disp, ws = (open(os.path.join(pdir, f)).read() for f in ("ft-core.diff", "ft-device.diff", "ft-dispatch.diff", "workspace.diff"))
    assert "+++ b/crates/ft-core/src/lib.rs" in core and "+    Hip," in core and "+    HipF32(Arc<HipBuffer>)," in core
    assert "+++ b/crates/ft-device/src/lib.rs" in dev and dev.count("+        (Device::") == 5
    assert "+    HIP = 6," in disp and "+const BACKEND_PRIORITY: [DispatchKey; 2] = [DispatchKey::HIP, DispatchKey::CPU];" in disp
    assert "+        Device::Hip => keyset.add(DispatchKey::HIP)," in disp and "ft_kernel_hip::softmax_dim_tensor_contiguous_f32(input, meta, dim)?" in disp
    assert '+  "crates/ft-kernel-hip",' in ws
    for p in (core, dev, disp, ws):
        for hunk in re.finditer(r"^@@ -(\d+),(\d+) \+(\d+),(\d+) @@", p, re.M):
            assert int(hunk.group(2)) > 0
