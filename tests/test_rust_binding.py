"""The Rust crate `native-hip` against the C header it binds, without a Rust toolchain.

`native-hip/src/lib.rs` declares the library's entry points in one `extern "C"` block.  Nothing in
this image can compile it, so what can go wrong between the two files is checked textually: every
declaration must name a function of include/native_hip.h with the same number of parameters, and
each parameter and return value must be of the same kind (pointer to const / to mutable of the same
pointee, size_t, uint32_t, int, float).  The crate's GemmKind -> ggml type map is held against the
reference's enum order (langtax/src/quant.rs:6646-6676) and the header's type ids, and the patch for
the reference workspace is checked to touch only the files it is documented to touch.
"""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "native_hip.h")
CRATE = os.path.join(ROOT, "native-hip")


def strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def c_kind(decl, has_name=True):
    """Kind of one C parameter or return type, read the way C declarators nest: the base type (with its
    constness), then every `*` makes a pointer to what stands left of it, `*const` a constant such pointer.
    A pointer is ('ptr', whether its pointee is const, the pointee's kind); the constness of the outermost
    object (the parameter variable itself) says nothing about the interface and is dropped."""
    tokens = re.findall(r"[A-Za-z_][A-Za-z0-9_]*|\*", decl)
    if has_name and tokens and tokens[-1] not in ("*", "const"):
        tokens = tokens[:-1]                       # the parameter's name
    const = False
    while tokens and tokens[0] == "const":
        const, tokens = True, tokens[1:]
    kind = base_kind(tokens[0])
    tokens = tokens[1:]
    while tokens and tokens[0] == "const":         # `T const`
        const, tokens = True, tokens[1:]
    while tokens:
        assert tokens[0] == "*", decl
        kind, tokens = ("ptr", const, kind), tokens[1:]
        const = False
        while tokens and tokens[0] == "const":
            const, tokens = True, tokens[1:]
    return kind


def base_kind(name):
    name = name.strip()
    table = {"size_t": "usize", "uint32_t": "u32", "uint8_t": "u8", "int": "int", "float": "f32", "double": "f64",
             "char": "char", "void": "void", "lnh_exec": "exec", "lnh_matrix": "matrix", "lnh_act": "act"}
    if name.startswith("const "):
        name = name[6:].strip()
    assert name in table, name
    return table[name]


def rust_kind(ty):
    ty = ty.strip()
    m = re.match(r"\*(const|mut)\s+(.*)$", ty)
    if m:
        return ("ptr", m.group(1) == "const", rust_kind(m.group(2)))
    table = {"usize": "usize", "u32": "u32", "u8": "u8", "c_int": "int", "f32": "f32", "f64": "f64", "c_char": "char",
             "c_void": "void", "LnhExec": "exec", "LnhMatrix": "matrix", "LnhAct": "act"}
    assert ty in table, ty
    return table[ty]


def header_functions():
    text = strip_c_comments(open(HEADER).read())
    text = re.sub(r"#define[^\n]*\n", "\n", text)
    out = {}
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(ln[hq]_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        plist = [] if params in ("", "void") else [p.strip() for p in params.split(",")]
        out[name] = (c_kind(ret, has_name=False), [c_kind(p) for p in plist])
    return out


def rust_functions():
    text = open(os.path.join(CRATE, "src", "lib.rs")).read()
    block = re.search(r'unsafe extern "C" \{(.*?)\n    \}', text, flags=re.S).group(1)
    out = {}
    for m in re.finditer(r"pub fn (ln[hq]_[a-z0-9_]+)\(([^)]*)\)\s*(->\s*([^;]+))?;", block):
        name, params, ret = m.group(1), m.group(2).strip(), m.group(4)
        plist = [] if not params else [p.split(":", 1)[1].strip() for p in params.split(",")]
        out[name] = (rust_kind(ret) if ret else "void", [rust_kind(p) for p in plist])
    return out


def test_every_extern_declaration_matches_the_header():
    c, r = header_functions(), rust_functions()
    assert len(c) >= 35 and len(r) >= 30
    for name, (ret, params) in r.items():
        assert name in c, f"{name} is not declared in include/native_hip.h"
        c_ret, c_params = c[name]
        assert len(params) == len(c_params), f"{name}: {len(params)} parameters in Rust, {len(c_params)} in C"
        for i, (a, b) in enumerate(zip(params, c_params)):
            assert a == b, f"{name}: parameter {i} is {a} in Rust and {b} in C"
        assert ret == c_ret, f"{name}: returns {ret} in Rust and {c_ret} in C"
    # what the wrappers of gpu.rs and the reference's call sites need is bound
    for needed in ("lnh_create", "lnh_destroy", "lnh_memory_info", "lnh_upload_f32", "lnh_upload_packed", "lnh_matrix_free",
                   "lnh_gemv", "lnh_gemm", "lnh_gemm_grouped", "lnh_last_error", "lnh_thread_error", "lnq_gemm",
                   "lnh_gemm_device_noalloc", "lnh_matrix_info", "lnh_resident_bytes"):
        assert needed in r, needed
    # measurement and test helpers of the header are deliberately left out of the binding
    assert set(c) - set(r) <= {"lnh_calibration_copy", "lnh_calibration_read", "lnq_parse_cache_bytes", "lnq_automatic_cache_bytes",
                               "lnq_admission_requires_eviction", "lnq_cache_stats", "lnq_reset"}


def test_wrappers_call_only_what_is_declared():
    r = rust_functions()
    gpu = open(os.path.join(CRATE, "src", "gpu.rs")).read()
    used = set(re.findall(r"ffi::(ln[hq]_[a-z0-9_]+)", gpu))
    assert used and used <= set(r)
    for method in ("pub fn new(", "pub fn memory_info(", "pub fn upload(", "pub fn upload_packed(", "pub fn gemv_resident(",
                   "pub fn gemv(", "pub fn gemm_resident(", "pub fn gemm_grouped("):
        assert method in gpu, method  # CudaGemv's method set (native-cuda/src/gpu.rs:148-417) plus the two extensions


def test_gemm_kind_map_agrees_with_the_reference_enum_and_the_header():
    # langtax/src/quant.rs:6646-6676: the order of `enum GemmKind`, whose discriminants `kind as u8` are
    kinds = ["F16", "BF16", "F32", "Q2K", "Q3K", "Q41", "Q50", "Q51", "MXFP4", "NVFP4", "Q10", "Q20", "Q40", "Q80", "Q81",
             "TQ10", "TQ20", "Q4K", "Q5K", "Q6K", "IQ1S", "IQ1M", "IQ2S", "IQ2XXS", "IQ2XS", "IQ3S", "IQ3XXS", "IQ4NL", "IQ4XS"]
    header = strip_c_comments(open(HEADER).read())
    ids = {m.group(1): int(m.group(2)) for m in re.finditer(r"LNH_TYPE_([A-Z0-9_]+)\s*=\s*(\d+)", header)}
    assert ids == {"F32": 0, "F16": 1, "Q4_0": 2, "Q5_0": 6, "Q5_1": 7, "Q8_0": 8, "Q4_K": 12, "Q6_K": 14}
    lib = open(os.path.join(CRATE, "src", "lib.rs")).read()
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"pub const ([A-Z0-9_]+): u32 = (\d+);", lib)}
    assert consts == ids
    arms = {int(m.group(1)): (m.group(2), m.group(3))
            for m in re.finditer(r"(\d+) => Some\(ggml_type::([A-Z0-9_]+)\),\s*// GemmKind::([A-Z0-9]+)", lib)}
    want = {"F16": "F16", "F32": "F32", "Q50": "Q5_0", "Q51": "Q5_1", "Q40": "Q4_0", "Q80": "Q8_0", "Q4K": "Q4_K", "Q6K": "Q6_K"}
    assert len(arms) == 8
    for disc, (ggml, kind) in arms.items():
        assert kinds[disc] == kind, (disc, kind)      # the discriminant is that kind's position in the enum
        assert want[kind] == ggml, (kind, ggml)


def test_patch_names_only_the_wiring_files():
    patch = open(os.path.join(CRATE, "langtax-native-hip.patch")).read()
    files = re.findall(r"^\+\+\+ b/(\S+)", patch, flags=re.M)
    assert files == ["Cargo.toml", "langtax/Cargo.toml", "langtax/src/lib.rs", "langtax/src/native_gpu.rs",
                     "langtax/src/quant.rs", "langtax/src/decode.rs"]
    added = [l[1:] for l in patch.splitlines() if l.startswith("+") and not l.startswith("+++")]
    assert any("upload_packed(ggml_type, rows, cols, packed)" in l for l in added)
    assert any('native-hip = ["dep:llama-native-hip", "llama-native-hip/hip"]' in l for l in added)
    assert any("LLAMA_HIP_CACHE_BYTES" in l for l in added)
    # the residency charge is the C++ twin's (llama-rust_amd/csrc/residency.cpp: resident, recharge): what the matrix
    # holds on the device plus the identity copy, asked from the library, and charged again after every product
    # because the figure grows when the multi-token layout appears - never a constant multiple of the packed size
    assert not any(re.search(r"checked_mul\(\s*\d+\s*\)", l) for l in added), "a constant multiple of the packed size"
    assert any("resident_bytes(t, rows, cols, tokens)" in l for l in added)
    assert any("device.checked_add(packed.len())" in l for l in added)
    assert any(".device_bytes()" in l for l in added) and sum("recharge_last(state);" in l for l in added) == 2
    # hunk headers are consistent with their bodies (a hand-edited patch that no longer applies shows up here)
    for m in re.finditer(r"^@@ -(\d+),(\d+) \+(\d+),(\d+) @@.*\n((?:[ +\-].*\n|\n)*)", patch, flags=re.M):
        old_n, new_n, body = int(m.group(2)), int(m.group(4)), m.group(5).splitlines()
        body = [l for l in body if not l.startswith(("--- ", "+++ "))]
        assert sum(1 for l in body if not l.startswith("+")) == old_n, m.group(0)[:40]
        assert sum(1 for l in body if not l.startswith("-")) == new_n, m.group(0)[:40]


@pytest.mark.skipif(not os.path.isdir("/root/reference/langtax"), reason="the reference checkout is only present where the crate was written")
def test_patch_applies_to_the_reference_checkout(tmp_path):
    import shutil
    import subprocess
    if shutil.which("patch") is None:
        pytest.skip("no patch(1)")
    for rel in ("Cargo.toml", "langtax/Cargo.toml", "langtax/src/lib.rs", "langtax/src/native_gpu.rs", "langtax/src/quant.rs",
                "langtax/src/decode.rs"):
        dst = tmp_path / rel
        dst.parent.mkdir(parents=True, exist_ok=True)
        shutil.copy(os.path.join("/root/reference", rel), dst)
    r = subprocess.run(["patch", "-p1", "--dry-run", "-i", os.path.join(CRATE, "langtax-native-hip.patch")], cwd=tmp_path,
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
