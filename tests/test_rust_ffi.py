"""The Rust FFI crate (rust/fastvideo-hip-sdpa) against the C header, without a Rust toolchain: every function
include/fv_sdpa_hip.h declares has one `extern "C"` declaration in src/ffi.rs with the same name, arity and
types; the `#[repr(C)]` structs list the header's fields in order; the constants agree; the Python loader's
ctypes table agrees with the header too; and src/lib.rs carries the reference's entry signatures
(crates/fastvideo-cudarc/src/rt/sdpa.rs:141, attn.rs:225, 526, 652, vsa.rs:358). The parsers here are
written apart from the crate's generator (gen_ffi.py), whose output must also be what is committed."""
import ctypes as C
import os
import re
import subprocess
import sys

from util import ROOT

from fv_sdpa import _lib

CRATE = os.path.join(ROOT, "rust", "fastvideo-hip-sdpa")
HEADER = os.path.join(ROOT, "include", "fv_sdpa_hip.h")

# C type (const-ness and pointer depth kept) -> (Rust type, ctypes class or None for void)
BASE = {"int": ("c_int", C.c_int), "float": ("f32", C.c_float), "double": ("f64", C.c_double),
        "size_t": ("usize", C.c_size_t), "long long": ("c_longlong", C.c_longlong), "uint64_t": ("u64", C.c_uint64)}
POINTEE = {"void": "c_void", "char": "c_char", "float": "f32", "uint16_t": "u16", "uint32_t": "u32", "int32_t": "i32",
           "uint64_t": "u64", "size_t": "usize", "int": "c_int", "fv_tensor": "FvTensor", "fv_plan": "FvPlan",
           "fv_kv_cache": "FvKvCache"}


def c_declarations():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    decls = {}
    for m in re.finditer(r"^([a-z_][a-z0-9_ ]*?[ \*]+)(fv_[a-z0-9_]+)\(([^)]*)\);", text, flags=re.M | re.S):
        ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        params = []
        if args != "void":
            for a in args.split(","):
                a = a.strip()
                arr = re.search(r"\[\d+\]$", a) is not None
                a = re.sub(r"\[\d+\]$", "", a)
                ctype, pname = re.match(r"^(.*?)([a-z_][a-z0-9_]*)$", a).groups()
                params.append((pname, ctype.strip(), arr))
        assert name not in decls
        decls[name] = (ret, params)
    return decls


def to_rust(ctype, arr=False):
    t = ctype.replace(" *", "*")
    const = t.startswith("const ")
    t = t[6:] if const else t
    if t.endswith("*") or arr:
        return ("*mut " if arr or not const else "*const ") + POINTEE[t.rstrip("*")]
    assert not const
    return BASE[t][0]


def to_ctypes(ctype, arr=False):
    t = ctype.replace(" *", "*")
    t = t[6:] if t.startswith("const ") else t
    if t == "char*":
        return C.c_char_p
    if t.endswith("*") or arr:
        return C.c_void_p
    return BASE[t][1]


def rust_declarations():
    text = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    block = re.search(r'#\[link\(name = "fv_sdpa_hip"\)\]\s*extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    decls = {}
    for m in re.finditer(r"pub fn (fv_[a-z0-9_]+)\(([^)]*)\)(?: -> ([^;]+))?;", block):
        name, args, ret = m.group(1), m.group(2).strip(), m.group(3)
        params = []
        if args:
            for a in args.split(","):
                pname, ptype = a.strip().split(": ", 1)
                params.append((pname, ptype))
        assert name not in decls
        decls[name] = (ret.strip() if ret else None, params)
    return text, decls


def test_every_header_function_has_a_matching_extern_declaration():
    cdecl = c_declarations()
    _, rdecl = rust_declarations()
    assert len(cdecl) >= 60
    assert set(cdecl) == set(rdecl), set(cdecl) ^ set(rdecl)
    for name, (ret, params) in cdecl.items():
        rret, rparams = rdecl[name]
        assert (None if ret == "void" else to_rust(ret)) == rret, name
        assert len(params) == len(rparams), name
        for (pname, ctype, arr), (rname, rtype) in zip(params, rparams):
            assert pname == rname and to_rust(ctype, arr) == rtype, (name, pname, ctype, rtype)


def test_repr_c_structs_and_constants_follow_the_header():
    header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    text, _ = rust_declarations()

    def c_fields(struct):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (struct, struct), header, flags=re.S).group(1)
        out = []
        for stmt in body.split(";"):
            stmt = " ".join(stmt.split())
            if not stmt:
                continue
            first, *rest = [x.strip() for x in stmt.split(",")]
            ctype, fname = re.match(r"^(.*?)([a-z_][a-z0-9_]*(?:\[\d+\])?)$", first).groups()
            for f in [fname] + rest:
                m = re.match(r"^([a-z_][a-z0-9_]*)(?:\[(\d+)\])?$", f)
                out.append((m.group(1), ctype.strip(), m.group(2)))
        return out

    def rust_fields(struct):
        body = re.search(r"pub struct %s \{(.*?)\n\}" % struct, text, flags=re.S).group(1)
        return re.findall(r"pub ([a-z_][a-z0-9_]*): ([^,\n]+),", body)

    for cname, rname in (("fv_tensor", "FvTensor"), ("fv_plan", "FvPlan")):
        cf, rf = c_fields(cname), rust_fields(rname)
        assert [f[0] for f in cf] == [f[0] for f in rf], (cf, rf)
        for (fname, ctype, n), (_, rtype) in zip(cf, rf):
            want = to_rust(ctype)
            assert rtype == (f"[{want}; {n}]" if n else want), (cname, fname, rtype)
        assert re.search(r"#\[repr\(C\)\]\s*(?:#\[derive\([^)]*\)\]\s*)?pub struct %s " % rname, text)
    consts = dict(re.findall(r"\b(FV_[A-Z_]+)\s*=\s*(\d+)", header))
    consts.update(dict(re.findall(r"#define (FV_(?:OK|DECLINED)) (\d+)", header)))
    assert len(consts) == 10
    for name, val in consts.items():
        assert re.search(r"pub const %s: c_int = %s;" % (name, val), text), name


def test_python_loader_table_agrees_with_the_header():
    cdecl = c_declarations()
    assert set(cdecl) == set(_lib.SIGNATURES)
    for name, (ret, params) in cdecl.items():
        res, args = _lib.SIGNATURES[name]
        assert res == (None if ret == "void" else to_ctypes(ret)), name
        assert args == [to_ctypes(t, arr) for _, t, arr in params], name


def test_committed_ffi_is_what_the_generator_writes(tmp_path):
    path = os.path.join(CRATE, "src", "ffi.rs")
    committed = open(path).read()
    before = os.stat(path).st_mtime_ns
    out = tmp_path / "ffi.rs"
    subprocess.check_call([sys.executable, os.path.join(CRATE, "gen_ffi.py"), str(out)])
    assert out.read_text() == committed
    assert os.stat(path).st_mtime_ns == before   # the tracked file is compared with, never written


def split_top_level(args):
    """Comma-separated pieces of a Rust argument list, commas inside (), [], {}, <> or || closures kept."""
    out, depth, cur, bars = [], 0, "", 0
    for i, ch in enumerate(args):
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        elif ch == "|" and depth == 0 and args[i - 1:i + 2] not in ("||",):
            bars ^= 1
        if ch == "," and depth == 0 and not bars:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def call_sites(src, prefix):
    """(name, argument list) of every `prefix::name(...)` call in `src`, matching parentheses."""
    sites = []
    for m in re.finditer(re.escape(prefix) + r"::([a-zA-Z0-9_]+)\(", src):
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(src[i], 0)
            i += 1
        sites.append((m.group(1), split_top_level(src[m.end():i - 1])))
    return sites


def test_every_ffi_call_site_passes_as_many_arguments_as_the_declaration_has():
    src = re.sub(r"//[^\n]*", "", open(os.path.join(CRATE, "src", "lib.rs")).read())
    _, rdecl = rust_declarations()
    sites = call_sites(src, "ffi")
    assert len(sites) >= 18
    for name, args in sites:
        assert name in rdecl, name
        assert len(args) == len(rdecl[name][1]), (name, len(args), len(rdecl[name][1]), args)
    # the HIP runtime calls of the crate against its own declarations (src/hip.rs)
    hip = re.sub(r"//[^\n]*", "", open(os.path.join(CRATE, "src", "hip.rs")).read())
    hdecl = {m.group(1): split_top_level(m.group(2)) for m in re.finditer(r"pub fn (hip[A-Za-z]+)\(([^)]*)\)", hip)}
    hsites = [c for c in call_sites(src, "hip") if c[0].startswith("hip")]
    assert len(hsites) >= 6
    for name, args in hsites:
        assert name in hdecl, name
        assert len(args) == len(hdecl[name]), (name, args, hdecl[name])


def test_shims_keep_the_reference_parameter_names_and_order():
    """Parameter names, in order, of the reference's entries (crates/fastvideo-cudarc/src/rt/sdpa.rs:56-141,
    attn.rs:225-231, 526-536, 652-659, vsa.rs:358-370; transcribed names only)."""
    src = " ".join(re.sub(r"//[^\n]*", "", open(os.path.join(CRATE, "src", "lib.rs")).read()).split())
    want = {
        "sdpa": ["q", "k", "v", "plan"],
        "device_mma_sdpa": ["q", "k", "v", "scale", "out_bf16"],
        "device_mma_sdpa_causal": ["q", "k", "v", "scale", "out_bf16", "mask"],
        "device_mma_sdpa_window": ["q", "k", "v", "scale", "out_bf16", "mask"],
        "vsa_attention_device": ["q", "k", "v", "gate", "plan", "topk", "bh", "seq", "dim", "scale", "group"],
        "dense": ["scale"], "masked": ["scale", "mask"], "fp8_first": ["self"], "composed": ["scale", "mask"],
        "block_causal": ["scale", "mask"], "vdn_window": ["scale", "mask"], "kv_window": [], "kv_window_with": ["flash"],
    }
    # two deliberate differences: no `sm_major` (attn.rs:112-119: one architecture here), and the two fields
    # `block_causal_for` reads from the model config (attn.rs:630-645) passed as plain numbers
    want["mma_sdpa_supported"] = ["b", "h", "sq", "sk", "d"]
    want["block_causal_for"] = ["num_frames_per_block", "local_attn_size", "frame_tokens"]
    for name, params in want.items():
        m = re.search(r"pub fn %s\(([^)]*)\)" % name, src)
        assert m, name
        got = [a.split(":")[0].strip() for a in split_top_level(m.group(1))]
        assert got == params, (name, got)


def test_shims_carry_the_reference_signatures():
    src = " ".join(open(os.path.join(CRATE, "src", "lib.rs")).read().split())
    for sig in (
        "pub fn sdpa(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, plan: &Plan<'_>) -> Result<CudaTensor>",
        "pub fn device_mma_sdpa(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, scale: Option<f32>, out_bf16: bool) "
        "-> Result<Option<CudaTensor>>",
        "pub fn device_mma_sdpa_causal( q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, scale: Option<f32>, out_bf16: bool, "
        "mask: BlockCausal, ) -> Result<Option<CudaTensor>>",
        "pub fn device_mma_sdpa_window( q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, scale: Option<f32>, out_bf16: bool, "
        "mask: VdnWindow, ) -> Result<Option<CudaTensor>>",
        "gate: Option<&HipSlice<f32>>, plan: &VsaPlanDev, topk: usize, bh: usize, seq: usize, dim: usize, scale: f32, "
        "group: usize, ) -> Result<HipSlice<f32>>",
        "pub fn dense(scale: Option<f32>) -> Self", "pub fn masked(scale: Option<f32>, mask: Option<&'a CudaTensor>) -> Self",
        "pub fn fp8_first(self) -> Self", "pub fn composed(scale: Option<f32>, mask: Option<&'a CudaTensor>) -> Self",
        "pub fn block_causal(scale: Option<f32>, mask: BlockCausal) -> Self",
        "pub fn vdn_window(scale: Option<f32>, mask: VdnWindow) -> Self", "pub fn kv_window() -> Self",
        "pub fn kv_window_with(flash: bool) -> Self",
    ):
        assert sig in src, sig
    # every ffi function a shim calls is declared
    _, rdecl = rust_declarations()
    for name in set(re.findall(r"ffi::(fv_[a-z0-9_]+)", src)):
        assert name in rdecl, name
    toml = open(os.path.join(CRATE, "Cargo.toml")).read()
    build = open(os.path.join(CRATE, "build.rs")).read()
    assert 'name = "fastvideo-hip-sdpa"' in toml and "cargo:rustc-link-lib=dylib=fv_sdpa_hip" in build
