"""The Rust host side (rust/qproj-sys, rust/qproj) cannot be compiled in this image (no cargo / rustc).  These
checks keep it in step with what IS built: the extern "C" block names exactly the functions include/qproj.h
declares, with the same number of arguments; the constants agree; build.rs compiles the Makefile's sources with
the Makefile's flags; the safe wrapper calls only functions the sys crate declares."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def read(*parts):
    return open(os.path.join(ROOT, *parts)).read()


def c_declarations():
    header = re.sub(r"/\*.*?\*/", "", read("include", "qproj.h"), flags=re.S)
    decls = {}
    for name, args in re.findall(r"\b(qproj_[a-z_0-9]+)\s*\(([^;{]*?)\)\s*;", header, flags=re.S):
        args = args.strip()
        decls[name] = 0 if args in ("", "void") else len(args.split(","))
    return decls


def rust_declarations():
    src = re.sub(r"//[^\n]*", "", read("rust", "qproj-sys", "src", "lib.rs"))
    block = src[src.index('extern "C" {'):]
    decls = {}
    for name, args in re.findall(r"pub fn (qproj_[a-z_0-9]+)\s*\(([^;]*?)\)\s*(?:->[^;]*)?;", block, flags=re.S):
        args = args.strip()
        decls[name] = 0 if not args else len([a for a in args.split(",") if a.strip()])
    return decls


def test_extern_block_matches_the_header():
    c, r = c_declarations(), rust_declarations()
    assert len(c) >= 28
    assert set(c) == set(r), set(c) ^ set(r)
    assert c == r, {k: (c[k], r[k]) for k in c if c[k] != r[k]}


def test_constants_agree():
    header = read("include", "qproj.h")
    rust = read("rust", "qproj-sys", "src", "lib.rs")
    for name, value in re.findall(r"\b(QPROJ_(?:OK|ERR_[A-Z_]+|ELIGIBILITY_[A-Z]+))\s*=\s*(\d+)", header):
        assert re.search(rf"pub const {name}: c_int = {value};", rust), name
    for name, value in re.findall(r"\b(QPROJ_(?:TYPE|ACT)_[A-Z0-9_]+)\s*=\s*(\d+)", header):
        assert re.search(rf"pub const {name}: c_int = {value};", rust), name
    assert "#define QPROJ_NOALLOC_SCRATCH_BYTES (64u << 20)" in header and "QPROJ_NOALLOC_SCRATCH_BYTES: usize = 64 << 20" in rust
    assert "#define QPROJ_PROBE_MAX_DEVICES 16" in header and "QPROJ_PROBE_MAX_DEVICES: usize = 16" in rust
    # the eligibility struct: same fields in the same order
    c_fields = re.findall(r"\b(state|driver_api|runtime_api|n_devices|architectures|hardware_labels|runtime_library|diagnostic)\b",
                          header[header.index("typedef struct qproj_eligibility"):header.index("} qproj_eligibility;")])
    r_fields = re.findall(r"pub (\w+):", rust[rust.index("pub struct qproj_eligibility"):rust.index('extern "C"')])
    assert c_fields == r_fields


def test_build_rs_compiles_what_the_makefile_compiles():
    mk = read("magnitude_amd", "csrc", "Makefile")
    rs = read("rust", "qproj-sys", "build.rs")
    mk_srcs = re.search(r"SRCS = (.*?)\nOBJS", mk, flags=re.S).group(1).replace("\\\n", " ").split()
    rs_srcs = re.findall(r'"([a-z_0-9]+\.hip)"', rs)
    assert sorted(mk_srcs) == sorted(rs_srcs)
    for f in mk_srcs:
        assert os.path.exists(os.path.join(ROOT, "magnitude_amd", "csrc", f))
    for flag in ("--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-packed-fp32-ops"):
        assert flag in rs and (flag in mk or flag == "--offload-arch=gfx950"), flag
    mk_hdrs = re.search(r"build/%\.o: %\.hip (.*)\n", mk).group(1).split()
    for h in mk_hdrs:
        if not h.startswith(".."):
            assert f'"{h}"' in rs, h


def test_safe_wrapper_calls_only_declared_functions():
    r = rust_declarations()
    wrapper = read("rust", "qproj", "src", "lib.rs")
    used = set(re.findall(r"sys::(qproj_[a-z_0-9]+)\(", wrapper))
    assert used and used <= set(r), used - set(r)
    assert 'qproj-sys = { path = "../qproj-sys" }' in read("rust", "qproj", "Cargo.toml")
