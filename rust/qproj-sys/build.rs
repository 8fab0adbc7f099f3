// Builds libqproj.so from the HIP sources with hipcc for gfx950 and links it.
// Same sources and flags as magnitude_amd/csrc/Makefile (a test keeps the two lists equal).
use std::{env, path::PathBuf, process::Command};

const SOURCES: &[&str] = &[
    "qproj_api.hip", "kernels_dequant.hip", "kernels_actquant.hip", "kernels_gemv.hip", "kernels_decode.hip",
    "kernels_gemv_mfma.hip", "kernels_gemv_f32.hip", "kernels_moe.hip", "kernels_moe_decode.hip", "kernels_gemm.hip", "kernels_gemm_q6k.hip",
    "kernels_rmsnorm.hip",
];
const HEADERS: &[&str] = &[
    "qproj_internal.h", "qproj_device.h", "gemv_frags.h", "actquant_device.h", "gemm_tiles.h", "lds_direct.h",
];
const HIPFLAGS: &[&str] = &[
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
];

fn main() {
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let csrc = manifest.join("../../magnitude_amd/csrc");
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into());
    let mut objects = vec![];
    for src in SOURCES {
        let obj = out.join(format!("{src}.o"));
        let ok = Command::new(&hipcc)
            .args(HIPFLAGS)
            .arg("-c")
            .arg(csrc.join(src))
            .arg("-o")
            .arg(&obj)
            .status()
            .expect("hipcc not found (set HIPCC)")
            .success();
        assert!(ok, "hipcc failed on {src}");
        objects.push(obj);
        println!("cargo:rerun-if-changed={}", csrc.join(src).display());
    }
    for h in HEADERS {
        println!("cargo:rerun-if-changed={}", csrc.join(h).display());
    }
    println!("cargo:rerun-if-changed={}", manifest.join("../../include/qproj.h").display());
    let lib = out.join("libqproj.so");
    let ok = Command::new(&hipcc)
        .args(["--offload-arch=gfx950", "-shared", "-fPIC", "-o"])
        .arg(&lib)
        .args(&objects)
        .status()
        .expect("hipcc link")
        .success();
    assert!(ok, "linking libqproj.so failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=qproj");
    println!("cargo:rustc-link-arg=-Wl,-rpath,$ORIGIN/../runtime"); // artifact-owned runtime libraries
}
