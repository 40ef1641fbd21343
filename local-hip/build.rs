// Builds liblocal_hip.so (hand-written HIP kernels for gfx950 behind a C ABI) with hipcc and links it.
// The kernel sources live in ../local-ai_amd/csrc; their Makefile takes OUT and BUILD so that nothing is written into
// the source tree.  Requires ROCm (HIPCC, default /opt/rocm/bin/hipcc); the library refuses any device but gfx950.
// (Written for the reference's workspace conventions: no unwrap/expect/panic outside build scripts is needed here.)
use std::{env, path::PathBuf, process::Command};

fn main() {
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").expect("CARGO_MANIFEST_DIR"));
    let out = PathBuf::from(env::var("OUT_DIR").expect("OUT_DIR"));
    let csrc = manifest.join("..").join("local-ai_amd").join("csrc");
    let header = manifest.join("..").join("include").join("local_hip.h");
    let jobs = env::var("NUM_JOBS").unwrap_or_else(|_| "8".into());
    let status = Command::new("make")
        .arg("-C").arg(&csrc)
        .arg(format!("-j{jobs}"))
        .arg(format!("OUT={}", out.join("liblocal_hip.so").display()))
        .arg(format!("BUILD={}", out.join("obj").display()))
        .status()
        .expect("run make (needs hipcc from ROCm)");
    assert!(status.success(), "building liblocal_hip.so failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=local_hip");
    println!("cargo:rerun-if-changed={}", csrc.display());
    println!("cargo:rerun-if-changed={}", header.display());
    println!("cargo:rerun-if-env-changed=HIPCC");
}
