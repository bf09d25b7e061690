// UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).
//
// Build script of the crate: one hipcc compilation of the attention library for gfx950 and nothing else, archived
// and linked statically, with the HIP runtime as the only dynamic dependency.  It takes the place of the part of
// flame-core's build.rs that loops nvcc over the CUDA sources and links cudart / cuBLAS / cuDNN
// (build.rs:251-347 there; the cuDNN discovery at :53-86 has no counterpart: nothing is discovered, nothing is
// optional).  Flags are the ones flame_amd/build.py uses, so that the archive is the library the tests ran.
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

fn run(cmd: &mut Command, what: &str) {
    let status = cmd.status().unwrap_or_else(|e| panic!("{what}: cannot start: {e}"));
    if !status.success() {
        panic!("{what} failed with {status:?}");
    }
}

fn main() {
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").expect("CARGO_MANIFEST_DIR"));
    let repo = manifest.parent().expect("the crate sits one level below the repository root").to_path_buf();
    let csrc = repo.join("flame_amd").join("csrc");
    let out = PathBuf::from(env::var("OUT_DIR").expect("OUT_DIR"));
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| format!("{rocm}/bin/hipcc"));
    if !Path::new(&hipcc).exists() {
        panic!("hipcc not found at {hipcc}: set HIPCC or ROCM_PATH (this crate builds for gfx950 only)");
    }

    for entry in std::fs::read_dir(&csrc).expect("flame_amd/csrc") {
        let path = entry.expect("dir entry").path();
        println!("cargo:rerun-if-changed={}", path.display());
    }
    println!("cargo:rerun-if-changed={}", repo.join("include").join("flame_attn.h").display());
    println!("cargo:rerun-if-env-changed=HIPCC");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");

    // the version string names the compiler, as the Python build does: the static checks of the hand-emitted
    // instructions only hold for the assembly that this compiler generates
    let version = Command::new(&hipcc).arg("--version").output().expect("hipcc --version");
    let text = String::from_utf8_lossy(&version.stdout);
    let hip = text
        .lines()
        .find_map(|l| l.strip_prefix("HIP version:"))
        .map(|s| s.trim().to_string())
        .unwrap_or_else(|| "?".to_string());

    let obj = out.join("flame_attn.o");
    let mut cc = Command::new(&hipcc);
    cc.args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC"])
        // packed fp32 vector operations stay off for every HIP source of this library
        .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
        .args(["-Wall", "-Wno-unused-function", "-Wno-inline-asm"])
        .arg(format!("-DFLAME_ATTN_HIPCC_VERSION=\"{hip} (cargo)\""))
        .arg("-c")
        .arg(csrc.join("flame_attn.hip"))
        .arg("-o")
        .arg(&obj);
    run(&mut cc, "hipcc flame_attn.hip");

    let lib = out.join("libflame_attn_hip.a");
    let _ = std::fs::remove_file(&lib);
    let mut ar = Command::new("ar");
    ar.arg("rcs").arg(&lib).arg(&obj);
    run(&mut ar, "ar");

    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=static=flame_attn_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
    // for dependents: where the header lives (DEP_FLAME_ATTN_HIP_INCLUDE)
    println!("cargo:include={}", repo.join("include").display());
}
