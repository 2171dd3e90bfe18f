// build.rs for the crate root: compiles the HIP sources of libag_hip.so for gfx950 with hipcc and
// links the result.  UNCOMPILED in this repository (no Rust toolchain in the image it was written
// in); the hipcc lines are the ones rust-autograd_amd/csrc/build.sh runs.
//
// Expects the sources under `ag_hip/` next to Cargo.toml: ag_hip/csrc = rust-autograd_amd/csrc,
// ag_hip/include = include/.  Needs ROCm's hipcc on PATH (or HIPCC set).
use std::{env, path::PathBuf, process::Command};

const SOURCES: &[&str] = &[
    "common", "im2col", "gemm", "gemm_dl", "conv", "conv_s2", "pool", "reduce", "adam", "elementwise",
];

fn main() {
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "hipcc".into());
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let src = PathBuf::from("ag_hip/csrc");
    let mut objects = Vec::new();
    for name in SOURCES {
        let object = out.join(format!("{name}.o"));
        let mut cmd = Command::new(&hipcc);
        cmd.args([
            "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
            // keep the compiler from forming packed-f32 instructions
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Iag_hip/include", "-Iag_hip/csrc", "-c",
        ]);
        match *name {
            // AdamOp's separately rounded multiplies and adds (gradient_descent_ops/adam.rs:16-50)
            "adam" => { cmd.arg("-ffp-contract=off"); }
            "gemm_dl" => { cmd.args(["-Wno-inline-asm", "-Wno-pass-failed"]); }
            _ => {}
        }
        cmd.arg(src.join(format!("{name}.hip"))).arg("-o").arg(&object);
        assert!(cmd.status().expect("hipcc not found").success(), "hipcc failed on {name}.hip");
        println!("cargo:rerun-if-changed=ag_hip/csrc/{name}.hip");
        objects.push(object);
    }
    let lib = out.join("libag_hip.so");
    let status = Command::new(&hipcc)
        .args(["--offload-arch=gfx950", "-shared", "-fPIC", "-o"])
        .arg(&lib)
        .args(&objects)
        .status()
        .expect("hipcc not found");
    assert!(status.success(), "linking libag_hip.so failed");
    println!("cargo:rerun-if-changed=ag_hip/include/ag_hip.h");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=ag_hip");
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
}
