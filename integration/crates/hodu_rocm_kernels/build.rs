//! Links the prebuilt `libhodu_rocm_kernels.so`, or builds it with hipcc from the kernel sources.
//!
//!   HODU_ROCM_KERNELS_LIB = directory that holds libhodu_rocm_kernels.so   -> link it
//!   HODU_ROCM_KERNELS_SRC = directory with the .hip / .cpp sources + include/ -> hipcc --offload-arch=gfx950
//!
//! The gfx950 code object is embedded in the shared library; nothing is compiled at run time (the CUDA sibling
//! embeds PTX and loads it through the driver: crates/hodu_cuda_kernels/build.rs:44-95).
use std::{env, path::PathBuf, process::Command};

fn main() {
    println!("cargo:rerun-if-env-changed=HODU_ROCM_KERNELS_LIB");
    println!("cargo:rerun-if-env-changed=HODU_ROCM_KERNELS_SRC");
    if let Ok(dir) = env::var("HODU_ROCM_KERNELS_LIB") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-lib=dylib=hodu_rocm_kernels");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
        return;
    }
    let src = PathBuf::from(env::var("HODU_ROCM_KERNELS_SRC").expect(
        "set HODU_ROCM_KERNELS_LIB (prebuilt library) or HODU_ROCM_KERNELS_SRC (kernel sources) to build hodu_rocm_kernels",
    ));
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let lib = out.join("libhodu_rocm_kernels.so");
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into());
    let mut cmd = Command::new(hipcc);
    cmd.args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared"])
        // no packed-f32 instruction forms, and the K loops are fully unrolled compile-time schedules
        .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
        .args(["-mllvm", "-pragma-unroll-threshold=200000"])
        .arg(format!("-I{}", src.join("include").display()))
        .arg(format!("-I{}", src.join("csrc").display()));
    for entry in std::fs::read_dir(src.join("csrc")).expect("csrc/ not found") {
        let path = entry.unwrap().path();
        match path.extension().and_then(|e| e.to_str()) {
            Some("hip") => { cmd.arg(&path); }
            Some("cpp") => { cmd.args(["-x", "hip"]).arg(&path); }
            _ => {}
        }
        println!("cargo:rerun-if-changed={}", path.display());
    }
    cmd.arg("-o").arg(&lib);
    let status = cmd.status().expect("hipcc could not be started");
    assert!(status.success(), "hipcc failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=hodu_rocm_kernels");
}
