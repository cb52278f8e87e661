// Builds librmlk_hip.so from the HIP sources with hipcc (gfx950) and links it.
// Replaces cuda/build.rs:11-35 of the reference (bindgen_cuda compiling src/ptx/*.cu to PTX):
// the HIP kernels are compiled to a code object inside one shared library, so there is no
// run-time module loading and no generated ptx.rs.
use std::{env, path::PathBuf, process::Command};

fn main() {
    let out = PathBuf::from(env::var("OUT_DIR").expect("OUT_DIR"));
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").expect("CARGO_MANIFEST_DIR"));
    // the kernel sources live next to the Python package of this repository
    let csrc = manifest.join("..").join("rmlk_amd").join("csrc");
    let lib_dir = match env::var("RMLK_HIP_LIB_DIR") {
        Ok(dir) if env::var("CARGO_FEATURE_PREBUILT").is_ok() => PathBuf::from(dir),
        _ => {
            let status = Command::new("make")
                .arg("-C")
                .arg(&csrc)
                .arg("-j16")
                .arg(format!("OUT_DIR={}", out.display()))
                .arg(format!("BUILD_DIR={}", out.join("obj").display()))
                .status()
                .expect("make / hipcc not found (ROCm 7 with /opt/rocm/bin/hipcc is required)");
            assert!(status.success(), "building librmlk_hip.so failed");
            out.clone()
        }
    };
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}", lib_dir.display());
    println!("cargo:rustc-link-lib=dylib=rmlk_hip");
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", lib_dir.display());
    println!("cargo:rerun-if-changed={}", csrc.display());
    println!("cargo:rerun-if-changed={}", manifest.join("..").join("include").join("rmlk_hip.h").display());
    println!("cargo:rerun-if-env-changed=RMLK_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
}
