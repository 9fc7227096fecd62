// build.rs for the reference crate with the `hip` feature: builds liblumen_hip.so with hipcc for gfx950 and links it.
//
//   LUMEN_HIP_SRC_DIR  the lumen_amd/csrc directory of this repository (its Makefile drives
//                      `hipcc --offload-arch=gfx950 -O3 ...` over the .hip sources and leaves ../lib/liblumen_hip.so);
//                      when set, the library is (re)built from there before it is linked
//   LUMEN_HIP_LIB_DIR  the directory that holds a library built beforehand (default: $LUMEN_HIP_SRC_DIR/../lib)
//   HIPCC              the compiler (default /opt/rocm/bin/hipcc)
//
// UNCOMPILED: no Rust toolchain exists where this library is built.
use std::path::PathBuf;
use std::process::Command;

fn main() {
    println!("cargo:rerun-if-env-changed=LUMEN_HIP_SRC_DIR");
    println!("cargo:rerun-if-env-changed=LUMEN_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=HIPCC");
    if std::env::var_os("CARGO_FEATURE_HIP").is_none() {
        return;
    }
    let src = std::env::var_os("LUMEN_HIP_SRC_DIR").map(PathBuf::from);
    if let Some(src) = &src {
        println!("cargo:rerun-if-changed={}", src.display());
        let hipcc = std::env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".to_string());
        let jobs = std::env::var("NUM_JOBS").unwrap_or_else(|_| "8".to_string());
        let status = Command::new("make")
            .arg("-C")
            .arg(src)
            .arg(format!("-j{jobs}"))
            .arg(format!("HIPCC={hipcc}"))
            .arg("ARCH=gfx950")
            .status()
            .expect("could not run make for liblumen_hip.so");
        assert!(status.success(), "building liblumen_hip.so with {hipcc} failed");
    }
    let dir = match (std::env::var_os("LUMEN_HIP_LIB_DIR"), &src) {
        (Some(d), _) => PathBuf::from(d),
        (None, Some(src)) => src.join("..").join("lib"),
        (None, None) => panic!("set LUMEN_HIP_SRC_DIR (build the library) or LUMEN_HIP_LIB_DIR (a built one)"),
    };
    let dir = dir.display();
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=lumen_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
}
