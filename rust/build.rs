// build.rs for the reference crate with the `hip` feature: links liblumen_hip.so.
// LUMEN_HIP_LIB_DIR = the directory that holds the library (…/lumen_amd/lib after `make -C lumen_amd/csrc`).
// UNCOMPILED: no Rust toolchain exists where this library is built.
fn main() {
    println!("cargo:rerun-if-env-changed=LUMEN_HIP_LIB_DIR");
    if std::env::var_os("CARGO_FEATURE_HIP").is_none() {
        return;
    }
    let dir = std::env::var("LUMEN_HIP_LIB_DIR").expect("set LUMEN_HIP_LIB_DIR to the directory of liblumen_hip.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=lumen_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
}
