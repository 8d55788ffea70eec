//! Link libstrix_mi355.so only when the `mi355` feature is on (the counterpart of
//! crates/strix-backend-rocm/build.rs).  The library itself is built by
//! `python strix.rs_amd/build.py` (hipcc, gfx950) and carries the HIP runtime dependency.

fn main() {
    println!("cargo:rerun-if-env-changed=STRIX_MI355_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    if std::env::var("CARGO_FEATURE_MI355").is_err() {
        return;
    }
    let manifest = std::env::var("CARGO_MANIFEST_DIR").unwrap_or_else(|_| ".".to_string());
    let dir = std::env::var("STRIX_MI355_LIB_DIR")
        .unwrap_or_else(|_| format!("{manifest}/../../strix.rs_amd"));
    let rocm = std::env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=strix_mi355");
    // the binary finds the library and the HIP runtime it depends on at run time
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{rocm}/lib");
}
