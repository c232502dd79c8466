//! Links `libnative_hip.so`, the C-ABI library of `include/native_hip.h`.
//!
//! The library is built from the HIP sources with
//! `python -c 'import __graft_entry__ as g; g.build()'` (plain `hipcc --offload-arch=gfx950`);
//! `NATIVE_HIP_LIB_DIR` names the directory that holds it (default: `../llama-rust_amd`).
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=NATIVE_HIP_LIB_DIR");
    if std::env::var_os("CARGO_FEATURE_HIP").is_none() {
        return; // host-only build: Shape, validate and their tests need no library
    }
    let dir = std::env::var_os("NATIVE_HIP_LIB_DIR")
        .map(PathBuf::from)
        .unwrap_or_else(|| {
            PathBuf::from(std::env::var_os("CARGO_MANIFEST_DIR").unwrap_or_default())
                .join("..")
                .join("llama-rust_amd")
        });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=native_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
