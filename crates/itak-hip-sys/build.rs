//! Links `libitak_hip_kv.so`. The library is built outside cargo (hipcc, gfx950) by
//! `python itak-torch-rebuild_amd/build.py`; `ITAK_HIP_KV_LIB_DIR` names the directory that
//! holds it (default: `itak-torch-rebuild_amd/lib` beside this workspace).

use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=ITAK_HIP_KV_LIB_DIR");
    let dir = env::var_os("ITAK_HIP_KV_LIB_DIR").map(PathBuf::from).unwrap_or_else(|| {
        let manifest = PathBuf::from(env::var_os("CARGO_MANIFEST_DIR").expect("cargo sets it"));
        manifest.join("..").join("..").join("itak-torch-rebuild_amd").join("lib")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=itak_hip_kv");
    // The HIP runtime the library itself links.
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
}
