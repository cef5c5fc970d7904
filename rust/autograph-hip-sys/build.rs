// Tells rustc where libautograph_hip.so lives: AUTOGRAPH_HIP_LIB_DIR, or the in-tree build
// directory of this repository (autograph_amd/lib, produced by `make -C autograph_amd/csrc`).
use std::{env, path::PathBuf};

fn main() {
    let dir = env::var("AUTOGRAPH_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../../autograph_amd/lib")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=autograph_hip");
    println!("cargo:rerun-if-env-changed=AUTOGRAPH_HIP_LIB_DIR");
}
