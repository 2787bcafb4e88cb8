// Tells cargo where libsaragossa_kv.so lives: SARAGOSSA_KV_LIB_DIR, or ../../saragossa_amd
// (where `make -C saragossa_amd/csrc` leaves it) relative to this crate.
use std::{env, path::PathBuf};

fn main() {
    let dir = env::var("SARAGOSSA_KV_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../../saragossa_amd")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=saragossa_kv");
    println!("cargo:rerun-if-env-changed=SARAGOSSA_KV_LIB_DIR");
}
