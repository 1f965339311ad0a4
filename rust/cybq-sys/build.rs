// Tells cargo where libcybq.so lives.  CYBQ_LIB_DIR overrides the default, which is the
// in-tree build output of this repository (cyb_amd/lib, two directories up from the crate).
use std::env;
use std::path::PathBuf;

fn main() {
    let dir = env::var_os("CYBQ_LIB_DIR").map(PathBuf::from).unwrap_or_else(|| {
        PathBuf::from(env::var_os("CARGO_MANIFEST_DIR").expect("cargo sets CARGO_MANIFEST_DIR"))
            .join("..")
            .join("..")
            .join("cyb_amd")
            .join("lib")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=cybq");
    println!("cargo:rerun-if-env-changed=CYBQ_LIB_DIR");
}
