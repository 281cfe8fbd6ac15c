// Points cargo at libturq.so.  TURQ_LIB_DIR names the directory that holds it (the `tur_amd/` directory of the libturq tree
// after `make -C tur_amd/csrc`); without it the library is expected next to this crate's tree, two levels up.
use std::env;
use std::path::PathBuf;

fn main() {
    let dir = env::var_os("TURQ_LIB_DIR")
        .map(PathBuf::from)
        .unwrap_or_else(|| PathBuf::from(env::var_os("CARGO_MANIFEST_DIR").unwrap()).join("../../tur_amd"));
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=turq");
    // the library finds the HIP runtime through its own rpath; the binary needs one for libturq itself
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    println!("cargo:rerun-if-env-changed=TURQ_LIB_DIR");
}
