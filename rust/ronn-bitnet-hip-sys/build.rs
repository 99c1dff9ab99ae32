// Tells cargo where libronn_bitnet_hip.so lives.
//
// RONN_BITNET_HIP_DIR names the directory that holds the built library (the `ronn_amd/`
// directory of its repository after `make -C ronn_amd/csrc`).  The directory is also put in
// the run-time search path of whatever links this crate, so test binaries find the library.
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=RONN_BITNET_HIP_DIR");
    let dir = match env::var("RONN_BITNET_HIP_DIR") {
        Ok(d) => PathBuf::from(d),
        Err(_) => panic!(
            "set RONN_BITNET_HIP_DIR to the directory that contains libronn_bitnet_hip.so \
             (built with `make -C ronn_amd/csrc` for gfx950)"
        ),
    };
    if !dir.join("libronn_bitnet_hip.so").exists() {
        panic!("{} does not contain libronn_bitnet_hip.so", dir.display());
    }
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=ronn_bitnet_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
