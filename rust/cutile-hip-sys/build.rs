// Tells rustc where libcutile_hip.so is.  CUTILE_HIP_LIB_DIR names the directory; without it the in-tree build
// output (cutile-rs_amd/lib, made by `python cutile-rs_amd/build.py`) is used.  The library carries its gfx950 code
// objects inside it and opens libamdhip64 itself on first use, so nothing else has to be linked.
// Not compiled in the environment this was written in (no Rust toolchain there).
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=CUTILE_HIP_LIB_DIR");
    println!("cargo:rerun-if-changed=../../include/cutile_hip.h");
    let dir = match env::var_os("CUTILE_HIP_LIB_DIR") {
        Some(d) => PathBuf::from(d),
        None => PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../../cutile-rs_amd/lib"),
    };
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=cutile_hip");
    // libcutile_hip_scratch.so (the device-resident scratch of the no-alloc entry point) is opened by the library
    // itself from its own directory; an rpath lets the final binary find both without LD_LIBRARY_PATH.
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
