// Links libtract_rocm.so, which `python -m tract_amd.build` makes with hipcc --offload-arch=gfx950.
// TRACT_ROCM_LIB_DIR names the directory that holds it; TRACT_ROCM_INCLUDE_DIR, when set, makes a change of the
// header rebuild the crate (src/ffi.rs is generated from that header by include/gen_rust_ffi.py --write).
fn main() {
    let dir = std::env::var("TRACT_ROCM_LIB_DIR")
        .expect("set TRACT_ROCM_LIB_DIR to the directory that holds libtract_rocm.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=tract_rocm");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    println!("cargo:rerun-if-env-changed=TRACT_ROCM_LIB_DIR");
    if let Ok(inc) = std::env::var("TRACT_ROCM_INCLUDE_DIR") {
        println!("cargo:rerun-if-changed={inc}/tract_rocm.h");
    }
}
