//! Tells the linker where liblng_hip.so is: `LNG_HIP_LIB_DIR` names the directory that
//! `python -m loadngo_amd.build` wrote the library into (`loadngo_amd/` of the library's repository).
//! The library's only run-time dependency is ROCm's libamdhip64.so.
fn main() {
    println!("cargo:rerun-if-env-changed=LNG_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("LNG_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=lng_hip");
}
