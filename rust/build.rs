// build.rs of the descent crate once `spark` and `shaderc` are gone: links libdescent_hip.so.
// DESCENT_HIP_LIB_DIR names the directory that holds the library (the backend repository builds it in
// descent_amd/csrc/ with `python descent_amd/csrc/build.py`); the HIP runtime and hipRTC are dependencies of that
// library, not of the crate.
fn main() {
    let dir = std::env::var("DESCENT_HIP_LIB_DIR").unwrap_or_else(|_| "/opt/descent_hip/lib".to_string());
    println!("cargo:rustc-link-search=native={}", dir);
    println!("cargo:rustc-link-lib=dylib=descent_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir);
    println!("cargo:rerun-if-env-changed=DESCENT_HIP_LIB_DIR");
}
