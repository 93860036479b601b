// Tells cargo where libtenferro_hip.so lives.  TENFERRO_HIP_LIB_DIR names the directory that holds the built library
// (the tenferro-rs_amd/ directory of the backend's source tree after `python tenferro-rs_amd/build.py`).
fn main() {
    println!("cargo:rerun-if-env-changed=TENFERRO_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("TENFERRO_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=tenferro_hip");
}
