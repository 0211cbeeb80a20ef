// Links libluminal_hip.so; LUMINAL_HIP_LIB_DIR points at the directory that holds it
// (luminal_amd/ in the backend's repository after `python -m luminal_amd.build`).
fn main() {
    if let Ok(dir) = std::env::var("LUMINAL_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=luminal_hip");
    println!("cargo:rerun-if-env-changed=LUMINAL_HIP_LIB_DIR");
}
