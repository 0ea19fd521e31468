// Links libcatgrad_hip.so.  CATGRAD_HIP_LIB_DIR names the directory that holds it
// (catgrad-rs_amd/csrc after `make -C catgrad-rs_amd/csrc`).
fn main() {
    println!("cargo:rerun-if-env-changed=CATGRAD_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("CATGRAD_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={}", dir);
        println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir);
    }
    println!("cargo:rustc-link-lib=dylib=catgrad_hip");
}
