// Source only (never compiled in this pipeline).  Links libeclat_hip.so, whose location is
// given by ECLAT_HIP_LIB_DIR (the directory holding the built library).
fn main() {
    if let Ok(dir) = std::env::var("ECLAT_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=eclat_hip");
    println!("cargo:rerun-if-env-changed=ECLAT_HIP_LIB_DIR");
}
